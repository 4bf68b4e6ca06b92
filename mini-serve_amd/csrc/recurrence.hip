// Linear recurrences over a matrix state per (request, head), token by token:
//     S_t = a_t S_(t-1) + b_t k_t v_t^T,   o_t = S_t^T q_t          (S: [D, E], k, q: [D], v: [E])
// in two forms that differ in where a_t and b_t come from:
//   MS_REC_DECAY: a_t = decay[head] (a constant per head), b_t = 1; o_t as above.
//   MS_REC_EXP_GATES: a log input gate i_t and a log forget gate f_t per head and token, made bounded by a soft cap,
//       i = cap tanh((x_i + bias_i) / cap), f = logsigmoid(cap tanh((x_f + bias_f) / cap)), and a running maximum
//       m_t = max(f_t + m_(t-1), i_t) (m starts at 0) that keeps the exponentials in range:
//       a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t); a vector n_t = a_t n_(t-1) + b_t k_t beside S;
//       o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
// q, k, v (and the gates' inputs) are columns of one float32 matrix x [tokens, ld] (the layer's projections);
// an activation (none or SiLU) is applied to q, k and v on the way in, q is then scaled by q_scale. Everything
// is float32. The state lives in S [slots, H, D, E] (and n [slots, H, D], m [slots, H]); a row whose
// sequence starts in this step (starts[row] == 0) begins from zero, every other row from its slot; the state after
// the row's last token is written back.
//
// One block of 256 threads per (row, head) walks the row's tokens in order with the state in registers:
// thread (s, e) holds S[d][e] for d = s, s + NS, ... (NS = 256 / EP slices, EP the power of two that holds E),
// adds its part of o_t[e], and the slices' parts meet in LDS in ascending s. What an output element is summed
// from, and in which order, depends on D and E alone: a token's result does not depend on how the sequence was
// cut into steps or batched.
#include "common.h"

#define MS_REC_DECAY 0
#define MS_REC_EXP_GATES 1

struct RecurrenceArgs {
  const float* x;
  int ld, q_off, k_off, v_off, i_off, f_off;
  int H, D, E, act, mode;
  float q_scale, cap;
  const float* decay;
  const void* i_bias;
  const void* f_bias;
  int bias_is_bf16;
  float* S;
  float* n;
  float* m;
  const int* row_start;
  const int* starts;
  const int* state_slots;
  float* out;
};

__device__ __forceinline__ float rec_act(float v, int act) { return act ? v / (1.f + expf(-v)) : v; }
__device__ __forceinline__ float rec_bias(const void* b, int is_bf16, int h) {
  if (b == nullptr) return 0.f;
  return is_bf16 ? to_f32(((const bf16*)b)[h]) : ((const float*)b)[h];
}
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int PM>
__global__ __launch_bounds__(256) void gated_recurrence_kernel(RecurrenceArgs a, int EP) {
  __shared__ float qs[2][256], ks[2][256];
  __shared__ float red[256];
  __shared__ float wred[2][4];
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int D = a.D, E = a.E;
  const int NS = 256 / EP, e = tid % EP, s = tid / EP;
  const int per = (D + NS - 1) / NS;
  const int t0 = a.row_start[b], t1 = a.row_start[b + 1];
  const bool fresh = a.starts[b] == 0;
  const size_t slot = (size_t)a.state_slots[b];
  float* Sg = a.S + (slot * a.H + h) * (size_t)D * E;
  const bool gates = a.mode == MS_REC_EXP_GATES;
  float S[PM];
#pragma unroll
  for (int i = 0; i < PM; ++i) {
    const int d = s + i * NS;
    S[i] = (!fresh && i < per && d < D && e < E) ? Sg[(size_t)d * E + e] : 0.f;
  }
  float nv = 0.f, m = 0.f;
  if (gates && !fresh) {
    if (tid < D) nv = a.n[(slot * a.H + h) * D + tid];
    m = a.m[slot * a.H + h];
  }
  const float decay = gates ? 0.f : a.decay[h];
  const float bi = gates ? rec_bias(a.i_bias, a.bias_is_bf16, h) : 0.f;
  const float bf = gates ? rec_bias(a.f_bias, a.bias_is_bf16, h) : 0.f;
  for (int t = t0; t < t1; ++t) {
    const float* xr = a.x + (size_t)t * a.ld;
    const int buf = (t - t0) & 1;
    float fs = decay, is = 1.f;
    if (gates) {
      const float gi = a.cap * tanhf((xr[a.i_off + h] + bi) / a.cap);
      const float gf = log_sigmoid(a.cap * tanhf((xr[a.f_off + h] + bf) / a.cap));
      const float m_new = fmaxf(gf + m, gi);
      fs = expf(gf + m - m_new);
      is = expf(gi - m_new);
      m = m_new;
    }
    float kd = 0.f, qd = 0.f;
    if (tid < D) {
      qd = rec_act(xr[a.q_off + h * D + tid], a.act) * a.q_scale;
      kd = rec_act(xr[a.k_off + h * D + tid], a.act);
      qs[buf][tid] = qd;
      ks[buf][tid] = kd;
    }
    if (gates) {
      nv = fs * nv + is * kd;  // threads beyond D carry zeros
      const float part = wave_sum(nv * qd);
      if (tid % WAVE == 0) wred[buf][tid / WAVE] = part;
    }
    const float v = e < E ? rec_act(xr[a.v_off + h * E + e], a.act) : 0.f;
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < PM; ++i) {
      const int d = s + i * NS;
      if (i < per && d < D) {
        S[i] = fs * S[i] + is * ks[buf][d] * v;
        acc += S[i] * qs[buf][d];
      }
    }
    if (NS > 1) {
      __syncthreads();  // the previous token's sums have been read
      red[tid] = acc;
      __syncthreads();
      if (s == 0) {
        acc = red[e];
        for (int j = 1; j < NS; ++j) acc += red[j * EP + e];
      }
    }
    if (s == 0 && e < E) {
      if (gates) {
        const float nq = (wred[buf][0] + wred[buf][1]) + (wred[buf][2] + wred[buf][3]);
        acc = acc / (fmaxf(fabsf(nq), expf(-m)) + 1e-6f);
      }
      a.out[(size_t)t * (a.H * E) + h * E + e] = acc;
    }
  }
#pragma unroll
  for (int i = 0; i < PM; ++i) {
    const int d = s + i * NS;
    if (i < per && d < D && e < E) Sg[(size_t)d * E + e] = S[i];
  }
  if (gates) {
    if (tid < D) a.n[(slot * a.H + h) * D + tid] = nv;
    if (tid == 0) a.m[slot * a.H + h] = m;
  }
}

extern "C" int ms_gated_recurrence(const float* x, int ld, int q_off, int k_off, int v_off, int i_off, int f_off, int H, int D,
                                   int E, int act, int mode, float q_scale, float cap, const float* decay, const void* i_bias,
                                   const void* f_bias, int bias_is_bf16, float* S, float* n, float* m, const int* row_start,
                                   const int* starts, const int* state_slots, float* out, int rows, hipStream_t st) {
  if (rows <= 0) return MS_OK;
  if (H <= 0 || D <= 0 || E <= 0 || x == nullptr || S == nullptr || out == nullptr || row_start == nullptr || starts == nullptr ||
      state_slots == nullptr || (act != 0 && act != 1) || q_off < 0 || k_off < 0 || v_off < 0 || q_off + H * D > ld ||
      k_off + H * D > ld || v_off + H * E > ld)
    return MS_BAD_ARG;
  if (mode == MS_REC_DECAY) {
    if (decay == nullptr) return MS_BAD_ARG;
  } else if (mode == MS_REC_EXP_GATES) {
    if (n == nullptr || m == nullptr || !(cap > 0.f) || i_off < 0 || f_off < 0 || i_off + H > ld || f_off + H > ld) return MS_BAD_ARG;
  } else {
    return MS_BAD_ARG;
  }
  if (D > 256 || E > 256 || H > 65535) return MS_UNSUPPORTED;
  int EP = 32;
  while (EP < E) EP *= 2;
  const int per = (D + 256 / EP - 1) / (256 / EP);
  RecurrenceArgs a{x, ld, q_off, k_off, v_off, i_off, f_off, H, D, E, act, mode, q_scale, cap, decay, i_bias, f_bias, bias_is_bf16,
                   S, n, m, row_start, starts, state_slots, out};
  const dim3 grid(rows, H);
  if (per <= 4) gated_recurrence_kernel<4><<<grid, 256, 0, st>>>(a, EP);
  else if (per <= 16) gated_recurrence_kernel<16><<<grid, 256, 0, st>>>(a, EP);
  else if (per <= 64) gated_recurrence_kernel<64><<<grid, 256, 0, st>>>(a, EP);
  else if (per <= 128) gated_recurrence_kernel<128><<<grid, 256, 0, st>>>(a, EP);
  else return MS_UNSUPPORTED;
  return launch_status();
}
