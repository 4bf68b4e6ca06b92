// Causal grouped-query attention over the paged cache, generic form: any query/key head size and any
// value head size up to 256, any head counts, float32 or bfloat16 storage, float32 arithmetic
// (scores, softmax weights and the weighted sum of the values).
//
// One wave per (token, query head); ``token_list`` (optional) names the flat token indices to run. Keys are visited in tiles of 64 aligned to absolute positions
// (tile boundaries at multiples of 64), so what a query computes depends only on its position, the
// window and the cache contents: not on how tokens were cut into steps or batched.
//   scores: lane = key; softmax: running maximum and sum (float32); values: lane = head element.
//
// Cache layouts: keys [pages, Hkv, page_size, D], values [pages, Hkv, Dv, page_size] (transposed
// within the page); block_table[row, i] = page of the row's tokens
// i * page_size .. ; a query at position p of row b sees keys max(0, p - window + 1) .. p
// (window == 0: all keys 0 .. p) and, with a window, the keys 0 .. keep_first - 1 as well (the
// sequence's first tokens stay visible; tiles that hold neither kind of key are skipped, and their
// pages are never read). Query head h reads KV head h / (Hq / Hkv).
//
// Options of the generic form (one wave, or several, per token and head):
//   softcap > 0     a scaled score s becomes softcap * tanh(s / softcap);
//   sinks           one float per query head whose exponential joins the softmax's denominator (it has no key and no
//                   value, is neither scaled nor capped and counts once);
//   value_share     this many consecutive key heads read the same value head (key head i: value head i / value_share;
//                   the value cache then has Hkv / value_share heads): several score maps over one set of values;
//   values_in_keys  the values are the first Dv elements of the key rows themselves (one vector per token serves as
//                   key and as value); no value cache is read;
//   out_f32         the result is written as float32 whatever the storage type (for a consumer that norms it).
// Head sizes up to 256, or, with at most eight waves, up to 1024.
#include "common.h"

#define MAX_HEAD_DIM 256
#define MAX_WIDE_HEAD_DIM 1024

template <typename T> struct Vec16;  // 16 bytes of T
template <> struct Vec16<float> { static constexpr int N = 4; };
template <> struct Vec16<bf16> { static constexpr int N = 8; };

// NW waves per (token, query head): wave w visits the tiles number w, w + NW, ... of those that hold visible keys,
// and the waves' running maxima, sums and outputs meet in LDS in wave order. NW == 1 is the plain form; more waves
// serve steps of few tokens (decode), where one wave per head would walk a long window alone.
template <typename T, int NW, int MAXD>
__global__ __launch_bounds__(NW * WAVE) void paged_attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ token_list,
    const int* __restrict__ token_row, const int* __restrict__ pos, T* __restrict__ out, int Hq, int Hkv, int D, int Dv,
    int page_size, float scale, int window, int keep_first, float softcap, const float* __restrict__ sinks, int value_share,
    int values_in_keys, float* __restrict__ out32) {
  __shared__ __attribute__((aligned(16))) float qs[MAXD];
  __shared__ float ps[NW][WAVE];
  __shared__ float ml[NW][2];
  __shared__ float os[NW > 1 ? NW : 1][NW > 1 ? MAXD : 1];
  constexpr int VN = Vec16<T>::N;
  constexpr int PER = MAXD / WAVE;
  const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int kvh = h / (Hq / Hkv);
  const int Hv = Hkv / value_share, vh = kvh / value_share;  // the value head this key head's scores weigh
  const int p = pos[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int kept = keep_first < lo ? keep_first : lo;  // keys 0 .. kept - 1 are visible beside lo .. p
  const bool vec = D % VN == 0;
  const int* table = block_table + (size_t)token_row[t] * table_width;

  const T* qv = q + (size_t)t * q_stride + (size_t)h * D;
  for (int e = threadIdx.x; e < D; e += NW * WAVE) qs[e] = to_f32(qv[e]);
  __syncthreads();

  float m_run = -INFINITY, l_run = 0.f;
  float o[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) o[i] = 0.f;

  // The tiles that hold a visible key: those of the kept keys, then those from the window's first key on.
  const int kept_tiles = (kept + WAVE - 1) / WAVE;
  const int first_window_tile = lo / WAVE > kept_tiles ? lo / WAVE : kept_tiles;
  const int tiles = kept_tiles + (p / WAVE - first_window_tile + 1);
  for (int ti = wave; ti < tiles; ti += NW) {
    const int j0 = (ti < kept_tiles ? ti : first_window_tile + (ti - kept_tiles)) * WAVE;
    const int j = j0 + lane;
    const bool valid = (j >= lo && j <= p) || j < kept;
    float s = -INFINITY;
    if (valid) {
      const int page = table[j / page_size];
      const T* kp = kc + (((size_t)page * Hkv + kvh) * page_size + (j % page_size)) * D;
      float dot = 0.f;
      if (vec) {
        for (int d = 0; d < D; d += VN) {
          alignas(16) T kv[VN];
          *reinterpret_cast<uint4*>(kv) = *reinterpret_cast<const uint4*>(kp + d);
#pragma unroll
          for (int i = 0; i < VN; ++i) dot = fmaf(qs[d + i], to_f32(kv[i]), dot);
        }
      } else {
        for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32(kp[d]), dot);
      }
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
    }
    const float m_new = fmaxf(m_run, wave_max(s));  // finite: every visited tile holds a visible key
    const float pj = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m_run - m_new);
    l_run = l_run * corr + wave_sum(pj);
    m_run = m_new;
    // A wave's own row of ps: its lanes run in lockstep, so the wave's order of LDS operations is enough.
    __builtin_amdgcn_wave_barrier();
    ps[wave][lane] = pj;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < PER; ++i) o[i] *= corr;
    const int je = j0 + WAVE - 1 < p ? j0 + WAVE - 1 : p;
    if (values_in_keys) {
      // Key by key: the lanes read a run of the key's own row, four keys' loads under way at a time.
      for (int jj = j0; jj <= je; jj += 4) {
        float w[4];
        const T* vp[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int ju = jj + u;
          const bool seen = ju <= je && (ju >= lo || ju < kept);
          w[u] = seen ? ps[wave][ju - j0] : 0.f;
          vp[u] = seen ? kc + (((size_t)table[ju / page_size] * Hkv + kvh) * page_size + (ju % page_size)) * D : nullptr;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int e = lane + i * WAVE;
          if (e >= Dv) continue;
          float vv[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) vv[u] = vp[u] ? to_f32(vp[u][e]) : 0.f;
#pragma unroll
          for (int u = 0; u < 4; ++u) o[i] = fmaf(w[u], vv[u], o[i]);
        }
      }
    } else if (page_size % VN == 0 && WAVE % page_size == 0) {
      // Page by page: a lane fetches the page's tokens of its element as 16-byte runs (the page keeps the tokens of
      // one element side by side). Keys that are not visible carry the weight 0, and fmaf(0, v, o) is o: the sum is
      // the one over the visible keys in ascending order. Pages that were given back are not read.
      for (int jp = j0; jp <= je; jp += page_size) {
        if (jp + page_size <= lo && jp >= kept) continue;  // wholly in the gap
        const int page = table[jp / page_size];
        if (page < 0) continue;
        const T* vp = vc + ((size_t)page * Hv + vh) * Dv * page_size;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int e = lane + i * WAVE;
          if (e >= Dv) continue;
          for (int u0 = 0; u0 < page_size; u0 += VN) {
            alignas(16) T vv[VN];
            *reinterpret_cast<uint4*>(vv) = *reinterpret_cast<const uint4*>(vp + (size_t)e * page_size + u0);
#pragma unroll
            for (int u = 0; u < VN; ++u) o[i] = fmaf(ps[wave][jp - j0 + u0 + u], to_f32(vv[u]), o[i]);
          }
        }
      }
    } else {
      for (int jj = j0; jj <= je; ++jj) {
        if (jj >= kept && jj < lo) {  // the gap inside a tile that holds kept keys or the window's first keys
          jj = lo - 1;
          continue;
        }
        const int page = table[jj / page_size];
        const T* vp = vc + ((size_t)page * Hv + vh) * Dv * page_size + (jj % page_size);
        const float w = ps[wave][jj - j0];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int e = lane + i * WAVE;
          if (e < Dv) o[i] = fmaf(w, to_f32(vp[(size_t)e * page_size]), o[i]);
        }
      }
    }
  }
  if (NW > 1) {
    if (lane == 0) {
      ml[wave][0] = m_run;
      ml[wave][1] = l_run;
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane + i * WAVE;
      if (e < Dv) os[wave][e] = o[i];
    }
    __syncthreads();
    if (wave != 0) return;
    float m_all = ml[0][0];  // wave 0 always has a tile
#pragma unroll
    for (int w = 1; w < NW; ++w) m_all = fmaxf(m_all, ml[w][0]);
    m_run = m_all;
    l_run = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) o[i] = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float c = expf(ml[w][0] - m_all);  // a wave without tiles: exp(-inf) = 0
      l_run += ml[w][1] * c;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int e = lane + i * WAVE;
        if (e < Dv) o[i] += os[w][e] * c;
      }
    }
  }
  T* ov = out + ((size_t)t * Hq + h) * Dv;
  float inv = 1.f / l_run;
  if (sinks) {
    // exp(sink) joins the denominator: both are brought to the larger of the two maxima first
    const float sink = sinks[h], m_all = fmaxf(m_run, sink);
    const float c = expf(m_run - m_all);
    inv = c / (l_run * c + expf(sink - m_all));
  }
  float* ov32 = out32 ? out32 + ((size_t)t * Hq + h) * Dv : nullptr;  // the result unrounded, whatever the storage
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + i * WAVE;
    if (e >= Dv) continue;
    if (ov32) ov32[e] = o[i] * inv;
    else ov[e] = from_f32<T>(o[i] * inv);
  }
}

extern "C" int ms_paged_attention_generic(const void* q, int q_stride, const void* kc, const void* vc, int is_bf16,
                                          const int* block_table, int table_width, const int* token_list,
                                          const int* token_row, const int* pos, void* out, int tokens, int Hq, int Hkv,
                                          int D, int Dv, int page_size, float scale, int window, int keep_first, int waves,
                                          float softcap, const float* sinks, int value_share, int values_in_keys,
                                          int out_f32, hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (D <= 0 || D > MAX_WIDE_HEAD_DIM || Dv <= 0 || Dv > MAX_WIDE_HEAD_DIM || Hq <= 0 || Hkv <= 0 || Hq % Hkv || page_size <= 0 ||
      window < 0 || keep_first < 0 || table_width <= 0 || Hq > 65535 || q_stride < Hq * D || (waves != 1 && waves != 8 && waves != 16) ||
      !(softcap >= 0.f) || value_share < 1 || Hkv % value_share || (values_in_keys && (Dv > D || value_share != 1)) ||
      (!values_in_keys && vc == nullptr))
    return MS_BAD_ARG;
  if (window == 0) keep_first = 0;  // every key is visible anyway
  const bool wide = D > MAX_HEAD_DIM || Dv > MAX_HEAD_DIM;
  if (wide && waves == 16) waves = 8;  // the waves' partial outputs must fit in LDS
  dim3 grid(tokens, Hq);
#define GA(T, NW, MAXD)                                                                                                      \
  paged_attention_generic_kernel<T, NW, MAXD><<<grid, NW * WAVE, 0, st>>>(                                                   \
      (const T*)q, q_stride, (const T*)kc, (const T*)vc, block_table, table_width, token_list, token_row, pos, (T*)out, Hq, Hkv, D, \
      Dv, page_size, scale, window, keep_first, softcap, sinks, value_share, values_in_keys, out_f32 ? (float*)out : nullptr)
  if (wide) {
    if (is_bf16) {
      if (waves == 8) GA(bf16, 8, MAX_WIDE_HEAD_DIM); else GA(bf16, 1, MAX_WIDE_HEAD_DIM);
    } else {
      if (waves == 8) GA(float, 8, MAX_WIDE_HEAD_DIM); else GA(float, 1, MAX_WIDE_HEAD_DIM);
    }
  } else if (is_bf16) {
    if (waves == 16) GA(bf16, 16, MAX_HEAD_DIM); else if (waves == 8) GA(bf16, 8, MAX_HEAD_DIM); else GA(bf16, 1, MAX_HEAD_DIM);
  } else {
    if (waves == 16) GA(float, 16, MAX_HEAD_DIM); else if (waves == 8) GA(float, 8, MAX_HEAD_DIM); else GA(float, 1, MAX_HEAD_DIM);
  }
#undef GA
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// The same attention for rows that bring several tokens: a block owns a tile of consecutive new tokens of one
// sequence and one KV head, that is up to 64 query rows (tokens x the heads of the group), and walks the tiles of 64
// keys that hold a key visible to any of them (absolute multiples of 64, as above: what a query computes does not
// depend on how the tokens were cut). Keys and values of a tile are widened to float32 in LDS, both transposed
// ([element][key], rows 65 apart) so that neither the stores nor the reads meet in a bank; scores, softmax weights
// and the weighted sums are float32 products on the vector units. Head sizes up to 128.
//   scores: thread (tid / 16, tid % 16) = rows 4 (tid / 16) .. + 3, keys tid % 16 + 16 k; a row's maximum and sum
//           meet over its 16 lanes by shuffles;
//   values: thread (tid / 32, tid % 32) = rows 8 (tid / 32) .. + 7, elements tid % 32 + 32 k.
#define TILED_ROWS 64
#define TILED_MAX_DIM 128

template <typename T>
__global__ __launch_bounds__(256) void paged_attention_tiled_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ tile_first,
    const int* __restrict__ tile_count, const int* __restrict__ token_row, const int* __restrict__ pos, T* __restrict__ out,
    int Hq, int Hkv, int D, int Dv, int page_size, float scale, int window, int keep_first) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  constexpr int CP = WAVE + 1;
  const int DQ = D | 1;
  float* Q = sm;                    // [TILED_ROWS][DQ]
  float* Kt = Q + TILED_ROWS * DQ;  // [D][CP]
  float* Vt = Kt + D * CP;          // [Dv][CP]
  float* P = Vt + Dv * CP;          // [TILED_ROWS][CP]
  float* corr = P + TILED_ROWS * CP;
  float* lsum = corr + TILED_ROWS;
  const int tid = threadIdx.x, kvh = blockIdx.y, g = Hq / Hkv;
  const int first = tile_first[blockIdx.x], count = tile_count[blockIdx.x], rows = count * g;
  const int* table = block_table + (size_t)token_row[first] * table_width;
  const int p_first = pos[first], p_last = p_first + count - 1;
  const int lo_first = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
  const int kept = keep_first < lo_first ? keep_first : lo_first;

  for (int i = tid; i < TILED_ROWS * D; i += 256) {
    const int r = i / D, d = i % D;
    Q[r * DQ + d] = r < rows ? to_f32(q[(size_t)(first + r / g) * q_stride + (size_t)(kvh * g + r % g) * D + d]) : 0.f;
  }
  const int r0 = (tid / 16) * 4, l16 = tid % 16;  // scores
  int pr[4], lor[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    pr[i] = r0 + i < rows ? p_first + (r0 + i) / g : -1;
    lor[i] = (window > 0 && pr[i] - window + 1 > 0) ? pr[i] - window + 1 : 0;
  }
  float m_run[4], l_run[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) m_run[i] = -INFINITY, l_run[i] = 0.f;
  const int ro = (tid / 32) * 8, l32 = tid % 32;  // values
  float o[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int k = 0; k < 4; ++k) o[i][k] = 0.f;

  const int kept_tiles = (kept + WAVE - 1) / WAVE;
  const int first_window_tile = lo_first / WAVE > kept_tiles ? lo_first / WAVE : kept_tiles;
  const int tiles = kept_tiles + (p_last / WAVE - first_window_tile + 1);
  for (int ti = 0; ti < tiles; ++ti) {
    const int j0 = (ti < kept_tiles ? ti : first_window_tile + (ti - kept_tiles)) * WAVE;
    __syncthreads();  // the tile before has been read
    constexpr int VN = Vec16<T>::N;
    if (D % VN == 0 && page_size % VN == 0 && WAVE % page_size == 0) {
      // 16 bytes a load, all of a thread's loads issued before the first is used: a key's run of VN elements, and a
      // page's run of VN tokens of one value element.
      const int kruns = D / VN, vruns = page_size / VN;
      for (int i0 = 0; i0 < WAVE * kruns; i0 += 4 * 256) {
        uint4 got[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 256 + tid, jj = i / kruns, d = (i % kruns) * VN, j = j0 + jj;
          got[u] = make_uint4(0, 0, 0, 0);
          if (i < WAVE * kruns && j <= p_last && (j >= lo_first || j < kept))
            got[u] = *reinterpret_cast<const uint4*>(kc + (((size_t)table[j / page_size] * Hkv + kvh) * page_size + (j % page_size)) * D + d);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 256 + tid, jj = i / kruns, d = (i % kruns) * VN;
          if (i >= WAVE * kruns) continue;
          alignas(16) T kv[VN];
          *reinterpret_cast<uint4*>(kv) = got[u];
#pragma unroll
          for (int w = 0; w < VN; ++w) Kt[(d + w) * CP + jj] = to_f32(kv[w]);
        }
      }
      const int per_page = Dv * vruns, total = (WAVE / page_size) * per_page;
      for (int i0 = 0; i0 < total; i0 += 4 * 256) {
        uint4 got[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 256 + tid, pg = i / per_page, e = (i % per_page) / vruns, part = i % vruns;
          const int jp = j0 + pg * page_size;  // the page's first key
          got[u] = make_uint4(0, 0, 0, 0);
          if (i < total && jp <= p_last && (jp + page_size > lo_first || jp < kept)) {
            const int page = table[jp / page_size];
            if (page >= 0) got[u] = *reinterpret_cast<const uint4*>(vc + (((size_t)page * Hkv + kvh) * Dv + e) * page_size + part * VN);
          }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * 256 + tid, pg = i / per_page, e = (i % per_page) / vruns, part = i % vruns;
          if (i >= total) continue;
          alignas(16) T vv[VN];
          *reinterpret_cast<uint4*>(vv) = got[u];
#pragma unroll
          for (int w = 0; w < VN; ++w) {
            const int jj = pg * page_size + part * VN + w, j = j0 + jj;
            Vt[e * CP + jj] = (j <= p_last && (j >= lo_first || j < kept)) ? to_f32(vv[w]) : 0.f;
          }
        }
      }
    } else {
      for (int i = tid; i < WAVE * D; i += 256) {
        const int jj = i / D, d = i % D, j = j0 + jj;
        float v = 0.f;
        if (j <= p_last && (j >= lo_first || j < kept))
          v = to_f32(kc[(((size_t)table[j / page_size] * Hkv + kvh) * page_size + (j % page_size)) * D + d]);
        Kt[d * CP + jj] = v;
      }
      for (int i = tid; i < WAVE * Dv; i += 256) {
        const int e = i / WAVE, jj = i % WAVE, j = j0 + jj;
        float v = 0.f;
        if (j <= p_last && (j >= lo_first || j < kept))
          v = to_f32(vc[(((size_t)table[j / page_size] * Hkv + kvh) * Dv + e) * page_size + (j % page_size)]);
        Vt[e * CP + jj] = v;
      }
    }
    __syncthreads();
    float s[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 4; ++k) s[i][k] = 0.f;
#pragma unroll 4
    for (int d = 0; d < D; ++d) {
      float qv[4], kv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) qv[i] = Q[(r0 + i) * DQ + d];
#pragma unroll
      for (int k = 0; k < 4; ++k) kv[k] = Kt[d * CP + l16 + 16 * k];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) s[i][k] = fmaf(qv[i], kv[k], s[i][k]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float mx = -INFINITY;
      bool ok[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int j = j0 + l16 + 16 * k;
        ok[k] = j <= pr[i] && (j >= lor[i] || j < keep_first);
        s[i][k] = ok[k] ? s[i][k] * scale : -INFINITY;
        mx = fmaxf(mx, s[i][k]);
      }
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 16));
      const float m_new = fmaxf(m_run[i], mx);
      const bool none = m_new == -INFINITY;  // no key of this row so far
      const float c = none ? 1.f : expf(m_run[i] - m_new);
      float sum = 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float pj = (ok[k] && !none) ? expf(s[i][k] - m_new) : 0.f;
        P[(r0 + i) * CP + l16 + 16 * k] = pj;
        sum += pj;
      }
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 16);
      l_run[i] = l_run[i] * c + sum;
      m_run[i] = m_new;
      if (l16 == 0) corr[r0 + i] = c;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float c = corr[ro + i];
#pragma unroll
      for (int k = 0; k < 4; ++k) o[i][k] *= c;
    }
    const int jn = p_last - j0 + 1 < WAVE ? p_last - j0 + 1 : WAVE;
#pragma unroll 4
    for (int jj = 0; jj < jn; ++jj) {
      float vv[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) vv[k] = l32 + 32 * k < Dv ? Vt[(l32 + 32 * k) * CP + jj] : 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float pv = P[(ro + i) * CP + jj];
#pragma unroll
        for (int k = 0; k < 4; ++k) o[i][k] = fmaf(pv, vv[k], o[i][k]);
      }
    }
  }
  if (l16 == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) lsum[r0 + i] = l_run[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = ro + i;
    if (r >= rows) continue;
    const float inv = 1.f / lsum[r];
    T* ov = out + ((size_t)(first + r / g) * Hq + (kvh * g + r % g)) * Dv;
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (l32 + 32 * k < Dv) ov[l32 + 32 * k] = from_f32<T>(o[i][k] * inv);
  }
}

// Tokens per tile for a group of `group` query heads per KV head (0: the tiled kernel does not take the shape).
extern "C" int ms_paged_attention_tiled_tokens(int group, int D, int Dv) {
  if (group < 1 || group > TILED_ROWS || D < 1 || Dv < 1 || D > TILED_MAX_DIM || Dv > TILED_MAX_DIM) return 0;
  return TILED_ROWS / group;
}

// tile_first / tile_count: `tiles` runs of at most ms_paged_attention_tiled_tokens consecutive new tokens of one sequence.
extern "C" int ms_paged_attention_tiled(const void* q, int q_stride, const void* kc, const void* vc, int is_bf16,
                                        const int* block_table, int table_width, const int* tile_first, const int* tile_count,
                                        int tiles, const int* token_row, const int* pos, void* out, int Hq, int Hkv, int D, int Dv,
                                        int page_size, float scale, int window, int keep_first, hipStream_t st) {
  if (tiles <= 0) return MS_OK;
  if (D <= 0 || Dv <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || page_size <= 0 || window < 0 || keep_first < 0 || table_width <= 0 ||
      Hkv > 65535 || q_stride < Hq * D || tile_first == nullptr || tile_count == nullptr)
    return MS_BAD_ARG;
  if (ms_paged_attention_tiled_tokens(Hq / Hkv, D, Dv) == 0) return MS_UNSUPPORTED;
  if (window == 0) keep_first = 0;
  const size_t lds = sizeof(float) * ((size_t)TILED_ROWS * (D | 1) + (size_t)(D + Dv + TILED_ROWS) * (WAVE + 1) + 2 * TILED_ROWS);
  dim3 grid(tiles, Hkv);
  if (is_bf16) {
    if (hipFuncSetAttribute((const void*)paged_attention_tiled_kernel<bf16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return MS_LAUNCH_FAILED;
    paged_attention_tiled_kernel<bf16><<<grid, 256, lds, st>>>((const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc, block_table,
                                                               table_width, tile_first, tile_count, token_row, pos, (bf16*)out, Hq,
                                                               Hkv, D, Dv, page_size, scale, window, keep_first);
  } else {
    if (hipFuncSetAttribute((const void*)paged_attention_tiled_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return MS_LAUNCH_FAILED;
    paged_attention_tiled_kernel<float><<<grid, 256, lds, st>>>((const float*)q, q_stride, (const float*)kc, (const float*)vc,
                                                                block_table, table_width, tile_first, tile_count, token_row, pos,
                                                                (float*)out, Hq, Hkv, D, Dv, page_size, scale, window, keep_first);
  }
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// The tiled form on the matrix cores, for bfloat16 storage with 16-token pages, head sizes that are multiples of 32
// (keys) and 16 (values) up to 128: the same tiles of tokens and of 64 keys, the same masks, float32 results of the
// same meaning. Queries and keys are bfloat16 as stored, so their products are exact in float32 and the scores are
// float32 sums of them (v_mfma_f32_16x16x32_bf16). The softmax weights stay float32: each is cut into three
// bfloat16 pieces (hi = bf16(p), mid = bf16(p - hi), lo = bf16(p - hi - mid): 24 bits of mantissa, p itself), and the
// second product runs once per piece into the same float32 accumulators, so what meets the values is the float32
// weight, not a rounding of it.
//   A wave owns 16 of the block's 64 query rows. Scores: A = 16 query rows x 32 elements, B = 32 elements x 16 keys,
//   both one 16-byte load per lane straight from global memory; a lane then holds one key of four rows
//   (rows 4 (lane / 16) + r), a row's maximum meets over the 16 lanes that share it; a row's sum of weights is one
//   more column of the second product (values of 1), so it is the sum of exactly the pieces that meet the values.
//   The weights go through a wave's own LDS rows to change hands (the second product wants a row's 8 consecutive keys in one lane); values:
//   B = 32 keys x 16 elements, 8 consecutive tokens of one element being one 16-byte load from the transposed page.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
#define MFMA_PAGE 16

__device__ __forceinline__ bf16x8 load_bf16x8(const bf16* p) {
  union { uint4 u; bf16x8 v; } x;
  x.u = *reinterpret_cast<const uint4*>(p);
  return x.v;
}
__device__ __forceinline__ bf16x8 zero_bf16x8() {
  union { uint4 u; bf16x8 v; } x;
  x.u = make_uint4(0, 0, 0, 0);
  return x.v;
}

// Maximum over a row of 16 lanes, the same bits in all of them: four rotations within the row (DPP row_ror 8, 4, 2, 1).
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false)));
  return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false)));
}
// e^x on the hardware's exp2 (about one unit in the last place, float32).
__device__ __forceinline__ float exp_fast(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

template <int D, int DV>
__global__ __launch_bounds__(256) void paged_attention_tiled_mfma_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ tile_first,
    const int* __restrict__ tile_count, const int* __restrict__ token_row, const int* __restrict__ pos, bf16* __restrict__ out,
    int Hq, int Hkv, float scale, int window, int keep_first) {
  constexpr int PS = WAVE + 4;  // floats between a wave's rows of weights
  __shared__ __attribute__((aligned(16))) float Pw[4][16][PS];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, l16 = lane % 16, grp = lane / 16;
  const int kvh = blockIdx.y, g = Hq / Hkv;
  const int first = tile_first[blockIdx.x], count = tile_count[blockIdx.x], rows = count * g;
  const int* table = block_table + (size_t)token_row[first] * table_width;
  const int p_first = pos[first], p_last = p_first + count - 1;
  const int lo_first = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
  const int kept = keep_first < lo_first ? keep_first : lo_first;

  // this lane's query row as the A operand: row 16 wave + l16, elements 32 kk + 8 grp .. + 7
  bf16x8 qf[D / 32];
  {
    const int r = wave * 16 + l16;
#pragma unroll
    for (int kk = 0; kk < D / 32; ++kk)
      qf[kk] = r < rows ? load_bf16x8(q + (size_t)(first + r / g) * q_stride + (size_t)(kvh * g + r % g) * D + kk * 32 + grp * 8)
                        : zero_bf16x8();
  }
  // the rows whose scores and outputs this lane holds: 16 wave + 4 grp + r
  int pr[4], lor[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = wave * 16 + grp * 4 + r;
    pr[r] = row < rows ? p_first + row / g : -1;
    lor[r] = (window > 0 && pr[r] - window + 1 > 0) ? pr[r] - window + 1 : 0;
  }
  float m_run[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) m_run[r] = -INFINITY;
  floatx4 o[DV / 16], l_run = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int et = 0; et < DV / 16; ++et) o[et] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 ones;
#pragma unroll
  for (int u = 0; u < 8; ++u) ones[u] = static_cast<bf16>(1.f);

  const int kept_tiles = (kept + WAVE - 1) / WAVE;
  const int first_window_tile = lo_first / WAVE > kept_tiles ? lo_first / WAVE : kept_tiles;
  const int tiles = kept_tiles + (p_last / WAVE - first_window_tile + 1);
  for (int ti = 0; ti < tiles; ++ti) {
    const int j0 = (ti < kept_tiles ? ti : first_window_tile + (ti - kept_tiles)) * WAVE;
    // The tile's four pages (a tile of 64 keys is four whole pages; table rows are padded to a multiple of four
    // entries): one load serves the keys' and the values' addresses.
    const int4 pg4 = *reinterpret_cast<const int4*>(table + j0 / MFMA_PAGE);
    const int pages[4] = {pg4.x, pg4.y, pg4.z, pg4.w};
    // keys and values are asked for together, ahead of the first product: the values do not wait for the softmax
    bf16x8 kf[4][D / 32], vf[2][DV / 16];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int j = j0 + t * 16 + l16;  // this lane's key as the B operand
      const bool seen = j <= p_last && (j >= lo_first || j < kept) && pages[t] >= 0;
      const bf16* kp = kc + (((size_t)(seen ? pages[t] : 0) * Hkv + kvh) * MFMA_PAGE + l16) * D + grp * 8;
#pragma unroll
      for (int kk = 0; kk < D / 32; ++kk) kf[t][kk] = seen ? load_bf16x8(kp + kk * 32) : zero_bf16x8();
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int jb = j0 + ks * 32 + grp * 8;  // this lane's 8 keys as the B operand: one run of a page
      const int page = pages[ks * 2 + grp / 2];
      const bool seen = jb <= p_last && (jb + 8 > lo_first || jb < kept) && page >= 0;
      const bf16* vp = vc + ((size_t)(seen ? page : 0) * Hkv + kvh) * DV * MFMA_PAGE + (jb % MFMA_PAGE);
#pragma unroll
      for (int et = 0; et < DV / 16; ++et) vf[ks][et] = seen ? load_bf16x8(vp + (size_t)(et * 16 + l16) * MFMA_PAGE) : zero_bf16x8();
    }
    // scores of 16 rows x 64 keys: four 16-key tiles
    floatx4 s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < D / 32; ++kk) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[kk], kf[t][kk], s[t], 0, 0, 0);
    }
    // masks, running maxima and sums; the weights into the wave's LDS rows
    float corr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float mx = -INFINITY;
      bool ok[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int j = j0 + t * 16 + l16;
        ok[t] = j <= pr[r] && (j >= lor[r] || j < keep_first);
        s[t][r] = ok[t] ? s[t][r] * scale : -INFINITY;
        mx = fmaxf(mx, s[t][r]);
      }
      mx = row16_max(mx);
      const float m_new = fmaxf(m_run[r], mx);
      const bool none = m_new == -INFINITY;  // no key of this row so far
      corr[r] = none ? 1.f : exp_fast(m_run[r] - m_new);
#pragma unroll
      for (int t = 0; t < 4; ++t) Pw[wave][grp * 4 + r][t * 16 + l16] = (ok[t] && !none) ? exp_fast(s[t][r] - m_new) : 0.f;
      l_run[r] *= corr[r];
      m_run[r] = m_new;
    }
#pragma unroll
    for (int et = 0; et < DV / 16; ++et)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[et][r] *= corr[r];
    __builtin_amdgcn_wave_barrier();  // a wave's own rows: its order of LDS operations is enough
    // weights x values, 32 keys a step: row l16's weights of keys 32 ks + 8 grp .. + 7 in three bfloat16 pieces
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const float4 a0 = *reinterpret_cast<const float4*>(&Pw[wave][l16][ks * 32 + grp * 8]);
      const float4 a1 = *reinterpret_cast<const float4*>(&Pw[wave][l16][ks * 32 + grp * 8 + 4]);
      const float pv[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
      bf16x8 hi, mid, low;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const bf16 h = static_cast<bf16>(pv[u]);
        const float r1 = pv[u] - static_cast<float>(h);
        const bf16 m = static_cast<bf16>(r1);
        hi[u] = h;
        mid[u] = m;
        low[u] = static_cast<bf16>(r1 - static_cast<float>(m));
      }
#pragma unroll
      for (int et = 0; et < DV / 16; ++et) {
        o[et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, vf[ks][et], o[et], 0, 0, 0);
        o[et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mid, vf[ks][et], o[et], 0, 0, 0);
        o[et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(low, vf[ks][et], o[et], 0, 0, 0);
      }
      l_run = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, ones, l_run, 0, 0, 0);
      l_run = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mid, ones, l_run, 0, 0, 0);
      l_run = __builtin_amdgcn_mfma_f32_16x16x32_bf16(low, ones, l_run, 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();  // the weights have been read before the next tile's are written
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = wave * 16 + grp * 4 + r;
    if (row >= rows) continue;
    const float inv = 1.f / l_run[r];
    bf16* ov = out + ((size_t)(first + row / g) * Hq + (kvh * g + row % g)) * DV;
#pragma unroll
    for (int et = 0; et < DV / 16; ++et) ov[et * 16 + l16] = static_cast<bf16>(o[et][r] * inv);
  }
}

// tanh on the hardware's exp2 and reciprocal: 1 - 2 / (1 + e^(2x)), about one unit in the last place of float32 near
// zero and exact at the ends (e^(2x) = inf gives 1, 0 gives -1).
__device__ __forceinline__ float tanh_fast(float x) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * 2.885390081777927f));
}

// The same kernel for heads of any size that is a multiple of 32 (keys) and 16 (values), and for the options of the
// generic form: a soft cap on the scores, a sink per query head, key heads that share a value head, float32 results.
// What differs: the key size D is a run-time number (the query fragments live in registers where D <= 32 NQ, NQ = 4 or
// 18, and are fetched again for every key tile where it is larger); a block owns DVC of a
// head's Dv value elements (blockIdx.z names the run), so a head of 512 values is two blocks that each form the scores
// again. A tile's keys go through LDS once for the block's four waves.
template <int DVC, bool SPLIT, int NQ>
__global__ __launch_bounds__(256) void paged_attention_tiled_mfma_wide_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ tile_first,
    const int* __restrict__ tile_count, const int* __restrict__ token_row, const int* __restrict__ pos, bf16* __restrict__ out,
    float* __restrict__ out32, int Hq, int Hkv, int D, int Dv, float scale, int window, int keep_first, float softcap,
    const float* __restrict__ sinks, int value_share, int splits, float* __restrict__ part_o, float* __restrict__ part_ml,
    int xcd_combos, int n_tiles) {
  constexpr int PS = WAVE + 4;  // floats between a wave's rows of weights
  __shared__ __attribute__((aligned(16))) float Pw[4][16][PS];
  __shared__ float Mo[SPLIT ? 4 : 1][SPLIT ? 16 : 1][SPLIT ? DVC : 1];  // SPLIT: the waves' outputs, maxima and sums meet here
  __shared__ float Mml[SPLIT ? 4 : 1][16][2];
  extern __shared__ __attribute__((aligned(16))) bf16 Ks[];  // not SPLIT: the tile's keys, [64][D + 8]
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, l16 = lane % 16, grp = lane / 16;
  // Which tile, key head and run of values the block owns. xcd_combos > 0 (not SPLIT, a one-dimensional grid): blocks go
  // to the chip's eight XCDs in turn, and every (key head, run of values) pair is given to XCDs of its own, so that an
  // XCD's L2 holds the keys and values of its pairs only: a prompt's tiles all walk the same keys, and what they walk
  // should stay in the 4 MB next to them.
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  if (!SPLIT && xcd_combos > 0) {
    const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8, runs_v = Dv / DVC;
    int combo, t;
    if (xcd_combos <= 8) {
      const int per = 8 / xcd_combos;  // XCDs that share a pair take its tiles in turn
      combo = xcd / per;
      t = slot * per + xcd % per;
    } else {
      const int groups = xcd_combos / 8;  // pairs an XCD owns
      combo = xcd + 8 * (slot % groups);
      t = slot / groups;
    }
    if (t >= n_tiles) return;
    bx = t;
    by = combo / runs_v;
    bz = combo % runs_v;
  }
  // SPLIT: a tile is one token, and a block owns up to 16 of a key head's query heads (blockIdx.y names key head and run)
  const int g = Hq / Hkv, e0 = bz * DVC, runs16 = SPLIT ? (g + 15) / 16 : 1;
  const int kvh = by / runs16, hoff = (by % runs16) * 16;
  const int Hv = Hkv / value_share, vh = kvh / value_share;
  const int tile = SPLIT ? bx / splits : bx, split = SPLIT ? bx % splits : 0;
  const int first = tile_first[tile], count = SPLIT ? 1 : tile_count[tile];
  const int rows = SPLIT ? (g - hoff < 16 ? g - hoff : 16) : count * g;
  const int rb = SPLIT ? 0 : wave * 16;  // SPLIT: every wave holds the tile's (at most 16) rows and takes every fourth key tile
  const int* table = block_table + (size_t)token_row[first] * table_width;
  const int p_first = pos[first], p_last = p_first + count - 1;
  const int lo_first = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
  const int kept = keep_first < lo_first ? keep_first : lo_first;
  const int chunks = D / 32;

  // this lane's query row as the A operand: row 16 wave + l16, elements 32 kk + 8 grp .. + 7
  const int qr = rb + l16;
  const bf16* qp = nullptr;
  if (qr < rows)
    qp = SPLIT ? q + (size_t)first * q_stride + (size_t)(kvh * g + hoff + qr) * D + grp * 8
               : q + (size_t)(first + qr / g) * q_stride + (size_t)(kvh * g + qr % g) * D + grp * 8;
  int pr[4], lor[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = rb + grp * 4 + r;
    pr[r] = row < rows ? (SPLIT ? p_first : p_first + row / g) : -1;
    lor[r] = (window > 0 && pr[r] - window + 1 > 0) ? pr[r] - window + 1 : 0;
  }
  // NQ > 0: the lane's query fragments live in registers (D <= 32 NQ); else they are fetched again for every key tile
  bf16x8 qreg[NQ > 0 ? NQ : 1];
  if (NQ > 0) {
#pragma unroll
    for (int kk = 0; kk < NQ; ++kk) qreg[kk] = (qp && kk < chunks) ? load_bf16x8(qp + kk * 32) : zero_bf16x8();
  }
  float m_run[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) m_run[r] = -INFINITY;
  floatx4 o[DVC / 16], l_run = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int et = 0; et < DVC / 16; ++et) o[et] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 ones;
#pragma unroll
  for (int u = 0; u < 8; ++u) ones[u] = static_cast<bf16>(1.f);
  const float cap_in = softcap > 0.f ? scale / softcap : 0.f;

  // where this thread's 16-byte runs of a key tile lie (not SPLIT: the tile goes through LDS)
  const int key_runs = D / 8;
  const int stage_key = threadIdx.x / key_runs, stage_run = threadIdx.x % key_runs, stage_dq = 256 / key_runs, stage_dr = 256 % key_runs;
  const int kept_tiles = (kept + WAVE - 1) / WAVE;
  const int first_window_tile = lo_first / WAVE > kept_tiles ? lo_first / WAVE : kept_tiles;
  const int tiles = kept_tiles + (p_last / WAVE - first_window_tile + 1);
  const int per_split = SPLIT ? (tiles + splits - 1) / splits : tiles;
  const int t_begin = SPLIT ? split * per_split + wave : 0;
  const int t_end = SPLIT ? ((split + 1) * per_split < tiles ? (split + 1) * per_split : tiles) : tiles;
  for (int ti = t_begin; ti < t_end; ti += SPLIT ? 4 : 1) {
    const int j0 = (ti < kept_tiles ? ti : first_window_tile + (ti - kept_tiles)) * WAVE;
    const int4 pg4 = *reinterpret_cast<const int4*>(table + j0 / MFMA_PAGE);
    const int pages[4] = {pg4.x, pg4.y, pg4.z, pg4.w};
    bf16x8 vf[2][DVC / 16];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int jb = j0 + ks * 32 + grp * 8;  // this lane's 8 keys as the B operand: one run of a page
      const int page = pages[ks * 2 + grp / 2];
      const bool seen = jb <= p_last && (jb + 8 > lo_first || jb < kept) && page >= 0;
      const bf16* vp = vc + (((size_t)(seen ? page : 0) * Hv + vh) * Dv + e0) * MFMA_PAGE + (jb % MFMA_PAGE);
#pragma unroll
      for (int et = 0; et < DVC / 16; ++et) vf[ks][et] = seen ? load_bf16x8(vp + (size_t)(et * 16 + l16) * MFMA_PAGE) : zero_bf16x8();
    }
    floatx4 s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    if (SPLIT) {
      // every wave has key tiles of its own: the keys come straight from memory, two runs of 32 elements under way
      const bf16* kp[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int j = j0 + t * 16 + l16;  // this lane's key as the B operand
        const bool seen = j <= p_last && (j >= lo_first || j < kept) && pages[t] >= 0;
        kp[t] = seen ? kc + (((size_t)pages[t] * Hkv + kvh) * MFMA_PAGE + l16) * D + grp * 8 : nullptr;
      }
      if (NQ > 0) {
#pragma unroll
        for (int kk = 0; kk < NQ; kk += 2) {
          if (kk >= chunks) continue;  // the same for every lane; no break, so that the loop unrolls and qreg stays in registers
          bf16x8 kf[2][4];
#pragma unroll
          for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int t = 0; t < 4; ++t)
              kf[c][t] = (kk + c < chunks && kp[t]) ? load_bf16x8(kp[t] + (kk + c) * 32) : zero_bf16x8();
#pragma unroll
          for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int t = 0; t < 4; ++t)
              if (kk + c < NQ) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qreg[kk + c < NQ ? kk + c : 0], kf[c][t], s[t], 0, 0, 0);
        }
      } else {
        for (int kk = 0; kk < chunks; kk += 2) {
          bf16x8 qf[2], kf[2][4];
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const bool in = kk + c < chunks;
            qf[c] = (in && qp) ? load_bf16x8(qp + (kk + c) * 32) : zero_bf16x8();
#pragma unroll
            for (int t = 0; t < 4; ++t) kf[c][t] = (in && kp[t]) ? load_bf16x8(kp[t] + (kk + c) * 32) : zero_bf16x8();
          }
#pragma unroll
          for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int t = 0; t < 4; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[c], kf[c][t], s[t], 0, 0, 0);
        }
      }
    } else {
      // The block's waves share the tile's keys: all of them are fetched at once into LDS, 16 bytes a thread and load
      // (rows D + 8 elements apart: the 16 lanes that read 16 keys' runs of 8 elements meet in no bank), so that a tile
      // waits for memory once and not once per run of elements. The query fragments come from the cache, the next
      // run's under way while this one is multiplied.
      __syncthreads();  // the tile before has been read
      const int ld = D + 8;
      // 16-byte loads of the tile a thread has under way at once: all of them where the queries' registers say how many
      // there are at most (keys of 128 elements: 4 a thread, of 576: 18), else 6 at a time
      constexpr int STAGE_BATCH = NQ == 4 ? 4 : NQ == 18 ? 18 : 6;
      int jj = stage_key, c = stage_run;  // thread's first 16-byte run; the next is 256 runs on (no division in the loop)
      for (int i0 = threadIdx.x; i0 < WAVE * key_runs; i0 += STAGE_BATCH * 256) {
        uint4 got[STAGE_BATCH];
        int at[STAGE_BATCH];
#pragma unroll
        for (int u = 0; u < STAGE_BATCH; ++u) {
          const int j = j0 + jj;
          const int page = jj < 16 ? pg4.x : jj < 32 ? pg4.y : jj < 48 ? pg4.z : pg4.w;
          at[u] = i0 + u * 256 < WAVE * key_runs ? jj * ld + c * 8 : -1;
          got[u] = make_uint4(0, 0, 0, 0);
          if (at[u] >= 0 && j <= p_last && (j >= lo_first || j < kept) && page >= 0)
            got[u] = *reinterpret_cast<const uint4*>(kc + (((size_t)page * Hkv + kvh) * MFMA_PAGE + jj % MFMA_PAGE) * D + c * 8);
          jj += stage_dq;
          c += stage_dr;
          if (c >= key_runs) {
            c -= key_runs;
            ++jj;
          }
        }
#pragma unroll
        for (int u = 0; u < STAGE_BATCH; ++u)
          if (at[u] >= 0) *reinterpret_cast<uint4*>(Ks + at[u]) = got[u];
      }
      bf16x8 qn = (NQ == 0 && qp && chunks > 0) ? load_bf16x8(qp) : zero_bf16x8();
      __syncthreads();
      if (NQ > 0) {
#pragma unroll
        for (int kk = 0; kk < NQ; ++kk) {
          if (kk >= chunks) continue;  // no break: the loop unrolls and qreg stays in registers
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            union { uint4 u; bf16x8 v; } kf;
            kf.u = *reinterpret_cast<const uint4*>(Ks + (size_t)(t * 16 + l16) * ld + kk * 32 + grp * 8);
            s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qreg[kk], kf.v, s[t], 0, 0, 0);
          }
        }
      } else {
        for (int kk = 0; kk < chunks; ++kk) {
          const bf16x8 qf = qn;
          qn = (qp && kk + 1 < chunks) ? load_bf16x8(qp + (kk + 1) * 32) : zero_bf16x8();
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            union { uint4 u; bf16x8 v; } kf;
            kf.u = *reinterpret_cast<const uint4*>(Ks + (size_t)(t * 16 + l16) * ld + kk * 32 + grp * 8);
            s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf, kf.v, s[t], 0, 0, 0);
          }
        }
      }
    }
    float corr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float mx = -INFINITY;
      bool ok[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int j = j0 + t * 16 + l16;
        ok[t] = j <= pr[r] && (j >= lor[r] || j < keep_first);
        const float sc = softcap > 0.f ? softcap * tanh_fast(s[t][r] * cap_in) : s[t][r] * scale;
        s[t][r] = ok[t] ? sc : -INFINITY;
        mx = fmaxf(mx, s[t][r]);
      }
      mx = row16_max(mx);
      const float m_new = fmaxf(m_run[r], mx);
      const bool none = m_new == -INFINITY;  // no key of this row so far
      corr[r] = none ? 1.f : exp_fast(m_run[r] - m_new);
#pragma unroll
      for (int t = 0; t < 4; ++t) Pw[wave][grp * 4 + r][t * 16 + l16] = (ok[t] && !none) ? exp_fast(s[t][r] - m_new) : 0.f;
      l_run[r] *= corr[r];
      m_run[r] = m_new;
    }
#pragma unroll
    for (int et = 0; et < DVC / 16; ++et)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[et][r] *= corr[r];
    __builtin_amdgcn_wave_barrier();  // a wave's own rows: its order of LDS operations is enough
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const float4 a0 = *reinterpret_cast<const float4*>(&Pw[wave][l16][ks * 32 + grp * 8]);
      const float4 a1 = *reinterpret_cast<const float4*>(&Pw[wave][l16][ks * 32 + grp * 8 + 4]);
      const float pv[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
      bf16x8 hi, mid, low;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const bf16 h = static_cast<bf16>(pv[u]);
        const float r1 = pv[u] - static_cast<float>(h);
        const bf16 m = static_cast<bf16>(r1);
        hi[u] = h;
        mid[u] = m;
        low[u] = static_cast<bf16>(r1 - static_cast<float>(m));
      }
#pragma unroll
      for (int et = 0; et < DVC / 16; ++et) {
        o[et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, vf[ks][et], o[et], 0, 0, 0);
        o[et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mid, vf[ks][et], o[et], 0, 0, 0);
        o[et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(low, vf[ks][et], o[et], 0, 0, 0);
      }
      l_run = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, ones, l_run, 0, 0, 0);
      l_run = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mid, ones, l_run, 0, 0, 0);
      l_run = __builtin_amdgcn_mfma_f32_16x16x32_bf16(low, ones, l_run, 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();  // the weights have been read before the next tile's are written
  }
  if (SPLIT) {
    // the four waves' partial results, brought to one maximum in wave order
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (l16 == 0) {
        Mml[wave][grp * 4 + r][0] = m_run[r];
        Mml[wave][grp * 4 + r][1] = l_run[r];
      }
#pragma unroll
      for (int et = 0; et < DVC / 16; ++et) Mo[wave][grp * 4 + r][et * 16 + l16] = o[et][r];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = grp * 4 + r;
      float m_all = -INFINITY;
#pragma unroll
      for (int w = 0; w < 4; ++w) m_all = fmaxf(m_all, Mml[w][row][0]);
      float l = 0.f;
#pragma unroll
      for (int et = 0; et < DVC / 16; ++et) o[et][r] = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float mw = Mml[w][row][0];
        const float c = mw == -INFINITY ? 0.f : expf(mw - m_all);  // a wave without a visible key
        l += Mml[w][row][1] * c;
#pragma unroll
        for (int et = 0; et < DVC / 16; ++et) o[et][r] += Mo[w][row][et * 16 + l16] * c;
      }
      m_run[r] = m_all;
      l_run[r] = l;
    }
    if (splits > 1) {
      // one part of the keys: unnormalised outputs, maximum and sum, for the merge kernel
      const size_t slot = (((size_t)tile * gridDim.y + blockIdx.y) * gridDim.z + blockIdx.z) * splits + split;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = grp * 4 + r;
        if (l16 == 0) {
          part_ml[(slot * 16 + row) * 2] = m_run[r];
          part_ml[(slot * 16 + row) * 2 + 1] = l_run[r];
        }
#pragma unroll
        for (int et = 0; et < DVC / 16; ++et) part_o[(slot * 16 + row) * DVC + et * 16 + l16] = o[et][r];
      }
      return;
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = rb + grp * 4 + r;
    if (row >= rows) continue;
    const int head = SPLIT ? kvh * g + hoff + row : kvh * g + row % g;
    float inv = 1.f / l_run[r];
    if (sinks) {  // exp(sink) joins the denominator: both are brought to the larger of the two maxima first
      const float sink = sinks[head], m_all = fmaxf(m_run[r], sink);
      const float c = expf(m_run[r] - m_all);
      inv = c / (l_run[r] * c + expf(sink - m_all));
    }
    const size_t at = ((size_t)(SPLIT ? first : first + row / g) * Hq + head) * Dv + e0;
#pragma unroll
    for (int et = 0; et < DVC / 16; ++et) {
      if (out32) out32[at + et * 16 + l16] = o[et][r] * inv;
      else out[at + et * 16 + l16] = static_cast<bf16>(o[et][r] * inv);
    }
  }
}

// The parts of the SPLIT form into the result: per row the parts' maxima, sums and outputs are brought to one maximum
// in ascending order of the parts, then the sink joins the denominator. One block per (token, key head and run of 16
// query heads, run of values).
template <int DVC>
__global__ __launch_bounds__(256) void paged_attention_mfma_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ tile_first,
    bf16* __restrict__ out, float* __restrict__ out32, int Hq, int Hkv, int Dv, int splits, const float* __restrict__ sinks) {
  extern __shared__ float coef[];  // [16 rows][splits + 1]: each part's factor, then the factor of the whole
  const int tile = blockIdx.x, g = Hq / Hkv, e0 = blockIdx.z * DVC, runs16 = (g + 15) / 16;
  const int kvh = blockIdx.y / runs16, hoff = (blockIdx.y % runs16) * 16;
  const int first = tile_first[tile], rows = g - hoff < 16 ? g - hoff : 16;
  const size_t slot0 = (((size_t)tile * gridDim.y + blockIdx.y) * gridDim.z + blockIdx.z) * splits;
  if (threadIdx.x < 16 && threadIdx.x < rows) {
    const int row = threadIdx.x;
    float m_all = -INFINITY;
    for (int sp = 0; sp < splits; ++sp) m_all = fmaxf(m_all, part_ml[((slot0 + sp) * 16 + row) * 2]);
    float l = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      const float mw = part_ml[((slot0 + sp) * 16 + row) * 2];
      const float c = mw == -INFINITY ? 0.f : expf(mw - m_all);  // a part without a visible key
      coef[row * (splits + 1) + sp] = c;
      l += part_ml[((slot0 + sp) * 16 + row) * 2 + 1] * c;
    }
    float inv = 1.f / l;
    if (sinks) {
      const float sink = sinks[kvh * g + hoff + row], m2 = fmaxf(m_all, sink);
      const float c = expf(m_all - m2);
      inv = c / (l * c + expf(sink - m2));
    }
    coef[row * (splits + 1) + splits] = inv;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 16 * DVC; i += 256) {
    const int row = i / DVC, e = i % DVC;
    if (row >= rows) continue;
    float acc = 0.f;
    for (int sp = 0; sp < splits; ++sp) acc += part_o[((slot0 + sp) * 16 + row) * DVC + e] * coef[row * (splits + 1) + sp];
    const size_t at = ((size_t)first * Hq + (kvh * g + hoff + row)) * Dv + e0 + e;
    const float v = acc * coef[row * (splits + 1) + splits];
    if (out32) out32[at] = v;
    else out[at] = static_cast<bf16>(v);
  }
}

// The run of value elements a block of the wide form owns (0: it does not take the shape): keys a multiple of 32,
// values a multiple of 16, up to 64 query heads per key head, 16-token pages.
extern "C" int ms_paged_attention_tiled_mfma_wide_chunk(int group, int D, int Dv, int page_size, int single) {
  if (page_size != MFMA_PAGE || group < 1 || group > TILED_ROWS || D < 32 || D % 32 || Dv < 16 || Dv % 16) return 0;
  // 256 values a block halve the times the scores of a head of 512 are formed again, at one wave per SIMD instead of two
  // (a head of 256 values gains nothing from it: 330 against 312 us at 2,048 tokens, fewer and slower blocks)
  if (!single && Dv % 256 == 0 && Dv > 256) return 256;
  return Dv % 128 == 0 ? 128 : Dv % 64 == 0 ? 64 : Dv % 32 == 0 ? 32 : 16;
}

// As ms_paged_attention_tiled_mfma, with the generic form's options; tiles of TILED_ROWS / group tokens. out_f32: the
// result is float32.
extern "C" int ms_paged_attention_tiled_mfma_wide(const void* q, int q_stride, const void* kc, const void* vc,
                                                  const int* block_table, int table_width, const int* tile_first,
                                                  const int* tile_count, int tiles, const int* token_row, const int* pos, void* out,
                                                  int out_f32, int Hq, int Hkv, int D, int Dv, int page_size, float scale, int window,
                                                  int keep_first, float softcap, const float* sinks, int value_share, int splits,
                                                  float* part_o, float* part_ml, hipStream_t st) {
  if (tiles <= 0) return MS_OK;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || window < 0 || keep_first < 0 || table_width <= 0 || table_width % 4 || Hkv > 65535 ||
      q_stride < Hq * D || q_stride % 8 || tile_first == nullptr || tile_count == nullptr || !(softcap >= 0.f) || value_share < 1 ||
      Hkv % value_share || splits < 0 || (splits > 1 && (part_o == nullptr || part_ml == nullptr)))
    return MS_BAD_ARG;
  const int chunk = ms_paged_attention_tiled_mfma_wide_chunk(Hq / Hkv, D, Dv, page_size, splits > 0);
  if (chunk == 0 || Dv / chunk > 65535) return MS_UNSUPPORTED;
  if (window == 0) keep_first = 0;
  bf16* o16 = out_f32 ? nullptr : (bf16*)out;
  float* o32 = out_f32 ? (float*)out : nullptr;
  // splits == 0: tiles of up to 64 rows, a wave 16 of them. splits >= 1: every tile is one token; a block owns up to 16 of
  // a key head's query heads, its waves share the key tiles, and `splits` blocks share a token's keys, their parts meeting
  // in the merge kernel.
  const int runs16 = (Hq / Hkv + 15) / 16;
  if ((long)Hkv * runs16 > 65535) return MS_BAD_ARG;
  // the tile's keys in LDS (not with splits): 64 rows of D + 8 elements, beside 17 KB of weights
  const size_t key_lds = (size_t)WAVE * (D + 8) * sizeof(bf16);
  if (splits == 0 && key_lds > 140 * 1024) return MS_UNSUPPORTED;
  dim3 grid(splits > 0 ? tiles * splits : tiles, splits > 0 ? Hkv * runs16 : Hkv, Dv / chunk);
  // rows of several tokens: (key head, run of values) pairs on XCDs of their own where their number divides 8 or is a
  // multiple of it (a one-dimensional grid of 8 x slots blocks; see the kernel)
  int combos = 0;
  if (splits == 0) {
    const long c = (long)Hkv * (Dv / chunk);
    if (c <= 8 ? 8 % c == 0 : c % 8 == 0) {
      combos = (int)c;
      const long blocks = c <= 8 ? 8L * ((tiles + 8 / c - 1) / (8 / c)) : (long)tiles * c;
      if (blocks > 0x7fffffffL) combos = 0;
      else grid = dim3((unsigned)blocks, 1, 1);
    }
  }
  const int nq = D <= 128 ? 4 : D <= 576 ? 18 : 0;  // 32-element runs of a query the kernel keeps in registers
#define TWQ(CC, SP, QQ)                                                                                                        \
  paged_attention_tiled_mfma_wide_kernel<CC, SP, QQ><<<grid, 256, SP ? 0 : key_lds, st>>>(                                     \
      (const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc, block_table, table_width, tile_first, tile_count, token_row, pos, \
      o16, o32, Hq, Hkv, D, Dv, scale, window, keep_first, softcap, sinks, value_share, SP ? splits : 1, SP ? part_o : nullptr,     \
      SP ? part_ml : nullptr, combos, tiles)
#define TW(CC)                                                                                                                 \
  do {                                                                                                                         \
    if (splits > 0) {                                                                                                          \
      if (nq == 4) TWQ(CC, true, 4); else if (nq == 18) TWQ(CC, true, 18); else TWQ(CC, true, 0);                              \
    } else {                                                                                                                   \
      const void* fn = nq == 4 ? (const void*)paged_attention_tiled_mfma_wide_kernel<CC, false, 4>                             \
                       : nq == 18 ? (const void*)paged_attention_tiled_mfma_wide_kernel<CC, false, 18>                         \
                                  : (const void*)paged_attention_tiled_mfma_wide_kernel<CC, false, 0>;                         \
      if (key_lds > 40 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)key_lds) != hipSuccess) \
        return MS_LAUNCH_FAILED;                                                                                               \
      if (nq == 4) TWQ(CC, false, 4); else if (nq == 18) TWQ(CC, false, 18); else TWQ(CC, false, 0);                           \
    }                                                                                                                          \
    if (splits > 1)                                                                                                            \
      paged_attention_mfma_merge_kernel<CC><<<dim3(tiles, Hkv * runs16, Dv / chunk), 256, 16 * (splits + 1) * sizeof(float), st>>>( \
          part_o, part_ml, tile_first, o16, o32, Hq, Hkv, Dv, splits, sinks);                                                   \
  } while (0)
  if (chunk == 256) {
    const void* fn = nq == 18 ? (const void*)paged_attention_tiled_mfma_wide_kernel<256, false, 18>
                              : (const void*)paged_attention_tiled_mfma_wide_kernel<256, false, 0>;
    if (key_lds > 40 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)key_lds) != hipSuccess)
      return MS_LAUNCH_FAILED;
    if (nq == 4 || nq == 18) TWQ(256, false, 18); else TWQ(256, false, 0);
  } else if (chunk == 128) TW(128);
  else if (chunk == 64) TW(64);
  else if (chunk == 32) TW(32);
  else TW(16);
#undef TWQ
#undef TW
  return launch_status();
}

// 1 where the matrix-core form of the tiled kernel takes the shape (bfloat16 storage).
extern "C" int ms_paged_attention_tiled_mfma_ok(int D, int Dv, int page_size) {
  return page_size == MFMA_PAGE && (D == 32 || D == 64 || D == 96 || D == 128) && (Dv == 16 || Dv == 32 || Dv == 64 || Dv == 128);
}

// As ms_paged_attention_tiled for bfloat16 and the shapes above.
extern "C" int ms_paged_attention_tiled_mfma(const void* q, int q_stride, const void* kc, const void* vc, const int* block_table,
                                             int table_width, const int* tile_first, const int* tile_count, int tiles,
                                             const int* token_row, const int* pos, void* out, int Hq, int Hkv, int D, int Dv,
                                             int page_size, float scale, int window, int keep_first, hipStream_t st) {
  if (tiles <= 0) return MS_OK;
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv || window < 0 || keep_first < 0 || table_width <= 0 || Hkv > 65535 || q_stride < Hq * D ||
      q_stride % 8 || tile_first == nullptr || tile_count == nullptr)
    return MS_BAD_ARG;
  if (!ms_paged_attention_tiled_mfma_ok(D, Dv, page_size) || ms_paged_attention_tiled_tokens(Hq / Hkv, D, Dv) == 0) return MS_UNSUPPORTED;
  if (window == 0) keep_first = 0;
  dim3 grid(tiles, Hkv);
#define TM(DD, EE)                                                                                                              \
  paged_attention_tiled_mfma_kernel<DD, EE><<<grid, 256, 0, st>>>((const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc, block_table, \
                                                                  table_width, tile_first, tile_count, token_row, pos, (bf16*)out, Hq, \
                                                                  Hkv, scale, window, keep_first)
#define TD(DD)                      \
  if (Dv == 16) TM(DD, 16);         \
  else if (Dv == 32) TM(DD, 32);    \
  else if (Dv == 64) TM(DD, 64);    \
  else TM(DD, 128)
  if (D == 32) { TD(32); }
  else if (D == 64) { TD(64); }
  else if (D == 96) { TD(96); }
  else { TD(128); }
#undef TD
#undef TM
  return launch_status();
}
