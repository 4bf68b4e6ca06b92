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
#include "common.h"

#define MAX_HEAD_DIM 256

template <typename T> struct Vec16;  // 16 bytes of T
template <> struct Vec16<float> { static constexpr int N = 4; };
template <> struct Vec16<bf16> { static constexpr int N = 8; };

// NW waves per (token, query head): wave w visits the tiles number w, w + NW, ... of those that hold visible keys,
// and the waves' running maxima, sums and outputs meet in LDS in wave order. NW == 1 is the plain form; more waves
// serve steps of few tokens (decode), where one wave per head would walk a long window alone.
template <typename T, int NW>
__global__ __launch_bounds__(NW * WAVE) void paged_attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ token_list,
    const int* __restrict__ token_row, const int* __restrict__ pos, T* __restrict__ out, int Hq, int Hkv, int D, int Dv,
    int page_size, float scale, int window, int keep_first) {
  __shared__ __attribute__((aligned(16))) float qs[MAX_HEAD_DIM];
  __shared__ float ps[NW][WAVE];
  __shared__ float ml[NW][2];
  __shared__ float os[NW > 1 ? NW : 1][NW > 1 ? MAX_HEAD_DIM : 1];
  constexpr int VN = Vec16<T>::N;
  constexpr int PER = MAX_HEAD_DIM / WAVE;
  const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int kvh = h / (Hq / Hkv);
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
    if (page_size % VN == 0 && WAVE % page_size == 0) {
      // Page by page: a lane fetches the page's tokens of its element as 16-byte runs (the page keeps the tokens of
      // one element side by side). Keys that are not visible carry the weight 0, and fmaf(0, v, o) is o: the sum is
      // the one over the visible keys in ascending order. Pages that were given back are not read.
      for (int jp = j0; jp <= je; jp += page_size) {
        if (jp + page_size <= lo && jp >= kept) continue;  // wholly in the gap
        const int page = table[jp / page_size];
        if (page < 0) continue;
        const T* vp = vc + ((size_t)page * Hkv + kvh) * Dv * page_size;
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
        const T* vp = vc + ((size_t)page * Hkv + kvh) * Dv * page_size + (jj % page_size);
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
  const float inv = 1.f / l_run;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = lane + i * WAVE;
    if (e < Dv) ov[e] = from_f32<T>(o[i] * inv);
  }
}

extern "C" int ms_paged_attention_generic(const void* q, int q_stride, const void* kc, const void* vc, int is_bf16,
                                          const int* block_table, int table_width, const int* token_list,
                                          const int* token_row, const int* pos, void* out, int tokens, int Hq, int Hkv,
                                          int D, int Dv, int page_size, float scale, int window, int keep_first, int waves,
                                          hipStream_t st) {
  if (tokens <= 0) return MS_OK;
  if (D <= 0 || D > MAX_HEAD_DIM || Dv <= 0 || Dv > MAX_HEAD_DIM || Hq <= 0 || Hkv <= 0 || Hq % Hkv || page_size <= 0 ||
      window < 0 || keep_first < 0 || table_width <= 0 || Hq > 65535 || q_stride < Hq * D || (waves != 1 && waves != 8 && waves != 16))
    return MS_BAD_ARG;
  if (window == 0) keep_first = 0;  // every key is visible anyway
  dim3 grid(tokens, Hq);
#define GA(T, NW)                                                                                                           \
  paged_attention_generic_kernel<T, NW><<<grid, NW * WAVE, 0, st>>>((const T*)q, q_stride, (const T*)kc, (const T*)vc, block_table, \
                                                                    table_width, token_list, token_row, pos, (T*)out, Hq, Hkv, D, Dv, \
                                                                    page_size, scale, window, keep_first)
  if (is_bf16) {
    if (waves == 16) GA(bf16, 16); else if (waves == 8) GA(bf16, 8); else GA(bf16, 1);
  } else {
    if (waves == 16) GA(float, 16); else if (waves == 8) GA(float, 8); else GA(float, 1);
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
