// Mixture of experts: the router, and the experts' products for the (token, choice) pairs.
//
//  * yalm_moe_route: per token, logits = W_router h in float32, scores = softmax over all experts, the
//    `top` largest (the lowest index on ties), with their scores as weights (optionally renormalised
//    to sum 1).  One wave a token.
//  * yalm_moe_pair_gate_up / yalm_moe_pair_down: every pair reads its expert's weights: a wave per output
//    row, the lanes along K with 16-byte loads.  What a decode step needs (few pairs, each bound by
//    the one pass over its expert), and correct for any number of tokens.
//    Expert unit: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit), mid = g sigmoid(alpha g) (u + 1)
//    (limit <= 0: no clamping); out[t] (+)= sum over the token's choices, in order, of weight * W_down mid.
#include "common.h"
#include "yalm_hip.h"

namespace {

constexpr int MOE_MAX_EXPERTS = 1024;
constexpr int PAIR_WAVES = 4;
constexpr int PAIR_ROWS = 32;             // output rows a workgroup

template <typename T>
__device__ __forceinline__ float dot_row(const T* __restrict__ w, const T* __restrict__ x, int K, int lane);

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ w, const float* __restrict__ x, int K, int lane) {
  float acc = 0.f;
  for (int k = lane; k < K; k += WAVE) acc += w[k] * x[k];
  return acc;
}
template <>
__device__ __forceinline__ float dot_row<bf16>(const bf16* __restrict__ w, const bf16* __restrict__ x, int K, int lane) {
  typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
  float acc = 0.f;
  if ((K & 7) == 0 && ((((uintptr_t)w) | ((uintptr_t)x)) & 15) == 0) {
    for (int k = lane * 8; k < K; k += WAVE * 8) {
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(w + k);
      const bf16x8 b = *reinterpret_cast<const bf16x8*>(x + k);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += static_cast<float>(a[j]) * static_cast<float>(b[j]);
    }
  } else {
    for (int k = lane; k < K; k += WAVE) acc += static_cast<float>(w[k]) * static_cast<float>(x[k]);
  }
  return acc;
}

// logits given (w null, h = float32 logits [T, E]) or made here, a dot product a wave at a time
template <typename T>
__global__ __launch_bounds__(WAVE) void moe_route_kernel(const T* __restrict__ h, const T* __restrict__ w, int* __restrict__ ids,
                                                         float* __restrict__ wts, int D, int E, int top, int renorm,
                                                         const float* __restrict__ bias) {
  __shared__ float score[MOE_MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x;
  if (w == nullptr) {
    for (int e = lane; e < E; e += WAVE) score[e] = to_f32(h[(size_t)t * E + e]) + (bias != nullptr ? bias[e] : 0.f);
  } else {
    const T* x = h + (size_t)t * D;
    for (int e = 0; e < E; ++e) {
      const float z = wave_sum(dot_row<T>(w + (size_t)e * D, x, D, lane));
      if (lane == 0) score[e] = z + (bias != nullptr ? bias[e] : 0.f);
    }
  }
  __syncthreads();
  if (renorm == 2) {
    // The experts with the largest LOGITS, weighted by the softmax over the chosen logits alone (no score is formed
    // over all experts, so that a logit far below the largest still takes its place in the order).
    float first = 0.f, total = 0.f;
    for (int k = 0; k < top; ++k) {
      float best = -3.4e38f;
      int at = 0x7fffffff;
      for (int e = lane; e < E; e += WAVE) {
        const float v = score[e];
        if (v > best) { best = v; at = e; }
      }
      for (int o = WAVE / 2; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, WAVE);
        const int oa = __shfl_xor(at, o, WAVE);
        if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
      }
      if (at == 0x7fffffff) at = 0;               // nothing finite is left
      if (k == 0) first = best;
      const float wk = expf(best - first);
      if (lane == 0) {
        ids[(size_t)t * top + k] = at;
        wts[(size_t)t * top + k] = wk;
        score[at] = -3.4e38f;                     // taken
      }
      total += wk;
      __syncthreads();
    }
    for (int k = lane; k < top; k += WAVE) wts[(size_t)t * top + k] /= total;
    return;
  }
  float m = -3.0e38f;
  for (int e = lane; e < E; e += WAVE) m = fmaxf(m, score[e]);
  m = wave_max(m);
  float s = 0.f;
  for (int e = lane; e < E; e += WAVE) s += expf(score[e] - m);
  s = wave_sum(s);
  __syncthreads();
  for (int e = lane; e < E; e += WAVE) score[e] = expf(score[e] - m) / s;
  __syncthreads();
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -1.f;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += WAVE) {
      const float v = score[e];
      if (v > best) { best = v; at = e; }         // the first of equals in a lane's run
    }
    for (int o = WAVE / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, WAVE);
      const int oa = __shfl_xor(at, o, WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (lane == 0) {
      ids[(size_t)t * top + k] = at;
      wts[(size_t)t * top + k] = best;
      score[at] = -2.f;                           // taken
    }
    total += best;
    __syncthreads();
  }
  if (renorm)
    for (int k = lane; k < top; k += WAVE) wts[(size_t)t * top + k] /= total;
}

template <typename T>
__global__ __launch_bounds__(PAIR_WAVES * WAVE) void moe_pair_gate_up_kernel(const T* __restrict__ h, const T* __restrict__ w_gate,
                                                                             const T* __restrict__ w_up, const int* __restrict__ ids,
                                                                             float limit, float alpha, float up_shift, T* __restrict__ mid, int top,
                                                                             int D, int F, int E) {
  const int pair = blockIdx.x;
  const int e = ids[pair];
  if (e < 0 || e >= E) return;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* x = h + (size_t)(pair / top) * D;
  const int f0 = blockIdx.y * PAIR_ROWS;
  for (int f = f0 + wave; f < min(F, f0 + PAIR_ROWS); f += PAIR_WAVES) {
    const size_t r = ((size_t)e * F + f) * D;
    float g = wave_sum(dot_row<T>(w_gate + r, x, D, lane));
    float u = wave_sum(dot_row<T>(w_up + r, x, D, lane));
    if (limit > 0.f) {
      g = fminf(g, limit);
      u = fminf(fmaxf(u, -limit), limit);
    }
    if (lane == 0) mid[(size_t)pair * F + f] = from_f32<T>(g / (1.0f + expf(-alpha * g)) * (u + up_shift));
  }
}

template <typename T>
__global__ __launch_bounds__(PAIR_WAVES * WAVE) void moe_pair_down_kernel(const T* __restrict__ mid, const T* __restrict__ w_down,
                                                                          const int* __restrict__ ids, const float* __restrict__ wts,
                                                                          float* __restrict__ out, int top, int D, int F, int E, int accumulate) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int d0 = blockIdx.y * PAIR_ROWS;
  for (int d = d0 + wave; d < min(D, d0 + PAIR_ROWS); d += PAIR_WAVES) {
    float acc = 0.f;
    for (int k0 = 0; k0 < top; k0 += 4) {          // four choices' rows at a time: their loads are in flight together
      float part[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + i;
        const int e = k < top ? ids[(size_t)t * top + k] : -1;
        part[i] = e >= 0 && e < E ? dot_row<T>(w_down + ((size_t)e * D + d) * F, mid + ((size_t)t * top + k) * F, F, lane) : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + i;
        const float v = wave_sum(part[i]);
        if (k < top) acc += wts[(size_t)t * top + k] * v;    // in the order of the choices
      }
    }
    if (lane == 0) out[(size_t)t * D + d] = accumulate ? out[(size_t)t * D + d] + acc : acc;
  }
}


// ---------------------------------------------------------------------------
// Many tokens (a step of whole prompts): the pairs are grouped by expert, every expert's rows padded to whole
// tiles of GR_TM rows, and one launch multiplies all tiles on the matrix cores, each with its expert's weights.
//
// moe_group_kernel (one workgroup): counts the pairs of every expert, lays the experts' row blocks one behind
// the other (each a multiple of GR_TM rows), and writes pair_of_row[row] (-1: padding), row_of_pair[pair] and
// tile_expert[tile] (-1: behind the last used tile).  The order of an expert's rows among themselves is not
// fixed, and no result depends on it: a row of a product depends on that row alone.
// ---------------------------------------------------------------------------
constexpr int GR_TM = 128, GR_TN = 256, GR_TK = 64, GR_ROW = GR_TK + 8, GR_THREADS = 256;
constexpr int GROUP_THREADS = 1024;

__global__ __launch_bounds__(GROUP_THREADS) void moe_group_kernel(const int* __restrict__ ids, int n_pairs, int E, int max_tiles,
                                                                  int* __restrict__ pair_of_row, int* __restrict__ row_of_pair,
                                                                  int* __restrict__ tile_expert) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int start[MOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += GROUP_THREADS) count[e] = 0;
  for (int r = tid; r < max_tiles * GR_TM; r += GROUP_THREADS) pair_of_row[r] = -1;
  for (int t = tid; t < max_tiles; t += GROUP_THREADS) tile_expert[t] = -1;
  __syncthreads();
  for (int p = tid; p < n_pairs; p += GROUP_THREADS) {
    const int e = ids[p];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at * GR_TM;
      const int tiles = (count[e] + GR_TM - 1) / GR_TM;
      for (int i = 0; i < tiles && at + i < max_tiles; ++i) tile_expert[at + i] = e;
      at += tiles;
      count[e] = 0;
    }
  }
  __syncthreads();
  for (int p = tid; p < n_pairs; p += GROUP_THREADS) {
    const int e = ids[p];
    if (e < 0 || e >= E) { row_of_pair[p] = -1; continue; }
    const int row = start[e] + atomicAdd(&count[e], 1);
    if (row < max_tiles * GR_TM) {
      pair_of_row[row] = p;
      row_of_pair[p] = row;
    } else {
      row_of_pair[p] = -1;
    }
  }
}

typedef __attribute__((ext_vector_type(8))) __bf16 gr_bf16x8;
typedef __attribute__((ext_vector_type(16))) float gr_f32x16;

// A tile of GR_TM rows x GR_TN weight rows, 4 waves in 2 x 2, each 64 rows x 128 weight rows: six fragment reads
// for eight matrix instructions (v_mfma_f32_32x32x16_bf16: operand rows = lane % 32, 8 k a lane at k offset
// 8 * (lane / 32); C: column = lane % 32, rows 8 (r / 4) + 4 (lane / 32) + r % 4).  One LDS buffer, the next k tile
// waits in registers.
// GATED: A rows are gathered (row -> pair -> token); a wave's 128 weight rows are 64 gate rows and the 64 up rows of
// the same hidden columns, and the epilogue writes mid[row, f] = act(g, u).  Else: A = mid rows as they lie, the
// weight rows are 256 rows of the expert's down matrix, and the epilogue stores float32 out[row, n].
template <bool GATED>
__global__ __launch_bounds__(GR_THREADS, 2) void moe_grouped_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W0,
                                                                    const bf16* __restrict__ W1, const int* __restrict__ tile_expert,
                                                                    const int* __restrict__ pair_of_row, int top, void* __restrict__ Cv,
                                                                    int N, int K, float limit, float alpha, float up_shift) {
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* As = reinterpret_cast<bf16*>(smem_raw);       // [GR_TM][GR_ROW]
  bf16* Ws = As + GR_TM * GR_ROW;                      // [GR_TN][GR_ROW]
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int wm = wave / 2, wn = wave % 2;
  const int li = lane % 32, lh = lane / 32;
  const int m0 = blockIdx.y * GR_TM;
  const int n0 = blockIdx.x * (GATED ? GR_TN / 2 : GR_TN);      // first output column of the tile
  constexpr int RPP = GR_THREADS / 8;                  // 32 rows a pass
  constexpr int LA = GR_TM / RPP, LB = GR_TN / RPP;    // chunks of 16 bytes a thread and operand
  const int lrow = tid / 8, lk = (tid % 8) * 8;
  const bf16* ap[LA];
  const bf16* wp[LB];
  bool aok[LA], wok[LB];
#pragma unroll
  for (int p = 0; p < LA; ++p) {
    const int row = m0 + lrow + RPP * p;
    const int pair = pair_of_row[row];
    aok[p] = pair >= 0;
    ap[p] = A + (size_t)(GATED ? (aok[p] ? pair / top : 0) : row) * K + lk;
  }
#pragma unroll
  for (int p = 0; p < LB; ++p) {
    const int j = lrow + RPP * p;                      // row of the weight tile
    int n;
    const bf16* base;
    if (GATED) {                                       // [gate 0..63 | up 0..63 | gate 64..127 | up 64..127]
      n = n0 + (j / 128) * 64 + j % 64;
      base = (j / 64) % 2 ? W1 : W0;
    } else {
      n = n0 + j;
      base = W0;
    }
    wok[p] = n < N;
    wp[p] = base + ((size_t)e * N + (wok[p] ? n : 0)) * K + lk;
  }
  gr_f32x16 acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  const gr_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  gr_bf16x8 ra[LA], rw[LB];
  const int nk = (K + GR_TK - 1) / GR_TK;
  {
    const bool kok = lk < K;
#pragma unroll
    for (int p = 0; p < LA; ++p) ra[p] = aok[p] && kok ? *reinterpret_cast<const gr_bf16x8*>(ap[p]) : zero;
#pragma unroll
    for (int p = 0; p < LB; ++p) rw[p] = wok[p] && kok ? *reinterpret_cast<const gr_bf16x8*>(wp[p]) : zero;
  }
  for (int kt = 0; kt < nk; ++kt) {
#pragma unroll
    for (int p = 0; p < LA; ++p) *reinterpret_cast<gr_bf16x8*>(&As[(lrow + RPP * p) * GR_ROW + lk]) = ra[p];
#pragma unroll
    for (int p = 0; p < LB; ++p) *reinterpret_cast<gr_bf16x8*>(&Ws[(lrow + RPP * p) * GR_ROW + lk]) = rw[p];
    __syncthreads();
    if (kt + 1 < nk) {
      const bool kok = (kt + 1) * GR_TK + lk < K;
#pragma unroll
      for (int p = 0; p < LA; ++p)
        ra[p] = aok[p] && kok ? *reinterpret_cast<const gr_bf16x8*>(ap[p] + (size_t)(kt + 1) * GR_TK) : zero;
#pragma unroll
      for (int p = 0; p < LB; ++p)
        rw[p] = wok[p] && kok ? *reinterpret_cast<const gr_bf16x8*>(wp[p] + (size_t)(kt + 1) * GR_TK) : zero;
    }
#pragma unroll
    for (int ks = 0; ks < GR_TK / 16; ++ks) {
      gr_bf16x8 fa[2], fw[4];
#pragma unroll
      for (int a = 0; a < 2; ++a)
        fa[a] = *reinterpret_cast<const gr_bf16x8*>(&As[(wm * 64 + a * 32 + li) * GR_ROW + ks * 16 + lh * 8]);
#pragma unroll
      for (int b = 0; b < 4; ++b)
        fw[b] = *reinterpret_cast<const gr_bf16x8*>(&Ws[(wn * 128 + b * 32 + li) * GR_ROW + ks * 16 + lh * 8]);
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[a], fw[b], acc[a][b], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < 2; ++a) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + wm * 64 + a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
      if (pair_of_row[row] < 0) continue;
      if (GATED) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const int f = n0 + wn * 64 + b * 32 + li;
          if (f >= N) continue;
          float g = acc[a][b][r], u = acc[a][b + 2][r];
          if (limit > 0.f) {
            g = fminf(g, limit);
            u = fminf(fmaxf(u, -limit), limit);
          }
          ((bf16*)Cv)[(size_t)row * N + f] = static_cast<bf16>(g / (1.0f + expf(-alpha * g)) * (u + up_shift));
        }
      } else {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int n = n0 + wn * 128 + b * 32 + li;
          if (n < N) ((float*)Cv)[(size_t)row * N + n] = acc[a][b][r];
        }
      }
    }
  }
}

// out[t, :] (+)= sum over k, in order, of wts[t, k] * y[row_of_pair[t * top + k], :]
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ row_of_pair,
                                                          const float* __restrict__ wts, float* __restrict__ out, int top, int D,
                                                          int accumulate) {
  const int t = blockIdx.x;
  for (int d = threadIdx.x; d < D; d += 256) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int row = row_of_pair[(size_t)t * top + k];
      if (row >= 0) acc += wts[(size_t)t * top + k] * y[(size_t)row * D + d];
    }
    out[(size_t)t * D + d] = accumulate ? out[(size_t)t * D + d] + acc : acc;
  }
}

}  // namespace

extern "C" int yalm_moe_route(const void* h, const void* w_router, int dtype, int* ids, float* wts, int T, int D, int E,
                              int top, int renorm, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || top > E) return YALM_ERR_ARG;
  if (dtype == YALM_BF16)
    moe_route_kernel<bf16><<<T, WAVE, 0, stream>>>((const bf16*)h, (const bf16*)w_router, ids, wts, D, E, top, renorm, nullptr);
  else if (dtype == YALM_F32)
    moe_route_kernel<float><<<T, WAVE, 0, stream>>>((const float*)h, (const float*)w_router, ids, wts, D, E, top, renorm, nullptr);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_moe_select(const float* logits, const float* bias, int* ids, float* wts, int T, int E, int top,
                               int renorm, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || top > E) return YALM_ERR_ARG;
  if (renorm < 0 || renorm > 2) return YALM_ERR_ARG;
  moe_route_kernel<float><<<T, WAVE, 0, stream>>>(logits, nullptr, ids, wts, E, E, top, renorm, bias);
  return launch_status();
}

extern "C" int yalm_moe_pair_gate_up(const void* h, const void* w_gate, const void* w_up, const int* ids, float limit,
                                     float alpha, float up_shift, void* mid, int T, int top, int D, int F, int E, int dtype,
                                     hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || F <= 0 || E <= 0 || top <= 0) return YALM_ERR_ARG;
  dim3 grid(T * top, ceil_div(F, PAIR_ROWS));
  if (dtype == YALM_BF16)
    moe_pair_gate_up_kernel<bf16><<<grid, PAIR_WAVES * WAVE, 0, stream>>>((const bf16*)h, (const bf16*)w_gate, (const bf16*)w_up,
                                                                          ids, limit, alpha, up_shift, (bf16*)mid, top, D, F, E);
  else if (dtype == YALM_F32)
    moe_pair_gate_up_kernel<float><<<grid, PAIR_WAVES * WAVE, 0, stream>>>((const float*)h, (const float*)w_gate,
                                                                           (const float*)w_up, ids, limit, alpha, up_shift, (float*)mid,
                                                                           top, D, F, E);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_moe_pair_down(const void* mid, const void* w_down, const int* ids, const float* wts, float* out, int T,
                                  int top, int D, int F, int E, int dtype, int accumulate, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || F <= 0 || E <= 0 || top <= 0) return YALM_ERR_ARG;
  dim3 grid(T, ceil_div(D, PAIR_ROWS));
  if (dtype == YALM_BF16)
    moe_pair_down_kernel<bf16><<<grid, PAIR_WAVES * WAVE, 0, stream>>>((const bf16*)mid, (const bf16*)w_down, ids, wts, out, top,
                                                                       D, F, E, accumulate);
  else if (dtype == YALM_F32)
    moe_pair_down_kernel<float><<<grid, PAIR_WAVES * WAVE, 0, stream>>>((const float*)mid, (const float*)w_down, ids, wts, out,
                                                                        top, D, F, E, accumulate);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

// The grouped path for many tokens (bfloat16; D and F multiples of 8).  max_tiles = yalm_moe_grouped_tiles(T * top, E);
// pair_of_row int32 [max_tiles * 128], row_of_pair int32 [T * top], tile_expert int32 [max_tiles], mid bfloat16
// [max_tiles * 128, F], y float32 [max_tiles * 128, D]: scratch of the caller.
extern "C" int yalm_moe_grouped_tiles(int n_pairs, int E) { return ceil_div(n_pairs, GR_TM) + E; }

extern "C" int yalm_moe_grouped(const void* h, const void* w_gate, const void* w_up, const void* w_down, const int* ids,
                                const float* wts, float limit, float alpha, float up_shift, int* pair_of_row, int* row_of_pair,
                                int* tile_expert, void* mid, float* y, float* out, int T, int top, int D, int F, int E,
                                int accumulate, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || F <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || (D & 7) || (F & 7) ||
      ((((uintptr_t)h) | ((uintptr_t)w_gate) | ((uintptr_t)w_up) | ((uintptr_t)w_down) | ((uintptr_t)mid)) & 15))
    return YALM_ERR_ARG;
  const long n_pairs = (long)T * top;
  if (n_pairs > (1l << 30)) return YALM_ERR_ARG;
  const int max_tiles = yalm_moe_grouped_tiles((int)n_pairs, E);
  if (max_tiles > 65535) return YALM_ERR_ARG;
  moe_group_kernel<<<1, GROUP_THREADS, 0, stream>>>(ids, (int)n_pairs, E, max_tiles, pair_of_row, row_of_pair, tile_expert);
  const size_t lds = (size_t)(GR_TM + GR_TN) * GR_ROW * sizeof(bf16);
  moe_grouped_kernel<true><<<dim3(ceil_div(F, GR_TN / 2), max_tiles), GR_THREADS, lds, stream>>>(
      (const bf16*)h, (const bf16*)w_gate, (const bf16*)w_up, tile_expert, pair_of_row, top, mid, F, D, limit, alpha, up_shift);
  moe_grouped_kernel<false><<<dim3(ceil_div(D, GR_TN), max_tiles), GR_THREADS, lds, stream>>>(
      (const bf16*)mid, (const bf16*)w_down, nullptr, tile_expert, pair_of_row, top, y, D, F, 0.f, 0.f, 0.f);
  moe_combine_kernel<<<T, 256, 0, stream>>>(y, row_of_pair, wts, out, top, D, accumulate);
  return launch_status();
}
