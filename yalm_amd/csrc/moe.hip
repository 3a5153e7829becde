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

template <typename T>
__global__ __launch_bounds__(WAVE) void moe_route_kernel(const T* __restrict__ h, const T* __restrict__ w, int* __restrict__ ids,
                                                         float* __restrict__ wts, int D, int E, int top, int renorm) {
  __shared__ float score[MOE_MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x;
  const T* x = h + (size_t)t * D;
  for (int e = 0; e < E; ++e) {
    const float z = wave_sum(dot_row<T>(w + (size_t)e * D, x, D, lane));
    if (lane == 0) score[e] = z;
  }
  __syncthreads();
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
                                                                             float limit, float alpha, T* __restrict__ mid, int top,
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
    if (lane == 0) mid[(size_t)pair * F + f] = from_f32<T>(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
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
    for (int k = 0; k < top; ++k) {
      const int e = ids[(size_t)t * top + k];
      if (e < 0 || e >= E) continue;
      const float v = wave_sum(dot_row<T>(w_down + ((size_t)e * D + d) * F, mid + ((size_t)t * top + k) * F, F, lane));
      acc += wts[(size_t)t * top + k] * v;
    }
    if (lane == 0) out[(size_t)t * D + d] = accumulate ? out[(size_t)t * D + d] + acc : acc;
  }
}

}  // namespace

extern "C" int yalm_moe_route(const void* h, const void* w_router, int dtype, int* ids, float* wts, int T, int D, int E,
                              int top, int renorm, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || top > E) return YALM_ERR_ARG;
  if (dtype == YALM_BF16)
    moe_route_kernel<bf16><<<T, WAVE, 0, stream>>>((const bf16*)h, (const bf16*)w_router, ids, wts, D, E, top, renorm);
  else if (dtype == YALM_F32)
    moe_route_kernel<float><<<T, WAVE, 0, stream>>>((const float*)h, (const float*)w_router, ids, wts, D, E, top, renorm);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_moe_pair_gate_up(const void* h, const void* w_gate, const void* w_up, const int* ids, float limit,
                                     float alpha, void* mid, int T, int top, int D, int F, int E, int dtype,
                                     hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || F <= 0 || E <= 0 || top <= 0) return YALM_ERR_ARG;
  dim3 grid(T * top, ceil_div(F, PAIR_ROWS));
  if (dtype == YALM_BF16)
    moe_pair_gate_up_kernel<bf16><<<grid, PAIR_WAVES * WAVE, 0, stream>>>((const bf16*)h, (const bf16*)w_gate, (const bf16*)w_up,
                                                                          ids, limit, alpha, (bf16*)mid, top, D, F, E);
  else if (dtype == YALM_F32)
    moe_pair_gate_up_kernel<float><<<grid, PAIR_WAVES * WAVE, 0, stream>>>((const float*)h, (const float*)w_gate,
                                                                           (const float*)w_up, ids, limit, alpha, (float*)mid,
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
