// Kernels of layers that norm a sublayer's OUTPUT before it joins the residual stream
// (x <- x + rms(y) * w), and of the PolyNorm activation.  Everything is float32 arithmetic on a row
// per workgroup; inputs from GEMMs are float32, outputs go to the compute dtype.
#include "common.h"
#include "yalm_hip.h"

namespace {

constexpr int ROW_THREADS = 256;
constexpr int ROW_WAVES = ROW_THREADS / WAVE;

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void cast_kernel(const float* __restrict__ x, T* __restrict__ out, long n) {
  long i = (long)blockIdx.x * ROW_THREADS + threadIdx.x;
  const long step = (long)gridDim.x * ROW_THREADS;
  for (; i < n; i += step) out[i] = from_f32<T>(x[i]);
}

// x[r] += y[r] * rsqrt(mean(y[r]^2) + eps) * w; if h is given: h[r] = T(x[r]), or with next_w the norm that reads
// the stream next, h[r] = T(x[r] * rsqrt(mean(x[r]^2) + next_eps) * next_w)
template <typename W, typename T, int NT, int PER>
__global__ __launch_bounds__(NT) void norm_add_kernel(const float* __restrict__ y, const W* __restrict__ w, float eps,
                                                      float* __restrict__ x, T* __restrict__ h, const float* __restrict__ next_w,
                                                      float next_eps, int D) {
  // PER > 0: the row fits PER values a thread; y is read once and the new x stays in registers for the second norm
  __shared__ float red[NT / WAVE];
  const size_t row = (size_t)blockIdx.x * D;
  float keep[PER > 0 ? PER : 1];
  float ss = 0.f;
  if (PER > 0) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * NT;
      keep[j] = i < D ? y[row + i] : 0.f;
      ss += keep[j] * keep[j];
    }
  } else {
    for (int i = threadIdx.x; i < D; i += NT) {
      const float v = y[row + i];
      ss += v * v;
    }
  }
  ss = block_sum<NT / WAVE>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)D + eps);
  float ss2 = 0.f;
  if (PER > 0) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * NT;
      if (i < D) {
        const float v = x[row + i] + keep[j] * scale * to_f32(w[i]);
        x[row + i] = v;
        keep[j] = v;
        ss2 += v * v;
        if (h != nullptr && next_w == nullptr) h[row + i] = from_f32<T>(v);
      }
    }
  } else {
    for (int i = threadIdx.x; i < D; i += NT) {
      const float v = x[row + i] + y[row + i] * scale * to_f32(w[i]);
      x[row + i] = v;
      ss2 += v * v;
      if (h != nullptr && next_w == nullptr) h[row + i] = from_f32<T>(v);
    }
  }
  if (h == nullptr || next_w == nullptr) return;
  ss2 = block_sum<NT / WAVE>(ss2, red);
  const float scale2 = 1.0f / sqrtf(ss2 / (float)D + next_eps);
  if (PER > 0) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * NT;
      if (i < D) h[row + i] = from_f32<T>(keep[j] * scale2 * next_w[i]);
    }
  } else {
    for (int i = threadIdx.x; i < D; i += NT) h[row + i] = from_f32<T>(x[row + i] * scale2 * next_w[i]);   // its own stores
  }
}

// out = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the row.  PER > 0: the row fits PER
// values a thread and is read once (kept in registers between the sums and the result); PER = 0: any width, read twice.
template <typename T, int NT, int PER>
__global__ __launch_bounds__(NT) void polynorm_kernel(const float* __restrict__ z, const float* __restrict__ coef, float eps,
                                                      T* __restrict__ out, int F) {
  constexpr int ROW_THREADS = NT, ROW_WAVES = NT / WAVE;
  __shared__ float red[ROW_WAVES];
  const size_t row = (size_t)blockIdx.x * F;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  float keep[PER > 0 ? PER : 1];
  if (PER > 0) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * ROW_THREADS;
      const float v = i < F ? z[row + i] : 0.f;
      keep[j] = v;
      const float v2 = v * v;
      s2 += v2;
      s4 += v2 * v2;
      s6 += v2 * v2 * v2;
    }
  } else {
    for (int i = threadIdx.x; i < F; i += ROW_THREADS) {
      const float v = z[row + i];
      const float v2 = v * v;
      s2 += v2;
      s4 += v2 * v2;
      s6 += v2 * v2 * v2;
    }
  }
  s2 = block_sum<ROW_WAVES>(s2, red);
  s4 = block_sum<ROW_WAVES>(s4, red);
  s6 = block_sum<ROW_WAVES>(s6, red);
  const float r1 = coef[0] / sqrtf(s2 / (float)F + eps);
  const float r2 = coef[1] / sqrtf(s4 / (float)F + eps);
  const float r3 = coef[2] / sqrtf(s6 / (float)F + eps);
  const float e = coef[3];
  if (PER > 0) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * ROW_THREADS;
      const float v = keep[j];
      if (i < F) out[row + i] = from_f32<T>(v * r1 + v * v * r2 + v * v * v * r3 + e);
    }
  } else {
    for (int i = threadIdx.x; i < F; i += ROW_THREADS) {
      const float v = z[row + i];
      out[row + i] = from_f32<T>(v * r1 + v * v * r2 + v * v * v * r3 + e);
    }
  }
}

template <typename T>
int polynorm_launch(const float* z, const float* coef, float eps, void* out, int R, int F, hipStream_t stream) {
  if (F < 2048) polynorm_kernel<T, 256, 8><<<R, 256, 0, stream>>>(z, coef, eps, (T*)out, F);
  else if (F <= 8192) polynorm_kernel<T, 1024, 8><<<R, 1024, 0, stream>>>(z, coef, eps, (T*)out, F);
  else if (F <= 32768) polynorm_kernel<T, 1024, 32><<<R, 1024, 0, stream>>>(z, coef, eps, (T*)out, F);
  else polynorm_kernel<T, 1024, 0><<<R, 1024, 0, stream>>>(z, coef, eps, (T*)out, F);
  return launch_status();
}

}  // namespace

extern "C" int yalm_cast(const float* x, void* out, long n, int out_dtype, hipStream_t stream) {
  if (n <= 0) return YALM_OK;
  const int blocks = (int)((n + ROW_THREADS - 1) / ROW_THREADS < 4096 ? (n + ROW_THREADS - 1) / ROW_THREADS : 4096);
  if (out_dtype == YALM_BF16)
    cast_kernel<bf16><<<blocks, ROW_THREADS, 0, stream>>>(x, (bf16*)out, n);
  else if (out_dtype == YALM_F32)
    cast_kernel<float><<<blocks, ROW_THREADS, 0, stream>>>(x, (float*)out, n);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

template <typename W, typename T>
static int norm_add_launch(const float* y, const void* w, float eps, float* x, void* h, const float* next_w, float next_eps,
                           int R, int D, hipStream_t stream) {
  if (D < 2048)
    norm_add_kernel<W, T, 256, 8><<<R, 256, 0, stream>>>(y, (const W*)w, eps, x, (T*)h, next_w, next_eps, D);
  else if (D <= 8192)
    norm_add_kernel<W, T, 1024, 8><<<R, 1024, 0, stream>>>(y, (const W*)w, eps, x, (T*)h, next_w, next_eps, D);
  else
    norm_add_kernel<W, T, 1024, 0><<<R, 1024, 0, stream>>>(y, (const W*)w, eps, x, (T*)h, next_w, next_eps, D);
  return launch_status();
}

extern "C" int yalm_norm_add(const float* y, const void* w, int w_dtype, float eps, float* x, void* h_out, int h_dtype,
                             const float* next_w, float next_eps, int R, int D, hipStream_t stream) {
  if (R <= 0) return YALM_OK;
  if (D <= 0) return YALM_ERR_ARG;
  if (w_dtype != YALM_F32 && w_dtype != YALM_BF16) return YALM_ERR_DTYPE;
  if (h_out != nullptr && h_dtype != YALM_F32 && h_dtype != YALM_BF16) return YALM_ERR_DTYPE;
  const bool hb = h_out != nullptr && h_dtype == YALM_BF16;
  if (w_dtype == YALM_F32)
    return hb ? norm_add_launch<float, bf16>(y, w, eps, x, h_out, next_w, next_eps, R, D, stream)
              : norm_add_launch<float, float>(y, w, eps, x, h_out, next_w, next_eps, R, D, stream);
  return hb ? norm_add_launch<bf16, bf16>(y, w, eps, x, h_out, next_w, next_eps, R, D, stream)
            : norm_add_launch<bf16, float>(y, w, eps, x, h_out, next_w, next_eps, R, D, stream);
}

extern "C" int yalm_polynorm(const float* z, const float* coef, float eps, void* out, int out_dtype, int R, int F,
                             hipStream_t stream) {
  if (R <= 0) return YALM_OK;
  if (F <= 0) return YALM_ERR_ARG;
  if (out_dtype == YALM_BF16) return polynorm_launch<bf16>(z, coef, eps, out, R, F, stream);
  if (out_dtype == YALM_F32) return polynorm_launch<float>(z, coef, eps, out, R, F, stream);
  return YALM_ERR_DTYPE;
}
