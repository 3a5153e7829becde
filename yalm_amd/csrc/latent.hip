// Latent attention: keys and values of all heads are functions of one small vector c per token, so the
// cache keeps one "head" a token, [rotated part | c | zeros up to the padded size], and attention runs in
// the latent space: a query head becomes [its rotated part | W_uk_h^T q_h], the result of a head is a mix
// of c vectors that W_uv_h turns into the head's values afterwards.  The attention kernels are the
// grouped-query ones with one KV head.
//
//  * yalm_latent_pack: per token, the RMS norm of the down projection's first `rank` columns, and the
//    head-shaped rows that the rotation kernel reads (query rotated parts scaled, key, value).
//  * yalm_head_matmul: out[t, h, :] = scale * in[t, h, :] Wt[h] for every head, Wt [H, K, N]
//    (optionally times sigmoid(gate)): the two per-head products (W_uk^T on queries, W_uv on results).
//    float32 arithmetic; a workgroup owns 16 tokens and 64 columns of a head's result, a lane a column.
//  * yalm_head_matmul_mfma: the same for many tokens on the matrix cores (bfloat16 weights [H, N, K]).
#include "common.h"
#include "yalm_hip.h"

namespace {

constexpr int HM_TOK = 16;                 // tokens a workgroup
constexpr int HM_THREADS = 256;
constexpr int HM_KMAX = 512;               // the most K the LDS tile holds

template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(HM_THREADS) void head_matmul_kernel(const TI* __restrict__ in, long in_row, int in_head, int in_off,
                                                                 const TW* __restrict__ wt, TO* __restrict__ out, long out_row,
                                                                 int out_head, int out_off, float scale,
                                                                 const float* __restrict__ gate, long gate_row, int T,
                                                                 int K, int N) {
  __shared__ float tile[HM_TOK][HM_KMAX];
  const int h = blockIdx.y;
  const int t0 = blockIdx.x * HM_TOK;
  const int tg = threadIdx.x / WAVE;        // a wave takes 4 of the 16 tokens
  const int lane = threadIdx.x % WAVE;
  const TW* w = wt + (size_t)h * K * N;
  const int n = blockIdx.z * WAVE + lane;          // a workgroup owns 64 columns of the head's result
  // the first 128 weights of the lane's column (all of them, at most sizes) and the gate's values are asked for
  // before the tokens' values, so that the waits for memory are one
  constexpr int FIRST = 128;
  TW w0[FIRST];
#pragma unroll
  for (int i = 0; i < FIRST; ++i) w0[i] = w[(size_t)min(i, K - 1) * N + min(n, N - 1)];
  float g4[4] = {0.f, 0.f, 0.f, 0.f};
  if (gate != nullptr) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      g4[j] = gate[(size_t)min(t0 + tg * 4 + j, T - 1) * gate_row + (size_t)h * N + min(n, N - 1)];
  }
  const int Kt = max(K, FIRST);                    // the tile is filled to FIRST columns at least, zeros behind K
  for (int i = threadIdx.x; i < HM_TOK * Kt; i += HM_THREADS) {
    const int tt = i / Kt, k = i % Kt;
    const int t = t0 + tt;
    tile[tt][k] = t < T && k < K ? to_f32(in[(size_t)t * in_row + (size_t)h * in_head + in_off + k]) : 0.f;
  }
  __syncthreads();
  if (n < N) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    // no branch in these 128 steps (behind K the tile holds zeros and the weights count as zero), so that the
    // reads of the tile run ahead of the products
#pragma unroll
    for (int i0 = 0; i0 < FIRST; i0 += 4) {
      float wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) wv[i] = i0 + i < K ? to_f32(w0[i0 + i]) : 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 a = *reinterpret_cast<const float4*>(&tile[tg * 4 + j][i0]);
        acc[j] += a.x * wv[0] + a.y * wv[1] + a.z * wv[2] + a.w * wv[3];
      }
    }
    int k = FIRST;
    for (; k + 32 <= K; k += 32) {                   // thirty-two loads in flight, then their products
      TW wv[32];
#pragma unroll
      for (int i = 0; i < 32; ++i) wv[i] = w[(size_t)(k + i) * N + n];
#pragma unroll
      for (int i = 0; i < 32; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] += tile[tg * 4 + j][k + i] * to_f32(wv[i]);
    }
    for (; k < K; ++k) {
      const float wv = to_f32(w[(size_t)k * N + n]);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += tile[tg * 4 + j][k] * wv;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = t0 + tg * 4 + j;
      if (t >= T) continue;
      float v = acc[j] * scale;
      if (gate != nullptr) v *= 1.0f / (1.0f + expf(-g4[j]));
      out[(size_t)t * out_row + (size_t)h * out_head + out_off + n] = from_f32<TO>(v);
    }
  }
}

// One wave a (token, job).  job < H: the rotated part of query head `job`, scaled, and zeros behind the
// latent part; job == H (has_kv only): the key and value rows.
template <typename TN>
__global__ __launch_bounds__(WAVE) void latent_pack_kernel(const float* __restrict__ proj, long proj_row, int q_head,
                                                           int q_rot_off, int kv_off, const TN* __restrict__ norm_w, float eps,
                                                           float q_scale, float* __restrict__ out, int H, int rot, int rank,
                                                           int Dk, int has_kv) {
  const int t = blockIdx.x, job = blockIdx.y, lane = threadIdx.x;
  const float* row = proj + (size_t)t * proj_row;
  float* dst = out + (size_t)t * (H + 2) * Dk;
  if (job < H) {
    float* q = dst + (size_t)job * Dk;
    for (int i = lane; i < rot; i += WAVE) q[i] = row[(size_t)job * q_head + q_rot_off + i] * q_scale;
    for (int i = rot + rank + lane; i < Dk; i += WAVE) q[i] = 0.f;
    return;
  }
  if (!has_kv) return;
  const float* d = row + kv_off;
  float ss = 0.f;
  for (int i = lane; i < rank; i += WAVE) ss += d[i] * d[i];
  ss = wave_sum(ss);
  const float s = 1.0f / sqrtf(ss / (float)rank + eps);
  float* k = dst + (size_t)H * Dk;
  float* v = k + Dk;
  for (int i = lane; i < rot; i += WAVE) {
    k[i] = d[rank + i];
    v[i] = 0.f;
  }
  for (int i = lane; i < rank; i += WAVE) {
    const float c = d[i] * s * to_f32(norm_w[i]);
    k[rot + i] = c;
    v[rot + i] = c;
  }
  for (int i = rot + rank + lane; i < Dk; i += WAVE) {
    k[i] = 0.f;
    v[i] = 0.f;
  }
}

// The same product on the matrix cores, for many tokens: wn [H, N, K] bfloat16 (a column's K values lie together), the
// tokens' values rounded to bfloat16 on their way into LDS, float32 sums.  A workgroup owns 128 tokens x 128
// columns of a head, 4 waves in 2 x 2 of 64 x 64 (v_mfma_f32_32x32x16_bf16), k tiles of 64 through one LDS buffer
// with the next tile waiting in registers.  Needs K a multiple of 8 and rows, heads and offsets that keep every
// 8 values of a token 16-byte aligned (32-byte for float32 input).
typedef __attribute__((ext_vector_type(8))) __bf16 hm_bf16x8;
typedef __attribute__((ext_vector_type(16))) float hm_f32x16;
constexpr int HG_TM = 128, HG_TN = 128, HG_TK = 64, HG_ROW = HG_TK + 8, HG_THREADS = 256;

__device__ __forceinline__ hm_bf16x8 load8_bf16(const bf16* p) { return *reinterpret_cast<const hm_bf16x8*>(p); }
__device__ __forceinline__ hm_bf16x8 load8_bf16(const float* p) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  hm_bf16x8 v = {static_cast<bf16>(a.x), static_cast<bf16>(a.y), static_cast<bf16>(a.z), static_cast<bf16>(a.w),
                 static_cast<bf16>(b.x), static_cast<bf16>(b.y), static_cast<bf16>(b.z), static_cast<bf16>(b.w)};
  return v;
}

template <typename TI, typename TO>
__global__ __launch_bounds__(HG_THREADS, 2) void head_mfma_kernel(const TI* __restrict__ in, long in_row, int in_head, int in_off,
                                                                  const bf16* __restrict__ wn, TO* __restrict__ out, long out_row,
                                                                  int out_head, int out_off, float scale,
                                                                  const float* __restrict__ gate, long gate_row, int T, int K,
                                                                  int N) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* As = reinterpret_cast<bf16*>(smem_raw);       // [HG_TM][HG_ROW]
  bf16* Ws = As + HG_TM * HG_ROW;                      // [HG_TN][HG_ROW]
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int wm = wave / 2, wnn = wave % 2, li = lane % 32, lh = lane / 32;
  const int h = blockIdx.y, m0 = blockIdx.x * HG_TM, n0 = blockIdx.z * HG_TN;
  constexpr int RPP = HG_THREADS / 8, LA = HG_TM / RPP, LB = HG_TN / RPP;
  const int lrow = tid / 8, lk = (tid % 8) * 8;
  const TI* ap[LA];
  const bf16* wp[LB];
  bool aok[LA], wok[LB];
#pragma unroll
  for (int p = 0; p < LA; ++p) {
    const int t = m0 + lrow + RPP * p;
    aok[p] = t < T;
    ap[p] = in + (size_t)(aok[p] ? t : 0) * in_row + (size_t)h * in_head + in_off + lk;
  }
#pragma unroll
  for (int p = 0; p < LB; ++p) {
    const int n = n0 + lrow + RPP * p;
    wok[p] = n < N;
    wp[p] = wn + ((size_t)h * N + (wok[p] ? n : 0)) * K + lk;
  }
  hm_f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  const hm_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  hm_bf16x8 ra[LA], rw[LB];
  const int nk = (K + HG_TK - 1) / HG_TK;
  {
    const bool kok = lk < K;
#pragma unroll
    for (int p = 0; p < LA; ++p) ra[p] = aok[p] && kok ? load8_bf16(ap[p]) : zero;
#pragma unroll
    for (int p = 0; p < LB; ++p) rw[p] = wok[p] && kok ? load8_bf16(wp[p]) : zero;
  }
  for (int kt = 0; kt < nk; ++kt) {
#pragma unroll
    for (int p = 0; p < LA; ++p) *reinterpret_cast<hm_bf16x8*>(&As[(lrow + RPP * p) * HG_ROW + lk]) = ra[p];
#pragma unroll
    for (int p = 0; p < LB; ++p) *reinterpret_cast<hm_bf16x8*>(&Ws[(lrow + RPP * p) * HG_ROW + lk]) = rw[p];
    __syncthreads();
    if (kt + 1 < nk) {
      const bool kok = (kt + 1) * HG_TK + lk < K;
#pragma unroll
      for (int p = 0; p < LA; ++p) ra[p] = aok[p] && kok ? load8_bf16(ap[p] + (kt + 1) * HG_TK) : zero;
#pragma unroll
      for (int p = 0; p < LB; ++p) rw[p] = wok[p] && kok ? load8_bf16(wp[p] + (kt + 1) * HG_TK) : zero;
    }
#pragma unroll
    for (int ks = 0; ks < HG_TK / 16; ++ks) {
      hm_bf16x8 fa[2], fw[2];
#pragma unroll
      for (int a = 0; a < 2; ++a)
        fa[a] = *reinterpret_cast<const hm_bf16x8*>(&As[(wm * 64 + a * 32 + li) * HG_ROW + ks * 16 + lh * 8]);
#pragma unroll
      for (int b = 0; b < 2; ++b)
        fw[b] = *reinterpret_cast<const hm_bf16x8*>(&Ws[(wnn * 64 + b * 32 + li) * HG_ROW + ks * 16 + lh * 8]);
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[a], fw[b], acc[a][b], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int t = m0 + wm * 64 + a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
      if (t >= T) continue;
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int n = n0 + wnn * 64 + b * 32 + li;
        if (n >= N) continue;
        float v = acc[a][b][r] * scale;
        if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[(size_t)t * gate_row + (size_t)h * N + n]));
        out[(size_t)t * out_row + (size_t)h * out_head + out_off + n] = from_f32<TO>(v);
      }
    }
}

template <typename TI, typename TW, typename TO>
int head_matmul_launch(const void* in, long in_row, int in_head, int in_off, const void* wt, void* out, long out_row,
                       int out_head, int out_off, float scale, const float* gate, long gate_row, int T, int H, int K,
                       int N, hipStream_t stream) {
  dim3 grid(ceil_div(T, HM_TOK), H, ceil_div(N, WAVE));
  head_matmul_kernel<TI, TW, TO><<<grid, HM_THREADS, 0, stream>>>((const TI*)in, in_row, in_head, in_off, (const TW*)wt,
                                                                  (TO*)out, out_row, out_head, out_off, scale, gate,
                                                                  gate_row, T, K, N);
  return launch_status();
}

}  // namespace

extern "C" int yalm_head_matmul(const void* in, int in_dtype, long in_row, int in_head, int in_off, const void* wt,
                                int w_dtype, void* out, int out_dtype, long out_row, int out_head, int out_off,
                                float scale, const float* gate, long gate_row, int T, int H, int K, int N,
                                hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (H <= 0 || K <= 0 || N <= 0 || K > HM_KMAX || in_off < 0 || out_off < 0 || in_off + K > in_head ||
      out_off + N > out_head || (long)H * in_head > in_row || (long)H * out_head > out_row ||
      (gate != nullptr && (long)H * N > gate_row))
    return YALM_ERR_ARG;
#define HM(TI, TW, TO) \
  return head_matmul_launch<TI, TW, TO>(in, in_row, in_head, in_off, wt, out, out_row, out_head, out_off, scale, gate, \
                                        gate_row, T, H, K, N, stream)
  if (in_dtype == YALM_F32 && w_dtype == YALM_F32 && out_dtype == YALM_F32) HM(float, float, float);
  if (in_dtype == YALM_F32 && w_dtype == YALM_BF16 && out_dtype == YALM_F32) HM(float, bf16, float);
  if (in_dtype == YALM_BF16 && w_dtype == YALM_BF16 && out_dtype == YALM_BF16) HM(bf16, bf16, bf16);
#undef HM
  return YALM_ERR_DTYPE;
}

extern "C" int yalm_head_matmul_mfma(const void* in, int in_dtype, long in_row, int in_head, int in_off, const void* wn,
                                     void* out, int out_dtype, long out_row, int out_head, int out_off, float scale,
                                     const float* gate, long gate_row, int T, int H, int K, int N, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (H <= 0 || K <= 0 || N <= 0 || in_off < 0 || out_off < 0 || in_off + K > in_head || out_off + N > out_head ||
      (long)H * in_head > in_row || (long)H * out_head > out_row || (gate != nullptr && (long)H * N > gate_row) ||
      H > 65535 || ceil_div(N, HG_TN) > 65535)
    return YALM_ERR_ARG;
  const int unit = in_dtype == YALM_F32 ? 8 : 8;            // 8 values a load: 32 bytes of float32, 16 of bfloat16
  const size_t bytes = in_dtype == YALM_F32 ? 4 : 2;
  if ((K % 8) || (in_row % unit) || (in_head % unit) || (in_off % unit) || (((uintptr_t)in) % (unit * bytes > 16 ? 16 : unit * bytes)) ||
      (((uintptr_t)wn) & 15))
    return YALM_ERR_ARG;
  dim3 grid(ceil_div(T, HG_TM), H, ceil_div(N, HG_TN));
  const size_t lds = (size_t)(HG_TM + HG_TN) * HG_ROW * sizeof(bf16);
#define HG(TI, TO) \
  head_mfma_kernel<TI, TO><<<grid, HG_THREADS, lds, stream>>>((const TI*)in, in_row, in_head, in_off, (const bf16*)wn, (TO*)out, \
                                                              out_row, out_head, out_off, scale, gate, gate_row, T, K, N)
  if (in_dtype == YALM_F32 && out_dtype == YALM_F32) HG(float, float);
  else if (in_dtype == YALM_BF16 && out_dtype == YALM_BF16) HG(bf16, bf16);
  else if (in_dtype == YALM_F32 && out_dtype == YALM_BF16) HG(float, bf16);
  else if (in_dtype == YALM_BF16 && out_dtype == YALM_F32) HG(bf16, float);
  else return YALM_ERR_DTYPE;
#undef HG
  return launch_status();
}

extern "C" int yalm_latent_pack(const float* proj, long proj_row, int q_head, int q_rot_off, int kv_off,
                                const void* norm_w, int norm_dtype, float eps, float q_scale, float* out, int T, int H,
                                int rot, int rank, int Dk, int has_kv, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (H <= 0 || rot < 0 || rank <= 0 || Dk < rot + rank || q_rot_off < 0 || q_rot_off + rot > q_head ||
      (long)H * q_head > proj_row || (has_kv && (norm_w == nullptr || kv_off < 0 || (long)kv_off + rank + rot > proj_row)))
    return YALM_ERR_ARG;
  dim3 grid(T, H + 1);
  if (norm_dtype == YALM_BF16)
    latent_pack_kernel<bf16><<<grid, WAVE, 0, stream>>>(proj, proj_row, q_head, q_rot_off, kv_off, (const bf16*)norm_w, eps,
                                                        q_scale, out, H, rot, rank, Dk, has_kv);
  else if (norm_dtype == YALM_F32)
    latent_pack_kernel<float><<<grid, WAVE, 0, stream>>>(proj, proj_row, q_head, q_rot_off, kv_off, (const float*)norm_w,
                                                         eps, q_scale, out, H, rot, rank, Dk, has_kv);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}
