// The matrix-memory recurrence (mLSTM) of a head: a state S [d, dv], a vector n [d] and a running maximum m per
// sequence and head, all float32, carried from token to token.
//
//   i = cap tanh((z_i + b_i) / cap),  f = logsigmoid(cap tanh((z_f + b_f) / cap))          (cap 0: uncapped)
//   m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k alone
//   o = S'^T q / (max(|n' . q|, exp(-m')) + floor)
//   out = o / rms(o) * w * sigmoid(g)                                                       (rms over the head's dv values)
//
// proj holds a token's projections side by side: q [H, d] | k [H, d] | v [H, dv] | g [H, dv] | z_i [H] | z_f [H];
// q is multiplied by q_scale here.  A workgroup owns one (sequence, head): it takes the state into LDS, walks the
// sequence's tokens of the step in order (one in a decode step) and puts the state back.  Threads stand as
// [row groups][columns]: a thread owns the rows k = group, group + groups, ... of one column of S, so that S needs no
// synchronisation of its own, and a column's sum over the groups is made through LDS.
#include "common.h"
#include "yalm_hip.h"

namespace {
constexpr int ML_THREADS = 256;
constexpr int ML_WAVES = ML_THREADS / WAVE;

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T>
__global__ __launch_bounds__(ML_THREADS) void mlstm_scan_kernel(
    const float* __restrict__ proj, const float* __restrict__ b_i, const float* __restrict__ b_f,
    const float* __restrict__ w_norm, float* __restrict__ state, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_slot, T* __restrict__ out, int H, int d, int dv, float q_scale, float cap, float floor_,
    float eps, int n_slots, int groups) {
  extern __shared__ float lds[];
  float* S = lds;                                 // [d][dv]
  float* nv = S + (size_t)d * dv;                 // [d]
  float* qs = nv + d;                             // [d]
  float* ks = qs + d;                             // [d]
  float* vs = ks + d;                             // [dv]
  float* part = vs + dv;                          // [groups][dv]
  __shared__ float red[ML_WAVES];
  __shared__ float gate[3];                       // keep, take, m
  const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int slot = seq_slot[b];
  if (slot < 0 || slot >= n_slots) return;        // a padding row: the whole workgroup leaves
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (t1 <= t0) return;
  const int per = d * dv + d + 1;
  float* st = state + ((size_t)slot * H + h) * per;
  for (int i = tid; i < d * dv + d; i += ML_THREADS) S[i] = st[i];      // S and n lie side by side
  float m = st[d * dv + d];
  const int N = 2 * H * d + 2 * H * dv + 2 * H;
  const int col = tid % dv, grp = tid / dv;       // threads beyond groups * dv only help with the loads and sums
  const bool owner = grp < groups;
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    const float* row = proj + (size_t)t * N;
    for (int i = tid; i < d; i += ML_THREADS) {
      qs[i] = row[h * d + i] * q_scale;
      ks[i] = row[H * d + h * d + i];
    }
    for (int i = tid; i < dv; i += ML_THREADS) vs[i] = row[2 * H * d + h * dv + i];
    if (tid == 0) {
      float zi = row[2 * H * d + 2 * H * dv + h] + b_i[h], zf = row[2 * H * d + 2 * H * dv + H + h] + b_f[h];
      if (cap > 0.f) {
        zi = cap * tanhf(zi / cap);
        zf = cap * tanhf(zf / cap);
      }
      const float f = log_sigmoid(zf);
      const float m_new = fmaxf(f + m, zi);
      gate[0] = expf(f + m - m_new);
      gate[1] = expf(zi - m_new);
      gate[2] = m_new;
    }
    __syncthreads();
    const float keep = gate[0], take = gate[1];
    m = gate[2];
    float nq = 0.f;
    for (int k = tid; k < d; k += ML_THREADS) {
      const float v = fmaf(keep, nv[k], take * ks[k]);
      nv[k] = v;
      nq = fmaf(v, qs[k], nq);
    }
    if (owner) {
      const float tv = take * vs[col];
      float acc = 0.f;
      for (int k = grp; k < d; k += groups) {
        const float s = fmaf(keep, S[(size_t)k * dv + col], ks[k] * tv);
        S[(size_t)k * dv + col] = s;
        acc = fmaf(s, qs[k], acc);
      }
      part[grp * dv + col] = acc;
    }
    nq = block_sum<ML_WAVES>(nq, red);            // its barriers also stand between part's writers and readers
    const float den = fmaxf(fabsf(nq), expf(-m)) + floor_;
    float o = 0.f, sq = 0.f;
    // a head's values may be more than the threads: a thread then takes several columns in turn
    for (int c = tid; c < dv; c += ML_THREADS) {
      float a = 0.f;
      for (int g2 = 0; g2 < groups; ++g2) a += part[g2 * dv + c];
      a /= den;
      sq = fmaf(a, a, sq);
      vs[c] = a;                                   // its value of this token is used up
    }
    sq = block_sum<ML_WAVES>(sq, red);
    const float rs = 1.0f / sqrtf(sq / (float)dv + eps);
    for (int c = tid; c < dv; c += ML_THREADS) {
      o = vs[c] * rs * w_norm[h * dv + c];
      const float g = row[2 * H * d + H * dv + h * dv + c];
      out[(size_t)t * H * dv + h * dv + c] = from_f32<T>(o / (1.0f + expf(-g)));
    }
    __syncthreads();                               // the next token's loads overwrite qs, ks, vs
  }
  for (int i = tid; i < d * dv + d; i += ML_THREADS) st[i] = S[i];
  if (tid == 0) st[d * dv + d] = m;
}

LdsAllowance ml_allow_f32, ml_allow_bf16;
}  // namespace

// proj float32 [T, 2 H d + 2 H dv + 2 H]; state float32 [n_slots, H, d dv + d + 1]; out `dtype` [T, H dv];
// cu_seqlens int32 [B + 1] (the tokens of sequence b are rows cu_seqlens[b] .. cu_seqlens[b + 1] - 1, in order),
// seq_slot int32 [B] (negative: a padding row, left alone).
extern "C" int yalm_mlstm_scan(const float* proj, const float* b_i, const float* b_f, const float* w_norm, float* state,
                               const int* cu_seqlens, const int* seq_slot, void* out, int B, int H, int d, int dv,
                               float q_scale, float cap, float floor_, float eps, int n_slots, int dtype,
                               hipStream_t stream) {
  if (B <= 0) return YALM_OK;
  if (H <= 0 || d <= 0 || dv <= 0 || n_slots <= 0 || cap < 0.f || H > 65535 || B > 65535) return YALM_ERR_ARG;
  const int fit = dv >= ML_THREADS ? 1 : ML_THREADS / dv;
  const int groups = fit < d ? fit : d;
  const size_t lds = ((size_t)d * dv + 3 * (size_t)d + dv + (size_t)groups * dv) * sizeof(float);
  if (lds > 150 * 1024) return YALM_ERR_ARG;
  if (dv > ML_THREADS) return YALM_ERR_ARG;       // a thread owns one column's rows
  dim3 grid(H, B);
  if (dtype == YALM_F32) {
    auto kernel = &mlstm_scan_kernel<float>;
    if (lds > 64 * 1024)
      if (int rc = allow_dynamic_lds(ml_allow_f32, (const void*)kernel, 150 * 1024); rc != YALM_OK) return rc;
    kernel<<<grid, ML_THREADS, lds, stream>>>(proj, b_i, b_f, w_norm, state, cu_seqlens, seq_slot, (float*)out, H, d, dv,
                                              q_scale, cap, floor_, eps, n_slots, groups);
  } else if (dtype == YALM_BF16) {
    auto kernel = &mlstm_scan_kernel<bf16>;
    if (lds > 64 * 1024)
      if (int rc = allow_dynamic_lds(ml_allow_bf16, (const void*)kernel, 150 * 1024); rc != YALM_OK) return rc;
    kernel<<<grid, ML_THREADS, lds, stream>>>(proj, b_i, b_f, w_norm, state, cu_seqlens, seq_slot, (bf16*)out, H, d, dv,
                                              q_scale, cap, floor_, eps, n_slots, groups);
  } else {
    return YALM_ERR_DTYPE;
  }
  return launch_status();
}
