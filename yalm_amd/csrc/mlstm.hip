// The matrix-memory recurrence (mLSTM) of a head: a state S [d, dv], a vector n [d] and a running maximum m per
// sequence and head, all float32, kept from one step of the sequence to the next.
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
#include <type_traits>
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
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (slot < 0 || slot >= n_slots) {              // a padding row: zeros, and the whole workgroup leaves
    for (int t = t0; t < t1; ++t)
      for (int c = tid; c < dv; c += ML_THREADS) out[(size_t)t * H * dv + h * dv + c] = from_f32<T>(0.f);
    return;
  }
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

// ---------------------------------------------------------------------------------------------------------------
// The same recurrence a chunk of L tokens at a time, on the matrix cores in float32 (v_mfma_f32_16x16x4_f32: products
// and sums of 32-bit floats).  With b_t the sum of the log forget gates from the chunk's start to t, w_s = i_s - b_s,
// g_t = max(m0, max_{s<=t} w_s) and m0 the running maximum before the chunk, the running maximum at t is b_t + g_t and
//   S_t^T q_t = exp(m0 - g_t) S0^T q_t + sum_{s<=t} exp(w_s - g_t) (k_s . q_t) v_s          (n_t . q_t likewise),
// every exponent at most 0; the state behind the chunk is exp(m0 - g_L) S0 + sum_s exp(w_s - g_L) k_s v_s^T.
// A workgroup owns 64 columns of one (sequence, head): the columns of S do not depend on each other, so a head's
// dv / 64 workgroups run side by side (each forms the scores q . k again).  It leaves num / den of every token in
// `raw` (float32 [T, H dv]); the norm over a head's dv values, which spans workgroups, is mlstm_finish_kernel's, and
// so is putting n and m back (they go through `nm`, [B, H, d + 1], because a head's other workgroups may still have to
// read the old ones).
typedef __attribute__((ext_vector_type(4))) float f32x4;
constexpr int DVS = 64;                           // columns of S a workgroup owns
constexpr int VROW = DVS + 16;                    // LDS row strides (floats)
constexpr float NEVER = -3.0e38f;

// A barrier that waits for the wave's LDS traffic only.  __syncthreads() carries a fence that also waits for every global
// load in flight, and the next chunk's operands are meant to stay in flight across the barriers of this chunk's work.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x3F | (0x7 << 4) | (0x0 << 8) | (0x3 << 14));      // lgkmcnt(0), nothing else
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int L>
__host__ __device__ constexpr size_t chunk_lds_floats(int d16) {
  return (size_t)d16 * VROW + 2 * (size_t)L * (d16 + 4) + (size_t)L * VROW + (size_t)L * (L + 4) + d16 + 8 * L;
}

template <int L>
__global__ __launch_bounds__(ML_THREADS) void mlstm_chunk_kernel(
    const float* __restrict__ proj, const float* __restrict__ b_i, const float* __restrict__ b_f,
    float* __restrict__ state, float* __restrict__ nm, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_slot, float* __restrict__ raw, int H, int d, int dv, float q_scale, float cap,
    float floor_, int n_slots) {
  extern __shared__ float lds[];
  const int d16 = (d + 15) / 16 * 16, QROW = d16 + 4, PROW = L + 4;
  float* Ss = lds;                                // [d16][VROW]
  float* Qs = Ss + (size_t)d16 * VROW;            // [L][QROW]
  float* Ks = Qs + (size_t)L * QROW;              // [L][QROW]
  float* Vs = Ks + (size_t)L * QROW;              // [L][VROW]
  float* Ps = Vs + (size_t)L * VROW;              // [L][PROW]
  float* nv = Ps + (size_t)L * PROW;              // [d16]
  float* wv = nv + d16;                           // [L] w_s
  float* gv = wv + L;                             // [L] g_t
  float* ev = gv + L;                             // [L] exp(m0 - g_t)
  float* mv = ev + L;                             // [L] the running maximum at t
  float* cv = mv + L;                             // [L] exp(w_s - g_L)
  float* rs = cv + L;                             // [L] sum_s P[t][s]
  float* qn = rs + L;                             // [L] q_t . n0
  float* bv = qn + L;                             // [L] b_t
  const int slice = blockIdx.x, h = blockIdx.y, b = blockIdx.z, tid = threadIdx.x;
  const int wave = tid / WAVE, lane = tid % WAVE, lr = lane % 16, lq = lane / 16;
  const int slot = seq_slot[b];
  if (slot < 0 || slot >= n_slots) return;        // a padding row (mlstm_finish_kernel writes its zeros)
  const int t_begin = cu_seqlens[b], t_end = cu_seqlens[b + 1];
  if (t_end <= t_begin) return;
  const int per = d * dv + d + 1;
  float* st = state + ((size_t)slot * H + h) * per;
  const int col0 = slice * DVS;
  // a wave takes rows wave, wave + 4, ... of the 64 columns, eight rows' loads in flight at a time
  for (int kb = wave; kb < d16; kb += 32) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = kb + 4 * j;
      v[j] = k < d && col0 + lane < dv ? st[(size_t)k * dv + col0 + lane] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (kb + 4 * j < d16) Ss[(kb + 4 * j) * VROW + lane] = v[j];
  }
  for (int k = tid; k < d16; k += ML_THREADS) nv[k] = k < d ? st[(size_t)d * dv + k] : 0.f;
  float m0 = st[(size_t)d * dv + d];
  const int N = 2 * H * d + 2 * H * dv + 2 * H;
  constexpr int RT = L / 16;                      // row tiles of a chunk

  // A chunk's queries, keys, values and gate inputs are asked for a chunk ahead and wait in registers while the
  // chunk before is worked (a workgroup has its compute unit alone: nobody else would hide the loads' latency).
  // Thread (wave, lane) holds tokens wave, wave + 4, ... and elements lane, lane + 64, ...
  constexpr int TJ = L / 4, KJ = L == 64 ? 2 : 5; // d16 <= 64 KJ where the LDS fits
  float qreg[TJ][KJ], kreg[TJ][KJ], vreg[TJ], zreg[2] = {0.f, 0.f};
  auto fetch = [&](int t0) {
    const int n_valid = min(L, t_end - t0);
#pragma unroll
    for (int jt = 0; jt < TJ; ++jt) {
      const int t = wave + 4 * jt;
      vreg[jt] = t < n_valid && col0 + lane < dv ? proj[(size_t)(t0 + t) * N + 2 * H * d + h * dv + col0 + lane] : 0.f;
#pragma unroll
      for (int jk = 0; jk < KJ; ++jk) {
        const int k = lane + WAVE * jk;
        const bool ok = t < n_valid && k < d;
        const float* row = proj + (size_t)(t0 + (ok ? t : 0)) * N + h * d + (ok ? k : 0);
        qreg[jt][jk] = ok ? row[0] : 0.f;
        kreg[jt][jk] = ok ? row[H * d] : 0.f;
      }
    }
    if (wave == 0 && lane < n_valid) {
      const float* row = proj + (size_t)(t0 + lane) * N + 2 * H * d + 2 * H * dv;
      zreg[0] = row[h];
      zreg[1] = row[H + h];
    }
  };
  fetch(t_begin);
  const float bias_i = b_i[h], bias_f = b_f[h];

  for (int t0 = t_begin; t0 < t_end; t0 += L) {
    const int n_valid = min(L, t_end - t0);
    __syncthreads();                              // the chunk before is done with Qs, Ks, Vs, Ps and the vectors
#pragma unroll
    for (int jt = 0; jt < TJ; ++jt) {
      const int t = wave + 4 * jt;
      Vs[t * VROW + lane] = vreg[jt];
#pragma unroll
      for (int jk = 0; jk < KJ; ++jk) {
        const int k = lane + WAVE * jk;
        if (k < d16) {
          Qs[t * QROW + k] = qreg[jt][jk] * q_scale;
          Ks[t * QROW + k] = kreg[jt][jk];
        }
      }
    }
    if (wave == 0) {                              // the gates of the chunk: sums and maxima along it, a lane a token
      float f = 0.f, zi = NEVER;
      if (lane < n_valid) {
        zi = zreg[0] + bias_i;
        float zf = zreg[1] + bias_f;
        if (cap > 0.f) {
          zi = cap * tanhf(zi / cap);
          zf = cap * tanhf(zf / cap);
        }
        f = log_sigmoid(zf);
      }
      float bsum = f;
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const float up = __shfl_up(bsum, o, WAVE);
        if (lane >= o) bsum += up;
      }
      const float w = lane < n_valid ? zi - bsum : NEVER;
      float a = w;
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const float up = __shfl_up(a, o, WAVE);
        if (lane >= o) a = fmaxf(a, up);
      }
      const float g = fmaxf(m0, a);
      const float gl = __shfl(g, n_valid - 1, WAVE);
      if (lane < L) {
        wv[lane] = w;
        gv[lane] = g;
        ev[lane] = expf(m0 - g);
        mv[lane] = bsum + g;
        bv[lane] = bsum;
        cv[lane] = lane < n_valid ? expf(w - gl) : 0.f;
      }
    }
    __syncthreads();
    if (t0 + L < t_end) fetch(t0 + L);             // the next chunk's loads fly while this one is worked
    if (tid < 4 * L) {                             // q_t . n0: four threads a token, a quarter of the elements each
      const int t = tid / 4, part = tid % 4;
      float a = 0.f;
      for (int k = part; k < d16; k += 4) a = fmaf(Qs[t * QROW + k], nv[k], a);
      a += __shfl_xor(a, 1, WAVE);
      a += __shfl_xor(a, 2, WAVE);
      if (part == 0) qn[t] = a;
    }
    // scores: P[t][s] = (q_t . k_s) exp(w_s - g_t) for s <= t; a wave a tile of 16 tokens
    if (wave < RT) {
      // the key tiles up to the diagonal side by side: independent sums keep the matrix cores busy, and a query
      // element is read once for all of them
      f32x4 acc[RT];
#pragma unroll
      for (int c = 0; c < RT; ++c) acc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const float* qa = Qs + (wave * 16 + lr) * QROW + lq;
      const float* kb = Ks + lr * QROW + lq;
      // the number of key tiles is the wave's own: a loop of its own for each number, so that none carries a branch
      // (a branch around every product keeps the loads of the next from being asked for under it)
      auto products = [&](auto nc) {
#pragma unroll 4
        for (int k0 = 0; k0 < d16; k0 += 4) {
          const float a = qa[k0];
#pragma unroll
          for (int c = 0; c < decltype(nc)::value; ++c)
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, kb[c * 16 * QROW + k0], acc[c], 0, 0, 0);
        }
      };
      if constexpr (RT == 4) {
        if (wave == 0) products(std::integral_constant<int, 1>{});
        else if (wave == 1) products(std::integral_constant<int, 2>{});
        else if (wave == 2) products(std::integral_constant<int, 3>{});
        else products(std::integral_constant<int, 4>{});
      } else {
        products(std::integral_constant<int, 1>{});
      }
      float sum[4] = {0.f, 0.f, 0.f, 0.f};        // of the rows lq * 4 + v over this lane's columns
#pragma unroll
      for (int c = 0; c < RT; ++c) {
        const int s_ = c * 16 + lr;
        const float ws = wv[s_];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int t = wave * 16 + lq * 4 + v;
          const float pv = s_ <= t ? acc[c][v] * expf(ws - gv[t]) : 0.f;
          Ps[t * PROW + s_] = pv;
          sum[v] += pv;
        }
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) sum[v] += __shfl_xor(sum[v], o, WAVE);
        if (lr == 0) rs[wave * 16 + lq * 4 + v] = sum[v];
      }
    }
    lds_barrier();
    // the tokens' results: P V + exp(m0 - g_t) Q S0, over the denominator
    if (wave < RT) {
      constexpr int CT = DVS / 16;                // the four column tiles side by side
      f32x4 acc[CT], acc2[CT];
#pragma unroll
      for (int c = 0; c < CT; ++c) acc[c] = acc2[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const float* pa = Ps + (wave * 16 + lr) * PROW + lq;
      const float* vb = Vs + lq * VROW + lr;
#pragma unroll 4
      for (int s0 = 0; s0 < (wave + 1) * 16; s0 += 4) {
        const float a = pa[s0];
#pragma unroll
        for (int c = 0; c < CT; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, vb[s0 * VROW + c * 16], acc[c], 0, 0, 0);
      }
      const float* qa = Qs + (wave * 16 + lr) * QROW + lq;
      const float* sb = Ss + lq * VROW + lr;
#pragma unroll 4
      for (int k0 = 0; k0 < d16; k0 += 4) {
        const float a = qa[k0];
#pragma unroll
        for (int c = 0; c < CT; ++c) acc2[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, sb[k0 * VROW + c * 16], acc2[c], 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int t = wave * 16 + lq * 4 + v;
        if (t < n_valid) {
          const float e = ev[t];
          const float inv = 1.0f / (fmaxf(fabsf(fmaf(e, qn[t], rs[t])), expf(-mv[t])) + floor_);
#pragma unroll
          for (int c = 0; c < CT; ++c) {
            const int col = col0 + c * 16 + lr;
            if (col < dv) raw[(size_t)(t0 + t) * H * dv + h * dv + col] = fmaf(e, acc2[c][v], acc[c][v]) * inv;
          }
        }
      }
    }
    lds_barrier();
    // the state behind the chunk: exp(m0 - g_L) S0 + (c K)^T V; wave w owns the column tile w of every row tile
    const float decay = ev[n_valid - 1];
    for (int r0 = 0; r0 < d16 / 16; r0 += 4) {    // four row tiles side by side: a value element is read once for them
      const int nr = min(4, d16 / 16 - r0);
      float* sp = Ss + (r0 * 16 + lq * 4) * VROW + wave * 16 + lr;
      f32x4 acc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float* p = sp + (j < nr ? j : 0) * 16 * VROW;
        acc[j] = (f32x4){p[0] * decay, p[VROW] * decay, p[2 * VROW] * decay, p[3 * VROW] * decay};
      }
      const float* ka = Ks + lq * QROW + r0 * 16 + lr;
      const float* vb = Vs + lq * VROW + wave * 16 + lr;
      if (nr == 4) {                              // the loop without a branch (see the scores' products)
#pragma unroll 4
        for (int s0 = 0; s0 < L; s0 += 4) {
          const float bvv = vb[s0 * VROW], cs = cv[s0 + lq];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[s0 * QROW + j * 16] * cs, bvv, acc[j], 0, 0, 0);
        }
      } else {
        for (int s0 = 0; s0 < L; s0 += 4) {
          const float bvv = vb[s0 * VROW], cs = cv[s0 + lq];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (j < nr) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[s0 * QROW + j * 16] * cs, bvv, acc[j], 0, 0, 0);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (j < nr) {
          float* p = sp + j * 16 * VROW;
          p[0] = acc[j][0];
          p[VROW] = acc[j][1];
          p[2 * VROW] = acc[j][2];
          p[3 * VROW] = acc[j][3];
        }
    }
    for (int k = tid; k < d16; k += ML_THREADS) {
      float a = nv[k] * decay;
#pragma unroll 8
      for (int s_ = 0; s_ < L; ++s_) a = fmaf(cv[s_], Ks[s_ * QROW + k], a);      // tokens behind the end weigh 0
      nv[k] = a;
    }
    m0 = mv[n_valid - 1];
  }
  __syncthreads();
  if (col0 + lane < dv)
    for (int k = wave; k < d; k += ML_WAVES) st[(size_t)k * dv + col0 + lane] = Ss[k * VROW + lane];
  if (slice == 0) {
    float* o = nm + ((size_t)b * H + h) * (d + 1);
    for (int k = tid; k < d; k += ML_THREADS) o[k] = nv[k];
    if (tid == 0) o[d] = m0;
  }
}

// out[t, head] = raw / rms(raw) * w * sigmoid(g) (a wave a token and head); the workgroup of a sequence's last token
// puts the head's n and m into the state; a padding row gets zeros.
template <typename T>
__global__ __launch_bounds__(WAVE) void mlstm_finish_kernel(const float* __restrict__ raw, const float* __restrict__ proj,
                                                            const float* __restrict__ w_norm, const float* __restrict__ nm,
                                                            float* __restrict__ state, const int* __restrict__ cu_seqlens,
                                                            const int* __restrict__ seq_slot, T* __restrict__ out, int B,
                                                            int H, int d, int dv, float eps, int n_slots) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  int lo = 0, hi = B - 1;                         // the sequence of token t
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_seqlens[mid] <= t) lo = mid; else hi = mid - 1;
  }
  const int b = lo, slot = seq_slot[b];
  T* o = out + (size_t)t * H * dv + h * dv;
  if (slot < 0 || slot >= n_slots) {
    for (int c = lane; c < dv; c += WAVE) o[c] = from_f32<T>(0.f);
    return;
  }
  const float* r = raw + (size_t)t * H * dv + h * dv;
  float sq = 0.f;
  for (int c = lane; c < dv; c += WAVE) sq = fmaf(r[c], r[c], sq);
  sq = wave_sum(sq);
  const float rsq = 1.0f / sqrtf(sq / (float)dv + eps);
  const float* g = proj + (size_t)t * (2 * H * d + 2 * H * dv + 2 * H) + 2 * H * d + H * dv + h * dv;
  for (int c = lane; c < dv; c += WAVE) o[c] = from_f32<T>(r[c] * rsq * w_norm[h * dv + c] / (1.0f + expf(-g[c])));
  if (t == cu_seqlens[b + 1] - 1) {
    const float* src = nm + ((size_t)b * H + h) * (d + 1);
    float* dst = state + ((size_t)slot * H + h) * ((size_t)d * dv + d + 1) + (size_t)d * dv;
    for (int k = lane; k <= d; k += WAVE) dst[k] = src[k];
  }
}

LdsAllowance ml_allow_chunk64, ml_allow_chunk16;
}  // namespace

// The recurrence a chunk at a time (see mlstm_chunk_kernel).  chunk: 64 (steps of whole prompts) or 16 (single tokens).
// raw: float32 [T, H dv] and nm: float32 [B, H (d + 1)], scratch of the caller.  Returns YALM_ERR_ARG where the sizes
// do not fit its LDS (yalm_mlstm_scan then serves).  T: the step's tokens, the last sequence's last token being T - 1.
extern "C" int yalm_mlstm_chunks(const float* proj, const float* b_i, const float* b_f, const float* w_norm, float* state,
                                 float* raw, float* nm, const int* cu_seqlens, const int* seq_slot, void* out, int T,
                                 int B, int H, int d, int dv, float q_scale, float cap, float floor_, float eps,
                                 int n_slots, int chunk, int dtype, hipStream_t stream) {
  if (B <= 0 || T <= 0) return YALM_OK;
  if (H <= 0 || d <= 0 || dv <= 0 || n_slots <= 0 || cap < 0.f || H > 65535 || B > 65535 ||
      (chunk != 64 && chunk != 16) || (dtype != YALM_F32 && dtype != YALM_BF16))
    return YALM_ERR_ARG;
  const int d16 = (d + 15) / 16 * 16;
  const size_t lds = (chunk == 64 ? chunk_lds_floats<64>(d16) : chunk_lds_floats<16>(d16)) * sizeof(float);
  if (lds > 150 * 1024) return YALM_ERR_ARG;
  dim3 grid(ceil_div(dv, DVS), H, B);
  if (chunk == 64) {
    auto kernel = &mlstm_chunk_kernel<64>;
    if (lds > 64 * 1024)
      if (int rc = allow_dynamic_lds(ml_allow_chunk64, (const void*)kernel, 150 * 1024); rc != YALM_OK) return rc;
    kernel<<<grid, ML_THREADS, lds, stream>>>(proj, b_i, b_f, state, nm, cu_seqlens, seq_slot, raw, H, d, dv, q_scale, cap,
                                              floor_, n_slots);
  } else {
    auto kernel = &mlstm_chunk_kernel<16>;
    if (lds > 64 * 1024)
      if (int rc = allow_dynamic_lds(ml_allow_chunk16, (const void*)kernel, 150 * 1024); rc != YALM_OK) return rc;
    kernel<<<grid, ML_THREADS, lds, stream>>>(proj, b_i, b_f, state, nm, cu_seqlens, seq_slot, raw, H, d, dv, q_scale, cap,
                                              floor_, n_slots);
  }
  if (int rc = launch_status(); rc != YALM_OK) return rc;
  if (dtype == YALM_F32)
    mlstm_finish_kernel<float><<<dim3(T, H), WAVE, 0, stream>>>(raw, proj, w_norm, nm, state, cu_seqlens, seq_slot, (float*)out,
                                                                B, H, d, dv, eps, n_slots);
  else
    mlstm_finish_kernel<bf16><<<dim3(T, H), WAVE, 0, stream>>>(raw, proj, w_norm, nm, state, cu_seqlens, seq_slot, (bf16*)out, B,
                                                               H, d, dv, eps, n_slots);
  return launch_status();
}

// the LDS bytes yalm_mlstm_chunks needs for key heads of d with chunks of `chunk` tokens
extern "C" long yalm_mlstm_chunks_lds(int d, int chunk) {
  const int d16 = (d + 15) / 16 * 16;
  return (long)((chunk == 64 ? chunk_lds_floats<64>(d16) : chunk_lds_floats<16>(d16)) * sizeof(float));
}

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
