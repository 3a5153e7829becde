// What stands between the q/k/v product and an attention without rotation: biases, RMS norms over the WHOLE query
// and key projections (all heads at once), a query factor that grows with the position, the blend of the values
// with those an earlier layer made for the same token, and the way into the cache.  A workgroup a token; the row
// waits in LDS between its sums and its results.
//
//   q = (qkv[:Q] + b_q);  q <- q / rms(q) * w_q            (w_q null: no norm)
//   q <- q * (1 + coef ln(floor((p + 1) / every) + 1)) * q_scale      (every 0: no factor)
//   k likewise with w_k (no factor);  v = qkv[Q + K:] + b_v
//   blend 1: v_first <- v;   blend 2: v <- (1 - lam) v + lam v_first      (lam a number on the device)
// Heads are written `pad` elements wide (key size d and value size dv may differ; zeros behind): q_out [T, heads,
// pad], keys into their page and the step's staging tile [row][pad], values transposed [pad][row].
#include "common.h"
#include "yalm_hip.h"

namespace {
// a row of a few hundred numbers takes 256 threads, a real model's thousands 1,024 (a decode step has few tokens, and a
// thread's loads wait for each other's results in turn: the fewer rounds the better)
template <typename T, int PACK_THREADS>
__global__ __launch_bounds__(PACK_THREADS) void qkv_pack_kernel(
    const float* __restrict__ qkv, const float* __restrict__ bias, const float* __restrict__ w_q,
    const float* __restrict__ w_k, float eps, float temp_coef, int temp_every, float q_scale, float* __restrict__ v_first,
    int blend, const float* __restrict__ lam_p, T* __restrict__ q_out, T* __restrict__ k_stage, T* __restrict__ v_stage,
    const int* __restrict__ seq_tile0, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, int ring_pages, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const int* __restrict__ seq_slot, const int* __restrict__ seq_len, int n_heads,
    int n_kv_heads, int d, int dv, int pad, int n_pages, int page_layout) {
  extern __shared__ float row[];                  // [Q + K + V]
  __shared__ float red[PACK_THREADS / WAVE];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int Q = n_heads * d, K = n_kv_heads * d, V = n_kv_heads * dv, N = Q + K + V;
  const float* src = qkv + (size_t)t * N;
  float sq = 0.f, sk = 0.f;
#pragma unroll 4
  for (int i = tid; i < N; i += PACK_THREADS) {
    const float v = src[i] + (bias != nullptr ? bias[i] : 0.f);
    row[i] = v;
    if (i < Q) sq = fmaf(v, v, sq);
    else if (i < Q + K) sk = fmaf(v, v, sk);
  }
  sq = block_sum<PACK_THREADS / WAVE>(sq, red);
  sk = block_sum<PACK_THREADS / WAVE>(sk, red);
  __syncthreads();
  const int pos = tok_pos[t];
  const int b = tok_seq[t];
  const int slot = b >= 0 ? seq_slot[b] : -1;

  // the queries
  float fq = q_scale;
  if (w_q != nullptr) fq *= 1.0f / sqrtf(sq / (float)Q + eps);
  if (temp_every > 0) fq *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  for (int i = tid; i < n_heads * pad; i += PACK_THREADS) {
    const int h = i / pad, e = i - h * pad;
    float v = 0.f;
    if (e < d) v = row[h * d + e] * fq * (w_q != nullptr ? w_q[h * d + e] : 1.0f);
    q_out[(size_t)t * n_heads * pad + i] = from_f32<T>(v);
  }

  // where this token's key and value go: its page in the cache (a ring keeps the last pages only) and the step's tile
  const int r = pos & (PAGE - 1);
  long page = -1, tile = -1;
  if (slot >= 0 && pos >= 0 && k_pages != nullptr) {
    const int ap = pos / PAGE, last_ap = (seq_len[b] - 1) / PAGE;
    if (ap > last_ap - ring_pages) {
      const int phys = block_table[(size_t)slot * table_stride + (ap % ring_pages)];
      if (phys >= 0 && phys < n_pages) page = phys;
    }
  }
  if (k_stage != nullptr && b >= 0 && pos >= 0) tile = (long)seq_tile0[b] + pos / PAGE;

  const float fk = w_k != nullptr ? 1.0f / sqrtf(sk / (float)K + eps) : 1.0f;
  const float lam = blend == 2 ? lam_p[0] : 0.f;
  for (int i = tid; i < n_kv_heads * pad; i += PACK_THREADS) {
    const int g = i / pad, e = i - g * pad;
    float kv = 0.f, vv = 0.f;
    if (e < d) kv = row[Q + g * d + e] * fk * (w_k != nullptr ? w_k[g * d + e] : 1.0f);
    if (e < dv) {
      vv = row[Q + K + g * dv + e];
      float* first = v_first != nullptr ? v_first + (size_t)t * V + g * dv + e : nullptr;
      if (blend == 1) *first = vv;
      else if (blend == 2) vv = (1.0f - lam) * vv + lam * *first;
    }
    const T kt = from_f32<T>(kv), vt = from_f32<T>(vv);
    if (tile >= 0) {
      const size_t base = ((size_t)tile * n_kv_heads + g) * PAGE * pad;
      k_stage[base + (size_t)r * pad + e] = kt;
      v_stage[base + (size_t)e * PAGE + r] = vt;
    }
    if (page >= 0) {
      const size_t base = ((size_t)page * n_kv_heads + g) * PAGE * pad;
      k_pages[base + page_k_offset(page_layout, r, e, pad)] = kt;
      v_pages[base + page_v_offset(page_layout, r, e, pad)] = vt;
    }
  }
}
}  // namespace

extern "C" int yalm_qkv_pack(const float* qkv, const float* bias, const float* w_q, const float* w_k, float eps,
                             float temp_coef, int temp_every, float q_scale, float* v_first, int blend,
                             const float* lam, void* q_out, void* k_stage, void* v_stage, const int* seq_tile0,
                             void* k_pages, void* v_pages, const int* block_table, int table_stride, int ring_pages,
                             const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* seq_len, int T,
                             int n_heads, int n_kv_heads, int d, int dv, int pad, int n_pages, int page_layout,
                             int dtype, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (n_heads <= 0 || n_kv_heads <= 0 || d <= 0 || dv <= 0 || pad < d || pad < dv || temp_every < 0 || blend < 0 ||
      blend > 2 || (blend != 0 && v_first == nullptr) || (blend == 2 && lam == nullptr) ||
      (k_stage != nullptr && (v_stage == nullptr || seq_tile0 == nullptr)) ||
      (k_pages != nullptr && (v_pages == nullptr || block_table == nullptr || ring_pages <= 0 || seq_len == nullptr)) ||
      !page_layout_ok(page_layout, pad))
    return YALM_ERR_ARG;
  const size_t lds = (size_t)(n_heads * d + n_kv_heads * (d + dv)) * sizeof(float);
  if (lds > 64 * 1024) return YALM_ERR_ARG;
  const bool wide = n_heads * d + n_kv_heads * (d + dv) >= 2048;
#define YALM_PACK(TYPE)                                                                                              \
  if (wide) YALM_PACK_N(TYPE, 1024); else YALM_PACK_N(TYPE, 256)
#define YALM_PACK_N(TYPE, NT)                                                                                        \
  qkv_pack_kernel<TYPE, NT><<<T, NT, lds, stream>>>(                                                                 \
      qkv, bias, w_q, w_k, eps, temp_coef, temp_every, q_scale, v_first, blend, lam, (TYPE*)q_out, (TYPE*)k_stage,    \
      (TYPE*)v_stage, seq_tile0, (TYPE*)k_pages, (TYPE*)v_pages, block_table, table_stride, ring_pages, tok_seq,     \
      tok_pos, seq_slot, seq_len, n_heads, n_kv_heads, d, dv, pad, n_pages, page_layout)
  if (dtype == YALM_F32) {
    YALM_PACK(float);
  } else if (dtype == YALM_BF16) {
    YALM_PACK(bf16);
  } else {
    return YALM_ERR_DTYPE;
  }
#undef YALM_PACK
#undef YALM_PACK_N
  return launch_status();
}
