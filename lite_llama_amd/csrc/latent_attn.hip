// Attention over a shared low-rank LATENT: what a token leaves in the cache is one normed latent row c [rank] plus one rotated
// key part k_r [rot] that all heads share.  The attention itself runs in the absorbed form on the ragged attention kernels
// (ragged_attn*.hip) as ONE key/value head of key width rank + rot and value width rank whose values are the first `rank`
// columns of the keys: per head the query becomes [W_uk^T q_unrotated | rotate(q_rotated)], and the head's output is
// W_uv (sum of weights times c).  This file holds the per-token work around the projections:
//
//   ll_latent_kv_prep   rows [.. | latent (rank) | k_r (rot) | ..] of the fused input projection -> the cache row
//                       [RMS-normed latent * weight | k_r rotated at the token's position]; optionally also the RMS norm of
//                       a query latent (another slice of the same rows)
//   ll_rotate_pairs     the rotated part of every query head, written behind the absorbed part of the query row
//
// Rotation: entry 2i pairs with entry 2i + 1 (interleaved layout), angle = position * freq[i] with a frequency table that the
// host prepares (frequency scaling is folded into it), cos and sin times an amplitude; entries past 2 * pairs pass unchanged.
// Positions, angles, cos / sin and the norms are fp32 in every storage dtype.
#include "common.h"

namespace {

template <int DT>
__device__ __forceinline__ float ldv(const void* p, int64_t i) {
  if constexpr (DT == LL_F32) return ((const float*)p)[i];
  else return to_f32<DT>(((const uint16_t*)p)[i]);
}
template <int DT>
__device__ __forceinline__ void stv(void* p, int64_t i, float v) {
  if constexpr (DT == LL_F32) ((float*)p)[i] = v;
  else ((uint16_t*)p)[i] = from_f32<DT>(v);
}

// One wave per (token, item): item 0 = latent norm -> cache, 1 = rotated key part -> cache, 2 = query latent norm.
template <int DT>
__global__ __launch_bounds__(256) void latent_kv_prep_kernel(
    const void* __restrict__ rows, int64_t ld, int64_t kv_off, int rank, int rot, const void* __restrict__ kv_norm_w, float eps,
    const float* __restrict__ freq, int pairs, float amp, const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ select,
    void* __restrict__ cache, int64_t cache_stride, int64_t q_off, int q_rank, const void* __restrict__ q_norm_w,
    void* __restrict__ q_out, int64_t n, int items) {
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= n * items) return;   // (wave-uniform)
  const int lane = threadIdx.x & 63;
  const int64_t t = w / items;
  const int item = (int)(w - t * items);
  if (item == 1) {
    const int64_t src = t * ld + kv_off + rank;
    const int64_t dst = (int64_t)select[t] * cache_stride + rank;
    const float pos = (float)tok_pos[t];
    for (int i = lane; i < pairs; i += 64) {
      const float a = pos * freq[i];
      const float cs = cosf(a) * amp, sn = sinf(a) * amp;
      const float u = ldv<DT>(rows, src + 2 * i), v = ldv<DT>(rows, src + 2 * i + 1);
      stv<DT>(cache, dst + 2 * i, u * cs - v * sn);
      stv<DT>(cache, dst + 2 * i + 1, v * cs + u * sn);
    }
    for (int i = 2 * pairs + lane; i < rot; i += 64) stv<DT>(cache, dst + i, ldv<DT>(rows, src + i));
    return;
  }
  const bool is_q = item == 2;
  const int width = is_q ? q_rank : rank;
  const int64_t src = t * ld + (is_q ? q_off : kv_off);
  float ss = 0.f;
  for (int i = lane; i < width; i += 64) {
    const float x = ldv<DT>(rows, src + i);
    ss += x * x;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  const void* wt = is_q ? q_norm_w : kv_norm_w;
  void* out = is_q ? q_out : cache;
  const int64_t dst = is_q ? t * (int64_t)q_rank : (int64_t)select[t] * cache_stride;
  for (int i = lane; i < width; i += 64) stv<DT>(out, dst + i, ldv<DT>(rows, src + i) * inv * ldv<DT>(wt, i));
}

// thread per (token, head, entry of the rotated part): q [n, heads, head_ld-strided] -> out[(t * heads + h) * out_ld + out_off + j]
// (out may be q: a pair is read and written by the same thread)
template <int DT>
__global__ __launch_bounds__(256) void rotate_pairs_kernel(const void* q, int64_t q_tok_stride, int64_t q_head_stride,
                                                           int64_t q_off, int rot, const float* __restrict__ freq, int pairs,
                                                           float amp, const int32_t* __restrict__ tok_pos, void* out,
                                                           int64_t out_head_stride, int64_t out_off, int64_t n, int heads) {
  const int half = (rot + 1) / 2;   // one thread per pair (or per single trailing entry)
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n * heads * half) return;
  const int i = (int)(idx % half);
  const int64_t th = idx / half;
  const int64_t t = th / heads;
  const int h = (int)(th - t * heads);
  const int64_t src = t * q_tok_stride + h * q_head_stride + q_off;
  const int64_t dst = th * out_head_stride + out_off;
  if (i < pairs) {
    const float a = (float)tok_pos[t] * freq[i];
    const float cs = cosf(a) * amp, sn = sinf(a) * amp;
    const float u = ldv<DT>(q, src + 2 * i), v = ldv<DT>(q, src + 2 * i + 1);
    stv<DT>(out, dst + 2 * i, u * cs - v * sn);
    stv<DT>(out, dst + 2 * i + 1, v * cs + u * sn);
  } else {
    if (2 * i < rot) stv<DT>(out, dst + 2 * i, ldv<DT>(q, src + 2 * i));
    if (2 * i + 1 < rot) stv<DT>(out, dst + 2 * i + 1, ldv<DT>(q, src + 2 * i + 1));
  }
}

}  // namespace

#define LL_BY_DTYPE(dtype, CALL)             \
  do {                                       \
    if (dtype == LL_F16) { CALL(LL_F16); }   \
    else if (dtype == LL_BF16) { CALL(LL_BF16); } \
    else { CALL(LL_F32); }                   \
  } while (0)

extern "C" int ll_latent_kv_prep(const void* rows, int64_t ld, int64_t kv_off, int64_t rank, int64_t rot, const void* kv_norm_w,
                                 float eps, const float* freq, int64_t pairs, float amp, const int32_t* tok_pos,
                                 const int32_t* select, void* cache, int64_t cache_stride, int64_t q_off, int64_t q_rank,
                                 const void* q_norm_w, void* q_out, int64_t n, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || rank < 1 || rot < 0 || pairs < 0 || 2 * pairs > rot || kv_off < 0 || ld < kv_off + rank + rot ||
      cache_stride < rank + rot || q_rank < 0 || (q_rank > 0 && (q_off < 0 || ld < q_off + q_rank)))
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!rows || !kv_norm_w || !tok_pos || !select || !cache || (pairs > 0 && !freq) || (q_rank > 0 && (!q_norm_w || !q_out)))
    return LL_ERR_ARG;
  const int items = q_rank > 0 ? 3 : 2;
  const dim3 grid((unsigned)((n * items + 3) / 4));
  hipStream_t st = (hipStream_t)stream;
#define CALL(DT)                                                                                                               \
  latent_kv_prep_kernel<DT><<<grid, 256, 0, st>>>(rows, ld, kv_off, (int)rank, (int)rot, kv_norm_w, eps, freq, (int)pairs, amp, \
                                                  tok_pos, select, cache, cache_stride, q_off, (int)q_rank, q_norm_w, q_out, n, \
                                                  items)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int ll_rotate_pairs(const void* q, int64_t q_tok_stride, int64_t q_head_stride, int64_t q_off, int64_t rot,
                               const float* freq, int64_t pairs, float amp, const int32_t* tok_pos, void* out,
                               int64_t out_head_stride, int64_t out_off, int64_t n, int64_t heads, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || heads < 1 || rot < 0 || pairs < 0 || 2 * pairs > rot || q_off < 0 || out_off < 0 || out_head_stride < out_off + rot)
    return LL_ERR_SHAPE;
  if (n == 0 || rot == 0) return LL_OK;
  if (!q || !out || !tok_pos || (pairs > 0 && !freq)) return LL_ERR_ARG;
  const int64_t threads = n * heads * ((rot + 1) / 2);
  const dim3 grid((unsigned)((threads + 255) / 256));
  hipStream_t st = (hipStream_t)stream;
#define CALL(DT)                                                                                                              \
  rotate_pairs_kernel<DT><<<grid, 256, 0, st>>>(q, q_tok_stride, q_head_stride, q_off, (int)rot, freq, (int)pairs, amp, tok_pos, \
                                                out, out_head_stride, out_off, n, (int)heads)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}
