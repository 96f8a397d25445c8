// Mixture of experts with a SIGMOID router over expert groups, for 16-bit and 32-bit storage dtypes (the softmax-router fp16
// path of moe.hip stays as it is):
//
//   ll_group_router   logits = W_router h in fp32, scores = sigmoid(logits); the experts form `group_count` equal groups of
//                     neighbours, a group's score is the sum of its two best scores, only the best `group_keep` groups stay
//                     eligible; the `top` best eligible experts are chosen, their scores divided by their sum (+ 1e-20) and
//                     multiplied by `route_scale`.  One more row of weights may give a per-token sigmoid scale (for a shared
//                     expert).  One wave per token; selection by ranks (ties: the lower index first), so slot k of a token holds
//                     its k-th best expert.
//   ll_moe_sort       slots (token, k) sorted by expert, every expert's run padded to the row-block size with a sentinel:
//                     sorted_ids / block_expert / num_post as in moe_align_block_size.  Deterministic: no atomics.
//   ll_moe_rows_gemm  the grouped products over sorted row blocks: either act = silu(a Wg_e^T) * (a Wu_e^T) (gate and up rows
//                     stacked in one matrix per expert) or out = (a W_e^T) * slot weight, fp32 accumulation.  MFMA form for
//                     16-bit storage with contraction widths that are multiples of 8, a plain tiled form otherwise.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

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

__device__ __forceinline__ float sigmoid_exact(float v) { return 1.0f / (1.0f + expf(-v)); }

// ------------------------------------------------------------------------------------------------------------------------
// router: one 64-thread workgroup per token.  LDS: scores [E], group score [G], group kept [G], chosen scores [top]
// ------------------------------------------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(64) void group_router_kernel(const void* __restrict__ h, int64_t h_ld, const void* __restrict__ w_router,
                                                          const void* __restrict__ w_extra, int width, int experts, int top,
                                                          int group_count, int group_keep, float route_scale,
                                                          int32_t* __restrict__ ids, float* __restrict__ weights,
                                                          float* __restrict__ extra_scale) {
  extern __shared__ float lds[];
  float* score = lds;                       // [experts]
  float* gscore = score + experts;          // [group_count]
  float* gkeep = gscore + group_count;      // [group_count]
  float* chosen = gkeep + group_count;      // [top]
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const int64_t hrow = t * h_ld;
  for (int e = 0; e < experts + (w_extra ? 1 : 0); ++e) {
    const bool extra = e == experts;
    const void* wr = extra ? w_extra : w_router;
    const int64_t wrow = extra ? 0 : (int64_t)e * width;
    float d = 0.f;
    for (int i = lane; i < width; i += 64) d += ldv<DT>(h, hrow + i) * ldv<DT>(wr, wrow + i);
    d = wave_sum(d);
    if (lane == 0) {
      const float s = sigmoid_exact(d);
      if (extra) extra_scale[t] = s;
      else score[e] = s;
    }
  }
  __syncthreads();
  const int per = experts / group_count;
  for (int g = lane; g < group_count; g += 64) {
    float b1 = -INFINITY, b2 = -INFINITY;   // the two largest of the group
    for (int j = 0; j < per; ++j) {
      const float s = score[g * per + j];
      if (s > b1) { b2 = b1; b1 = s; }
      else if (s > b2) b2 = s;
    }
    gscore[g] = per > 1 ? b1 + b2 : b1;
  }
  __syncthreads();
  for (int g = lane; g < group_count; g += 64) {
    const float mine = gscore[g];
    int rank = 0;
    for (int o = 0; o < group_count; ++o) {
      const float s = gscore[o];
      rank += (s > mine || (s == mine && o < g)) ? 1 : 0;
    }
    gkeep[g] = rank < group_keep ? 1.0f : 0.0f;
  }
  __syncthreads();
  for (int e = lane; e < experts; e += 64) {
    if (gkeep[e / per] == 0.0f) continue;
    const float mine = score[e];
    int rank = 0;
    for (int o = 0; o < experts; ++o) {
      const float s = score[o];
      rank += (gkeep[o / per] != 0.0f && (s > mine || (s == mine && o < e))) ? 1 : 0;
    }
    if (rank < top) {
      ids[t * top + rank] = e;
      chosen[rank] = mine;
    }
  }
  __syncthreads();
  float sum = 0.f;
  for (int k = 0; k < top; ++k) sum += chosen[k];
  for (int k = lane; k < top; k += 64) weights[t * top + k] = chosen[k] / (sum + 1e-20f) * route_scale;
}

// ------------------------------------------------------------------------------------------------------------------------
// sort by expert: one workgroup per expert, twice (count, then place)
// ------------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_count_kernel(const int32_t* __restrict__ ids, int num_slots, int32_t* __restrict__ counts) {
  __shared__ int part[4];
  const int e = blockIdx.x, tid = threadIdx.x;
  int c = 0;
  for (int i = tid; i < num_slots; i += 256) c += ids[i] == e ? 1 : 0;
  for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
  if ((tid & 63) == 0) part[tid >> 6] = c;
  __syncthreads();
  if (tid == 0) counts[e] = part[0] + part[1] + part[2] + part[3];
}

__global__ __launch_bounds__(256) void moe_place_kernel(const int32_t* __restrict__ ids, int num_slots, int experts, int block_m,
                                                        const int32_t* __restrict__ counts, int32_t* __restrict__ sorted,
                                                        int32_t* __restrict__ block_expert, int32_t* __restrict__ num_post) {
  __shared__ int wtot[4];
  const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int base = 0;
  for (int o = 0; o < e; ++o) base += (counts[o] + block_m - 1) / block_m * block_m;
  const int mine = counts[e];
  const int padded = (mine + block_m - 1) / block_m * block_m;
  int running = 0;
  for (int at = 0; at < num_slots; at += 256) {
    const int i = at + tid;
    const bool hit = i < num_slots && ids[i] == e;
    const unsigned long long mask = __ballot(hit);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    __syncthreads();   // (the previous round's totals have been read)
    if (lane == 0) wtot[wave] = __popcll(mask);
    __syncthreads();
    int off = running;
    for (int w = 0; w < wave; ++w) off += wtot[w];
    if (hit) sorted[base + off + before] = i;
    running += wtot[0] + wtot[1] + wtot[2] + wtot[3];
  }
  for (int i = mine + tid; i < padded; i += 256) sorted[base + i] = num_slots;
  for (int b = tid; b < padded / block_m; b += 256) block_expert[base / block_m + b] = e;
  if (e == experts - 1 && tid == 0) num_post[0] = base + padded;
}

// ------------------------------------------------------------------------------------------------------------------------
// grouped products, plain tiled form: 32 sorted rows x 64 columns per workgroup, 32 contraction entries per pass
// ------------------------------------------------------------------------------------------------------------------------
template <int DT, bool GLU>
__global__ __launch_bounds__(256) void moe_rows_gemm_kernel(const void* __restrict__ a, int64_t a_ld, int a_div,
                                                            const void* __restrict__ w, int64_t w_stride_e, int K, int N,
                                                            const float* __restrict__ slot_weight, void* __restrict__ out,
                                                            int64_t out_ld, const int32_t* __restrict__ sorted,
                                                            const int32_t* __restrict__ block_expert,
                                                            const int32_t* __restrict__ num_post, int num_slots) {
  constexpr int BM = 32, BN = 64, BK = 32;
  __shared__ float As[BM][BK + 1];
  __shared__ int rows[BM];
  const int block = blockIdx.x;
  if (block * BM >= num_post[0]) return;
  const int e = block_expert[block];
  const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
  if (tid < BM) rows[tid] = sorted[block * BM + tid];
  const int col = blockIdx.y * BN + tx;
  const bool colok = col < N;
  const int64_t wg_at = (int64_t)e * w_stride_e + (int64_t)col * K;
  const int64_t wu_at = (int64_t)e * w_stride_e + (int64_t)(N + col) * K;
  float acc_g[8], acc_u[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) acc_g[r] = acc_u[r] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < BM * BK / 256; ++u) {
      const int idx = tid + 256 * u, r = idx / BK, kk = idx - r * BK;
      const int slot = rows[r];
      As[r][kk] = (slot < num_slots && k0 + kk < K) ? ldv<DT>(a, (int64_t)(slot / a_div) * a_ld + k0 + kk) : 0.f;
    }
    __syncthreads();
    if (colok) {
      const int kn = K - k0 < BK ? K - k0 : BK;
      for (int kk = 0; kk < kn; ++kk) {
        const float wg = ldv<DT>(w, wg_at + k0 + kk);
        const float wu = GLU ? ldv<DT>(w, wu_at + k0 + kk) : 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const float av = As[ty * 8 + r][kk];
          acc_g[r] += av * wg;
          if (GLU) acc_u[r] += av * wu;
        }
      }
    }
  }
  if (!colok) return;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int slot = rows[ty * 8 + r];
    if (slot >= num_slots) continue;
    float v;
    if (GLU) {
      const float sg = DT == LL_F32 ? sigmoid_exact(acc_g[r]) : ll_sigmoidf(acc_g[r]);
      v = acc_g[r] * sg * acc_u[r];
    } else {
      v = slot_weight ? acc_g[r] * slot_weight[slot] : acc_g[r];
    }
    stv<DT>(out, (int64_t)slot * out_ld + col, v);
  }
}

// ------------------------------------------------------------------------------------------------------------------------
// grouped products, MFMA form (16-bit storage, K a multiple of 8, 16-byte aligned rows): one wave per 32 sorted rows x 32
// columns (gate and up: 32 + 32).  Both operands are contraction-contiguous, so a lane's fragment is ONE 16-byte load: lane
// (t, c) holds entries 8 c .. 8 c + 7 (+ 32 per pass) of row / column t.  Rows = columns of the MFMA (B operand), weight rows
// = MFMA rows (A operand): the accumulator of lane (t, c) holds weight rows 4 c .. 4 c + 3 of sorted row t.
// ------------------------------------------------------------------------------------------------------------------------
struct alignas(16) Q4 {
  uint32_t x, y, z, w;
};
template <int DT>
__device__ __forceinline__ f32x4 mfma16(const Q4& a, const Q4& b, f32x4 c) {
  if constexpr (DT == LL_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

template <int DT, bool GLU>
__global__ __launch_bounds__(64) void moe_rows_gemm_mfma_kernel(const uint16_t* __restrict__ a, int64_t a_ld, int a_div,
                                                                const uint16_t* __restrict__ w, int64_t w_stride_e, int K, int N,
                                                                const float* __restrict__ slot_weight, uint16_t* __restrict__ out,
                                                                int64_t out_ld, const int32_t* __restrict__ sorted,
                                                                const int32_t* __restrict__ block_expert,
                                                                const int32_t* __restrict__ num_post, int num_slots) {
  constexpr int BM = 32, BN = 32;
  constexpr int NW = GLU ? 4 : 2;   // weight-row tiles of 16: gate 0..1, up 2..3
  const int block = blockIdx.x;
  if (block * BM >= num_post[0]) return;
  const int e = block_expert[block];
  const int lane = threadIdx.x, t = lane & 15, c = lane >> 4;
  const int n0 = blockIdx.y * BN;
  int slot[2];
  const uint16_t* arow[2];
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    slot[m] = sorted[block * BM + 16 * m + t];
    arow[m] = slot[m] < num_slots ? a + (int64_t)(slot[m] / a_div) * a_ld : nullptr;
  }
  const uint16_t* wrow[NW];
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    const int col = n0 + 16 * (j & 1) + t;
    const int64_t r = (GLU && j >= 2) ? (int64_t)N + col : col;
    wrow[j] = col < N ? w + (int64_t)e * w_stride_e + r * K : nullptr;
  }
  f32x4 acc[NW][2];
#pragma unroll
  for (int j = 0; j < NW; ++j) acc[j][0] = acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int ch = k0 + 8 * c;
    const bool in = ch < K;
    Q4 af[2], wf[NW];
#pragma unroll
    for (int m = 0; m < 2; ++m) af[m] = (in && arow[m]) ? *reinterpret_cast<const Q4*>(arow[m] + ch) : Q4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < NW; ++j) wf[j] = (in && wrow[j]) ? *reinterpret_cast<const Q4*>(wrow[j] + ch) : Q4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      acc[j][0] = mfma16<DT>(wf[j], af[0], acc[j][0]);
      acc[j][1] = mfma16<DT>(wf[j], af[1], acc[j][1]);
    }
  }
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    if (slot[m] >= num_slots) continue;
    const float sw = (!GLU && slot_weight) ? slot_weight[slot[m]] : 1.0f;
    uint16_t* orow = out + (int64_t)slot[m] * out_ld;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = n0 + 16 * j + 4 * c + r;
        if (col >= N) continue;
        float v;
        if (GLU) {
          const float g = acc[j][m][r];
          v = g * ll_sigmoidf(g) * acc[j + 2][m][r];
        } else {
          v = acc[j][m][r] * sw;
        }
        orow[col] = from_f32<DT>(v);
      }
    }
  }
}

}  // namespace

#define LL_BY_DTYPE(dtype, CALL)             \
  do {                                       \
    if (dtype == LL_F16) { CALL(LL_F16); }   \
    else if (dtype == LL_BF16) { CALL(LL_BF16); } \
    else { CALL(LL_F32); }                   \
  } while (0)

extern "C" int ll_group_router(const void* h, int64_t h_ld, const void* w_router, const void* w_extra, int64_t n, int64_t width,
                               int64_t experts, int64_t top, int64_t group_count, int64_t group_keep, float route_scale,
                               int32_t* ids, float* weights, float* extra_scale, int dtype, void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (n < 0 || width < 1 || h_ld < width || experts < 1 || experts > 4096 || top < 1 || top > experts || top > 64 || group_count < 1 ||
      experts % group_count || group_keep < 1 || group_keep > group_count || group_keep * (experts / group_count) < top)
    return LL_ERR_SHAPE;
  if (n == 0) return LL_OK;
  if (!h || !w_router || !ids || !weights || (w_extra && !extra_scale)) return LL_ERR_ARG;
  const size_t lds = sizeof(float) * (size_t)(experts + 2 * group_count + top);
  hipStream_t st = (hipStream_t)stream;
#define CALL(DT)                                                                                                                  \
  group_router_kernel<DT><<<dim3((unsigned)n), 64, lds, st>>>(h, h_ld, w_router, w_extra, (int)width, (int)experts, (int)top,      \
                                                              (int)group_count, (int)group_keep, route_scale, ids, weights, extra_scale)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}

extern "C" int64_t ll_moe_rows_block(void) { return 32; }

// counts: int32 scratch [experts].  sorted [num_slots + experts * (block - 1)], block_expert [ceil(that / block)], num_post [1]
extern "C" int ll_moe_sort(const int32_t* ids, int64_t num_slots, int64_t experts, int32_t* counts, int32_t* sorted,
                           int32_t* block_expert, int32_t* num_post, void* stream) {
  if (num_slots < 0 || experts < 1 || experts > 65535 || num_slots + experts * 32 >= (1ll << 31)) return LL_ERR_SHAPE;
  if (!ids || !counts || !sorted || !block_expert || !num_post) return LL_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  moe_count_kernel<<<dim3((unsigned)experts), 256, 0, st>>>(ids, (int)num_slots, counts);
  moe_place_kernel<<<dim3((unsigned)experts), 256, 0, st>>>(ids, (int)num_slots, (int)experts, 32, counts, sorted, block_expert,
                                                            num_post);
  return LL_LAUNCH_CHECK();
}

// glu != 0: w [experts][2 N][K] (gate rows, then up rows), out[slot][N] = silu(a_row Wg^T) * (a_row Wu^T) with a_row =
// a[slot / a_div]; glu == 0: w [experts][N][K], out[slot][N] = (a[slot / a_div] W^T) * slot_weight[slot] (NULL: 1).
extern "C" int ll_moe_rows_gemm(const void* a, int64_t a_ld, int64_t a_div, const void* w, int64_t w_stride_e, int64_t K, int64_t N,
                                int glu, const float* slot_weight, void* out, int64_t out_ld, const int32_t* sorted,
                                const int32_t* block_expert, const int32_t* num_post, int64_t num_slots, int64_t experts, int dtype,
                                void* stream) {
  if (dtype != LL_F16 && dtype != LL_BF16 && dtype != LL_F32) return LL_ERR_DTYPE;
  if (num_slots < 0 || K < 1 || N < 1 || a_div < 1 || a_ld < K || out_ld < N || w_stride_e < (glu ? 2 : 1) * N * K || experts < 1)
    return LL_ERR_SHAPE;
  if (num_slots == 0) return LL_OK;
  if (!a || !w || !out || !sorted || !block_expert || !num_post) return LL_ERR_ARG;
  const int64_t max_blocks = (num_slots + experts * 31 + 31) / 32;
  hipStream_t st = (hipStream_t)stream;
  static const bool no_mfma = getenv("LL_MOE_ROWS_VALU") != nullptr;   // A/B knob, read once
  const bool mfma = !no_mfma && dtype != LL_F32 && K % 8 == 0 && a_ld % 8 == 0 && w_stride_e % 8 == 0 && ll_aligned16(a) && ll_aligned16(w);
  if (mfma) {
    const dim3 grid((unsigned)max_blocks, (unsigned)((N + 31) / 32));
#define CALL_M(DT, G)                                                                                                         \
  moe_rows_gemm_mfma_kernel<DT, G><<<grid, 64, 0, st>>>((const uint16_t*)a, a_ld, (int)a_div, (const uint16_t*)w, w_stride_e, \
                                                        (int)K, (int)N, slot_weight, (uint16_t*)out, out_ld, sorted, block_expert, \
                                                        num_post, (int)num_slots)
    if (dtype == LL_F16) { if (glu) CALL_M(LL_F16, true); else CALL_M(LL_F16, false); }
    else { if (glu) CALL_M(LL_BF16, true); else CALL_M(LL_BF16, false); }
#undef CALL_M
    return LL_LAUNCH_CHECK();
  }
  const dim3 grid((unsigned)max_blocks, (unsigned)((N + 63) / 64));
#define CALL(DT)                                                                                                             \
  if (glu) moe_rows_gemm_kernel<DT, true><<<grid, 256, 0, st>>>(a, a_ld, (int)a_div, w, w_stride_e, (int)K, (int)N, slot_weight, \
                                                                out, out_ld, sorted, block_expert, num_post, (int)num_slots);    \
  else moe_rows_gemm_kernel<DT, false><<<grid, 256, 0, st>>>(a, a_ld, (int)a_div, w, w_stride_e, (int)K, (int)N, slot_weight,   \
                                                             out, out_ld, sorted, block_expert, num_post, (int)num_slots)
  LL_BY_DTYPE(dtype, CALL);
#undef CALL
  return LL_LAUNCH_CHECK();
}
