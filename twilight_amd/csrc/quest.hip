// Quest page selector: page scores from min/max metadata, then top-k pages per row.
//
// Restates twilight/pyimpl/quest.py:17-122. The reference recomputes, every step,
// amax over each 16-token chunk of K*sign(q) and multiplies by q*sign(q) (quest.py:37-84); since
// max_t(K_t*s) is max_t K_t for s=+1 and -min_t K_t for s=-1, the same number is
//     score(page) = sum_d q_d * (q_d > 0 ? max_d : min_d)
// over per-page channel-wise min / max kept as metadata (512 B per page and kv head instead of
// 4 KiB of K). Kernel 1 streams the metadata (the largest HBM term of the decode layer): one
// 16-byte load per lane covers 4 channels' min and max, so a wavefront scores 2 pages per load
// instruction; the max/min choice is one bit-select per channel pair because sign(q) is fixed for
// the row, and products are accumulated in fp32. The k best pages of a row are then selected with
// an MSB-first radix select on order-preserving keys held in registers and emitted in ascending
// page order (ties at the k-th score go to the lower page number; torch.topk leaves that order
// unspecified, quest.py:99). (Letting the last scoring workgroup of a row do the selection, to
// save the second launch, was measured and is slower: the device-scope stores and the ticket
// keep every scoring workgroup alive for a memory round trip longer.)
#include "quest_select_core.h"

namespace twl {

struct QuestArgs {
  const void* q;
  const uint8_t* meta;
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  uint32_t num_q_heads, num_kv_heads;
  uint32_t max_pages;  // pages per request the grid and the score row are sized for
  float* page_scores;
  uint32_t score_stride;
  uint32_t token_budget;
  int32_t* sel_pages;
  uint32_t sel_stride;
  int32_t* sel_count;
  int group_max;  // GROUP > 1: every q head of a group receives the group's largest score per page
};

constexpr int kQsThreads = 256;
constexpr int kQsPagesPerWave = 32;
constexpr int kQsPagesPerBlock = kQsPagesPerWave * (kQsThreads / kWave);  // 128
constexpr int kQsUnroll = 4;  // load instructions in flight per wave (2 pages each)

// Top-k pages of one (batch, q head) row.
template <int THREADS, int VPT>
__device__ __forceinline__ void quest_select_row(const QuestArgs& a, uint32_t row, SelSmem& sm) {
  const uint32_t b = row / a.num_q_heads;
  const int n_pages = min(a.kv_page_indptr[b + 1] - a.kv_page_indptr[b],
                          min((int)a.max_pages, THREADS * VPT));
  const int k = min(quest_budget_pages(a.token_budget), n_pages);
  if (threadIdx.x == 0) a.sel_count[row] = max(k, 0);
  if (k <= 0) return;
  select_row_topk<THREADS, VPT>(a.page_scores + (size_t)row * a.score_stride, n_pages, k,
                                a.sel_pages + (size_t)row * a.sel_stride, nullptr, sm);
}

template <int THREADS, int VPT>
__global__ __launch_bounds__(THREADS) void quest_select_kernel(QuestArgs a) {
  __shared__ SelSmem sm;
  select_smem_init<THREADS>(sm);
  __syncthreads();
  quest_select_row<THREADS, VPT>(a, blockIdx.x, sm);
}

// GROUP q heads share one kv head (GQA): a workgroup row is one (batch, kv head) and every metadata
// record is loaded once and scored against the GROUP queries. GROUP == 1 also serves group sizes
// without a specialisation: then a row is one (batch, q head) and records are re-read per q head.
template <int DT, int GROUP>
__global__ __launch_bounds__(kQsThreads) void quest_score_kernel(QuestArgs a) {
  const uint32_t rows_per_batch = GROUP == 1 ? a.num_q_heads : a.num_kv_heads;
  const uint32_t b = blockIdx.y / rows_per_batch;
  const uint32_t r = blockIdx.y - b * rows_per_batch;
  const uint32_t kvh = GROUP == 1 ? r / (a.num_q_heads / a.num_kv_heads) : r;
  const uint32_t row0 = b * a.num_q_heads + (GROUP == 1 ? r : r * GROUP);  // first q-head row
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int pg_begin = a.kv_page_indptr[b];
  const int n_pages = min(max(a.kv_page_indptr[b + 1] - pg_begin, 0), (int)a.max_pages);
  const int p0 = blockIdx.x * kQsPagesPerBlock + wave * kQsPagesPerWave;
  const int np = min(kQsPagesPerWave, n_pages - p0);  // <= 0: this wave has nothing to stream
  if (np <= 0) return;

  const int c = lane & 31;     // channel chunk: dims 4c..4c+3
  const int half = lane >> 5;  // which of the 2 pages of a load
  // q for dims 4c..4c+3 and the per-half select mask (all ones where q > 0), per q head
  uint32_t qw[GROUP][2];
#pragma unroll
  for (int g = 0; g < GROUP; ++g) {
    u32x2 v = *(const u32x2*)((const uint16_t*)a.q + (size_t)(row0 + g) * TWL_HEAD_DIM + 4 * c);
    qw[g][0] = v.x; qw[g][1] = v.y;
  }
  int my_phys = 0;
  if (lane < np) my_phys = a.kv_page_indices[pg_begin + p0 + lane];
  float qf[GROUP][4];
  uint32_t selmask[GROUP][2];
#pragma unroll
  for (int g = 0; g < GROUP; ++g)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      qf[g][2 * j] = bits16_to_f32<DT>(qw[g][j] & 0xFFFFu);
      qf[g][2 * j + 1] = bits16_to_f32<DT>(qw[g][j] >> 16);
      selmask[g][j] = (qf[g][2 * j] > 0.0f ? 0x0000FFFFu : 0u) |
                      (qf[g][2 * j + 1] > 0.0f ? 0xFFFF0000u : 0u);
    }
  const size_t rec_stride = (size_t)a.num_kv_heads * TWL_META_RECORD_BYTES;
  const uint8_t* base = a.meta + (size_t)kvh * TWL_META_RECORD_BYTES + 16 * c;
  float keep[GROUP];  // lane i ends up with the score of page p0 + i
#pragma unroll
  for (int g = 0; g < GROUP; ++g) keep[g] = 0.0f;

#pragma unroll
  for (int i0 = 0; i0 < kQsPagesPerWave; i0 += 2 * kQsUnroll) {
    if (i0 >= np) break;
    u32x4 mm[kQsUnroll];
#pragma unroll
    for (int u = 0; u < kQsUnroll; ++u) {
      const int ia = i0 + 2 * u, ib = ia + 1;
      const int pa = __builtin_amdgcn_readlane(my_phys, (ia < np) ? ia : 0);
      const int pb = __builtin_amdgcn_readlane(my_phys, (ib < np) ? ib : 0);
      const int phys = half ? pb : pa;
      mm[u] = __builtin_nontemporal_load((const u32x4*)(base + (size_t)phys * rec_stride));
    }
#pragma unroll
    for (int u = 0; u < kQsUnroll; ++u) {
      const int ia = i0 + 2 * u;
#pragma unroll
      for (int g = 0; g < GROUP; ++g) {
        // words: x,y = min[4c..4c+3], z,w = max[4c..4c+3]
        const uint32_t s0 = (mm[u].z & selmask[g][0]) | (mm[u].x & ~selmask[g][0]);
        const uint32_t s1 = (mm[u].w & selmask[g][1]) | (mm[u].y & ~selmask[g][1]);
        float acc;
        if (DT == TWL_F16) {
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, s0),
                                       __builtin_bit_cast(half2_t, qw[g][0]), 0.0f, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, s1),
                                       __builtin_bit_cast(half2_t, qw[g][1]), acc, false);
        } else {
          acc = qf[g][0] * as_f32(s0 << 16);
          acc = fmaf(qf[g][1], as_f32(s0 & 0xFFFF0000u), acc);
          acc = fmaf(qf[g][2], as_f32(s1 << 16), acc);
          acc = fmaf(qf[g][3], as_f32(s1 & 0xFFFF0000u), acc);
        }
        acc = row16_allreduce<OpSum>(acc);
        acc += dpp<kDppBcast15, 0xA>(0.0f, acc);  // lanes 16..31 / 48..63 now hold a page total
        const float sa = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 31));
        const float sb = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 63));
        keep[g] = (lane == ia) ? sa : keep[g];
        keep[g] = (lane == ia + 1) ? sb : keep[g];
      }
    }
  }
  if (GROUP > 1 && a.group_max) {
    float mx = keep[0];
#pragma unroll
    for (int g = 1; g < GROUP; ++g) mx = fmaxf(mx, keep[g]);
#pragma unroll
    for (int g = 0; g < GROUP; ++g) keep[g] = mx;
  }
  // one store per wave and q head: 32 consecutive scores
  if (lane < np) {
#pragma unroll
    for (int g = 0; g < GROUP; ++g)
      a.page_scores[(size_t)(row0 + g) * a.score_stride + p0 + lane] = keep[g];
  }
}

}  // namespace twl

static int check_quest_common(const void* q, int q_dtype, const void* meta,
                              const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                              uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                              uint32_t max_pages_per_req, const float* page_scores,
                              uint32_t score_stride) {
  if (!q || !meta || !kv_page_indices || !kv_page_indptr || !page_scores) return TWL_ENULL;
  if (q_dtype != TWL_F16 && q_dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (max_pages_per_req == 0 || max_pages_per_req > 16384 || score_stride < max_pages_per_req)
    return TWL_EINVAL;
  if ((uint64_t)batch * num_q_heads > 65535u) return TWL_EINVAL;
  if ((((uintptr_t)q) & 7u) || (((uintptr_t)meta) & 15u) || (((uintptr_t)page_scores) & 3u))
    return TWL_EALIGN;
  return TWL_OK;
}

static int check_budget(uint32_t token_budget, uint32_t max_pages_per_req, uint32_t sel_stride) {
  if (token_budget == 0) return TWL_EINVAL;
  uint64_t k = (token_budget / TWL_PAGE ? token_budget / TWL_PAGE : 1) +
               (token_budget % TWL_PAGE ? 1 : 0);
  if (k > max_pages_per_req) k = max_pages_per_req;
  return sel_stride < k ? TWL_EINVAL : TWL_OK;
}

template <int GROUP>
static void launch_score_g(int q_dtype, dim3 grid, hipStream_t s, const twl::QuestArgs& a) {
  if (q_dtype == TWL_F16)
    hipLaunchKernelGGL((twl::quest_score_kernel<TWL_F16, GROUP>), grid, dim3(twl::kQsThreads), 0,
                       s, a);
  else
    hipLaunchKernelGGL((twl::quest_score_kernel<TWL_BF16, GROUP>), grid, dim3(twl::kQsThreads), 0,
                       s, a);
}

static void launch_score(int q_dtype, uint32_t batch, hipStream_t s, const twl::QuestArgs& a) {
  const uint32_t gx = (a.max_pages + twl::kQsPagesPerBlock - 1) / twl::kQsPagesPerBlock;
  const uint32_t group = a.num_q_heads / a.num_kv_heads;
  if (group == 2) launch_score_g<2>(q_dtype, dim3(gx, batch * a.num_kv_heads), s, a);
  else if (group == 4) launch_score_g<4>(q_dtype, dim3(gx, batch * a.num_kv_heads), s, a);
  else if (group == 8) launch_score_g<8>(q_dtype, dim3(gx, batch * a.num_kv_heads), s, a);
  else launch_score_g<1>(q_dtype, dim3(gx, batch * a.num_q_heads), s, a);
}

int twl::quest_page_scores_ex(const void* q, int q_dtype, const void* meta,
                              const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                              uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                              uint32_t max_pages_per_req, float* page_scores,
                              uint32_t score_stride, int group_max, void* stream) {
  if (group_max) {
    const uint32_t group = num_kv_heads ? num_q_heads / num_kv_heads : 0;
    if (group != 2 && group != 4 && group != 8) return TWL_EINVAL;
  }
  int rc = check_quest_common(q, q_dtype, meta, kv_page_indices, kv_page_indptr, batch,
                              num_q_heads, num_kv_heads, max_pages_per_req, page_scores,
                              score_stride);
  if (rc != TWL_OK) return rc;
  twl::QuestArgs a{};
  a.q = q; a.meta = (const uint8_t*)meta; a.kv_page_indices = kv_page_indices;
  a.kv_page_indptr = kv_page_indptr; a.num_q_heads = num_q_heads; a.num_kv_heads = num_kv_heads;
  a.max_pages = max_pages_per_req; a.page_scores = page_scores; a.score_stride = score_stride;
  a.group_max = group_max;
  launch_score(q_dtype, batch, (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_quest_page_scores(const void* q, int q_dtype, const void* meta,
                                     const int32_t* kv_page_indices,
                                     const int32_t* kv_page_indptr, uint32_t batch,
                                     uint32_t num_q_heads, uint32_t num_kv_heads,
                                     uint32_t max_pages_per_req, float* page_scores,
                                     uint32_t score_stride, void* stream) {
  return twl::quest_page_scores_ex(q, q_dtype, meta, kv_page_indices, kv_page_indptr, batch,
                                   num_q_heads, num_kv_heads, max_pages_per_req, page_scores,
                                   score_stride, 0, stream);
}

extern "C" int twl_quest_topk_pages(const float* page_scores, uint32_t score_stride,
                                    const int32_t* kv_page_indptr, uint32_t batch,
                                    uint32_t num_q_heads, uint32_t token_budget,
                                    uint32_t max_pages_per_req, int32_t* sel_pages,
                                    uint32_t sel_stride, int32_t* sel_count, void* stream) {
  if (!page_scores || !kv_page_indptr || !sel_pages || !sel_count) return TWL_ENULL;
  if (batch == 0 || num_q_heads == 0) return TWL_EINVAL;
  if (max_pages_per_req == 0 || max_pages_per_req > 16384 || score_stride < max_pages_per_req)
    return TWL_EINVAL;
  int rc = check_budget(token_budget, max_pages_per_req, sel_stride);
  if (rc != TWL_OK) return rc;
  if ((uint64_t)batch * num_q_heads > 65535u) return TWL_EINVAL;
  if (((uintptr_t)page_scores) & 3u) return TWL_EALIGN;
  hipStream_t s = (hipStream_t)stream;
  const uint32_t rows = batch * num_q_heads;
  twl::QuestArgs a{};
  a.page_scores = const_cast<float*>(page_scores); a.score_stride = score_stride;
  a.kv_page_indptr = kv_page_indptr; a.num_q_heads = num_q_heads; a.max_pages = max_pages_per_req;
  a.token_budget = token_budget; a.sel_pages = sel_pages; a.sel_stride = sel_stride;
  a.sel_count = sel_count;
  const uint32_t n = max_pages_per_req;
  if (n <= 512)
    hipLaunchKernelGGL((twl::quest_select_kernel<256, 2>), dim3(rows), dim3(256), 0, s, a);
  else if (n <= 2048)
    hipLaunchKernelGGL((twl::quest_select_kernel<1024, 2>), dim3(rows), dim3(1024), 0, s, a);
  else if (n <= 4096)
    hipLaunchKernelGGL((twl::quest_select_kernel<1024, 4>), dim3(rows), dim3(1024), 0, s, a);
  else if (n <= 8192)
    hipLaunchKernelGGL((twl::quest_select_kernel<1024, 8>), dim3(rows), dim3(1024), 0, s, a);
  else
    hipLaunchKernelGGL((twl::quest_select_kernel<1024, 16>), dim3(rows), dim3(1024), 0, s, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_quest_select(const void* q, int q_dtype, const void* meta,
                                const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                                uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                                uint32_t token_budget, uint32_t max_pages_per_req,
                                int32_t* sel_pages, uint32_t sel_stride, int32_t* sel_count,
                                float* page_scores, uint32_t score_stride, void* stream) {
  if (!sel_pages || !sel_count) return TWL_ENULL;
  int rc = check_budget(token_budget, max_pages_per_req, sel_stride);
  if (rc != TWL_OK) return rc;
  rc = twl_quest_page_scores(q, q_dtype, meta, kv_page_indices, kv_page_indptr, batch,
                             num_q_heads, num_kv_heads, max_pages_per_req, page_scores,
                             score_stride, stream);
  if (rc != TWL_OK) return rc;
  return twl_quest_topk_pages(page_scores, score_stride, kv_page_indptr, batch, num_q_heads,
                              token_budget, max_pages_per_req, sel_pages, sel_stride, sel_count,
                              stream);
}
