// Fused estimator + pruner: INT4-K score GEMV, fp32 softmax, top-p bisection and ordered
// compaction of one (batch, head) row in one workgroup, the scores never leaving registers
// (fused_row_core.h). This kernel takes the row's page list from memory; keeping the row in one
// workgroup removes a launch, the write-back of the score matrix at the end of the GEMV (4 bytes
// per candidate cost about as much time as 20 bytes of reads on this HBM) and its re-read.
#include "fused_row_core.h"

namespace twl {

template <int QDT, int THREADS, int VPT>
__global__ __launch_bounds__(THREADS) void gemv_top_p_kernel(FusedArgs a) {
  constexpr int PW = 4 * VPT;
  constexpr int RUNS = (PW + 63) / 64;
  __shared__ FusedSmem fsm;
  const uint32_t row = blockIdx.x;
  const uint32_t b = row / a.num_q_heads;
  const uint32_t h = row - b * a.num_q_heads;
  const uint32_t kvh = h / (a.num_q_heads / a.num_kv_heads);
  const int lane = lane_id();
  const int e0 = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave) * PW;
  // everything that depends only on the kernel arguments is requested at once
  const int pg_begin = a.kv_page_indptr[b];
  const int pg_end = a.kv_page_indptr[b + 1];
  const int last_len = a.kv_last_page_len[b];
  const int sel_n = a.sel_count ? a.sel_count[row] : (int)a.sel_stride;
  int my_logical[RUNS];
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    const int e = e0 + 64 * r + lane;
    my_logical[r] = (64 * r + lane < PW && (uint32_t)e < a.sel_stride)
                        ? a.sel_pages[(size_t)row * a.sel_stride + e] : 0;
  }
  u32x4 qraw[4];
  fused_load_q(a.q, row, lane & 3, qraw);
  estimate_prune_row<QDT, THREADS, VPT>(a, fsm, row, kvh, pg_begin, pg_end - pg_begin, last_len,
                                        sel_n, my_logical, qraw);
}

template <int QDT>
static void launch_fused(const FusedArgs& a, uint32_t rows, hipStream_t s) {
  const uint32_t k = a.max_pages;
#define TWL_FUSED_CASE(T, V) \
  hipLaunchKernelGGL((gemv_top_p_kernel<QDT, T, V>), dim3(rows), dim3(T), 0, s, a)
  if (k <= 16) TWL_FUSED_CASE(256, 1);
  else if (k <= 32) TWL_FUSED_CASE(256, 2);
  else if (k <= 64) TWL_FUSED_CASE(256, 4);
  else if (k <= 128) TWL_FUSED_CASE(256, 8);
  else if (k <= 256) TWL_FUSED_CASE(256, 16);
  else if (k <= 512) TWL_FUSED_CASE(512, 16);  // measured faster than 1024 x 8
  else if (k <= 1024) TWL_FUSED_CASE(1024, 16);
  else TWL_FUSED_CASE(1024, 32);
#undef TWL_FUSED_CASE
}

}  // namespace twl

int twl::gemv_top_p_ex(const void* q, int q_dtype, const void* k_int4,
                              const int32_t* sel_pages, const int32_t* sel_count,
                              uint32_t sel_stride, const int32_t* kv_page_indices,
                              const int32_t* kv_page_indptr, const int32_t* kv_last_page_len,
                              uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                              uint32_t max_pages_per_row, float sm_scale, const float* p_arr,
                              float p, int high_mode, int32_t* idx, uint32_t idx_stride,
                              int32_t* count, float* scores_out, uint32_t score_stride,
                              int32_t* cand_count, float* low_out, float* surv_probs,
                              void* stream) {
  if (!q || !k_int4 || !sel_pages || !kv_page_indices || !kv_page_indptr || !kv_last_page_len ||
      !idx || !count)
    return TWL_ENULL;
  if (q_dtype != TWL_F16 && q_dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (max_pages_per_row == 0 || max_pages_per_row > TWL_MAX_CANDIDATES / TWL_PAGE)
    return TWL_EINVAL;
  if (sel_stride < max_pages_per_row) return TWL_EINVAL;
  if ((uint64_t)max_pages_per_row * TWL_PAGE > idx_stride) return TWL_EINVAL;
  if (scores_out && (uint64_t)max_pages_per_row * TWL_PAGE > score_stride) return TWL_EINVAL;
  if (high_mode != TWL_HIGH_FIRST && high_mode != TWL_HIGH_MAX) return TWL_EINVAL;
  if (!p_arr && !(p > 0.0f && p <= 1.0f)) return TWL_EINVAL;
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k_int4) & 15u) || (((uintptr_t)scores_out) & 3u))
    return TWL_EALIGN;
  twl::FusedArgs a{};
  a.q = q; a.k_int4 = (const uint8_t*)k_int4; a.sel_pages = sel_pages; a.sel_count = sel_count;
  a.sel_stride = sel_stride; a.kv_page_indices = kv_page_indices; a.kv_page_indptr = kv_page_indptr;
  a.kv_last_page_len = kv_last_page_len; a.num_q_heads = num_q_heads;
  a.num_kv_heads = num_kv_heads; a.max_pages = max_pages_per_row; a.sm_scale = sm_scale;
  a.p_arr = p_arr; a.p = p; a.high_mode = high_mode; a.idx = idx; a.idx_stride = idx_stride;
  a.count = count; a.scores_out = scores_out; a.score_stride = score_stride;
  a.cand_count = cand_count; a.low_out = low_out; a.surv_probs = surv_probs;
  const uint32_t rows = batch * num_q_heads;
  if (q_dtype == TWL_F16) twl::launch_fused<TWL_F16>(a, rows, (hipStream_t)stream);
  else twl::launch_fused<TWL_BF16>(a, rows, (hipStream_t)stream);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_gemv_top_p(const void* q, int q_dtype, const void* k_int4,
                              const int32_t* sel_pages, const int32_t* sel_count,
                              uint32_t sel_stride, const int32_t* kv_page_indices,
                              const int32_t* kv_page_indptr, const int32_t* kv_last_page_len,
                              uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                              uint32_t max_pages_per_row, float sm_scale, const float* p_arr,
                              float p, int high_mode, int32_t* idx, uint32_t idx_stride,
                              int32_t* count, float* scores_out, uint32_t score_stride,
                              int32_t* cand_count, float* low_out, void* stream) {
  return twl::gemv_top_p_ex(q, q_dtype, k_int4, sel_pages, sel_count, sel_stride, kv_page_indices,
                            kv_page_indptr, kv_last_page_len, batch, num_q_heads, num_kv_heads,
                            max_pages_per_row, sm_scale, p_arr, p, high_mode, idx, idx_stride,
                            count, scores_out, score_stride, cand_count, low_out, nullptr, stream);
}
