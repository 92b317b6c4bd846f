// Selector + estimator + pruner of one (batch, head) row in ONE workgroup and one launch:
// Quest page scores from the min/max metadata, top-k pages, INT4 score GEMV over those pages,
// softmax, top-p bisection and compaction (twilight/pyimpl/quest.py:17-122,
// twilight/pyimpl/attention.py:252-255, twilight/pyimpl/top_p.py:10-15, attention.py:280-281).
//
// Every stage of a row depends only on that row, so a workgroup that owns the row from start to
// end needs no synchronisation with any other workgroup: the page scores live in LDS, the page
// list in LDS and registers, the candidate scores in registers. Compared with the three launches
// (twl_quest_page_scores, twl_quest_topk_pages, twl_gemv_top_p) this removes two launches with
// their dependent argument -> page table -> record load chains and the page-score / page-list
// round trips through memory. It pays off when there is about one row per CU (rows <= CUs);
// with GQA the three-launch form shares each metadata record between the q heads of a group,
// which this kernel cannot, so the caller chooses.
//
// 1024 threads: 16 wavefronts each score 32 pages per pass (lane = 4 channels x 2 pages per
// 16-byte load, as quest_score_kernel does), then select_row_topk and estimate_prune_row run with
// the same 1024 threads.
#include "fused_row_core.h"
#include "quest_select_core.h"

namespace twl {

struct RowArgs {
  FusedArgs f;              // estimator / pruner part (sel_pages / sel_count unused)
  const uint8_t* meta;
  uint32_t token_budget;
  uint32_t max_pages_req;
  int32_t* sel_pages_out;   // [rows, f.sel_stride]
  int32_t* sel_count_out;
  float* page_scores_out;   // nullable
  uint32_t page_score_stride;
  const uint16_t* planes;   // PLANES: metadata in plane layout (meta_planes.hip)
  uint32_t plane_cap;
  const int32_t* plane_slots;  // nullable: slot of each batch position (else slot = position)
  uint32_t plane_num_slots;
};

constexpr int kRowThreads = 1024;
constexpr int kRowWaves = kRowThreads / kWave;
constexpr int kRowUnroll = 4;  // 16-byte loads in flight per lane (2 pages each)

// PLANES: page scores from the plane layout (half the metadata bytes: only the run the sign of
// q_d selects is read, 2 pages per lane, channels in ascending order), else from the 512-byte
// records through the page table.
template <int QDT, int VPT, int SEL_VPT, bool PLANES>
__global__ __launch_bounds__(kRowThreads) void select_estimate_prune_kernel(RowArgs a) {
  constexpr int PW = 4 * VPT;
  constexpr int RUNS = (PW + 63) / 64;
  constexpr int PASSES = 2 * SEL_VPT;  // 512 pages per pass of the whole workgroup
  __shared__ FusedSmem fsm;
  __shared__ SelSmem ssm;
  __shared__ float ps_lds[kRowThreads * SEL_VPT];
  __shared__ int32_t sel_lds[kRowWaves * PW];

  select_smem_init<kRowThreads>(ssm);  // the barrier after the scoring phase orders it
  uint32_t row = blockIdx.x;
  {
    // q heads that share a kv head go to the same XCD (workgroups are dealt to the 8 XCDs round
    // robin; each XCD has its own L2), so that the group's metadata comes from HBM once and the
    // other heads of the group find it in that L2: 65 -> 56 us at 8 x 32 q heads on 8 kv heads.
    // Only the placement depends on how the hardware deals workgroups; the result does not.
    const uint32_t grp = a.f.num_q_heads / a.f.num_kv_heads;
    if (grp > 1 && gridDim.x % (8 * grp) == 0) {
      const uint32_t xcd = blockIdx.x & 7u, s = blockIdx.x >> 3;
      row = ((s / grp) * 8 + xcd) * grp + s % grp;
    }
  }
  const uint32_t b = row / a.f.num_q_heads;
  const uint32_t h = row - b * a.f.num_q_heads;
  const uint32_t kvh = h / (a.f.num_q_heads / a.f.num_kv_heads);
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);

  const int pg_begin = a.f.kv_page_indptr[b];
  const int pg_end = a.f.kv_page_indptr[b + 1];
  const int last_len = a.f.kv_last_page_len[b];
  const int c = lane & 31;     // channel chunk: dims 4c..4c+3
  const int half = lane >> 5;  // which of the 2 pages of a load
  uint32_t qw[2];
  {
    u32x2 v = *(const u32x2*)((const uint16_t*)a.f.q + (size_t)row * TWL_HEAD_DIM + 4 * c);
    qw[0] = v.x; qw[1] = v.y;
  }
  const int req_pages = pg_end - pg_begin;
  const int n_req = min(max(req_pages, 0), min((int)a.max_pages_req, kRowThreads * SEL_VPT));
  const int sel_n = min(min(quest_budget_pages(a.token_budget), n_req), (int)a.f.max_pages);
  // a request no longer than the budget keeps every page: its metadata is not read at all (unless
  // the caller asked for the page scores)
  const int n_score = (sel_n < n_req || a.page_scores_out) ? n_req : 0;

  // ---- 1. Quest page scores into LDS ---------------------------------------------------------
  if constexpr (PLANES) {
    // lane l keeps q[l] and q[64 + l]; q_d reaches every lane as a scalar
    const uint16_t* qrow = (const uint16_t*)a.f.q + (size_t)row * TWL_HEAD_DIM;
    const float q_lo = bits16_to_f32<QDT>(qrow[lane]);
    const float q_hi = bits16_to_f32<QDT>(qrow[64 + lane]);
    const uint32_t slot = plane_slot(a.plane_slots, a.plane_num_slots, b);
    const uint16_t* pl =
        a.planes + ((size_t)slot * a.f.num_kv_heads + kvh) * (TWL_HEAD_DIM * 2) * a.plane_cap;
    constexpr int PL_PASSES = (SEL_VPT + 1) / 2;  // 16 waves x 128 pages = 2048 pages per pass
    // The request's last pages are scored from their metadata records (plane_scored_pages): the
    // appending side keeps the record of the last page current token by token and writes its
    // plane entries once, when the page is full.
    const int np = plane_scored_pages(n_score);
    // tail pages np + wave, np + wave + 16, ... of this wavefront (at most 8): their records are
    // requested now and folded after the plane passes
    const int tail = n_score - np - wave;              // wave-uniform
    const int tail_cnt = tail > 0 ? min((tail + kRowWaves - 1) / kRowWaves, 8) : 0;
    RecordBatch8 rb;
    if (tail_cnt > 0)
      record_pages_load8(rb, a.meta + (size_t)kvh * TWL_META_RECORD_BYTES,
                         (size_t)a.f.num_kv_heads * TWL_META_RECORD_BYTES,
                         a.f.kv_page_indices + pg_begin, np + wave, kRowWaves, tail_cnt);
#pragma unroll
    for (int pass = 0; pass < PL_PASSES; ++pass) {
      const int w0 = (pass * kRowWaves + wave) * 128;  // first page of this wave's slice
      if (w0 < np) {                                     // wave-uniform
        const int pg0 = w0 + 2 * lane;                 // this lane's two pages
        const int pgc = min(pg0, (int)a.plane_cap - 2);  // loads stay inside the run
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll 16
        for (int d = 0; d < TWL_HEAD_DIM; ++d) {
          const float qd =
              as_f32(__builtin_amdgcn_readlane(as_i32(d < 64 ? q_lo : q_hi), d & 63));
          const int plane = qd > 0.0f ? 1 : 0;         // max run for q_d > 0, else min run
          const uint32_t w = __builtin_nontemporal_load(
              (const uint32_t*)(pl + (size_t)(2 * d + plane) * a.plane_cap + pgc));
          s0 = fmaf(qd, bits16_to_f32<QDT>(w & 0xFFFFu), s0);
          s1 = fmaf(qd, bits16_to_f32<QDT>(w >> 16), s1);
        }
        if (pg0 < np) ps_lds[pg0] = s0;
        if (pg0 + 1 < np) ps_lds[pg0 + 1] = s1;
        if (a.page_scores_out) {
          float* po = a.page_scores_out + (size_t)row * a.page_score_stride;
          if (pg0 < np) po[pg0] = s0;
          if (pg0 + 1 < np) po[pg0 + 1] = s1;
        }
      }
    }
    if (tail_cnt > 0) {
      const uint32_t qw2 = *(const uint32_t*)(qrow + 2 * lane);
      float sc[8];
      record_pages_fold8<QDT>(rb, tail_cnt, bits16_to_f32<QDT>(qw2 & 0xFFFFu), bits16_to_f32<QDT>(qw2 >> 16), sc);
      if (lane == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (i < tail_cnt) {
            const int pg = np + wave + i * kRowWaves;
            ps_lds[pg] = sc[i];
            if (a.page_scores_out) a.page_scores_out[(size_t)row * a.page_score_stride + pg] = sc[i];
          }
        }
      }
    }
  } else {
    // page ids of all passes first: register r, lane l <-> pass 2r + l/32, page l%32 of the wave's
    // 32-page slice of that pass
    int ids[SEL_VPT];
#pragma unroll
    for (int r = 0; r < SEL_VPT; ++r) {
      const int pg = ((2 * r + half) * kRowWaves + wave) * 32 + c;
      ids[r] = (pg < n_score) ? a.f.kv_page_indices[pg_begin + pg] : 0;
    }
    float qf[4];
    uint32_t selmask[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      qf[2 * j] = bits16_to_f32<QDT>(qw[j] & 0xFFFFu);
      qf[2 * j + 1] = bits16_to_f32<QDT>(qw[j] >> 16);
      selmask[j] = (qf[2 * j] > 0.0f ? 0x0000FFFFu : 0u) | (qf[2 * j + 1] > 0.0f ? 0xFFFF0000u : 0u);
    }
    const size_t meta_stride = (size_t)a.f.num_kv_heads * TWL_META_RECORD_BYTES;
    const uint8_t* mbase = a.meta + (size_t)kvh * TWL_META_RECORD_BYTES + 16 * c;
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const int p0 = (pass * kRowWaves + wave) * 32;
      const int np = min(32, n_score - p0);  // wave-uniform
      if (np > 0) {
        const int lbase = (pass & 1) * 32;
        float keep = 0.0f;  // lane i ends up with the score of page p0 + i
#pragma unroll
        for (int i0 = 0; i0 < 32; i0 += 2 * kRowUnroll) {
          if (i0 < np) {
            u32x4 mm[kRowUnroll];
#pragma unroll
            for (int u = 0; u < kRowUnroll; ++u) {
              const int ia = i0 + 2 * u, ib = ia + 1;
              // pages past the slice reuse its first page: a valid address, result discarded
              const int pa = __builtin_amdgcn_readlane(ids[pass / 2], lbase + ((ia < np) ? ia : 0));
              const int pb = __builtin_amdgcn_readlane(ids[pass / 2], lbase + ((ib < np) ? ib : 0));
              const int phys = half ? pb : pa;
              mm[u] = __builtin_nontemporal_load((const u32x4*)(mbase + (size_t)phys * meta_stride));
            }
#pragma unroll
            for (int u = 0; u < kRowUnroll; ++u) {
              const int ia = i0 + 2 * u;
              // words: x,y = min[4c..4c+3], z,w = max[4c..4c+3]; q > 0 takes the max, else the min
              const uint32_t s0 = (mm[u].z & selmask[0]) | (mm[u].x & ~selmask[0]);
              const uint32_t s1 = (mm[u].w & selmask[1]) | (mm[u].y & ~selmask[1]);
              float acc;
              if (QDT == TWL_F16) {
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, s0),
                                             __builtin_bit_cast(half2_t, qw[0]), 0.0f, false);
                acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, s1),
                                             __builtin_bit_cast(half2_t, qw[1]), acc, false);
              } else {
                acc = qf[0] * as_f32(s0 << 16);
                acc = fmaf(qf[1], as_f32(s0 & 0xFFFF0000u), acc);
                acc = fmaf(qf[2], as_f32(s1 << 16), acc);
                acc = fmaf(qf[3], as_f32(s1 & 0xFFFF0000u), acc);
              }
              acc = row16_allreduce<OpSum>(acc);
              acc += dpp<kDppBcast15, 0xA>(0.0f, acc);  // lanes 16..31 / 48..63 hold a page total
              const float sa = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 31));
              const float sb = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 63));
              keep = (lane == ia) ? sa : keep;
              keep = (lane == ia + 1) ? sb : keep;
            }
          }
        }
        if (lane < np) {
          ps_lds[p0 + lane] = keep;
          if (a.page_scores_out)
            a.page_scores_out[(size_t)row * a.page_score_stride + p0 + lane] = keep;
        }
      }
    }
  }
  __syncthreads();

  // ---- 2. top-k pages: list to LDS (and to memory for the caller) ----------------------------
  // the estimator's slice of q is requested here: the selection hides the round trip, and the 16
  // registers are not held through the scoring passes
  u32x4 qraw[4];
  fused_load_q(a.f.q, row, lane & 3, qraw);
  if (threadIdx.x == 0) a.sel_count_out[row] = sel_n;
  if (sel_n > 0)
    select_row_topk<kRowThreads, SEL_VPT>(ps_lds, n_req, sel_n,
                                          a.sel_pages_out + (size_t)row * a.f.sel_stride, sel_lds,
                                          ssm);
  __syncthreads();

  // ---- 3. estimator + pruner over the list ---------------------------------------------------
  int my_logical[RUNS];
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    const int e = wave * PW + 64 * r + lane;
    my_logical[r] = (64 * r + lane < PW && e < sel_n) ? sel_lds[e] : 0;
  }
  estimate_prune_row<QDT, kRowThreads, VPT>(a.f, fsm, row, kvh, pg_begin, req_pages, last_len,
                                            sel_n, my_logical, qraw);
}

template <int QDT, int SEL_VPT, bool PLANES>
static void launch_row(const RowArgs& a, uint32_t rows, hipStream_t s) {
  const uint32_t k = a.f.max_pages;
#define TWL_ROW_CASE(V)                                                                         \
  hipLaunchKernelGGL((select_estimate_prune_kernel<QDT, V, SEL_VPT, PLANES>), dim3(rows),       \
                     dim3(kRowThreads), 0, s, a)
  if (k <= 64) TWL_ROW_CASE(1);
  else if (k <= 128) TWL_ROW_CASE(2);
  else if (k <= 256) TWL_ROW_CASE(4);
  else if (k <= 512) TWL_ROW_CASE(8);
  else if (k <= 1024) TWL_ROW_CASE(16);
  else TWL_ROW_CASE(32);
#undef TWL_ROW_CASE
}

}  // namespace twl

int twl::select_estimate_prune_ex(
    const void* q, int dtype, const void* meta, const void* k_int4, const int32_t* kv_page_indices,
    const int32_t* kv_page_indptr, const int32_t* kv_last_page_len, uint32_t batch,
    uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t token_budget,
    uint32_t max_pages_per_req, float sm_scale, const float* p_arr, float p, int high_mode,
    int32_t* sel_pages, uint32_t sel_stride, int32_t* sel_count, int32_t* idx, uint32_t idx_stride,
    int32_t* count, float* page_scores_out, uint32_t page_score_stride, float* scores_out,
    uint32_t score_stride, int32_t* cand_count, const void* meta_planes,
    uint32_t plane_cap_pages, const int32_t* plane_slots, uint32_t plane_num_slots,
    float* surv_probs, void* stream) {
  if (!q || !meta || !k_int4 || !kv_page_indices || !kv_page_indptr || !kv_last_page_len ||
      !sel_pages || !sel_count || !idx || !count)
    return TWL_ENULL;
  if (dtype != TWL_F16 && dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (token_budget == 0 || max_pages_per_req == 0 || max_pages_per_req > 8192) return TWL_EINVAL;
  uint64_t k = (token_budget / TWL_PAGE ? token_budget / TWL_PAGE : 1) +
               (token_budget % TWL_PAGE ? 1 : 0);
  if (k > max_pages_per_req) k = max_pages_per_req;
  if (k * TWL_PAGE > TWL_MAX_CANDIDATES) return TWL_EINVAL;
  if (sel_stride < k || k * TWL_PAGE > idx_stride) return TWL_EINVAL;
  if (scores_out && k * TWL_PAGE > score_stride) return TWL_EINVAL;
  if (page_scores_out && page_score_stride < max_pages_per_req) return TWL_EINVAL;
  if (high_mode != TWL_HIGH_FIRST && high_mode != TWL_HIGH_MAX) return TWL_EINVAL;
  if (!p_arr && !(p > 0.0f && p <= 1.0f)) return TWL_EINVAL;
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k_int4) & 15u) || (((uintptr_t)meta) & 15u) ||
      (((uintptr_t)scores_out) & 3u) || (((uintptr_t)page_scores_out) & 3u) ||
      (((uintptr_t)meta_planes) & 15u))
    return TWL_EALIGN;
  if (meta_planes && (plane_cap_pages < max_pages_per_req || (plane_cap_pages & 7u)))
    return TWL_EINVAL;
  if (meta_planes && plane_slots && plane_num_slots == 0) return TWL_EINVAL;
  twl::RowArgs a{};
  a.f.q = q; a.f.k_int4 = (const uint8_t*)k_int4; a.f.sel_stride = sel_stride;
  a.f.kv_page_indices = kv_page_indices; a.f.kv_page_indptr = kv_page_indptr;
  a.f.kv_last_page_len = kv_last_page_len; a.f.num_q_heads = num_q_heads;
  a.f.num_kv_heads = num_kv_heads; a.f.max_pages = (uint32_t)k; a.f.sm_scale = sm_scale;
  a.f.p_arr = p_arr; a.f.p = p; a.f.high_mode = high_mode; a.f.idx = idx;
  a.f.idx_stride = idx_stride; a.f.count = count; a.f.scores_out = scores_out;
  a.f.score_stride = score_stride; a.f.cand_count = cand_count; a.f.surv_probs = surv_probs;
  a.meta = (const uint8_t*)meta; a.token_budget = token_budget;
  a.max_pages_req = max_pages_per_req; a.sel_pages_out = sel_pages; a.sel_count_out = sel_count;
  a.page_scores_out = page_scores_out; a.page_score_stride = page_score_stride;
  a.planes = (const uint16_t*)meta_planes; a.plane_cap = plane_cap_pages;
  a.plane_slots = plane_slots; a.plane_num_slots = plane_num_slots;
  const uint32_t rows = batch * num_q_heads;
  hipStream_t s = (hipStream_t)stream;
  // page scores per thread of the selection: 2 up to 2048 pages (32k tokens), 4 up to 4096, else 8
  const int vpt = max_pages_per_req <= 2048 ? 2 : (max_pages_per_req <= 4096 ? 4 : 8);
#define TWL_ROW_LAUNCH(DT)                                              \
  do {                                                                  \
    if (meta_planes) {                                                  \
      if (vpt == 2) twl::launch_row<DT, 2, true>(a, rows, s);           \
      else if (vpt == 4) twl::launch_row<DT, 4, true>(a, rows, s);      \
      else twl::launch_row<DT, 8, true>(a, rows, s);                    \
    } else {                                                            \
      if (vpt == 2) twl::launch_row<DT, 2, false>(a, rows, s);          \
      else if (vpt == 4) twl::launch_row<DT, 4, false>(a, rows, s);     \
      else twl::launch_row<DT, 8, false>(a, rows, s);                   \
    }                                                                   \
  } while (0)
  if (dtype == TWL_F16) TWL_ROW_LAUNCH(TWL_F16);
  else TWL_ROW_LAUNCH(TWL_BF16);
#undef TWL_ROW_LAUNCH
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_select_estimate_prune(
    const void* q, int dtype, const void* meta, const void* k_int4, const int32_t* kv_page_indices,
    const int32_t* kv_page_indptr, const int32_t* kv_last_page_len, uint32_t batch,
    uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t token_budget,
    uint32_t max_pages_per_req, float sm_scale, const float* p_arr, float p, int high_mode,
    int32_t* sel_pages, uint32_t sel_stride, int32_t* sel_count, int32_t* idx, uint32_t idx_stride,
    int32_t* count, float* page_scores_out, uint32_t page_score_stride, float* scores_out,
    uint32_t score_stride, int32_t* cand_count, const void* meta_planes,
    uint32_t plane_cap_pages, const int32_t* plane_slots, uint32_t plane_num_slots, void* stream) {
  return twl::select_estimate_prune_ex(
      q, dtype, meta, k_int4, kv_page_indices, kv_page_indptr, kv_last_page_len, batch, num_q_heads,
      num_kv_heads, token_budget, max_pages_per_req, sm_scale, p_arr, p, high_mode, sel_pages,
      sel_stride, sel_count, idx, idx_stride, count, page_scores_out, page_score_stride, scores_out,
      score_stride, cand_count, meta_planes, plane_cap_pages, plane_slots, plane_num_slots, nullptr,
      stream);
}
