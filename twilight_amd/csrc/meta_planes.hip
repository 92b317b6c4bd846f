// Quest metadata in plane layout, for the selector's scoring pass.
//
// The page score of twilight/pyimpl/quest.py:37-84 in its min/max form is
//     score(page) = sum_d q_d * (q_d > 0 ? max_d(page) : min_d(page)),
// so for a given query only ONE of the two numbers kept per (page, channel) is ever read. The
// 512-byte record layout (min and max of 4 channels side by side, records indexed by physical
// page) forces both through memory. The plane layout stores, per (request slot, kv head, channel),
// the minima of all pages of the request contiguously and the maxima contiguously,
//     planes[slot][kv_head][d][0 = min, 1 = max][logical page],   16-bit values, `cap` pages,
// so a row of the decode batch streams 128 runs of `pages` values — the min run or the max run of
// each channel, chosen by the sign of q_d — and touches half the bytes. Planes are indexed by
// LOGICAL page of a request slot (slot = position in the batch), not by physical page: they are a
// per-request side buffer next to the paged K / V, updated by twl_kv_append. The slot of a request is its position in the batch, or, with a slot
// table (plane_slots), any slot of the buffer: then a batch whose composition changes keeps the
// planes of its requests where they are.
#include "twl_common.h"

namespace twl {

struct PlanesArgs {
  const uint8_t* meta;   // records [pages, kv_heads, 512]
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  uint32_t num_kv_heads;
  uint16_t* planes;
  uint32_t cap;          // pages per run
  const int32_t* slots;  // nullable: slot of each batch position
  uint32_t num_slots;
};

constexpr int kPlTile = 64;  // pages per workgroup

// Records -> planes for the pages of the current page table. One workgroup per (64 logical pages,
// kv head, request): the records go through LDS and leave as 128-byte runs per (channel, plane).
__global__ __launch_bounds__(256) void meta_planes_build_kernel(PlanesArgs a) {
  __shared__ uint16_t tile[kPlTile][256 + 2];  // +2: rows fall on different banks
  const uint32_t b = blockIdx.z, kvh = blockIdx.y;
  const int p0 = blockIdx.x * kPlTile;
  const int pg_begin = a.kv_page_indptr[b];
  const int n_pages = min(a.kv_page_indptr[b + 1] - pg_begin, (int)a.cap);
  if (p0 >= n_pages) return;  // uniform
  const int np = min(kPlTile, n_pages - p0);
  const int tx = threadIdx.x;
  // 64 records x 512 B = 2048 16-byte pieces, 8 per thread
  for (int i = tx; i < np * 32; i += 256) {
    const int pg = i >> 5, piece = i & 31;
    const int phys = a.kv_page_indices[pg_begin + p0 + pg];
    const u32x4 v = *(const u32x4*)(a.meta + ((size_t)phys * a.num_kv_heads + kvh) *
                                                 TWL_META_RECORD_BYTES + 16 * piece);
    uint32_t* dst = (uint32_t*)&tile[pg][8 * piece];
    dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
  }
  __syncthreads();
  const int lane = tx & 63, wave = tx >> 6;
  const uint32_t slot = plane_slot(a.slots, a.num_slots, b);
  uint16_t* out = a.planes + ((size_t)slot * a.num_kv_heads + kvh) * (TWL_HEAD_DIM * 2) * a.cap;
  // run r = d * 2 + plane; record element of (d, plane) = (d / 4) * 8 + plane * 4 + d % 4
  for (int r = wave; r < TWL_HEAD_DIM * 2; r += 4) {
    const int d = r >> 1, plane = r & 1;
    const int col = (d >> 2) * 8 + plane * 4 + (d & 3);
    if (lane < np) out[(size_t)r * a.cap + p0 + lane] = tile[lane][col];
  }
}

}  // namespace twl

extern "C" int twl_meta_planes_build(const void* meta, const int32_t* kv_page_indices,
                                     const int32_t* kv_page_indptr, uint32_t batch,
                                     uint32_t num_kv_heads, uint32_t max_pages_per_req,
                                     void* planes, uint32_t plane_cap_pages,
                                     const int32_t* plane_slots, uint32_t plane_num_slots,
                                     void* stream) {
  if (!meta || !kv_page_indices || !kv_page_indptr || !planes) return TWL_ENULL;
  if (batch == 0 || num_kv_heads == 0 || max_pages_per_req == 0) return TWL_EINVAL;
  if (plane_cap_pages == 0 || (plane_cap_pages & 7u) || max_pages_per_req > plane_cap_pages)
    return TWL_EINVAL;
  if (batch > 65535u || num_kv_heads > 65535u) return TWL_EINVAL;
  if (plane_slots && plane_num_slots == 0) return TWL_EINVAL;
  if ((((uintptr_t)meta) & 15u) || (((uintptr_t)planes) & 15u)) return TWL_EALIGN;
  twl::PlanesArgs a{};
  a.meta = (const uint8_t*)meta; a.kv_page_indices = kv_page_indices;
  a.kv_page_indptr = kv_page_indptr; a.num_kv_heads = num_kv_heads;
  a.planes = (uint16_t*)planes; a.cap = plane_cap_pages;
  a.slots = plane_slots; a.num_slots = plane_num_slots;
  const dim3 grid((max_pages_per_req + twl::kPlTile - 1) / twl::kPlTile, num_kv_heads, batch);
  hipLaunchKernelGGL(twl::meta_planes_build_kernel, grid, dim3(256), 0, (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

namespace twl {

struct PlaneScoreArgs {
  const void* q;
  const uint16_t* planes;
  uint32_t cap;
  const int32_t* slots;  // nullable: slot of each batch position
  uint32_t num_slots;
  const uint8_t* meta;             // records: a request's last page is scored from its record
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  uint32_t num_q_heads, num_kv_heads;
  uint32_t max_pages;
  float* page_scores;
  uint32_t score_stride;
};

constexpr int kPsThreads = 256;
constexpr int kPsPagesPerBlock = 2 * kPsThreads;  // 2 pages per lane

// Page scores of one (batch, q head) row from the plane layout: lane = 2 pages, the 128 channels
// in ascending order, per channel the run (min or max) that the sign of q_d selects. The same
// arithmetic as the scoring phase of select_estimate_prune_kernel, as a kernel of its own for the
// batch sizes where the stages run as separate launches. UNROLL = loads a lane keeps in flight: 64
// where the launch has few wavefronts per SIMD (measured 9.7 -> 6.6 us at 32 rows x 2048 pages),
// 32 otherwise.
template <int DT, int UNROLL>
__global__ __launch_bounds__(kPsThreads) void quest_score_planes_kernel(PlaneScoreArgs a) {
  const uint32_t row = blockIdx.y;
  const uint32_t b = row / a.num_q_heads;
  const uint32_t h = row - b * a.num_q_heads;
  const uint32_t kvh = h / (a.num_q_heads / a.num_kv_heads);
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int n_req = min(max(a.kv_page_indptr[b + 1] - a.kv_page_indptr[b], 0),
                        min((int)a.max_pages, (int)a.cap));
  const int w0 = blockIdx.x * kPsPagesPerBlock + wave * 128;
  const uint16_t* qrow = (const uint16_t*)a.q + (size_t)row * TWL_HEAD_DIM;
  float* po = a.page_scores + (size_t)row * a.score_stride;
  // pages from np on are scored from their records (plane_scored_pages), by the wavefronts of the
  // workgroup whose slice begins at np (np is a multiple of that slice whenever more than the
  // last page is left) or by the wavefront that owns the last page
  const int np = plane_scored_pages(n_req);
  if (n_req - np > 1) {
    if ((int)(blockIdx.x * kPsPagesPerBlock) == np) {   // workgroup-uniform
      constexpr int kWaves = kPsThreads / kWave;
      const uint32_t qw2 = *(const uint32_t*)(qrow + 2 * lane);
      const float q0 = bits16_to_f32<DT>(qw2 & 0xFFFFu), q1 = bits16_to_f32<DT>(qw2 >> 16);
      for (int first = np + wave; first < n_req; first += 8 * kWaves) {
        const int cnt = min((n_req - first + kWaves - 1) / kWaves, 8);
        RecordBatch8 rb;
        record_pages_load8(rb, a.meta + (size_t)kvh * TWL_META_RECORD_BYTES,
                           (size_t)a.num_kv_heads * TWL_META_RECORD_BYTES,
                           a.kv_page_indices + a.kv_page_indptr[b], first, kWaves, cnt);
        float sc[8];
        record_pages_fold8<DT>(rb, cnt, q0, q1, sc);
        if (lane == 0) {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (i < cnt) po[first + i * kWaves] = sc[i];
        }
      }
      return;
    }
  }
  if (w0 >= n_req || (n_req - np > 1 && w0 >= np)) return;
  const float q_lo = bits16_to_f32<DT>(qrow[lane]);
  const float q_hi = bits16_to_f32<DT>(qrow[64 + lane]);
  const uint32_t slot = plane_slot(a.slots, a.num_slots, b);
  const uint16_t* pl =
      a.planes + ((size_t)slot * a.num_kv_heads + kvh) * (TWL_HEAD_DIM * 2) * a.cap;
  const int pg0 = w0 + 2 * lane;
  const int pgc = min(pg0, (int)a.cap - 2);
  float s0 = 0.0f, s1 = 0.0f;
#pragma unroll UNROLL
  for (int d = 0; d < TWL_HEAD_DIM; ++d) {
    const float qd = as_f32(__builtin_amdgcn_readlane(as_i32(d < 64 ? q_lo : q_hi), d & 63));
    const int plane = qd > 0.0f ? 1 : 0;
    const uint32_t w = __builtin_nontemporal_load(
        (const uint32_t*)(pl + (size_t)(2 * d + plane) * a.cap + pgc));
    s0 = fmaf(qd, bits16_to_f32<DT>(w & 0xFFFFu), s0);
    s1 = fmaf(qd, bits16_to_f32<DT>(w >> 16), s1);
  }
  const int last_pg = n_req - 1;  // scored from its record, by the wavefront that owns it
  if (pg0 < np) po[pg0] = s0;
  if (pg0 + 1 < np) po[pg0 + 1] = s1;
  if (np == last_pg && last_pg >= w0 && last_pg < w0 + 128) {  // wave-uniform
    const uint32_t qw2 = *(const uint32_t*)(qrow + 2 * lane);
    const int phys = a.kv_page_indices[a.kv_page_indptr[b] + last_pg];
    const float s_last = record_page_score<DT>(
        a.meta + ((size_t)phys * a.num_kv_heads + kvh) * TWL_META_RECORD_BYTES,
        bits16_to_f32<DT>(qw2 & 0xFFFFu), bits16_to_f32<DT>(qw2 >> 16));
    if (lane == 0) po[last_pg] = s_last;
  }
}

}  // namespace twl

extern "C" int twl_quest_page_scores_planes(const void* q, int q_dtype, const void* meta_planes,
                                            uint32_t plane_cap_pages,
                                            const int32_t* plane_slots, uint32_t plane_num_slots,
                                            const void* meta, const int32_t* kv_page_indices,
                                            const int32_t* kv_page_indptr, uint32_t batch,
                                            uint32_t num_q_heads, uint32_t num_kv_heads,
                                            uint32_t max_pages_per_req, float* page_scores,
                                            uint32_t score_stride, void* stream) {
  if (!q || !meta_planes || !meta || !kv_page_indices || !kv_page_indptr || !page_scores)
    return TWL_ENULL;
  if (q_dtype != TWL_F16 && q_dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (max_pages_per_req == 0 || max_pages_per_req > 16384 || score_stride < max_pages_per_req)
    return TWL_EINVAL;
  if (plane_cap_pages < max_pages_per_req || (plane_cap_pages & 7u)) return TWL_EINVAL;
  if (plane_slots && plane_num_slots == 0) return TWL_EINVAL;
  if ((uint64_t)batch * num_q_heads > 65535u) return TWL_EINVAL;
  if ((((uintptr_t)q) & 3u) || (((uintptr_t)meta_planes) & 15u) || (((uintptr_t)meta) & 15u) ||
      (((uintptr_t)page_scores) & 3u))
    return TWL_EALIGN;
  twl::PlaneScoreArgs a{};
  a.q = q; a.planes = (const uint16_t*)meta_planes; a.cap = plane_cap_pages;
  a.slots = plane_slots; a.num_slots = plane_num_slots;
  a.meta = (const uint8_t*)meta; a.kv_page_indices = kv_page_indices;
  a.kv_page_indptr = kv_page_indptr; a.num_q_heads = num_q_heads; a.num_kv_heads = num_kv_heads;
  a.max_pages = max_pages_per_req; a.page_scores = page_scores; a.score_stride = score_stride;
  const dim3 grid((max_pages_per_req + twl::kPsPagesPerBlock - 1) / twl::kPsPagesPerBlock,
                  batch * num_q_heads);
  int cus = 256;
  (void)twl::device_cu_count(&cus);
  const bool few_waves = (uint64_t)grid.x * grid.y * (twl::kPsThreads / twl::kWave) <
                         16ull * (uint64_t)cus;
  const dim3 blk(twl::kPsThreads);
  hipStream_t st = (hipStream_t)stream;
  if (q_dtype == TWL_F16) {
    if (few_waves) hipLaunchKernelGGL((twl::quest_score_planes_kernel<TWL_F16, 64>), grid, blk, 0, st, a);
    else hipLaunchKernelGGL((twl::quest_score_planes_kernel<TWL_F16, 32>), grid, blk, 0, st, a);
  } else {
    if (few_waves) hipLaunchKernelGGL((twl::quest_score_planes_kernel<TWL_BF16, 64>), grid, blk, 0, st, a);
    else hipLaunchKernelGGL((twl::quest_score_planes_kernel<TWL_BF16, 32>), grid, blk, 0, st, a);
  }
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
