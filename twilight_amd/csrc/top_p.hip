// Top-p pruner: one workgroup per (batch, head) row, the row held in registers.
//
// Follows the bisection of csrc/include/sampling.cuh:156-231 iteration by iteration
// (low = 0, high = probs[row][0] or the row maximum; mid = (low+high)/2; S = sum of probs > mid;
// min_gt_low / max_le_high bracket; stop when the bracket is narrower than 1e-5; keep
// probs > low), but reads the row from HBM exactly once: every thread keeps VPT values in
// VGPRs, the three block reductions of an iteration are DPP wave reductions plus one LDS hop,
// and the result is emitted as a byte mask and/or as an ascending index list with its count
// (the stream compaction that replaces `mask & pruned_mask`, twilight/pyimpl/attention.py:280-281).
//
// The fused entry additionally computes the fp32 softmax of raw scores in the same registers
// (twilight/pyimpl/top_p.py:10-15), so scores are read once and probabilities never hit HBM.
//
// Cost model: an iteration is VPT compare/accumulate steps per thread plus one block reduction, and
// the reduction (wave DPP trees, an LDS hop, a barrier) is the expensive part, so the row is spread
// over few, fat threads (256-512 threads x up to 32 values), the loop is branch-free with its
// state in vector registers (no lane reads into scalar registers), and min{p > low} /
// max{p <= high} are found with one unsigned-integer search that runs only for the bound the
// previous iteration moved.
#include "top_p_core.h"

namespace twl {

struct TopPArgs {
  const void* in;        // fp32 probabilities or raw fp32 scores
  uint32_t in_stride;    // elements between rows
  const int32_t* lens;   // nullable: per-row length (<= d)
  uint32_t d;
  const float* p_arr;    // nullable
  float p;
  int high_mode;
  uint8_t* mask;         // nullable [rows, d]
  int32_t* idx;          // nullable [rows, idx_stride]
  uint32_t idx_stride;
  int32_t* count;        // nullable [rows]
  const int32_t* sel_pages;  // nullable: position -> token mapping through a page list
  uint32_t sel_stride;
  float* probs_out;      // nullable [rows, in_stride] (fused entry only)
  float* low_out;        // nullable [rows]
  int32_t* iters_out;    // nullable [rows]
  float* surv_probs;     // nullable [rows, idx_stride]: the value of survivor j beside idx
};

// Element e of the row is held by thread (e/4) % THREADS, slot 4*((e/4)/THREADS) + e%4:
// consecutive threads read consecutive 16-byte groups.
template <int DT, int THREADS, int VPT, bool FUSED_SOFTMAX>
__global__ __launch_bounds__(THREADS) void top_p_kernel(TopPArgs a) {
  constexpr int NWAVES = THREADS / kWave;
  constexpr int CHUNKS = VPT / 4;
  __shared__ float red[2][2][16];

  const uint32_t row = blockIdx.x;
  const int tx = threadIdx.x;
  const int lane = lane_id();
  const int wave = tx / kWave;
  const uint32_t len = a.lens ? min((uint32_t)max(a.lens[row], 0), a.d) : a.d;

  // ---- load the row once ----------------------------------------------------------------
  float x[VPT];
  const float fill = FUSED_SOFTMAX ? -__builtin_inff() : 0.0f;
  {
    static_assert(DT == TWL_F32, "16-bit probabilities have a kernel of their own (top_p_dtype.hip)");
    const float* src = (const float*)a.in + (size_t)row * a.in_stride;
    const bool vec_ok = ((((uintptr_t)src) & 15u) == 0);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const uint32_t e0 = 4u * (uint32_t)(tx + THREADS * c);
      if (vec_ok && e0 + 4 <= len) {
        f32x4 v = *(const f32x4*)(src + e0);
        x[4 * c + 0] = v.x; x[4 * c + 1] = v.y; x[4 * c + 2] = v.z; x[4 * c + 3] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) x[4 * c + j] = (e0 + j < len) ? src[e0 + j] : fill;
      }
    }
  }

  int buf = 0;
  // ---- softmax in registers (fused entry) -------------------------------------------------
  float max_prob = 0.0f;
  if (FUSED_SOFTMAX) {
    max_prob = softmax_regs<THREADS, VPT>(x, red, buf);
    if (a.probs_out) {
      float* dst = a.probs_out + (size_t)row * a.in_stride;
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) {
        const uint32_t e0 = 4u * (uint32_t)(tx + THREADS * c);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (e0 + j < len) dst[e0 + j] = x[4 * c + j];
      }
    }
  }

  // ---- bisection (sampling.cuh:156-217) ----------------------------------------------------
  const float p = round_to<DT>(a.p_arr ? a.p_arr[row] : a.p);
  float high;
  if (a.high_mode == TWL_HIGH_FIRST) {
    // element 0 lives in thread 0, slot 0. With a page list it stands for token 0 of the context
    // (what csrc/include/sampling.cuh:156-159 reads on its full-length row) only when logical
    // page 0 heads the ascending list; a token outside the list has probability 0 there.
    __shared__ float first;
    if (tx == 0) {
      const bool is_token0 = !a.sel_pages || a.sel_pages[(size_t)row * a.sel_stride] == 0;
      first = (len > 0 && is_token0) ? x[0] : 0.0f;
    }
    __syncthreads();
    high = first;
  } else if (FUSED_SOFTMAX) {
    high = max_prob;  // the row maximum, without another reduction
  } else {
    high = row_max_regs<THREADS, VPT>(x, red, buf);
  }
  int iters = 0;
  __shared__ BisectSmem bsm;
  const float low = bisect_regs<DT, THREADS, VPT>(x, p, high, red, buf, iters, bsm,
                                                 a.high_mode != TWL_HIGH_FIRST);

  if (tx == 0) {
    if (a.low_out) a.low_out[row] = low;
    if (a.iters_out) a.iters_out[row] = iters;
  }

  // ---- emit: mask and / or ordered index list ----------------------------------------------
  if (a.mask) {
    uint8_t* dst = a.mask + (size_t)row * a.d;
    const bool vec_ok = ((((uintptr_t)dst) & 3u) == 0);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const uint32_t e0 = 4u * (uint32_t)(tx + THREADS * c);
      if (vec_ok && e0 + 4 <= a.d) {
        uint32_t w = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) w |= (x[4 * c + j] > low ? 1u : 0u) << (8 * j);
        *(uint32_t*)(dst + e0) = w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (e0 + j < a.d) dst[e0 + j] = (x[4 * c + j] > low) ? 1 : 0;
      }
    }
  }
  if (a.idx || a.count) {
    int32_t* dst = a.idx ? a.idx + (size_t)row * a.idx_stride : nullptr;
    float* wdst = (a.idx && a.surv_probs) ? a.surv_probs + (size_t)row * a.idx_stride : nullptr;
    const int32_t* pages = a.sel_pages ? a.sel_pages + (size_t)row * a.sel_stride : nullptr;
    // every chunk's wave totals go to LDS first, so the whole emission needs one barrier
    __shared__ int chunk_tot[CHUNKS][16];
    int mine[CHUNKS], excl[CHUNKS];
    uint32_t keep[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      keep[c] = (x[4 * c + 0] > low ? 1u : 0u) | (x[4 * c + 1] > low ? 2u : 0u) |
                (x[4 * c + 2] > low ? 4u : 0u) | (x[4 * c + 3] > low ? 8u : 0u);
      mine[c] = __builtin_popcount(keep[c]);
      const int scan = wave_inclusive_scan(mine[c]);   // in lane order
      excl[c] = scan - mine[c];
      if (lane == kWave - 1) chunk_tot[c][wave] = scan;
    }
    if (NWAVES > 1) __syncthreads();
    int base = 0;  // survivors emitted by earlier chunks (uniform)
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const uint32_t e0 = 4u * (uint32_t)(tx + THREADS * c);
      int before = 0, total = 0;
#pragma unroll
      for (int w = 0; w < NWAVES; ++w) {
        const int t = chunk_tot[c][w];
        before += (w < wave) ? t : 0;
        total += t;
      }
      if (dst && mine[c]) {
        int pos = base + before + excl[c];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (keep[c] & (1u << j)) {
            const uint32_t e = e0 + j;
            if (wdst) wdst[pos] = x[4 * c + j];
            dst[pos++] = pages ? (pages[e >> 4] * TWL_PAGE + (int)(e & 15u)) : (int)e;
          }
        }
      }
      base += total;
    }
    if (tx == 0 && a.count) a.count[row] = base;
  }
}

template <int DT, bool FUSED>
static int launch_top_p(const TopPArgs& a, uint32_t rows, hipStream_t s) {
  const uint32_t d = a.d;
  if (d <= 1024) {
    hipLaunchKernelGGL((top_p_kernel<DT, 256, 4, FUSED>), dim3(rows), dim3(256), 0, s, a);
  } else if (d <= 2048) {
    hipLaunchKernelGGL((top_p_kernel<DT, 256, 8, FUSED>), dim3(rows), dim3(256), 0, s, a);
  } else if (d <= 4096) {
    hipLaunchKernelGGL((top_p_kernel<DT, 256, 16, FUSED>), dim3(rows), dim3(256), 0, s, a);
  } else if (d <= 8192) {
    hipLaunchKernelGGL((top_p_kernel<DT, 512, 16, FUSED>), dim3(rows), dim3(512), 0, s, a);
  } else if (d <= 16384) {
    hipLaunchKernelGGL((top_p_kernel<DT, 512, 32, FUSED>), dim3(rows), dim3(512), 0, s, a);
  } else {
    hipLaunchKernelGGL((top_p_kernel<DT, 1024, 32, FUSED>), dim3(rows), dim3(1024), 0, s, a);
  }
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

}  // namespace twl

using twl::TopPArgs;

// `any_p`: the drop-in mask entries take whatever p the reference takes (csrc/src/sampling.cu:22-63
// checks nothing: p >= 1 makes every comparison S >= p fail, so the search ends with low = 0 and
// every positive probability kept; p <= 0 makes every one succeed); only NaN is refused.
static int check_top_p_common(const void* in, uint8_t* mask, int32_t* idx, int32_t* count,
                              float p, const float* p_arr, uint32_t rows, uint32_t d,
                              uint32_t idx_stride, int high_mode, bool any_p = false) {
  if (!in) return TWL_ENULL;
  if (!mask && !idx && !count) return TWL_ENULL;
  if (idx && !count) return TWL_ENULL;
  if (rows == 0 || d == 0 || d > TWL_MAX_CANDIDATES) return TWL_EINVAL;
  if (idx && idx_stride < d) return TWL_EINVAL;
  if (high_mode != TWL_HIGH_FIRST && high_mode != TWL_HIGH_MAX) return TWL_EINVAL;
  if (!p_arr && (any_p ? (p != p) : !(p > 0.0f && p <= 1.0f))) return TWL_EINVAL;
  return TWL_OK;
}

extern "C" int twl_top_p_f32(const float* probs, uint8_t* mask, int32_t* idx, int32_t* count,
                             const float* p_arr, float p, uint32_t rows, uint32_t d,
                             uint32_t idx_stride, int high_mode, float* low_out,
                             int32_t* iters_out, void* stream) {
  int rc = check_top_p_common(probs, mask, idx, count, p, p_arr, rows, d, idx_stride, high_mode,
                              true);
  if (rc != TWL_OK) return rc;
  if (((uintptr_t)probs) & 3u) return TWL_EALIGN;
  TopPArgs a{};
  a.in = probs; a.in_stride = d; a.lens = nullptr; a.d = d; a.p_arr = p_arr; a.p = p;
  a.high_mode = high_mode; a.mask = mask; a.idx = idx; a.idx_stride = idx_stride; a.count = count;
  a.low_out = low_out; a.iters_out = iters_out;
  return twl::launch_top_p<TWL_F32, false>(a, rows, (hipStream_t)stream);
}

int twl::softmax_top_p_ex(const float* scores, uint32_t score_stride, const int32_t* lens,
                          uint32_t rows, uint32_t d, const float* p_arr, float p, int high_mode,
                          const int32_t* sel_pages, uint32_t sel_stride, int32_t* idx,
                          uint32_t idx_stride, int32_t* count, float* probs_out, float* low_out,
                          float* surv_probs, void* stream) {
  int rc = check_top_p_common(scores, nullptr, idx, count, p, p_arr, rows, d, idx_stride, high_mode);
  if (rc != TWL_OK) return rc;
  if (score_stride < d) return TWL_EINVAL;
  if (sel_pages && (uint64_t)sel_stride * TWL_PAGE < d) return TWL_EINVAL;
  if (((uintptr_t)scores) & 3u) return TWL_EALIGN;
  TopPArgs a{};
  a.in = scores; a.in_stride = score_stride; a.lens = lens; a.d = d; a.p_arr = p_arr; a.p = p;
  a.high_mode = high_mode; a.mask = nullptr; a.idx = idx; a.idx_stride = idx_stride;
  a.count = count; a.sel_pages = sel_pages; a.sel_stride = sel_stride; a.probs_out = probs_out;
  a.low_out = low_out; a.surv_probs = surv_probs;
  return twl::launch_top_p<TWL_F32, true>(a, rows, (hipStream_t)stream);
}

extern "C" int twl_softmax_top_p_f32(const float* scores, uint32_t score_stride,
                                     const int32_t* lens, uint32_t rows, uint32_t d,
                                     const float* p_arr, float p, int high_mode,
                                     const int32_t* sel_pages, uint32_t sel_stride, int32_t* idx,
                                     uint32_t idx_stride, int32_t* count, float* probs_out,
                                     float* low_out, void* stream) {
  return twl::softmax_top_p_ex(scores, score_stride, lens, rows, d, p_arr, p, high_mode, sel_pages,
                               sel_stride, idx, idx_stride, count, probs_out, low_out, nullptr,
                               stream);
}
