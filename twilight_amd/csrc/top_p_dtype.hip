// Top-p mask kernel in the arithmetic of the probabilities' own type: TopPReturnMaskKernel<1024,
// BLOCK_REDUCE_WARP_REDUCTIONS, VEC, DType> (csrc/include/sampling.cuh:119-231) as instantiated for
// half and nv_bfloat16 (csrc/src/sampling.cu:22-43) and for float (csrc/src/sampling.cu:45-63),
// with the arithmetic and the order of additions each instantiation has. The 16-bit case:
//
// There p, low, high, mid, the tolerance 1e-5, the bracket width and EVERY partial sum are values
// of the 16-bit type, each addition rounding to nearest even. A sum of thousands of 16-bit
// numbers depends on the order of the additions, so the kernel below adds in the order CUB's
// block reduction does (cub::BlockReduce with BLOCK_REDUCE_WARP_REDUCTIONS, sampling.cuh:54):
//   - a workgroup has the reference's 1024 threads; thread t owns, in chunk i, the
//     VEC = gcd(16 / sizeof(DType), d) elements from (i * 1024 + t) * VEC on
//     (sampling.cuh:176-181,239-243), zeros past the end of the row;
//   - a thread folds its VEC masked items left to right (cub::ThreadReduce);
//   - a CUDA warp is 32 consecutive threads = half a wavefront: its five shuffle-down steps
//     (offsets 1, 2, 4, 8, 16; lane l adds lane l + offset) are four row-shift DPP steps inside each
//     row of 16 lanes and one addition of the two row results. Only lane 0 of a warp is used by
//     CUB, and lane 0 of a row only ever needs lanes of its own row, so the lanes whose shifted
//     source falls outside the row may hold anything;
//   - the 32 warp results go through LDS and are added one after the other, warp 0 first, as
//     CUB's thread 0 does; every thread here repeats that chain so no second barrier is needed;
//   - the block sums of successive chunks are added to the running sum in chunk order
//     (sampling.cuh:191-193).
// Minima, maxima and comparisons are exact in any order. The row is read from HBM once and kept
// in registers (at most 32 values per thread); an iteration costs one barrier.
//
// A 16-bit addition is computed as an fp32 addition rounded to the 16-bit type: fp32 carries
// 24 >= 2 * 11 + 2 significand bits, so the double rounding equals the single one. For float the
// rounding step is the identity and what remains is the order of the additions, which is what
// makes the float op reproduce the reference's masks row for row (the faster fp32 kernel of
// top_p.hip adds in another order and can differ where a sum meets p within rounding).
#include "twl_common.h"

namespace twl {

struct TopPDtArgs {
  const void* probs;       // [rows, d] of the kernel's element type
  uint32_t d;
  const float* p_arr;      // nullable
  float p;
  int high_mode;
  uint8_t* mask;           // nullable [rows, d]
  int32_t* idx;            // nullable [rows, idx_stride]
  uint32_t idx_stride;
  int32_t* count;          // nullable [rows]
  float* low_out;          // nullable [rows]
  int32_t* iters_out;      // nullable [rows]
};

constexpr int kCubThreads = 1024;              // BLOCK_THREADS of the reference's launcher
constexpr int kCubWaves = kCubThreads / kWave;  // 16 wavefronts
constexpr int kCubWarps = kCubThreads / 32;     // 32 CUDA warps
constexpr int kCubMaxVals = TWL_MAX_CANDIDATES / kCubThreads;  // 32 values per thread

constexpr int kDppRowShl1 = 0x101, kDppRowShl2 = 0x102, kDppRowShl4 = 0x104, kDppRowShl8 = 0x108;

template <int DT>
__device__ __forceinline__ float dt_add(float a, float b) {
  return round_to<DT>(a + b);
}

template <int DT, int VEC>
__global__ __launch_bounds__(kCubThreads) void top_p_dtype_kernel(TopPDtArgs a) {
  constexpr int MAXC = kCubMaxVals / VEC;
  __shared__ float wagg[2][MAXC][kCubWarps];
  __shared__ float wmin[2][kCubWaves], wmax[2][kCubWaves];
  __shared__ float first_val;
  __shared__ int chunk_tot[MAXC][kCubWaves];

  const uint32_t row = blockIdx.x;
  const int tx = threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tx / kWave);
  const uint32_t d = a.d;
  const int nchunks = (int)((d + kCubThreads * VEC - 1) / (kCubThreads * VEC));  // <= MAXC

  // ---- the row, once (VEC divides d, so a thread's VEC elements are all inside or all outside)
  constexpr uint32_t ESZ = (DT == TWL_F32) ? 4u : 2u;
  const uint8_t* src = (const uint8_t*)a.probs + (size_t)row * d * ESZ;
  const bool vec_ok = ((((uintptr_t)src) & (ESZ * VEC - 1u)) == 0);
  float x[MAXC][VEC];
  bool valid[MAXC];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const uint32_t e0 = ((uint32_t)c * kCubThreads + (uint32_t)tx) * VEC;
    valid[c] = c < nchunks && e0 < d;
    float raw[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) raw[j] = 0.0f;
    if (valid[c]) {
      if constexpr (DT == TWL_F32) {
        const float* s32 = (const float*)src;
        if (VEC == 4 && vec_ok) {
          const f32x4 v = *(const f32x4*)(s32 + e0);
          const float w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int j = 0; j < VEC; ++j) raw[j] = w[j % 4];
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) raw[j] = s32[e0 + j];
        }
      } else {
        const uint16_t* s16 = (const uint16_t*)src;
        uint32_t bits[VEC];
        if (VEC == 8 && vec_ok) {
          const u32x4 v = *(const u32x4*)(s16 + e0);
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int j = 0; j < VEC; ++j) bits[j] = (w[(j / 2) % 4] >> (16 * (j & 1))) & 0xFFFFu;
        } else if (VEC == 4 && vec_ok) {
          const u32x2 v = *(const u32x2*)(s16 + e0);
          const uint32_t w[2] = {v.x, v.y};
#pragma unroll
          for (int j = 0; j < VEC; ++j) bits[j] = (w[(j / 2) % 2] >> (16 * (j & 1))) & 0xFFFFu;
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) bits[j] = s16[e0 + j];
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) raw[j] = bits16_to_f32<DT>(bits[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      x[c][j] = (raw[j] > 0.0f) ? raw[j] : 0.0f;   // probabilities; negative, -0 and NaN count as 0
  }

  // ---- bounds (sampling.cuh:156-162) ----------------------------------------------------------
  const float p = round_to<DT>(a.p_arr ? a.p_arr[row] : a.p);
  const float eps = round_to<DT>(1e-5f);
  float low = 0.0f, high;
  if (a.high_mode == TWL_HIGH_FIRST) {
    if (tx == 0) first_val = x[0][0];
    __syncthreads();
    high = first_val;
  } else {
    float m = 0.0f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c)
#pragma unroll
      for (int j = 0; j < VEC; ++j) m = fmaxf(m, x[c][j]);
    m = wave_allreduce<OpMax>(m);
    if (lane == 0) wmax[1][wave] = m;
    __syncthreads();
    high = 0.0f;
#pragma unroll
    for (int w = 0; w < kCubWaves; ++w) high = fmaxf(high, wmax[1][w]);
    // the loop's first iteration writes buffer 0; buffer 1 is written again only after the
    // barrier of that iteration, which every wave reaches after these reads
  }

  // ---- bisection (sampling.cuh:171-217) -------------------------------------------------------
  int iters = 0, buf = 0;
  bool more;
  do {
    const float mid = round_to<DT>(round_to<DT>(low + high) * 0.5f);   // :173
    float mn = high, mx = low;                                          // :174-175
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nchunks) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float v = x[c][j];
          const float g = (v > mid) ? v : 0.0f;                         // :183
          acc = (j == 0) ? g : dt_add<DT>(acc, g);                      // cub::ThreadReduce
          if (valid[c]) {
            if (v > low) mn = fminf(mn, v);                             // :184-186
            if (v <= high) mx = fmaxf(mx, v);                           // :187-189
          }
        }
        // a CUDA warp's shuffle-down tree, as far as its lane 0 sees it
        acc = dt_add<DT>(acc, dpp<kDppRowShl1>(0.0f, acc));
        acc = dt_add<DT>(acc, dpp<kDppRowShl2>(0.0f, acc));
        acc = dt_add<DT>(acc, dpp<kDppRowShl4>(0.0f, acc));
        acc = dt_add<DT>(acc, dpp<kDppRowShl8>(0.0f, acc));
        const float r0 = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 0));
        const float r1 = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 16));
        const float r2 = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 32));
        const float r3 = as_f32(__builtin_amdgcn_readlane(as_i32(acc), 48));
        if (lane == 0) {
          wagg[buf][c][2 * wave] = dt_add<DT>(r0, r1);
          wagg[buf][c][2 * wave + 1] = dt_add<DT>(r2, r3);
        }
      }
    }
    mn = wave_allreduce<OpMin>(mn);
    mx = wave_allreduce<OpMax>(mx);
    if (lane == 0) {
      wmin[buf][wave] = mn;
      wmax[buf][wave] = mx;
    }
    __syncthreads();
    float total = 0.0f;                                                 // threadlocal_sum, :172
    for (int c = 0; c < nchunks; ++c) {
      float agg = wagg[buf][c][0];                                      // thread 0 of CUB's block
#pragma unroll
      for (int w = 1; w < kCubWarps; ++w) agg = dt_add<DT>(agg, wagg[buf][c][w]);
      total = dt_add<DT>(total, agg);                                   // :191-193
    }
    float min_gt_low = high, max_le_high = low;
#pragma unroll
    for (int w = 0; w < kCubWaves; ++w) {
      min_gt_low = fminf(min_gt_low, wmin[buf][w]);
      max_le_high = fmaxf(max_le_high, wmax[buf][w]);
    }
    if (total >= p) {                                                   // :211-216
      low = mid;
    } else {
      high = fminf(mid, max_le_high);
    }
    ++iters;
    more = round_to<DT>(max_le_high - min_gt_low) > eps && iters < 4096;  // :217
    buf ^= 1;
  } while (more);

  if (tx == 0) {
    if (a.low_out) a.low_out[row] = low;
    if (a.iters_out) a.iters_out[row] = iters;
  }

  // ---- mask (sampling.cuh:219-230) --------------------------------------------------------------
  if (a.mask) {
    uint8_t* dst = a.mask + (size_t)row * d;
    const bool st_ok = VEC >= 4 && ((((uintptr_t)dst) & 3u) == 0);
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (valid[c]) {
        const uint32_t e0 = ((uint32_t)c * kCubThreads + (uint32_t)tx) * VEC;
        if (st_ok) {
#pragma unroll
          for (int j0 = 0; j0 < VEC; j0 += 4) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j)
              w |= (x[c][(j0 + j) % VEC] > low ? 1u : 0u) << (8 * j);
            *(uint32_t*)(dst + e0 + j0) = w;
          }
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) dst[e0 + j] = (x[c][j] > low) ? 1 : 0;
        }
      }
    }
  }

  // ---- ordered index list (the stream compaction of twilight/pyimpl/attention.py:280-281) ------
  if (a.idx || a.count) {
    int32_t* dst = a.idx ? a.idx + (size_t)row * a.idx_stride : nullptr;
    uint32_t keep[MAXC];
    int excl[MAXC];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      keep[c] = 0;
#pragma unroll
      for (int j = 0; j < VEC; ++j) keep[c] |= (valid[c] && x[c][j] > low) ? (1u << j) : 0u;
      const int mine = __builtin_popcount(keep[c]);
      const int scan = wave_inclusive_scan(mine);
      excl[c] = scan - mine;
      if (lane == kWave - 1) chunk_tot[c][wave] = scan;
    }
    __syncthreads();
    int base = 0;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nchunks) {
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kCubWaves; ++w) {
          const int t = chunk_tot[c][w];
          before += (w < wave) ? t : 0;
          total += t;
        }
        if (dst && keep[c]) {
          int pos = base + before + excl[c];
          const uint32_t e0 = ((uint32_t)c * kCubThreads + (uint32_t)tx) * VEC;
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            if (keep[c] & (1u << j)) dst[pos++] = (int)(e0 + j);
        }
        base += total;
      }
    }
    if (tx == 0 && a.count) a.count[row] = base;
  }
}

template <int DT>
static int launch_top_p_dtype(const TopPDtArgs& a, uint32_t rows, hipStream_t s) {
  const dim3 grid(rows), block(kCubThreads);
  // VEC_SIZE = gcd(16 / sizeof(DType), d), sampling.cuh:239
  if constexpr (DT != TWL_F32) {
    if (a.d % 8 == 0) {
      hipLaunchKernelGGL((top_p_dtype_kernel<DT, 8>), grid, block, 0, s, a);
      return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
    }
  }
  if (a.d % 4 == 0) hipLaunchKernelGGL((top_p_dtype_kernel<DT, 4>), grid, block, 0, s, a);
  else if (a.d % 2 == 0) hipLaunchKernelGGL((top_p_dtype_kernel<DT, 2>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((top_p_dtype_kernel<DT, 1>), grid, block, 0, s, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

}  // namespace twl

static int check_top_p_dtype(const void* probs, const uint8_t* mask, const int32_t* idx,
                             const int32_t* count, const float* p_arr, float p, uint32_t rows,
                             uint32_t d, uint32_t idx_stride, int high_mode) {
  if (!probs) return TWL_ENULL;
  if (!mask && !idx && !count) return TWL_ENULL;
  if (idx && !count) return TWL_ENULL;
  if (rows == 0 || d == 0 || d > TWL_MAX_CANDIDATES) return TWL_EINVAL;
  if (idx && idx_stride < d) return TWL_EINVAL;
  if (high_mode != TWL_HIGH_FIRST && high_mode != TWL_HIGH_MAX) return TWL_EINVAL;
  if (!p_arr && p != p) return TWL_EINVAL;   // any p the reference takes; see twl_top_p_f32
  return TWL_OK;
}

extern "C" int twl_top_p_f16(const void* probs, int dtype, uint8_t* mask, int32_t* idx,
                             int32_t* count, const float* p_arr, float p, uint32_t rows,
                             uint32_t d, uint32_t idx_stride, int high_mode, float* low_out,
                             int32_t* iters_out, void* stream) {
  const int rc = check_top_p_dtype(probs, mask, idx, count, p_arr, p, rows, d, idx_stride, high_mode);
  if (rc != TWL_OK) return rc;
  if (dtype != TWL_F16 && dtype != TWL_BF16) return TWL_EDTYPE;
  if (((uintptr_t)probs) & 1u) return TWL_EALIGN;
  twl::TopPDtArgs a{};
  a.probs = probs; a.d = d; a.p_arr = p_arr; a.p = p; a.high_mode = high_mode;
  a.mask = mask; a.idx = idx; a.idx_stride = idx_stride; a.count = count; a.low_out = low_out;
  a.iters_out = iters_out;
  if (dtype == TWL_F16) return twl::launch_top_p_dtype<TWL_F16>(a, rows, (hipStream_t)stream);
  return twl::launch_top_p_dtype<TWL_BF16>(a, rows, (hipStream_t)stream);
}

// The float instantiation of the same kernel (csrc/src/sampling.cu:45-63): fp32 arithmetic with the
// additions in cub::BlockReduce's order, VEC = gcd(4, d).
extern "C" int twl_top_p_f32_exact(const float* probs, uint8_t* mask, int32_t* idx, int32_t* count,
                                   const float* p_arr, float p, uint32_t rows, uint32_t d,
                                   uint32_t idx_stride, int high_mode, float* low_out,
                                   int32_t* iters_out, void* stream) {
  const int rc = check_top_p_dtype(probs, mask, idx, count, p_arr, p, rows, d, idx_stride, high_mode);
  if (rc != TWL_OK) return rc;
  if (((uintptr_t)probs) & 3u) return TWL_EALIGN;
  twl::TopPDtArgs a{};
  a.probs = probs; a.d = d; a.p_arr = p_arr; a.p = p; a.high_mode = high_mode;
  a.mask = mask; a.idx = idx; a.idx_stride = idx_stride; a.count = count; a.low_out = low_out;
  a.iters_out = iters_out;
  return twl::launch_top_p_dtype<TWL_F32>(a, rows, (hipStream_t)stream);
}
