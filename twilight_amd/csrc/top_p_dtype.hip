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
//     CUB's thread 0 does, by one wavefront per chunk;
//   - the block sums of successive chunks are added to the running sum in chunk order
//     (sampling.cuh:191-193).
// Minima, maxima and comparisons are exact in any order, so they are made on bit patterns with
// integer instructions. The row is read from HBM once and kept in registers (at most 32 values
// per thread); an iteration costs two barriers.
//
// A binary16 addition is the hardware's; a bfloat16 addition is an fp32 addition rounded to
// bfloat16 (fp32 carries 24 >= 2 * 8 + 2 significand bits, so the double rounding equals the
// single one). For float what remains is the order of the additions, which is what makes the
// float op reproduce the reference's masks row for row (the faster fp32 kernel of top_p.hip adds
// in another order and can differ where a sum meets p within rounding).
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

// The arithmetic of one element type. The kernel carries a probability as its key: the bit
// pattern of the value in its own type for binary16 (16 bits, zero-extended), the bit pattern of
// the equal float for bfloat16 and float. Keys of non-negative numbers order like the numbers, so
// comparisons and the minimum / maximum searches are integer operations; additions are made in
// T, where `add` rounds to the element type: natively for binary16 and float, as a float
// addition rounded to bfloat16 otherwise (24 >= 2 * 8 + 2 significand bits: the double rounding
// equals the single one). `box` / `unbox` carry a T through a 32-bit register or LDS word.
template <int DT>
struct DtNum {   // float and bfloat16
  using T = float;
  static constexpr uint32_t kInfKey = 0x7F800000u;
  static __device__ __forceinline__ uint32_t key(float f) { return as_u32(f); }
  static __device__ __forceinline__ float keyf(uint32_t k) { return as_f32(k); }
  static __device__ __forceinline__ T unbox(uint32_t k) { return as_f32(k); }
  static __device__ __forceinline__ uint32_t box(T v) { return as_u32(v); }
  static __device__ __forceinline__ T add(T a, T b) { return round_to<DT>(a + b); }
  static __device__ __forceinline__ float f32(T v) { return v; }
};
template <>
struct DtNum<TWL_F16> {
  using T = _Float16;
  static constexpr uint32_t kInfKey = 0x7C00u;
  static __device__ __forceinline__ uint32_t key(float f) { return f32_to_f16_bits(f); }
  static __device__ __forceinline__ float keyf(uint32_t k) { return f16_bits_to_f32(k); }
  static __device__ __forceinline__ T unbox(uint32_t k) {
    return __builtin_bit_cast(_Float16, (uint16_t)k);
  }
  static __device__ __forceinline__ uint32_t box(T v) {
    return (uint32_t)__builtin_bit_cast(uint16_t, v);
  }
  static __device__ __forceinline__ T add(T a, T b) { return a + b; }
  static __device__ __forceinline__ float f32(T v) { return (float)v; }
};

__device__ __forceinline__ uint32_t wave_min_u32_to_lane63(uint32_t v) {
  v = min(v, (uint32_t)dpp<kDppXor1>((int)0xFFFFFFFF, (int)v));
  v = min(v, (uint32_t)dpp<kDppXor2>((int)0xFFFFFFFF, (int)v));
  v = min(v, (uint32_t)dpp<kDppHalfMirror>((int)0xFFFFFFFF, (int)v));
  v = min(v, (uint32_t)dpp<kDppMirror>((int)0xFFFFFFFF, (int)v));
  v = min(v, (uint32_t)dpp<kDppBcast15, 0xA>((int)0xFFFFFFFF, (int)v));
  v = min(v, (uint32_t)dpp<kDppBcast31, 0xC>((int)0xFFFFFFFF, (int)v));
  return v;
}
// the smallest of the 16 per-wavefront keys in `slots`, in every lane
__device__ __forceinline__ uint32_t fold16_min_u32(const uint32_t* slots, int lane) {
  uint32_t t = slots[lane & (kCubWaves - 1)];
  t = min(t, (uint32_t)dpp<kDppXor1>((int)0xFFFFFFFF, (int)t));
  t = min(t, (uint32_t)dpp<kDppXor2>((int)0xFFFFFFFF, (int)t));
  t = min(t, (uint32_t)dpp<kDppHalfMirror>((int)0xFFFFFFFF, (int)t));
  t = min(t, (uint32_t)dpp<kDppMirror>((int)0xFFFFFFFF, (int)t));
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)t);
}

template <int DT, int VEC>
__global__ __launch_bounds__(kCubThreads) void top_p_dtype_kernel(TopPDtArgs a) {
  using N = DtNum<DT>;
  using T = typename N::T;
  constexpr int MAXC = kCubMaxVals / VEC;
  __shared__ __align__(16) uint32_t wagg[MAXC][kCubWarps];   // warp aggregates of a chunk, boxed
  __shared__ uint32_t cagg[MAXC];                            // block aggregate of a chunk, boxed
  __shared__ uint32_t wkey[kCubWaves], wkey0[kCubWaves];
  __shared__ uint32_t first_key;
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
  uint32_t xk[MAXC][VEC];
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
      xk[c][j] = (raw[j] > 0.0f) ? N::key(raw[j]) : 0u;   // negative, -0 and NaN count as 0
  }

  // ---- bounds (sampling.cuh:156-162) ----------------------------------------------------------
  // A = min{x > low} and B = max{x <= high} as keys, without the reference's caps (it starts the
  // two searches from `high` and `low`, sampling.cuh:174-175; the caps are applied where the
  // values are used). One search pattern serves both:
  //   k = x - c   (c = key(low) + 1)   smallest k -> A = c + k
  //   k = c - x   (c = key(high))      smallest k -> B = c - k
  // in wrapping unsigned arithmetic, where elements on the wrong side of the bound wrap to
  // k >= 2^31. A only moves when `low` moves and B only when `high` moves, so an iteration runs
  // the search for whichever bound the iteration before it changed. Zeros past the end of the
  // row never enter either result: they are not above `low`, and a B of 0 is capped by `low`.
  const float p = round_to<DT>(a.p_arr ? a.p_arr[row] : a.p);
  const float eps = round_to<DT>(1e-5f);
  float low = 0.0f, high;
  uint32_t A_key = N::kInfKey, B_key = 0u;
  auto min_search = [&](uint32_t c, bool below) -> uint32_t {   // `below` is uniform
    uint32_t kmin = 0xFFFFFFFFu;
    if (__builtin_amdgcn_readfirstlane((int)below)) {
#pragma unroll
      for (int cc = 0; cc < MAXC; ++cc)
        if (cc < nchunks) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) kmin = min(kmin, c - xk[cc][j]);
        }
    } else {
#pragma unroll
      for (int cc = 0; cc < MAXC; ++cc)
        if (cc < nchunks) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) kmin = min(kmin, xk[cc][j] - c);
        }
    }
    return wave_min_u32_to_lane63(kmin);
  };
  if (a.high_mode == TWL_HIGH_FIRST) {
    if (tx == 0) first_key = xk[0][0];
    __syncthreads();
    const uint32_t c = first_key;
    high = N::keyf(c);
    const uint32_t k = min_search(c, true);
    if (lane == kWave - 1) wkey0[wave] = k;
    __syncthreads();
    const uint32_t kk = fold16_min_u32(wkey0, lane);
    B_key = (kk < 0x80000000u) ? c - kk : 0u;
  } else {
    // the row's maximum: the largest key below infinity's successor
    const uint32_t c = N::kInfKey;
    const uint32_t k = min_search(c, true);
    if (lane == kWave - 1) wkey0[wave] = k;
    __syncthreads();
    const uint32_t kk = fold16_min_u32(wkey0, lane);
    B_key = (kk < 0x80000000u) ? c - kk : 0u;
    high = N::keyf(B_key);
  }

  // ---- bisection (sampling.cuh:171-217) -------------------------------------------------------
  // Two barriers per iteration: warp aggregates and the wavefronts' search keys meet in LDS at the
  // first; then ONE wavefront per chunk adds the chunk's 32 warp aggregates one after the other,
  // warp 0 first (CUB's thread 0), while every wavefront folds the keys; the chunk aggregates
  // meet at the second.
  int iters = 0;
  bool sel_a = true;
  bool more;
  do {
    const float mid = round_to<DT>(round_to<DT>(low + high) * 0.5f);   // :173
    const uint32_t midk = N::key(mid);
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      if (c < nchunks) {
        T acc = N::unbox(0u);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const T g = N::unbox((xk[c][j] > midk) ? xk[c][j] : 0u);     // :183
          acc = (j == 0) ? g : N::add(acc, g);                          // cub::ThreadReduce
        }
        // a CUDA warp's shuffle-down tree, as far as its lane 0 sees it
        acc = N::add(acc, N::unbox((uint32_t)dpp<kDppRowShl1>(0, (int)N::box(acc))));
        acc = N::add(acc, N::unbox((uint32_t)dpp<kDppRowShl2>(0, (int)N::box(acc))));
        acc = N::add(acc, N::unbox((uint32_t)dpp<kDppRowShl4>(0, (int)N::box(acc))));
        acc = N::add(acc, N::unbox((uint32_t)dpp<kDppRowShl8>(0, (int)N::box(acc))));
        const int ab = (int)N::box(acc);
        const T r0 = N::unbox((uint32_t)__builtin_amdgcn_readlane(ab, 0));
        const T r1 = N::unbox((uint32_t)__builtin_amdgcn_readlane(ab, 16));
        const T r2 = N::unbox((uint32_t)__builtin_amdgcn_readlane(ab, 32));
        const T r3 = N::unbox((uint32_t)__builtin_amdgcn_readlane(ab, 48));
        if (lane == 0) {
          wagg[c][2 * wave] = N::box(N::add(r0, r1));
          wagg[c][2 * wave + 1] = N::box(N::add(r2, r3));
        }
      }
    }
    const uint32_t sc = sel_a ? N::key(low) + 1u : N::key(high);        // :184-189
    const uint32_t wk = min_search(sc, !sel_a);
    if (lane == kWave - 1) wkey[wave] = wk;
    __syncthreads();
    for (int c = wave; c < nchunks; c += kCubWaves) {
      const u32x4* pv = (const u32x4*)&wagg[c][0];
      uint32_t wv[kCubWarps];
#pragma unroll
      for (int i = 0; i < kCubWarps / 4; ++i) {
        const u32x4 v = pv[i];
        wv[4 * i] = v.x; wv[4 * i + 1] = v.y; wv[4 * i + 2] = v.z; wv[4 * i + 3] = v.w;
      }
      T agg = N::unbox(wv[0]);
#pragma unroll
      for (int w = 1; w < kCubWarps; ++w) agg = N::add(agg, N::unbox(wv[w]));
      if (lane == 0) cagg[c] = N::box(agg);
    }
    const uint32_t kmin = fold16_min_u32(wkey, lane);
    __syncthreads();
    T total = N::unbox(cagg[0]);                                        // threadlocal_sum, :172
    for (int c = 1; c < nchunks; ++c) total = N::add(total, N::unbox(cagg[c]));   // :191-193
    const bool found = kmin < 0x80000000u;
    if (sel_a) A_key = found ? sc + kmin : N::kInfKey;
    else B_key = found ? sc - kmin : 0u;
    const float min_gt_low = fminf(high, N::keyf(A_key));               // :174,184-186
    const float max_le_high = fmaxf(low, N::keyf(B_key));               // :175,187-189
    const bool accept = N::f32(total) >= p;                             // :211-216
    low = accept ? mid : low;
    high = accept ? high : fminf(mid, max_le_high);
    sel_a = accept;
    ++iters;
    more = round_to<DT>(max_le_high - min_gt_low) > eps && iters < 4096;  // :217
  } while (more);
  const uint32_t lowk = N::key(low);

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
              w |= (xk[c][(j0 + j) % VEC] > lowk ? 1u : 0u) << (8 * j);
            *(uint32_t*)(dst + e0 + j0) = w;
          }
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) dst[e0 + j] = (xk[c][j] > lowk) ? 1 : 0;
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
      for (int j = 0; j < VEC; ++j) keep[c] |= (valid[c] && xk[c][j] > lowk) ? (1u << j) : 0u;
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
