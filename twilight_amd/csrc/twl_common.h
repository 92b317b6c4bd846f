// Device-side helpers shared by the kernels of libtwilight_hip (gfx950, wave64 only).
#ifndef TWL_COMMON_H_
#define TWL_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/twilight_hip.h"

namespace twl {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

__device__ __forceinline__ float as_f32(int v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ float as_f32(uint32_t v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ int as_i32(float v) { return __builtin_bit_cast(int, v); }
__device__ __forceinline__ uint32_t as_u32(float v) { return __builtin_bit_cast(uint32_t, v); }

__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// ---- 16-bit float conversions (exact widenings; narrowing is round-to-nearest-even) ----------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return as_f32(b << 16); }
// round to nearest even by the hardware convert (v_cvt_pk_bf16_f32); a NaN stays a NaN
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}
template <int DT>
__device__ __forceinline__ float bits16_to_f32(uint32_t b) {
  return DT == TWL_F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
}
template <int DT>
__device__ __forceinline__ uint32_t f32_to_bits16(float f) {
  return DT == TWL_F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f);
}
// round a float to the value set of element type DT (TWL_F32: identity)
template <int DT>
__device__ __forceinline__ float round_to(float f) {
  if (DT == TWL_F16) return f16_bits_to_f32(f32_to_f16_bits(f));
  if (DT == TWL_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(f));
  return f;
}

// (x & m) | o in one VALU operation. The compiler splits the expression into v_and + v_or when
// both constants are literals (a three-operand instruction cannot carry a literal on this
// target), so the mask travels in a scalar register and `o` in a vector register.
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t m, uint32_t o) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(m), "v"(o));
  return r;
}

// A query value as the INT4 estimator's fp16 dot products take it. fp16 queries pass unchanged.
// A bf16 query is converted to fp16: exact for 2^-17 <= |q| <= 65504 (8 significand bits fit 11),
// rounded to a multiple of 2^-24 below that, and SATURATED to +-65504 above (so that a score can
// never become inf - inf = NaN; attention queries are nowhere near that magnitude).
__device__ __forceinline__ _Float16 q_to_half(float v) {
  return (_Float16)__builtin_fminf(__builtin_fmaxf(v, -65504.0f), 65504.0f);
}

// eight 16-bit values of a 16-byte load, widened to fp32 (element order = memory order)
template <int DT>
__device__ __forceinline__ void unpack8(const u32x4& v, float* f) {
  const uint32_t ws[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = bits16_to_f32<DT>(ws[j] & 0xFFFFu);
    f[2 * j + 1] = bits16_to_f32<DT>(ws[j] >> 16);
  }
}

// ---- DPP data movement -----------------------------------------------------------------------
// Lanes disabled by ROW_MASK / out-of-range sources receive `old`.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp(float old, float v) {
  return as_f32(__builtin_amdgcn_update_dpp(as_i32(old), as_i32(v), CTRL, ROW_MASK, 0xF, false));
}
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ int dpp(int old, int v) {
  return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xF, false);
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8 lanes
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each row of 16
constexpr int kDppBcast15 = 0x142;    // lane 15 of each row -> next row
constexpr int kDppBcast31 = 0x143;    // lane 31 -> rows 2 and 3

struct OpSum {
  static __device__ __forceinline__ float id() { return 0.0f; }
  static __device__ __forceinline__ float ap(float a, float b) { return a + b; }
};
struct OpMax {
  static __device__ __forceinline__ float id() { return -__builtin_inff(); }
  static __device__ __forceinline__ float ap(float a, float b) { return fmaxf(a, b); }
};
struct OpMin {
  static __device__ __forceinline__ float id() { return __builtin_inff(); }
  static __device__ __forceinline__ float ap(float a, float b) { return fminf(a, b); }
};

// After this every lane of a quad holds the quad's reduction.
template <class Op>
__device__ __forceinline__ float quad_allreduce(float v) {
  v = Op::ap(v, dpp<kDppXor1>(Op::id(), v));
  v = Op::ap(v, dpp<kDppXor2>(Op::id(), v));
  return v;
}
// After this every lane of a 16-lane row holds the row's reduction (fixed order: deterministic).
template <class Op>
__device__ __forceinline__ float row16_allreduce(float v) {
  v = quad_allreduce<Op>(v);
  v = Op::ap(v, dpp<kDppHalfMirror>(Op::id(), v));
  v = Op::ap(v, dpp<kDppMirror>(Op::id(), v));
  return v;
}
// Reduction over the 64 lanes, returned in every lane (wave-uniform value).
template <class Op>
__device__ __forceinline__ float wave_allreduce(float v) {
  v = row16_allreduce<Op>(v);
  v = Op::ap(v, dpp<kDppBcast15, 0xA>(Op::id(), v));  // rows 1,3 += rows 0,2
  v = Op::ap(v, dpp<kDppBcast31, 0xC>(Op::id(), v));  // row 3 += rows 0,1
  return as_f32(__builtin_amdgcn_readlane(as_i32(v), 63));
}

// Block-wide reduction through a caller-provided LDS slot array of `NWAVES` floats.
// All threads receive the result. Callers alternate between two slot arrays (or put a barrier
// between uses) so that a fast wave cannot overwrite values a slow wave still has to read.
template <class Op, int NWAVES>
__device__ __forceinline__ float block_allreduce(float v, float* slots) {
  static_assert(NWAVES <= 16 && (NWAVES & (NWAVES - 1)) == 0, "NWAVES must be a power of 2 <= 16");
  v = wave_allreduce<Op>(v);
  if (NWAVES == 1) return v;
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  if (lane == 0) slots[wave] = v;
  __syncthreads();
  float t = slots[lane & (NWAVES - 1)];
  // lanes hold NWAVES distinct partials, repeated with period NWAVES inside each row of 16
  if (NWAVES >= 2) t = Op::ap(t, dpp<kDppXor1>(Op::id(), t));
  if (NWAVES >= 4) t = Op::ap(t, dpp<kDppXor2>(Op::id(), t));
  if (NWAVES >= 8) t = Op::ap(t, dpp<kDppHalfMirror>(Op::id(), t));
  if (NWAVES >= 16) t = Op::ap(t, dpp<kDppMirror>(Op::id(), t));
  return t;
}

// inclusive scan of an int across the 64 lanes, in lane order
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  int t;
  t = dpp<0x111>(0, v); v += t;
  t = dpp<0x112>(0, v); v += t;
  t = dpp<0x114>(0, v); v += t;
  t = dpp<0x118>(0, v); v += t;
  t = dpp<kDppBcast15, 0xA>(0, v); v += t;
  t = dpp<kDppBcast31, 0xC>(0, v); v += t;
  return v;
}

// Quest score of ONE page from its 512-byte metadata record (chunks of min[4c..4c+3],
// max[4c..4c+3]) by a whole wavefront: lane l takes channels 2l and 2l + 1 (q0, q1 = the query
// there) and the sum is folded in a fixed order. The plane-layout scoring passes use it for a
// request's LAST page, whose plane entries are only written when the page is complete.
template <int DT>
__device__ __forceinline__ float record_page_score(const uint8_t* rec, float q0, float q1) {
  const int lane = lane_id();
  const int c = lane >> 1, o = (lane & 1) * 4;
  const uint32_t mn = *(const uint32_t*)(rec + 16 * c + o);
  const uint32_t mx = *(const uint32_t*)(rec + 16 * c + 8 + o);
  const float v0 = bits16_to_f32<DT>((q0 > 0.0f ? mx : mn) & 0xFFFFu);
  const float v1 = bits16_to_f32<DT>((q1 > 0.0f ? mx : mn) >> 16);
  return wave_allreduce<OpSum>(fmaf(q1, v1, q0 * v0));
}

// Up to 8 pages at once, same arithmetic per page, in two steps so that a caller can put other
// work between the loads and the folds: page i of the batch is logical page first + i * step of
// the table `pages` (i < count <= 8; the other slots stay untouched). rec0 points at
// the kv head's record of physical page 0, `stride` = bytes from one physical page's record to
// the next one's.
struct RecordBatch8 {
  uint32_t mn[8], mx[8];
};
__device__ __forceinline__ void record_pages_load8(RecordBatch8& r, const uint8_t* rec0,
                                                   size_t stride, const int32_t* pages, int first,
                                                   int step, int count) {
  const int lane = lane_id();
  const int c = lane >> 1, o = (lane & 1) * 4;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (i < count) {   // wave-uniform
      const int phys = pages[first + i * step];
      const uint8_t* rec = rec0 + (size_t)phys * stride;
      r.mn[i] = *(const uint32_t*)(rec + 16 * c + o);
      r.mx[i] = *(const uint32_t*)(rec + 16 * c + 8 + o);
    }
  }
}
template <int DT>
__device__ __forceinline__ void record_pages_fold8(const RecordBatch8& r, int count, float q0,
                                                   float q1, float* out) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (i < count) {   // wave-uniform
      const float v0 = bits16_to_f32<DT>((q0 > 0.0f ? r.mx[i] : r.mn[i]) & 0xFFFFu);
      const float v1 = bits16_to_f32<DT>((q1 > 0.0f ? r.mx[i] : r.mn[i]) >> 16);
      out[i] = wave_allreduce<OpSum>(fmaf(q1, v1, q0 * v0));
    }
  }
}

// The plane-layout scoring passes read a request's first plane_scored_pages(n) pages from the
// planes and the rest from the metadata records: always the last page (its plane entries are only
// written when it is complete), and a whole tail of up to kPlaneTailMax pages beyond the last
// multiple of kPlaneBlock, so that a request a little longer than a multiple of what one pass of
// a workgroup covers does not pay a whole pass for a handful of pages.
constexpr int kPlaneBlock = 2048, kPlaneTailMax = 128;
__host__ __device__ __forceinline__ int plane_scored_pages(int n) {
  if (n <= 0) return 0;
  const int full = ((n - 1) / kPlaneBlock) * kPlaneBlock;
  return (n - full <= kPlaneTailMax) ? full : n - 1;
}

// Slot of a request's plane-layout metadata: the request's position in the batch, or, with a slot
// table, the entry of that position (clamped, so that a corrupt table cannot leave the buffer).
__device__ __forceinline__ uint32_t plane_slot(const int32_t* slots, uint32_t num_slots, uint32_t b) {
  if (!slots) return b;
  const int s = slots[b];
  return (uint32_t)min(max(s, 0), (int)num_slots - 1);
}

// compute units of the current device, looked up once per device (the only process-wide state of
// the library; written with relaxed atomics, any racing writers store the same value)
inline int device_cu_count(int* out) {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return TWL_ENODEVICE;
  }
  if (dev >= 0 && dev < 64) {
    const int c = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (c > 0) {
      *out = c;
      return TWL_OK;
    }
  }
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return TWL_ENODEVICE;
  }
  if (dev >= 0 && dev < 64) __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
  *out = n;
  return TWL_OK;
}

// The exported estimator / pruner entry points with one more output: `surv_probs` (nullable,
// float [rows, idx_stride]) receives, beside idx[row, j], the softmax probability the estimator
// gave survivor j. Everything else is the exported function of the same name.
int gemv_top_p_ex(const void* q, int q_dtype, const void* k_int4, const int32_t* sel_pages,
                  const int32_t* sel_count, uint32_t sel_stride, const int32_t* kv_page_indices,
                  const int32_t* kv_page_indptr, const int32_t* kv_last_page_len, uint32_t batch,
                  uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t max_pages_per_row,
                  float sm_scale, const float* p_arr, float p, int high_mode, int32_t* idx,
                  uint32_t idx_stride, int32_t* count, float* scores_out, uint32_t score_stride,
                  int32_t* cand_count, float* low_out, float* surv_probs, void* stream);
int select_estimate_prune_ex(
    const void* q, int dtype, const void* meta, const void* k_int4, const int32_t* kv_page_indices,
    const int32_t* kv_page_indptr, const int32_t* kv_last_page_len, uint32_t batch,
    uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t token_budget,
    uint32_t max_pages_per_req, float sm_scale, const float* p_arr, float p, int high_mode,
    int32_t* sel_pages, uint32_t sel_stride, int32_t* sel_count, int32_t* idx, uint32_t idx_stride,
    int32_t* count, float* page_scores_out, uint32_t page_score_stride, float* scores_out,
    uint32_t score_stride, int32_t* cand_count, const void* meta_planes,
    uint32_t plane_cap_pages, const int32_t* plane_slots, uint32_t plane_num_slots,
    float* surv_probs, void* stream);
// twl_quest_page_scores; with group_max every q head of a kv head's group receives the largest
// of the group's scores for each page (2, 4 or 8 q heads per kv head)
int quest_page_scores_ex(const void* q, int q_dtype, const void* meta,
                         const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                         uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                         uint32_t max_pages_per_req, float* page_scores, uint32_t score_stride,
                         int group_max, void* stream);
int softmax_top_p_ex(const float* scores, uint32_t score_stride, const int32_t* lens,
                     uint32_t rows, uint32_t d, const float* p_arr, float p, int high_mode,
                     const int32_t* sel_pages, uint32_t sel_stride, int32_t* idx,
                     uint32_t idx_stride, int32_t* count, float* probs_out, float* low_out,
                     float* surv_probs, void* stream);

}  // namespace twl
#endif  // TWL_COMMON_H_
