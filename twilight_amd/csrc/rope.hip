// Rotary position embedding of one decode token's query and key heads, in place, one launch.
//
// Restates apply_rotary_pos_emb as the reference's attention forward calls it
// (twilight/pyimpl/attention.py:118-123; the half-split convention of the Llama models):
//     out[d]      = x[d]      * cos[d]      - x[d + 64] * sin[d]            d < 64
//     out[d + 64] = x[d + 64] * cos[d + 64] + x[d]      * sin[d + 64]
// with every elementary operation rounded to the tensor dtype, as the chain of element-wise
// tensor operations rounds it (two products, one sum), so the result equals the unfused form
// bit for bit.
#include "twl_common.h"

namespace twl {

struct RopeArgs {
  uint16_t* q;          // [batch, num_q_heads, 128]
  uint16_t* k;          // [batch, num_kv_heads, 128]
  const uint16_t* cos;  // [batch, 128]
  const uint16_t* sin;  // [batch, 128]
  uint32_t num_q_heads, num_kv_heads;
};

// One wavefront per (request, head); lane d owns the pair (d, d + 64).
template <int DT>
__global__ __launch_bounds__(256) void rope_qk_kernel(RopeArgs a, uint32_t total) {
  // no fused multiply-add here: a product and the sum contracted into one operation (the compiler
  // does it in half precision) would round once less than the tensor form
#pragma clang fp contract(off)
  const uint32_t w = blockIdx.x * 4 + threadIdx.x / kWave;
  if (w >= total) return;
  const uint32_t heads = a.num_q_heads + a.num_kv_heads;
  const uint32_t b = w / heads, h = w - b * heads;
  uint16_t* x = h < a.num_q_heads
                    ? a.q + ((size_t)b * a.num_q_heads + h) * TWL_HEAD_DIM
                    : a.k + ((size_t)b * a.num_kv_heads + (h - a.num_q_heads)) * TWL_HEAD_DIM;
  const int d = lane_id();
  const float x1 = bits16_to_f32<DT>(x[d]), x2 = bits16_to_f32<DT>(x[d + 64]);
  const float c1 = bits16_to_f32<DT>(a.cos[(size_t)b * TWL_HEAD_DIM + d]);
  const float c2 = bits16_to_f32<DT>(a.cos[(size_t)b * TWL_HEAD_DIM + d + 64]);
  const float s1 = bits16_to_f32<DT>(a.sin[(size_t)b * TWL_HEAD_DIM + d]);
  const float s2 = bits16_to_f32<DT>(a.sin[(size_t)b * TWL_HEAD_DIM + d + 64]);
  // products of two 16-bit values are exact in fp32, so one rounding each, like the tensor ops
  const float o1 = round_to<DT>(x1 * c1) + round_to<DT>(-x2 * s1);
  const float o2 = round_to<DT>(x2 * c2) + round_to<DT>(x1 * s2);
  x[d] = (uint16_t)f32_to_bits16<DT>(o1);
  x[d + 64] = (uint16_t)f32_to_bits16<DT>(o2);
}

}  // namespace twl

extern "C" int twl_rope_qk(void* q, void* k, const void* cos, const void* sin, int dtype,
                           uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                           void* stream) {
  if (!q || !k || !cos || !sin) return TWL_ENULL;
  if (dtype != TWL_F16 && dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0) return TWL_EINVAL;
  const uint64_t total = (uint64_t)batch * (num_q_heads + num_kv_heads);
  if (total > 0x7FFFFFFFull) return TWL_EINVAL;
  if ((((uintptr_t)q) | ((uintptr_t)k) | ((uintptr_t)cos) | ((uintptr_t)sin)) & 1u) return TWL_EALIGN;
  twl::RopeArgs a{(uint16_t*)q, (uint16_t*)k, (const uint16_t*)cos, (const uint16_t*)sin,
                  num_q_heads, num_kv_heads};
  const dim3 grid((uint32_t)((total + 3) / 4));
  if (dtype == TWL_F16)
    hipLaunchKernelGGL((twl::rope_qk_kernel<TWL_F16>), grid, dim3(256), 0, (hipStream_t)stream, a,
                       (uint32_t)total);
  else
    hipLaunchKernelGGL((twl::rope_qk_kernel<TWL_BF16>), grid, dim3(256), 0, (hipStream_t)stream, a,
                       (uint32_t)total);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
