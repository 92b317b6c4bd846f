// Double-Sparse label ops: heavy-channel gather and the int8 label-cache GEMV.
//
//   twl_get_label_tensor  Out[l,h,c] = X[l,h,channel[h,c]]      (twilight/kernel/triton/channel.py:11-79)
//   twl_bgemv_int8        Out[b,h,n] = (sum_c q[b,h,c] * k[b*N+n,h,c]) * scale[b*N+n,h]
//                                                               (twilight/kernel/triton/bgemv_int8.py:12-75)
// Both are pure data movement (a label row is r <= 64 bytes), so the only design point is
// coalescing: threads walk (token, head, channel) in memory order on the read side, and the GEMV
// turns its [token][head] results through LDS so that the [head][token] output is written in runs.
#include "twl_common.h"

namespace twl {

struct LabelArgs {
  const void* x;
  const int64_t* channel;
  void* out;
  int64_t sx_l, sx_h, sx_d;     // element strides
  int64_t sc_h, sc_c;
  int64_t so_l, so_h, so_c;
  uint32_t L, H, r;
};

template <typename T>
__global__ __launch_bounds__(256) void get_label_tensor_kernel(LabelArgs a) {
  const uint64_t total = (uint64_t)a.L * a.H * a.r;
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (uint64_t)gridDim.x * 256) {
    const uint32_t c = (uint32_t)(i % a.r);
    const uint64_t lh = i / a.r;
    const uint32_t h = (uint32_t)(lh % a.H);
    const uint64_t l = lh / a.H;
    const int64_t ch = a.channel[h * a.sc_h + c * a.sc_c];
    ((T*)a.out)[l * a.so_l + h * a.so_h + c * a.so_c] =
        ((const T*)a.x)[l * a.sx_l + h * a.sx_h + ch * a.sx_d];
  }
}

struct BgemvArgs {
  const uint16_t* q;       // fp16 [B,H,r]
  const int8_t* k;         // int8 [B*N,H,r]
  const uint16_t* scales;  // fp16 [B*N,H]
  uint16_t* out;           // fp16 [B,H,N]
  int64_t sq_b, sq_h, sq_d;
  int64_t sk_t, sk_h, sk_d;
  int64_t ss_t, ss_h;
  int64_t so_b, so_h, so_n;
  uint32_t B, H, r, N;
};

constexpr int kBgTokens = 64;  // tokens per workgroup tile

__global__ __launch_bounds__(256) void bgemv_int8_kernel(BgemvArgs a) {
  extern __shared__ float tile[];  // [H][kBgTokens + 1]
  const uint32_t b = blockIdx.y;
  const uint32_t n0 = blockIdx.x * kBgTokens;
  const uint32_t nt = min((uint32_t)kBgTokens, a.N - n0);
  // (token, head) pairs in memory order of K_Label
  for (uint32_t i = threadIdx.x; i < nt * a.H; i += 256) {
    const uint32_t h = i % a.H, t = i / a.H;
    const uint64_t tok = (uint64_t)b * a.N + n0 + t;
    const int8_t* kp = a.k + tok * a.sk_t + h * a.sk_h;
    const uint16_t* qp = a.q + b * a.sq_b + h * a.sq_h;
    float acc = 0.0f;
    for (uint32_t c = 0; c < a.r; ++c)
      acc = fmaf(f16_bits_to_f32(qp[c * a.sq_d]), (float)kp[c * a.sk_d], acc);
    tile[h * (kBgTokens + 1) + t] = acc * f16_bits_to_f32(a.scales[tok * a.ss_t + h * a.ss_h]);
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < nt * a.H; i += 256) {
    const uint32_t t = i % nt, h = i / nt;
    a.out[b * a.so_b + h * a.so_h + (uint64_t)(n0 + t) * a.so_n] =
        (uint16_t)f32_to_f16_bits(tile[h * (kBgTokens + 1) + t]);
  }
}

}  // namespace twl

extern "C" int twl_get_label_tensor(const void* x, const int64_t* channel, void* out,
                                    uint32_t elem_bytes, uint32_t L, uint32_t H, uint32_t r,
                                    int64_t sx_l, int64_t sx_h, int64_t sx_d, int64_t sc_h,
                                    int64_t sc_c, int64_t so_l, int64_t so_h, int64_t so_c,
                                    void* stream) {
  if (!x || !channel || !out) return TWL_ENULL;
  if (elem_bytes != 2 && elem_bytes != 4) return TWL_EDTYPE;
  if (L == 0 || H == 0 || r == 0) return TWL_EINVAL;
  if ((((uintptr_t)x) | ((uintptr_t)out)) & (elem_bytes - 1)) return TWL_EALIGN;
  if (((uintptr_t)channel) & 7u) return TWL_EALIGN;
  twl::LabelArgs a{x, channel, out, sx_l, sx_h, sx_d, sc_h, sc_c, so_l, so_h, so_c, L, H, r};
  const uint64_t total = (uint64_t)L * H * r;
  const uint32_t blocks = (uint32_t)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
  if (elem_bytes == 2)
    hipLaunchKernelGGL(twl::get_label_tensor_kernel<uint16_t>, dim3(blocks), dim3(256), 0,
                       (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL(twl::get_label_tensor_kernel<uint32_t>, dim3(blocks), dim3(256), 0,
                       (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_bgemv_int8(const void* q_label, const int8_t* k_label, const void* k_scales,
                              void* out, uint32_t B, uint32_t H, uint32_t r, uint32_t n_ctx,
                              int64_t sq_b, int64_t sq_h, int64_t sq_d, int64_t sk_t, int64_t sk_h,
                              int64_t sk_d, int64_t ss_t, int64_t ss_h, int64_t so_b, int64_t so_h,
                              int64_t so_n, void* stream) {
  if (!q_label || !k_label || !k_scales || !out) return TWL_ENULL;
  if (B == 0 || H == 0 || r == 0 || n_ctx == 0 || B > 65535u || H > 1024u) return TWL_EINVAL;
  if ((((uintptr_t)q_label) | ((uintptr_t)k_scales) | ((uintptr_t)out)) & 1u) return TWL_EALIGN;
  twl::BgemvArgs a{(const uint16_t*)q_label, k_label, (const uint16_t*)k_scales, (uint16_t*)out,
                   sq_b, sq_h, sq_d, sk_t, sk_h, sk_d, ss_t, ss_h, so_b, so_h, so_n, B, H, r, n_ctx};
  const size_t lds = (size_t)H * (twl::kBgTokens + 1) * sizeof(float);
  dim3 grid((n_ctx + twl::kBgTokens - 1) / twl::kBgTokens, B);
  if (lds > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)twl::bgemv_int8_kernel,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  hipLaunchKernelGGL(twl::bgemv_int8_kernel, grid, dim3(256), lds, (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
