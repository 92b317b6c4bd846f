// Token-granular paged score GEMVs in the tensor layouts of the reference's efficiency benchmark
// (benchmark/efficiency/bench_gemv.py): K cache [max_pages, page_size, num_heads, 128] as fp16
// (:211-241), as uint8 = int8 + 128 with per-token fp16 scale / zero (:80-144), or as packed
// 4-bit pairs [.., 64] with per-token scale / zero (:390-454); one page list per request shared by
// all heads; fp16 output. Dequantisation follows bench_gemv.py:181: k * scale + zero.
//
// These are the drop-in call shapes of ftka.cuda_ops.gemv; the decode layer itself uses the
// page-record kernel of gemv_int4.hip. A token-head row is 256 / 128 / 64 contiguous bytes, read by
// 16 / 8 / 4 lanes with one 16-byte load each, so a wavefront scores 4 / 8 / 16 tokens per step.
#include "twl_common.h"

namespace twl {

enum { kNhdF16 = 0, kNhdInt8 = 1, kNhdInt4 = 2 };

struct GemvNhdArgs {
  const uint16_t* q;
  uint16_t* o;
  uint32_t o_stride;
  const uint8_t* k;
  const uint16_t* scales;
  const uint16_t* zeros;
  const int32_t* kv_page_indices;  // NULL: physical page = logical page
  const int32_t* kv_page_indptr;   // NULL: a single request of n_tok_single tokens
  const int32_t* kv_last_page_len;
  uint32_t num_heads;
  uint32_t page_size;
  uint32_t max_tok;  // tokens per request the grid and the output row are sized for
  uint32_t n_tok_single;
  float sm_scale;
};

constexpr int kNhdThreads = 256;
constexpr int kNhdSteps = 4;

template <int KIND>
__global__ __launch_bounds__(kNhdThreads) void gemv_nhd_kernel(GemvNhdArgs a) {
  constexpr int LPT = KIND == kNhdF16 ? 16 : (KIND == kNhdInt8 ? 8 : 4);  // lanes per token
  constexpr int TPS = kWave / LPT;                                        // tokens per wave step
  constexpr int EPL = KIND == kNhdF16 ? 8 : (KIND == kNhdInt8 ? 16 : 32); // elements per lane
  constexpr int ROW_BYTES = KIND == kNhdF16 ? 256 : (KIND == kNhdInt8 ? 128 : 64);
  const uint32_t row = blockIdx.y;
  const uint32_t b = row / a.num_heads;
  const uint32_t h = row - b * a.num_heads;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int sub = lane % LPT;  // which 16-byte slice of the token
  const int tsl = lane / LPT;  // which token of the step

  int pg_begin = 0, n_tok = (int)a.n_tok_single;
  if (a.kv_page_indptr) {
    pg_begin = a.kv_page_indptr[b];
    const int req_pages = a.kv_page_indptr[b + 1] - pg_begin;
    if (req_pages <= 0) return;
    n_tok = (req_pages - 1) * (int)a.page_size + a.kv_last_page_len[b];
  }
  n_tok = min(n_tok, (int)a.max_tok);

  // this lane's slice of q, as fp32 and (for the 16-bit paths) as half2 pairs
  float qf[EPL];
  float qsum = 0.0f;
  {
    const uint16_t* qrow = a.q + (size_t)row * TWL_HEAD_DIM + EPL * sub;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      qf[i] = f16_bits_to_f32(qrow[i]);
      qsum += qf[i];
    }
  }
  half2_t qp[EPL / 2];
  if (KIND == kNhdInt4) {
    // nibble pairs (n0,n4),(n1,n5),(n2,n6),(n3,n7) of each dword
#pragma unroll
    for (int w = 0; w < EPL / 8; ++w)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        half2_t pr = {(_Float16)qf[8 * w + s], (_Float16)qf[8 * w + s + 4]};
        qp[4 * w + s] = pr;
      }
  } else {
#pragma unroll
    for (int i = 0; i < EPL / 2; ++i) {
      half2_t pr = {(_Float16)qf[2 * i], (_Float16)qf[2 * i + 1]};
      qp[i] = pr;
    }
  }

  const int n0 = (blockIdx.x * (kNhdThreads / kWave) + wave) * (TPS * kNhdSteps);
#pragma unroll
  for (int s = 0; s < kNhdSteps; ++s) {
    const int n = n0 + TPS * s + tsl;
    if (n < n_tok) {  // uniform over the LPT lanes of a token
      const int lp = n / (int)a.page_size;
      const int slot = n - lp * (int)a.page_size;
      const int phys = a.kv_page_indices ? a.kv_page_indices[pg_begin + lp] : lp;
      const size_t tok = ((size_t)phys * a.page_size + slot) * a.num_heads + h;
      const u32x4 v = __builtin_nontemporal_load((const u32x4*)(a.k + tok * ROW_BYTES + 16 * sub));
      const uint32_t ws[4] = {v.x, v.y, v.z, v.w};
      float part;
      if (KIND == kNhdF16) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ws[j]), qp[j], acc, false);
        part = acc;
      } else if (KIND == kNhdInt8) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc = fmaf(qf[4 * j + 0], (float)(ws[j] & 0xFFu), acc);
          acc = fmaf(qf[4 * j + 1], (float)((ws[j] >> 8) & 0xFFu), acc);
          acc = fmaf(qf[4 * j + 2], (float)((ws[j] >> 16) & 0xFFu), acc);
          acc = fmaf(qf[4 * j + 3], (float)(ws[j] >> 24), acc);
        }
        const float scale = f16_bits_to_f32(a.scales[tok]);
        const float zero = f16_bits_to_f32(a.zeros[tok]);
        // stored byte = int8 value + 128 (bench_gemv.py:78,93)
        part = fmaf(scale, fmaf(-128.0f, qsum, acc), zero * qsum);
      } else {
        float acc = 0.0f;
        const uint32_t m = 0x00F000F0u, one = 0x3C003C00u;  // fp16 1 + n/64, see gemv_int4.hip
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = ws[j];
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ((w << 4) & m) | one), qp[4 * j + 0], acc, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, (w & m) | one), qp[4 * j + 1], acc, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ((w >> 4) & m) | one), qp[4 * j + 2], acc, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ((w >> 8) & m) | one), qp[4 * j + 3], acc, false);
        }
        const float scale = f16_bits_to_f32(a.scales[tok]);
        const float zero = f16_bits_to_f32(a.zeros[tok]);
        part = fmaf(scale * 64.0f, acc - qsum, zero * qsum);
      }
      // fold the LPT lanes of the token (they are contiguous and aligned inside a DPP row)
      part += dpp<kDppXor1>(0.0f, part);
      part += dpp<kDppXor2>(0.0f, part);
      if (LPT >= 8) part += dpp<kDppHalfMirror>(0.0f, part);
      if (LPT >= 16) part += dpp<kDppMirror>(0.0f, part);
      if (sub == 0) a.o[(size_t)row * a.o_stride + n] = (uint16_t)f32_to_f16_bits(part * a.sm_scale);
    }
  }
}

}  // namespace twl

static int launch_nhd(int kind, const void* q, void* o, uint32_t o_stride, const void* k,
                      const void* scales, const void* zeros, const int32_t* kv_page_indices,
                      const int32_t* kv_page_indptr, const int32_t* kv_last_page_len,
                      uint32_t batch, uint32_t num_heads, uint32_t page_size, uint64_t max_tok,
                      uint32_t n_tok_single, float sm_scale, void* stream) {
  if (!q || !o || !k) return TWL_ENULL;
  if (kind != twl::kNhdF16 && (!scales || !zeros)) return TWL_ENULL;
  if ((kv_page_indptr == nullptr) != (kv_last_page_len == nullptr)) return TWL_ENULL;
  if (kv_page_indptr && !kv_page_indices) return TWL_ENULL;
  if (batch == 0 || num_heads == 0 || page_size == 0 || max_tok == 0) return TWL_EINVAL;
  if (max_tok > o_stride || max_tok > 0x7FFFFFFFull) return TWL_EINVAL;
  if ((uint64_t)batch * num_heads > 65535u) return TWL_EINVAL;
  if ((((uintptr_t)k) & 15u) || (((uintptr_t)q) & 1u) || (((uintptr_t)o) & 1u)) return TWL_EALIGN;
  twl::GemvNhdArgs a{};
  a.q = (const uint16_t*)q; a.o = (uint16_t*)o; a.o_stride = o_stride; a.k = (const uint8_t*)k;
  a.scales = (const uint16_t*)scales; a.zeros = (const uint16_t*)zeros;
  a.kv_page_indices = kv_page_indices; a.kv_page_indptr = kv_page_indptr;
  a.kv_last_page_len = kv_last_page_len; a.num_heads = num_heads; a.page_size = page_size;
  a.max_tok = (uint32_t)max_tok; a.n_tok_single = n_tok_single; a.sm_scale = sm_scale;
  const int lpt = kind == twl::kNhdF16 ? 16 : (kind == twl::kNhdInt8 ? 8 : 4);
  const uint64_t tok_per_block = (uint64_t)(64 / lpt) * twl::kNhdSteps * (twl::kNhdThreads / 64);
  dim3 grid((uint32_t)((max_tok + tok_per_block - 1) / tok_per_block), batch * num_heads);
  hipStream_t s = (hipStream_t)stream;
  if (kind == twl::kNhdF16)
    hipLaunchKernelGGL((twl::gemv_nhd_kernel<twl::kNhdF16>), grid, dim3(twl::kNhdThreads), 0, s, a);
  else if (kind == twl::kNhdInt8)
    hipLaunchKernelGGL((twl::gemv_nhd_kernel<twl::kNhdInt8>), grid, dim3(twl::kNhdThreads), 0, s, a);
  else
    hipLaunchKernelGGL((twl::gemv_nhd_kernel<twl::kNhdInt4>), grid, dim3(twl::kNhdThreads), 0, s, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_gemv_int4_nhd(const void* q, void* o, uint32_t o_stride, const uint8_t* k_u8,
                                 const void* scales, const void* zeros,
                                 const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                                 const int32_t* kv_last_page_len, uint32_t batch,
                                 uint32_t num_heads, uint32_t page_size,
                                 uint32_t max_pages_per_req, float sm_scale, void* stream) {
  if (!kv_page_indices || !kv_page_indptr || !kv_last_page_len) return TWL_ENULL;
  return launch_nhd(twl::kNhdInt4, q, o, o_stride, k_u8, scales, zeros, kv_page_indices,
                    kv_page_indptr, kv_last_page_len, batch, num_heads, page_size,
                    (uint64_t)max_pages_per_req * page_size, 0, sm_scale, stream);
}

extern "C" int twl_gemv_int8_nhd(const void* q, void* o, uint32_t o_stride, const uint8_t* k_u8,
                                 const void* scales, const void* zeros,
                                 const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                                 const int32_t* kv_last_page_len, uint32_t batch,
                                 uint32_t num_heads, uint32_t page_size,
                                 uint32_t max_pages_per_req, float sm_scale, void* stream) {
  if (!kv_page_indices || !kv_page_indptr || !kv_last_page_len) return TWL_ENULL;
  return launch_nhd(twl::kNhdInt8, q, o, o_stride, k_u8, scales, zeros, kv_page_indices,
                    kv_page_indptr, kv_last_page_len, batch, num_heads, page_size,
                    (uint64_t)max_pages_per_req * page_size, 0, sm_scale, stream);
}

extern "C" int twl_gemv_f16_nhd(const void* q, void* o, uint32_t o_stride, const void* k_cache,
                                const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                                const int32_t* kv_last_page_len, uint32_t batch,
                                uint32_t num_heads, uint32_t page_size,
                                uint32_t max_pages_per_req, float sm_scale, void* stream) {
  if (!kv_page_indices || !kv_page_indptr || !kv_last_page_len) return TWL_ENULL;
  return launch_nhd(twl::kNhdF16, q, o, o_stride, k_cache, nullptr, nullptr, kv_page_indices,
                    kv_page_indptr, kv_last_page_len, batch, num_heads, page_size,
                    (uint64_t)max_pages_per_req * page_size, 0, sm_scale, stream);
}

extern "C" int twl_gemv_f16_single(const void* q, void* o, const void* k, uint32_t num_heads,
                                   uint32_t seq_len, float sm_scale, void* stream) {
  return launch_nhd(twl::kNhdF16, q, o, seq_len, k, nullptr, nullptr, nullptr, nullptr, nullptr, 1,
                    num_heads, 1, seq_len, seq_len, sm_scale, stream);
}
