// Token-granular paged score GEMVs in the tensor layouts of the reference's efficiency benchmark
// (benchmark/efficiency/bench_gemv.py): K cache [max_pages, page_size, num_heads, 128] as fp16
// (:211-241), as uint8 = int8 + 128 with per-token fp16 scale / zero (:80-144), or as packed
// 4-bit pairs [.., 64] with per-token scale / zero (:390-454); one page list per request shared by
// all heads; fp16 output. Dequantisation follows bench_gemv.py:181: k * scale + zero.
//
// These are the drop-in call shapes of ftka.cuda_ops.gemv; the decode layer itself uses the
// page-record kernel of gemv_int4.hip. A token is num_heads * 256 / 128 / 64 contiguous bytes, so a
// workgroup takes a tile of tokens of ONE request with all their heads and streams every token as
// one contiguous run (a workgroup per head would fetch a 256 / 128 / 64-byte piece every
// num_heads * 256 bytes: measured 0.55 / 0.47 / 0.38 of the HBM peak). A token-head row is read by
// 16 / 8 / 4 lanes with one 16-byte load each (32 bytes per lane was measured slower: half-used
// load instructions) and folded by DPP; the [token][head] results are
// turned through LDS so that the [head][token] output leaves as runs of up to 256 bytes per head.
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
  uint32_t tile_tok;  // tokens per workgroup, a multiple of 8
  int vec_out;        // output rows allow 16-byte stores
  float sm_scale;
};

constexpr int kNhdThreads = 256;
constexpr int kNhdUnroll = 4;   // 16-byte pieces in flight per lane
constexpr int kNhdTilePad = 8;  // halves between the rows of the output tile
// q rows in LDS are 16 bytes longer than a head: the lanes of a wavefront read the same slice of
// up to 16 different heads at once, and rows a multiple of 256 bytes apart share their banks
constexpr int kNhdQRow = TWL_HEAD_DIM + 8;

template <int KIND>
__global__ __launch_bounds__(kNhdThreads) void gemv_nhd_kernel(GemvNhdArgs a) {
  constexpr int LPT = KIND == kNhdF16 ? 16 : (KIND == kNhdInt8 ? 8 : 4);  // lanes per token-head
  constexpr int EPL = KIND == kNhdF16 ? 8 : (KIND == kNhdInt8 ? 16 : 32); // elements per lane
  extern __shared__ __align__(16) uint8_t smem[];
  const uint32_t H = a.num_heads, T = a.tile_tok, TP = T + kNhdTilePad;
  uint16_t* qs = (uint16_t*)smem;                              // [H][kNhdQRow], int4: nibble-pair order
  float* qsl = (float*)(smem + (size_t)H * kNhdQRow * 2);      // [H][LPT] sums of a lane's q slice
  uint32_t* tbase = (uint32_t*)(qsl + H * LPT);                // [T] token row = phys * page_size + slot
  uint16_t* tile = (uint16_t*)(tbase + T);                     // [H][TP] results as fp16
  const uint32_t b = blockIdx.y;
  const uint32_t n0 = blockIdx.x * T;
  const uint32_t tid = threadIdx.x;

  int pg_begin = 0, n_tok = (int)a.n_tok_single;
  if (a.kv_page_indptr) {
    pg_begin = a.kv_page_indptr[b];
    const int req_pages = a.kv_page_indptr[b + 1] - pg_begin;
    if (req_pages <= 0) return;
    n_tok = (req_pages - 1) * (int)a.page_size + a.kv_last_page_len[b];
  }
  n_tok = min(n_tok, (int)a.max_tok);
  if ((int)n0 >= n_tok) return;  // uniform
  const uint32_t nt = min(T, (uint32_t)n_tok - n0);

  // ---- stage: q of the request's heads, slice sums, token rows ------------------------------
  const uint16_t* qg = a.q + (size_t)b * H * TWL_HEAD_DIM;
  for (uint32_t i = tid; i < H * TWL_HEAD_DIM; i += kNhdThreads) {
    uint32_t dst = i;
    if (KIND == kNhdInt4) {
      // a dword holds nibbles n0..n7 of elements 8w..8w+7 and is consumed as the pairs
      // (n0,n4),(n1,n5),(n2,n6),(n3,n7): element 8w+e sits at 8w + 2*(e%4) + e/4
      const uint32_t e = i & 7u;
      dst = (i & ~7u) + 2u * (e & 3u) + (e >> 2);
    }
    qs[(dst >> 7) * kNhdQRow + (dst & 127u)] = qg[i];
  }
  for (uint32_t i = tid; i < H * LPT; i += kNhdThreads) {
    float sum = 0.0f;
    for (int e = 0; e < EPL; ++e) sum += f16_bits_to_f32(qg[(size_t)i * EPL + e]);
    qsl[i] = sum;
  }
  for (uint32_t t = tid; t < nt; t += kNhdThreads) {
    const uint32_t n = n0 + t;
    const uint32_t lp = n / a.page_size;
    const uint32_t slot = n - lp * a.page_size;
    const uint32_t phys = a.kv_page_indices ? (uint32_t)a.kv_page_indices[pg_begin + (int)lp] : lp;
    tbase[t] = phys * a.page_size + slot;
  }
  __syncthreads();

  // ---- stream -------------------------------------------------------------------------------
  // The tile is nt tokens x P 16-byte pieces (piece = LPT-aligned slice of a token-head row).
  // consume(): one piece against the lane's q slice, folded over the LPT lanes of the token-head.
  const uint32_t P = H * LPT;
  auto consume = [&](const u32x4& v, uint16_t scb, uint16_t zrb, const uint32_t (&qd)[EPL / 2],
                     float qsum, uint32_t h, uint32_t sub, uint32_t t) {
    // (vector components go through arrays: __builtin_bit_cast of `v.y` itself reads component 0
    // with this compiler)
    const uint32_t ws[4] = {v.x, v.y, v.z, v.w};
    float acc = 0.0f;
    float part;
    if (KIND == kNhdF16) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, ws[j]),
                                     __builtin_bit_cast(half2_t, qd[j]), acc, false);
      part = acc;
    } else {
      const float scale = f16_bits_to_f32(scb);
      const float zero = f16_bits_to_f32(zrb);
      if (KIND == kNhdInt8) {
        // byte b as fp16 bits 0x6400 | b = 1024 + b exactly: two bytes per v_perm, then dot2
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, ws[j], 0x07010700u);
          const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, ws[j], 0x07030702u);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, lo),
                                       __builtin_bit_cast(half2_t, qd[(2 * j) % (EPL / 2)]), acc, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, hi),
                                       __builtin_bit_cast(half2_t, qd[(2 * j + 1) % (EPL / 2)]), acc, false);
        }
        // stored byte = int8 value + 128 (bench_gemv.py:78,93); acc = sum q * (1024 + byte)
        part = fmaf(scale, fmaf(-(1024.0f + 128.0f), qsum, acc), zero * qsum);
      } else {
        const uint32_t m = 0x00F000F0u, one = 0x3C003C00u;  // fp16 1 + n/64, see gemv_int4.hip
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = ws[j];
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w << 4, m, one)),
                                       __builtin_bit_cast(half2_t, qd[(4 * j) % (EPL / 2)]), acc, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w, m, one)),
                                       __builtin_bit_cast(half2_t, qd[(4 * j + 1) % (EPL / 2)]), acc, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w >> 4, m, one)),
                                       __builtin_bit_cast(half2_t, qd[(4 * j + 2) % (EPL / 2)]), acc, false);
          acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w >> 8, m, one)),
                                       __builtin_bit_cast(half2_t, qd[(4 * j + 3) % (EPL / 2)]), acc, false);
        }
        part = fmaf(scale * 64.0f, acc - qsum, zero * qsum);
      }
    }
    part += dpp<kDppXor1>(0.0f, part);
    part += dpp<kDppXor2>(0.0f, part);
    if (LPT >= 8) part += dpp<kDppHalfMirror>(0.0f, part);
    if (LPT >= 16) part += dpp<kDppMirror>(0.0f, part);
    if (sub == 0) tile[(size_t)h * TP + t] = (uint16_t)f32_to_f16_bits(part * a.sm_scale);
  };
  auto load_q = [&](uint32_t h, uint32_t sub, uint32_t (&qd)[EPL / 2]) {
    const uint32_t* qw = (const uint32_t*)(qs + (size_t)h * kNhdQRow + sub * EPL);
#pragma unroll
    for (int j = 0; j < EPL / 2; ++j) qd[j] = qw[j];
  };

  if (P % kNhdThreads == 0 || kNhdThreads % P == 0) {
    // A thread keeps ONE slice (head, 16-byte piece) and walks the tokens of the tile: its q slice
    // and its sum stay in registers, a piece costs an address, the dot products and the fold.
    const uint32_t phases = P >= kNhdThreads ? P / kNhdThreads : 1u;
    const uint32_t tstep = P >= kNhdThreads ? 1u : kNhdThreads / P;
    for (uint32_t ph = 0; ph < phases; ++ph) {
      const uint32_t rem = P >= kNhdThreads ? tid + ph * kNhdThreads : tid % P;
      const uint32_t t_first = P >= kNhdThreads ? 0u : tid / P;
      const uint32_t h = rem / LPT, sub = rem % LPT;
      uint32_t qd[EPL / 2];
      load_q(h, sub, qd);
      const float qsum = qsl[h * LPT + sub];
      const uint8_t* col = a.k + (size_t)rem * 16u;
      for (uint32_t t0 = t_first; t0 < nt; t0 += tstep * kNhdUnroll) {
        u32x4 v[kNhdUnroll];
        uint16_t sc[kNhdUnroll], zr[kNhdUnroll];
#pragma unroll
        for (int u = 0; u < kNhdUnroll; ++u) {
          const uint32_t t = min(t0 + u * tstep, nt - 1);  // past the tile: a valid piece, unused
          const uint32_t row = tbase[t];
          v[u] = __builtin_nontemporal_load((const u32x4*)(col + (size_t)row * P * 16u));
          if (KIND != kNhdF16) {
            sc[u] = a.scales[(size_t)row * H + h];
            zr[u] = a.zeros[(size_t)row * H + h];
          } else {
            sc[u] = 0; zr[u] = 0;
          }
        }
#pragma unroll
        for (int u = 0; u < kNhdUnroll; ++u) {
          const uint32_t t = t0 + u * tstep;
          if (t < nt) consume(v[u], sc[u], zr[u], qd, qsum, h, sub, t);  // same for the LPT lanes
        }
      }
    }
  } else {
    // any other head count: the tile as a flat sequence of pieces, slice looked up per piece
    const uint32_t total = nt * P;  // a multiple of LPT: the lanes of a token-head stay together
    const uint32_t dtok = kNhdThreads / P, drem = kNhdThreads % P;
    uint32_t tok = tid / P, rem = tid - tok * P;
    for (uint32_t g = tid; g < total; g += kNhdThreads) {
      const uint32_t row = tbase[tok];
      const uint32_t h = rem / LPT, sub = rem % LPT;
      const u32x4 v = __builtin_nontemporal_load((const u32x4*)(a.k + ((size_t)row * P + rem) * 16u));
      uint16_t scb = 0, zrb = 0;
      if (KIND != kNhdF16) {
        scb = a.scales[(size_t)row * H + h];
        zrb = a.zeros[(size_t)row * H + h];
      }
      uint32_t qd[EPL / 2];
      load_q(h, sub, qd);
      consume(v, scb, zrb, qd, qsl[h * LPT + sub], h, sub, tok);
      tok += dtok; rem += drem;
      if (rem >= P) { rem -= P; ++tok; }
    }
  }
  __syncthreads();

  // ---- the tile leaves head by head: runs of up to T fp16 values ------------------------------
  const uint32_t chunks = T / 8;
  for (uint32_t i = tid; i < H * chunks; i += kNhdThreads) {
    const uint32_t h = i / chunks, c = i - h * chunks;
    const uint32_t t0 = 8 * c;
    if (t0 >= nt) continue;
    uint16_t* dst = a.o + ((size_t)b * H + h) * a.o_stride + n0 + t0;
    const uint16_t* src = tile + (size_t)h * TP + t0;
    if (a.vec_out && t0 + 8 <= nt) {
      *(u32x4*)dst = *(const u32x4*)src;
    } else {
      for (uint32_t e = 0; e < 8 && t0 + e < nt; ++e) dst[e] = src[e];
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
  if (batch > 65535u || num_heads > 128u) return TWL_EINVAL;  // q of all heads lives in LDS
  if ((((uintptr_t)k) & 15u) || (((uintptr_t)q) & 1u) || (((uintptr_t)o) & 1u)) return TWL_EALIGN;
  twl::GemvNhdArgs a{};
  a.q = (const uint16_t*)q; a.o = (uint16_t*)o; a.o_stride = o_stride; a.k = (const uint8_t*)k;
  a.scales = (const uint16_t*)scales; a.zeros = (const uint16_t*)zeros;
  a.kv_page_indices = kv_page_indices; a.kv_page_indptr = kv_page_indptr;
  a.kv_last_page_len = kv_last_page_len; a.num_heads = num_heads; a.page_size = page_size;
  a.max_tok = (uint32_t)max_tok; a.n_tok_single = n_tok_single; a.sm_scale = sm_scale;
  const uint32_t lpt = kind == twl::kNhdF16 ? 16 : (kind == twl::kNhdInt8 ? 8 : 4);
  // tokens per workgroup: the fp16 output tile [heads][tokens] stays near 16 KB of LDS
  uint32_t tile = (8192u / num_heads) & ~7u;
  tile = tile < 8u ? 8u : (tile > 128u ? 128u : tile);
  // ... and the launch keeps a few workgroups per compute unit (a single short request)
  int cus = 256;
  (void)twl::device_cu_count(&cus);
  while (tile > 16u && (uint64_t)batch * ((max_tok + tile - 1) / tile) < 4ull * (uint64_t)cus) tile >>= 1;
  tile &= ~7u;
  a.tile_tok = tile;
  a.vec_out = ((((uintptr_t)o) & 15u) == 0 && (o_stride & 7u) == 0) ? 1 : 0;
  const size_t lds = (size_t)num_heads * twl::kNhdQRow * 2 + (size_t)num_heads * lpt * 4 + (size_t)tile * 4 +
                     (size_t)num_heads * (tile + twl::kNhdTilePad) * 2;
  dim3 grid((uint32_t)((max_tok + tile - 1) / tile), batch);
  hipStream_t s = (hipStream_t)stream;
  if (kind == twl::kNhdF16)
    hipLaunchKernelGGL((twl::gemv_nhd_kernel<twl::kNhdF16>), grid, dim3(twl::kNhdThreads), lds, s, a);
  else if (kind == twl::kNhdInt8)
    hipLaunchKernelGGL((twl::gemv_nhd_kernel<twl::kNhdInt8>), grid, dim3(twl::kNhdThreads), lds, s, a);
  else
    hipLaunchKernelGGL((twl::gemv_nhd_kernel<twl::kNhdInt4>), grid, dim3(twl::kNhdThreads), lds, s, a);
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
