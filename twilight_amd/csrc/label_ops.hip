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

// Dense 16-bit X [L][H][D]: rows are read whole and coalesced (the channels of a head are spread
// over the row, so every 32-byte sector of it is touched anyway), parked in LDS and picked from
// there; Out [L][H][r] leaves in memory order. Measured against the element-wise gather above at
// 262144 x 32 rows of 128 channels, 16 picked: 490 -> 423 us (5.7 TB/s over the rows and the output).
constexpr int kLabRows = 32;  // (l, h) rows per tile

struct LabelFastArgs {
  const uint16_t* x;
  const int64_t* channel;
  uint16_t* out;
  int64_t sc_h, sc_c;
  uint64_t rows;  // L * H
  uint32_t H, r, D;
};

__global__ __launch_bounds__(256) void get_label_tensor_rows_kernel(LabelFastArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  uint16_t* chan = (uint16_t*)smem;                 // [H][r] channel numbers
  uint16_t* tile = chan + ((a.H * a.r + 7u) & ~7u); // [kLabRows][D]
  const uint32_t tid = threadIdx.x;
  for (uint32_t i = tid; i < a.H * a.r; i += 256) {
    const uint32_t h = i / a.r, c = i - h * a.r;
    chan[i] = (uint16_t)a.channel[h * a.sc_h + c * a.sc_c];
  }
  const uint32_t ppr = a.D / 8;  // 16-byte pieces per row
  const uint64_t tiles = (a.rows + kLabRows - 1) / kLabRows;
  for (uint64_t tl = blockIdx.x; tl < tiles; tl += gridDim.x) {
    const uint64_t row0 = tl * kLabRows;
    const uint32_t nr = (uint32_t)min((uint64_t)kLabRows, a.rows - row0);
    __syncthreads();  // the previous tile has been read (first round: the channel table is there)
    for (uint32_t i = tid; i < nr * ppr; i += 256)
      ((u32x4*)tile)[i] = __builtin_nontemporal_load((const u32x4*)(a.x + row0 * a.D) + i);
    __syncthreads();
    for (uint32_t i = tid; i < nr * a.r; i += 256) {
      const uint32_t rw = i / a.r, c = i - rw * a.r;
      const uint32_t h = (uint32_t)((row0 + rw) % a.H);
      a.out[row0 * a.r + i] = tile[rw * a.D + chan[h * a.r + c]];
    }
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

// Contiguous labels (K_Label [B*N][H][R] dense, R = 8 / 16 / 32 / 64 channels): the layout of
// twilight/pyimpl/double_sparse.py. A workgroup takes a tile of tokens of one request with all
// their heads (a token is H * R contiguous bytes); a thread keeps one 16-byte (R = 8: 8-byte) slice of one head
// (its q values and their sum in registers) and walks the tokens of the tile; results are turned
// through LDS so that Out [B][H][N] leaves as runs of tokens per head.
constexpr int kBgFastThreads = 256;
constexpr int kBgFastUnroll = 4;
constexpr int kBgTilePad = 8;

struct BgemvFastArgs {
  const uint16_t* q;       // fp16 [B,H,R]
  const uint8_t* k;        // int8 [B*N,H,R]
  const uint16_t* scales;  // fp16 [B*N,H]
  uint16_t* out;           // fp16 [B,H,N]
  uint32_t H, N, tile_tok;
  int vec_out;
};

template <int R>
__global__ __launch_bounds__(kBgFastThreads) void bgemv_int8_fast_kernel(BgemvFastArgs a) {
  constexpr int PB = R >= 16 ? 16 : 8;  // bytes of a piece
  constexpr int PW = PB / 4;            // dwords of a piece
  constexpr int LPT = R / PB;           // lanes per token-head
  extern __shared__ __align__(16) uint8_t smem[];
  const uint32_t H = a.H, T = a.tile_tok, TP = T + kBgTilePad;
  const uint32_t P = H * LPT;  // pieces per token
  uint16_t* tile = (uint16_t*)smem;  // [H][TP]
  const uint32_t b = blockIdx.y, n0 = blockIdx.x * T, tid = threadIdx.x;
  const uint32_t nt = min(T, a.N - n0);
  const uint32_t phases = P >= kBgFastThreads ? P / kBgFastThreads : 1u;
  const uint32_t tstep = P >= kBgFastThreads ? 1u : kBgFastThreads / P;
  for (uint32_t ph = 0; ph < phases; ++ph) {
    const uint32_t rem = P >= kBgFastThreads ? tid + ph * kBgFastThreads : tid % P;
    const uint32_t t_first = P >= kBgFastThreads ? 0u : tid / P;
    const uint32_t h = rem / LPT, sub = rem % LPT;
    // q slice as half2 pairs, and its sum (for the + 128 bias below)
    uint32_t qd[2 * PW];
    float qsum = 0.0f;
    {
      const uint16_t* qp = a.q + ((size_t)b * H + h) * R + PB * sub;
#pragma unroll
      for (int j = 0; j < 2 * PW; ++j) {
        const uint32_t lo = qp[2 * j], hi = qp[2 * j + 1];
        qd[j] = lo | (hi << 16);
        qsum += f16_bits_to_f32(lo) + f16_bits_to_f32(hi);
      }
    }
    const uint8_t* col = a.k + ((size_t)b * a.N + n0) * P * PB + (size_t)rem * PB;
    const uint16_t* scol = a.scales + ((size_t)b * a.N + n0) * H + h;
    for (uint32_t t0 = t_first; t0 < nt; t0 += tstep * kBgFastUnroll) {
      uint32_t v[kBgFastUnroll][PW];
      uint16_t sc[kBgFastUnroll];
#pragma unroll
      for (int u = 0; u < kBgFastUnroll; ++u) {
        const uint32_t t = min(t0 + u * tstep, nt - 1);  // past the tile: a valid piece, unused
        if (PW == 4) {
          const u32x4 x = __builtin_nontemporal_load((const u32x4*)(col + (size_t)t * P * PB));
          v[u][0] = x.x; v[u][1] = x.y; v[u][2 % PW] = x.z; v[u][3 % PW] = x.w;
        } else {
          const u32x2 x = __builtin_nontemporal_load((const u32x2*)(col + (size_t)t * P * PB));
          v[u][0] = x.x; v[u][1] = x.y;
        }
        sc[u] = scol[(size_t)t * H];
      }
#pragma unroll
      for (int u = 0; u < kBgFastUnroll; ++u) {
        const uint32_t t = t0 + u * tstep;
        if (t < nt) {  // the same for the LPT lanes of a token-head
          float acc = 0.0f;
#pragma unroll
          for (int j = 0; j < PW; ++j) {
            // int8 c -> byte c + 128 -> fp16 bits 0x6400 | byte = 1152 + c exactly
            const uint32_t w = v[u][j] ^ 0x80808080u;
            const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, w, 0x07010700u);
            const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, w, 0x07030702u);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, lo),
                                         __builtin_bit_cast(half2_t, qd[2 * j]), acc, false);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, hi),
                                         __builtin_bit_cast(half2_t, qd[2 * j + 1]), acc, false);
          }
          float part = fmaf(-1152.0f, qsum, acc);
          if (LPT >= 2) part += dpp<kDppXor1>(0.0f, part);
          if (LPT >= 4) part += dpp<kDppXor2>(0.0f, part);
          if (sub == 0)
            tile[(size_t)h * TP + t] = (uint16_t)f32_to_f16_bits(part * f16_bits_to_f32(sc[u]));
        }
      }
    }
  }
  __syncthreads();
  const uint32_t chunks = T / 8;
  for (uint32_t i = tid; i < H * chunks; i += kBgFastThreads) {
    const uint32_t h = i / chunks, c = i - h * chunks;
    const uint32_t t0 = 8 * c;
    if (t0 >= nt) continue;
    uint16_t* dst = a.out + ((size_t)b * H + h) * a.N + n0 + t0;
    const uint16_t* src = tile + (size_t)h * TP + t0;
    if (a.vec_out && t0 + 8 <= nt) {
      *(u32x4*)dst = *(const u32x4*)src;
    } else {
      for (uint32_t e = 0; e < 8 && t0 + e < nt; ++e) dst[e] = src[e];
    }
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
  // dense 16-bit rows of D = sx_h channels (a multiple of 8, so that rows are 16-byte pieces)
  const bool dense = elem_bytes == 2 && sx_d == 1 && H > 1 && sx_h > 0 && sx_h <= 1024 &&
                     (sx_h & 7) == 0 && sx_l == (int64_t)H * sx_h && so_c == 1 &&
                     so_h == (int64_t)r && so_l == (int64_t)H * r && r <= (uint32_t)sx_h &&
                     (uint64_t)H * r <= 16384 && (((uintptr_t)x) & 15u) == 0;
  if (dense) {
    twl::LabelFastArgs f{(const uint16_t*)x, channel, (uint16_t*)out, sc_h, sc_c,
                         (uint64_t)L * H, H, r, (uint32_t)sx_h};
    const uint64_t tiles = (f.rows + twl::kLabRows - 1) / twl::kLabRows;
    const uint32_t blocks = (uint32_t)(tiles < 8192 ? tiles : 8192);
    const size_t lds = (((size_t)H * r + 7) & ~(size_t)7) * 2 + (size_t)twl::kLabRows * f.D * 2;
    hipLaunchKernelGGL(twl::get_label_tensor_rows_kernel, dim3(blocks), dim3(256), lds,
                       (hipStream_t)stream, f);
    return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
  }
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
  // dense operands of the Double-Sparse layout: the streaming kernel
  const uint32_t pieces = H * (r >= 16 ? r / 16 : 1);
  const bool dense = (r == 8 || r == 16 || r == 32 || r == 64) && sq_d == 1 && sq_h == (int64_t)r &&
                     sq_b == (int64_t)H * r && sk_d == 1 && sk_h == (int64_t)r &&
                     sk_t == (int64_t)H * r && ss_h == 1 && ss_t == (int64_t)H && so_n == 1 &&
                     so_h == (int64_t)n_ctx && so_b == (int64_t)H * n_ctx && H <= 128 &&
                     (pieces % twl::kBgFastThreads == 0 || twl::kBgFastThreads % pieces == 0) &&
                     (((uintptr_t)k_label) & 15u) == 0 && (((uintptr_t)q_label) & 1u) == 0;
  if (dense) {
    uint32_t tile = (8192u / H) & ~7u;
    tile = tile < 8u ? 8u : (tile > 128u ? 128u : tile);
    int cus = 256;
    (void)twl::device_cu_count(&cus);
    while (tile > 16u && (uint64_t)B * ((n_ctx + tile - 1) / tile) < 4ull * (uint64_t)cus) tile >>= 1;
    tile &= ~7u;
    twl::BgemvFastArgs f{(const uint16_t*)q_label, (const uint8_t*)k_label,
                         (const uint16_t*)k_scales, (uint16_t*)out, H, n_ctx, tile,
                         ((((uintptr_t)out) & 15u) == 0 && (n_ctx & 7u) == 0) ? 1 : 0};
    const size_t lds_f = (size_t)H * (tile + twl::kBgTilePad) * 2;
    const dim3 grid_f((n_ctx + tile - 1) / tile, B);
    const dim3 blk(twl::kBgFastThreads);
    hipStream_t st = (hipStream_t)stream;
    if (r == 8) hipLaunchKernelGGL((twl::bgemv_int8_fast_kernel<8>), grid_f, blk, lds_f, st, f);
    else if (r == 16) hipLaunchKernelGGL((twl::bgemv_int8_fast_kernel<16>), grid_f, blk, lds_f, st, f);
    else if (r == 32) hipLaunchKernelGGL((twl::bgemv_int8_fast_kernel<32>), grid_f, blk, lds_f, st, f);
    else hipLaunchKernelGGL((twl::bgemv_int8_fast_kernel<64>), grid_f, blk, lds_f, st, f);
    return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
  }
  const size_t lds = (size_t)H * (twl::kBgTokens + 1) * sizeof(float);
  dim3 grid((n_ctx + twl::kBgTokens - 1) / twl::kBgTokens, B);
  if (lds > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)twl::bgemv_int8_kernel,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  hipLaunchKernelGGL(twl::bgemv_int8_kernel, grid, dim3(256), lds, (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
