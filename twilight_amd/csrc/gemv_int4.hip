// INT4-K score GEMV: out[row, c] = sm_scale * sum_d q[row, d] * (nibble * scale + zero).
//
// Restates the estimator matmul of twilight/pyimpl/attention.py:252-254 over the candidate pages
// only, reading the INT4 shadow records defined in twilight_hip.h. It is a pure HBM stream
// (80 bytes per token-head for 256 flops), so there is no MFMA: one wavefront owns a run of
// candidate pages of one (batch, head) row and, per page, issues one 16-byte load per lane
// (64 lanes x 16 B = the page's 1 KiB of nibbles) plus one 4-byte load per lane (its fp16 scale /
// zero pair). Lane l holds token l/4, quantisation group l%4 — exactly the 32 nibbles that share
// one scale — so dequantisation factors out of the inner loop:
//     partial = scale * sum_j q_j * nibble_j + zero * sum_j q_j
// with sum_j q_j precomputed once per row. Nibbles become exact fp16 values with one shift and one
// v_and_or, products are accumulated in fp32 by v_dot2, a two-step DPP quad reduction yields the
// token's score, and the 64 scores of four pages leave in one 256-byte store. The kernel is close
// to co-limited by VALU issue (about 100 instructions per page fit under the HBM stream at 7 TB/s),
// which is why the unpack is kept to 11 instructions per 8 nibbles.
#include "twl_common.h"

namespace twl {

struct GemvArgs {
  const void* q;
  float* out;
  uint32_t out_stride;
  int32_t* out_count;
  const uint8_t* k_int4;
  const int32_t* sel_pages;
  const int32_t* sel_count;
  uint32_t sel_stride;
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  const int32_t* kv_last_page_len;
  uint32_t num_q_heads;
  uint32_t num_kv_heads;
  uint32_t max_pages;  // pages per row the grid and the output row are sized for
  float sm_scale;
};

// launch shape, chosen by sweeps over (threads, pages per wave, unroll) at 8 x 32 x 32768 and
// 8 x 32 x 8192 candidates
constexpr int kGemvThreads = 256;       // 4 wavefronts
// pages per wavefront (the PW template argument, <= 64: one lane per page id): 64 when the grid
// fills the chip anyway (long runs, few large store bursts); 16 or 8 for small batches, where a
// wavefront's groups of four pages are serial memory round trips and the launch needs more
// wavefronts, not longer ones
constexpr int kGemvUnroll = 4;          // pages in flight per wavefront

// 8 nibbles of one dword against 8 q values held as 4 half2 pairs (n0,n4),(n1,n5),(n2,n6),(n3,n7).
// A nibble moved to mantissa bits 4..7 of an fp16 with exponent 0 is exactly 1 + n/64, so one
// shift and one v_and_or turn two nibbles into a half2 and v_dot2 accumulates
// sum q*(1 + n/64) in fp32; the caller removes the bias with sum q (a number of the same size:
// the cancellation costs about one fp32 ulp of sum q).
__device__ __forceinline__ float dot8_nibbles(uint32_t w, const half2_t* qp, float acc) {
  const uint32_t m = 0x00F000F0u, one = 0x3C003C00u;
  half2_t a0 = __builtin_bit_cast(half2_t, and_or(w << 4, m, one));
  half2_t a1 = __builtin_bit_cast(half2_t, and_or(w, m, one));
  half2_t a2 = __builtin_bit_cast(half2_t, and_or(w >> 4, m, one));
  half2_t a3 = __builtin_bit_cast(half2_t, and_or(w >> 8, m, one));
  acc = __builtin_amdgcn_fdot2(a0, qp[0], acc, false);
  acc = __builtin_amdgcn_fdot2(a1, qp[1], acc, false);
  acc = __builtin_amdgcn_fdot2(a2, qp[2], acc, false);
  acc = __builtin_amdgcn_fdot2(a3, qp[3], acc, false);
  return acc;
}

// score of one page for this lane's token: 32 nibbles of one group against the lane's q slice
__device__ __forceinline__ float page_partial(const u32x4& nib, uint32_t sz, const half2_t* qp,
                                              float qsum) {
  float acc = 0.0f;
  acc = dot8_nibbles(nib.x, qp + 0, acc);
  acc = dot8_nibbles(nib.y, qp + 4, acc);
  acc = dot8_nibbles(nib.z, qp + 8, acc);
  acc = dot8_nibbles(nib.w, qp + 12, acc);
  // sum q*nibble = 64 * (acc - sum q);  partial = scale * sum q*nibble + zero * sum q
  const float scale64 = f16_bits_to_f32(sz & 0xFFFFu) * 64.0f;
  const float zero = f16_bits_to_f32(sz >> 16);
  return quad_allreduce<OpSum>(fmaf(scale64, acc - qsum, zero * qsum));
}

// HAS_SEL: the row has its own page list (sel_pages / sel_count); otherwise every page of the
// request is a candidate.
template <int QDT, bool HAS_SEL, int PW>
__global__ __launch_bounds__(kGemvThreads) void gemv_int4_kernel(GemvArgs a) {
  constexpr int U = kGemvUnroll;
  constexpr int G = PW / U;  // load groups per wavefront
  static_assert(PW % U == 0 && PW <= 64, "one lane per page id, whole groups");
  const uint32_t row = blockIdx.y;
  const uint32_t b = row / a.num_q_heads;
  const uint32_t h = row - b * a.num_q_heads;
  const uint32_t kvh = h / (a.num_q_heads / a.num_kv_heads);
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int p0 = (blockIdx.x * (kGemvThreads / kWave) + wave) * PW;

  // everything that depends only on the kernel arguments is requested at once
  const int pg_begin = a.kv_page_indptr[b];
  const int pg_end = a.kv_page_indptr[b + 1];
  const int last_len = a.kv_last_page_len[b];
  const int sel_n = HAS_SEL ? (a.sel_count ? a.sel_count[row] : (int)a.sel_stride) : 0;
  int my_logical = p0 + lane;
  if (HAS_SEL) {
    // read ahead of the count: the slot exists whenever it is inside the row's stride
    my_logical = (lane < PW && (uint32_t)(p0 + lane) < a.sel_stride)
                     ? a.sel_pages[(size_t)row * a.sel_stride + p0 + lane] : 0;
  }
  const int g = lane & 3;
  const int t = lane >> 2;
  u32x4 qraw[4];
  {
    const uint16_t* qrow = (const uint16_t*)a.q + (size_t)row * TWL_HEAD_DIM + 32 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) qraw[i] = *(const u32x4*)(qrow + 8 * i);
  }

  const int req_pages = pg_end - pg_begin;
  int n_pages = HAS_SEL ? sel_n : req_pages;
  n_pages = min(max(n_pages, 0), (int)a.max_pages);
  if (req_pages <= 0) n_pages = 0;
  if (blockIdx.x == 0 && threadIdx.x == 0 && a.out_count) a.out_count[row] = n_pages * TWL_PAGE;
  if (p0 >= n_pages) return;
  const int np = min(PW, n_pages - p0);

  // ---- page ids of this wave's run: lane i owns run entry i ---------------------------------
  my_logical = min(max(my_logical, 0), req_pages - 1);  // a corrupt list must not leave the table
  int my_phys = 0;
  if (lane < np) my_phys = a.kv_page_indices[pg_begin + my_logical];

  // ---- q: lane (t = l/4, g = l%4) keeps q[32g .. 32g+32) as 16 half2 pairs -------------------
  half2_t qp[16];
  float qsum = 0.0f;
  {
    float qf[32];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t ws[4] = {qraw[i].x, qraw[i].y, qraw[i].z, qraw[i].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        qf[8 * i + 2 * j] = bits16_to_f32<QDT>(ws[j] & 0xFFFFu);
        qf[8 * i + 2 * j + 1] = bits16_to_f32<QDT>(ws[j] >> 16);
      }
    }
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        half2_t pr = {q_to_half(qf[8 * w + s]), q_to_half(qf[8 * w + s + 4])};
        qp[4 * w + s] = pr;
      }
#pragma unroll
    for (int i = 0; i < 32; ++i) qsum += (float)q_to_half(qf[i]);
  }

  const size_t rec_stride = (size_t)a.num_kv_heads * TWL_INT4_RECORD_BYTES;
  const uint8_t* base = a.k_int4 + (size_t)kvh * TWL_INT4_RECORD_BYTES + 16 * lane;
  float* orow = a.out + (size_t)row * a.out_stride + (size_t)p0 * TWL_PAGE;
  const float ninf = -__builtin_inff();

  // ---- stream: the four pages of a group are requested together, then consumed. (Requesting
  // group k+1 before consuming group k was measured and does not help: enough wavefronts are
  // resident to cover the latency.)
  u32x4 nib[U];
  uint32_t sz[U];
  static_assert(U == 4, "the output transpose below moves 4 pages x 16 tokens per store");
  // lane l stores element l of the group's 64 scores (page l/16, token l%16); it takes that value
  // from the lane that owns token l%16 and whose group index equals the page: lane 4*(l%16)+l/16
  const int src_lane4 = 4 * (4 * (lane & 15) + (lane >> 4));
  float held[G];  // the wave's scores stay in registers until its run is done
#pragma unroll
  for (int grp = 0; grp < G; ++grp) {
    if (grp * U < np) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = grp * U + u;
        // entries past the run reuse entry 0: a valid address, result discarded
        const int phys = __builtin_amdgcn_readlane(my_phys, (i < np) ? i : 0);
        const uint8_t* rec = base + (size_t)phys * rec_stride;
        // read-once stream: keep it out of the way of the data the other kernels reuse
        nib[u] = __builtin_nontemporal_load((const u32x4*)rec);
        sz[u] = __builtin_nontemporal_load((const uint32_t*)(rec + 1024 - 12 * lane));
      }
      float mine = 0.0f;  // the score this lane hands over: page g of the group, token t
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = grp * U + u;
        const float part = page_partial(nib[u], sz[u], qp, qsum);
        const int logical = __builtin_amdgcn_readlane(my_logical, (i < np) ? i : 0);
        const int valid = (logical == req_pages - 1) ? last_len : TWL_PAGE;
        const float val = (t < valid) ? part * a.sm_scale : ninf;
        mine = (g == u) ? val : mine;
      }
      held[grp] = as_f32(__builtin_amdgcn_ds_bpermute(src_lane4, as_i32(mine)));
    }
  }
  // The wave's whole run (up to 4 KiB of scores) leaves in one burst of 256-byte stores; pages
  // past the run are masked off. Writes interleaved with the read stream cost this kernel ~20 %
  // of its time; one burst per wave (instead of a store per group) and long runs recover a third.
#pragma unroll
  for (int grp = 0; grp < G; ++grp)
    if (grp * U + (lane >> 4) < np) orow[grp * U * TWL_PAGE + lane] = held[grp];
}

// The q heads of a kv head over ONE page list (that of the group's first q head): every INT4
// record is fetched once and meets the group's queries on the matrix cores. Per page and per
// quantisation group the estimator is a [heads x 32] x [32 x 16 tokens] product; four of them
// (the page's four quantisation groups) share one v_mfma_f32_16x16x32_f16 by giving each
// (head, group) pair a ROW of the A operand that is zero outside its own group:
//   A (16 x 32)  row 4*h + c', k-block c (lanes 16c..16c+15): q[h, 32c + 8j .. +8] if c == c', else 0
//   B (32 x 16)  column t (token), k-block c: the 8 nibbles of dword j of group c, as the exact
//                fp16 values 1 + n/64 (one shift and one v_and_or per two nibbles)
//   C (16 x 16)  lane (r, t) holds rows 4r .. 4r+3 = (head r, groups 0..3) of token t
// accumulated over the group's four dwords j. A lane (r, t) therefore ends with the four per-group
// dot products of ONE (head, token) pair: scale and zero (four fp16 pairs = one 16-byte load per
// token) are applied and summed inside the lane, no cross-lane step at all:
//     score = sm_scale * sum_c' ( 64 scale[t,c'] (C[c'] - qsum[h,c']) + zero[t,c'] qsum[h,c'] )
// About 55 vector instructions and 4 matrix instructions per page for up to four heads (the
// per-head arithmetic on the vector unit took about 130), eight heads take two A operands. The
// products are exact and accumulate in fp32 as before, in the matrix unit's order: scores agree
// with twl_gemv_int4 within fp32 rounding of the sums, not bit for bit.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

template <int QDT, int GROUP, int PW, int U>
__global__ __launch_bounds__(kGemvThreads) void gemv_int4_group_kernel(GemvArgs a) {
  constexpr int G = PW / U;
  constexpr int SETS = (GROUP + 3) / 4;          // A operands of four heads each
  constexpr int NW = kGemvThreads / kWave;
  static_assert(PW % U == 0 && PW <= 64, "one lane per page id, whole groups");
  __shared__ float qs_lds[NW][SETS][4][4];                // [wave][set][head of set][group]
  __shared__ __align__(16) float sc_lds[NW][4 * SETS][PW * TWL_PAGE];
  const uint32_t b = blockIdx.y / a.num_kv_heads;
  const uint32_t kvh = blockIdx.y - b * a.num_kv_heads;
  const uint32_t row0 = b * a.num_q_heads + kvh * GROUP;  // the group's first q-head row
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int p0 = (blockIdx.x * NW + wave) * PW;

  const int pg_begin = a.kv_page_indptr[b];
  const int pg_end = a.kv_page_indptr[b + 1];
  const int last_len = a.kv_last_page_len[b];
  const int sel_n = a.sel_count ? a.sel_count[row0] : (int)a.sel_stride;
  int my_logical = (lane < PW && (uint32_t)(p0 + lane) < a.sel_stride)
                       ? a.sel_pages[(size_t)row0 * a.sel_stride + p0 + lane] : 0;
  const int req_pages = pg_end - pg_begin;
  int n_pages = min(max(sel_n, 0), (int)a.max_pages);
  if (req_pages <= 0) n_pages = 0;
  if (blockIdx.x == 0 && threadIdx.x < GROUP && a.out_count)
    a.out_count[row0 + threadIdx.x] = n_pages * TWL_PAGE;
  const int np = max(0, min(PW, n_pages - p0));            // 0: this wavefront only keeps the barriers
  my_logical = min(max(my_logical, 0), max(req_pages - 1, 0));
  int my_phys = 0;
  if (lane < np) my_phys = a.kv_page_indices[pg_begin + my_logical];

  const int c = lane >> 4;          // k-block of both operands; as a C lane: head of the set
  const int t = lane & 15;          // B column / C column: token of the page
  const int hl = t >> 2, cq = t & 3;  // as an A lane: head of the set, quantisation group of the row

  // ---- A operands: lane = (k-block c, row 4*hl + c') ------------------------------------------
  half8_t aop[SETS][4];
#pragma unroll
  for (int st = 0; st < SETS; ++st) {
    const int h = 4 * st + hl;
    const bool live = (c == cq) && h < GROUP;
    float qsum = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (live)
        v = *(const u32x4*)((const uint16_t*)a.q + (size_t)(row0 + h) * TWL_HEAD_DIM + 32 * c + 8 * j);
      float qf[8];
      unpack8<QDT>(v, qf);
      _Float16 qh[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        qh[i] = q_to_half(qf[i]);
        qsum += (float)qh[i];
      }
      // element order of the unpacked nibbles: n0 n4 n1 n5 n2 n6 n3 n7
      aop[st][j] = half8_t{qh[0], qh[4], qh[1], qh[5], qh[2], qh[6], qh[3], qh[7]};
    }
    if (live) qs_lds[wave][st][hl][cq] = qsum;
    else if (c == cq) qs_lds[wave][st][hl][cq] = 0.0f;
  }
  __syncthreads();
  float qs[SETS][4];                // as a C lane (head c of the set): sum of q over each group
#pragma unroll
  for (int st = 0; st < SETS; ++st)
#pragma unroll
    for (int i = 0; i < 4; ++i) qs[st][i] = qs_lds[wave][st][c][i];

  const size_t rec_stride = (size_t)a.num_kv_heads * TWL_INT4_RECORD_BYTES;
  // B lane (k-block c, token t): the 16 bytes of token t's quantisation group c; C lane (head c,
  // token t): the token's four (scale, zero) pairs
  const uint8_t* base = a.k_int4 + (size_t)kvh * TWL_INT4_RECORD_BYTES;
  const uint32_t nib_off = 64u * (uint32_t)t + 16u * (uint32_t)c;
  const uint32_t sz_off = 1024u + 16u * (uint32_t)t;
  const float ninf = -__builtin_inff();
  // the mask in a scalar register and the exponent pattern in a vector register, both opaque to
  // the compiler, so that (x & m) | one is one v_and_or_b32 (it cannot carry two literals)
  uint32_t m = 0x00F000F0u, one = 0x3C003C00u;
  asm volatile("" : "+s"(m));
  asm volatile("" : "+v"(one));
  // (Requesting the first pages before the queries are converted was measured: 12.9 against
  // 12.1 us; the wavefronts of a compute unit are not in step, so the phases overlap anyway.)
  u32x4 nib[U], sz[U];
#pragma unroll
  for (int grp = 0; grp < G; ++grp) {
    if (grp * U < np) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = grp * U + u;
        const int phys = __builtin_amdgcn_readlane(my_phys, (i < np) ? i : 0);
        const uint8_t* rec = base + (size_t)phys * rec_stride;
        nib[u] = __builtin_nontemporal_load((const u32x4*)(rec + nib_off));
        sz[u] = __builtin_nontemporal_load((const u32x4*)(rec + sz_off));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = grp * U + u;
        const uint32_t ws[4] = {nib[u].x, nib[u].y, nib[u].z, nib[u].w};
        const uint32_t sw[4] = {sz[u].x, sz[u].y, sz[u].z, sz[u].w};
        half8_t bop[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // plain C here, not the and_or() helper: the matrix instruction that reads these
          // registers needs wait states after a vector write, which the compiler inserts for
          // instructions it knows and cannot for the text of an asm statement
          const u32x4 e = {((ws[j] << 4) & m) | one, (ws[j] & m) | one,
                           ((ws[j] >> 4) & m) | one, ((ws[j] >> 8) & m) | one};
          bop[j] = __builtin_bit_cast(half8_t, e);
        }
        const int logical = __builtin_amdgcn_readlane(my_logical, (i < np) ? i : 0);
        const int valid = (logical == req_pages - 1) ? last_len : TWL_PAGE;
#pragma unroll
        for (int st = 0; st < SETS; ++st) {
          f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop[st][j], bop[j], acc, 0, 0, 0);
          const float cv[4] = {acc.x, acc.y, acc.z, acc.w};
          float v = 0.0f;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float scale64 = f16_bits_to_f32(sw[g] & 0xFFFFu) * 64.0f;
            const float zero = f16_bits_to_f32(sw[g] >> 16);
            v = fmaf(scale64, cv[g] - qs[st][g], v);
            v = fmaf(zero, qs[st][g], v);
          }
          sc_lds[wave][4 * st + c][i * TWL_PAGE + t] = (t < valid) ? v * a.sm_scale : ninf;
        }
      }
    }
  }
  __syncthreads();
  // a head's PW pages x 16 scores leave as one run: a lane stores 16 bytes, a wavefront 1 KiB
  if (np > 0) {
#pragma unroll
    for (int h = 0; h < GROUP; ++h) {
      float* orow = a.out + (size_t)(row0 + h) * a.out_stride + (size_t)p0 * TWL_PAGE;
      const bool wide = (((uintptr_t)orow) & 15u) == 0;
#pragma unroll
      for (int e = 0; e < (4 * PW + kWave - 1) / kWave; ++e) {
        const int f4 = e * kWave + lane;               // which group of four scores
        if (f4 < 4 * PW && (f4 >> 2) < np) {
          const f32x4 v = *(const f32x4*)&sc_lds[wave][h][4 * f4];
          if (wide) {
            *(f32x4*)(orow + 4 * f4) = v;
          } else {
            orow[4 * f4] = v.x; orow[4 * f4 + 1] = v.y; orow[4 * f4 + 2] = v.z;
            orow[4 * f4 + 3] = v.w;
          }
        }
      }
    }
  }
}

// One workgroup of 16 wavefronts per (batch, head) row, the row's scores parked in LDS and written
// out in one burst when the row is done. With about one row per compute unit (the stand-alone
// benchmark shape: 256 rows of 2048 pages) every compute unit streams for the whole kernel and
// the score writes (4 bytes per token, 5 % of the bytes) no longer interleave with the read
// stream, which costs this HBM far more than their share: see the dispatch in twl_gemv_int4.
constexpr int kGemvRowThreads = 1024;

template <int QDT, bool HAS_SEL>
__global__ __launch_bounds__(kGemvRowThreads) void gemv_int4_rows_kernel(GemvArgs a, int wide) {
  constexpr int U = kGemvUnroll;
  constexpr int PW = 64;
  constexpr int G = PW / U;
  extern __shared__ __align__(16) float row_scores[];  // [max_pages * 16]
  const uint32_t row = blockIdx.x;
  const uint32_t b = row / a.num_q_heads;
  const uint32_t h = row - b * a.num_q_heads;
  const uint32_t kvh = h / (a.num_q_heads / a.num_kv_heads);
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int pg_begin = a.kv_page_indptr[b];
  const int pg_end = a.kv_page_indptr[b + 1];
  const int last_len = a.kv_last_page_len[b];
  const int sel_n = HAS_SEL ? (a.sel_count ? a.sel_count[row] : (int)a.sel_stride) : 0;
  const int g = lane & 3;
  const int t = lane >> 2;
  u32x4 qraw[4];
  {
    const uint16_t* qrow = (const uint16_t*)a.q + (size_t)row * TWL_HEAD_DIM + 32 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) qraw[i] = *(const u32x4*)(qrow + 8 * i);
  }
  const int req_pages = pg_end - pg_begin;
  int n_pages = HAS_SEL ? sel_n : req_pages;
  n_pages = min(max(n_pages, 0), (int)a.max_pages);
  if (req_pages <= 0) n_pages = 0;
  if (threadIdx.x == 0 && a.out_count) a.out_count[row] = n_pages * TWL_PAGE;
  if (n_pages == 0) return;  // uniform

  half2_t qp[16];
  float qsum = 0.0f;
  {
    float qf[32];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t ws[4] = {qraw[i].x, qraw[i].y, qraw[i].z, qraw[i].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        qf[8 * i + 2 * j] = bits16_to_f32<QDT>(ws[j] & 0xFFFFu);
        qf[8 * i + 2 * j + 1] = bits16_to_f32<QDT>(ws[j] >> 16);
      }
    }
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        half2_t pr = {q_to_half(qf[8 * w + s]), q_to_half(qf[8 * w + s + 4])};
        qp[4 * w + s] = pr;
      }
#pragma unroll
    for (int i = 0; i < 32; ++i) qsum += (float)q_to_half(qf[i]);
  }
  const size_t rec_stride = (size_t)a.num_kv_heads * TWL_INT4_RECORD_BYTES;
  const uint8_t* base = a.k_int4 + (size_t)kvh * TWL_INT4_RECORD_BYTES + 16 * lane;
  const float ninf = -__builtin_inff();
  const int src_lane4 = 4 * (4 * (lane & 15) + (lane >> 4));

  for (int p0 = wave * PW; p0 < n_pages; p0 += (kGemvRowThreads / kWave) * PW) {
    const int np = min(PW, n_pages - p0);
    int my_logical = p0 + lane;
    if (HAS_SEL)
      my_logical = ((uint32_t)(p0 + lane) < a.sel_stride)
                       ? a.sel_pages[(size_t)row * a.sel_stride + p0 + lane] : 0;
    my_logical = min(max(my_logical, 0), req_pages - 1);
    int my_phys = 0;
    if (lane < np) my_phys = a.kv_page_indices[pg_begin + my_logical];
    u32x4 nib[U];
    uint32_t sz[U];
#pragma unroll
    for (int grp = 0; grp < G; ++grp) {
      if (grp * U < np) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = grp * U + u;
          const int phys = __builtin_amdgcn_readlane(my_phys, (i < np) ? i : 0);
          const uint8_t* rec = base + (size_t)phys * rec_stride;
          nib[u] = __builtin_nontemporal_load((const u32x4*)rec);
          sz[u] = __builtin_nontemporal_load((const uint32_t*)(rec + 1024 - 12 * lane));
        }
        float mine = 0.0f;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = grp * U + u;
          const float part = page_partial(nib[u], sz[u], qp, qsum);
          const int logical = __builtin_amdgcn_readlane(my_logical, (i < np) ? i : 0);
          const int valid = (logical == req_pages - 1) ? last_len : TWL_PAGE;
          const float val = (t < valid) ? part * a.sm_scale : ninf;
          mine = (g == u) ? val : mine;
        }
        const float v = as_f32(__builtin_amdgcn_ds_bpermute(src_lane4, as_i32(mine)));
        if (grp * U + (lane >> 4) < np) row_scores[(p0 + grp * U) * TWL_PAGE + lane] = v;
      }
    }
  }
  __syncthreads();
  float* orow = a.out + (size_t)row * a.out_stride;
  const int total = n_pages * TWL_PAGE;  // a multiple of 16
  if (wide) {
    for (int i = 4 * threadIdx.x; i < total; i += 4 * kGemvRowThreads)
      *(f32x4*)(orow + i) = *(const f32x4*)(row_scores + i);
  } else {
    for (int i = threadIdx.x; i < total; i += kGemvRowThreads) orow[i] = row_scores[i];
  }
}

template <int QDT, bool HAS_SEL>
static void launch_gemv(const GemvArgs& a, uint32_t rows, int pw, hipStream_t st) {
  const dim3 blk(kGemvThreads);
  const uint32_t per_block = (uint32_t)pw * (kGemvThreads / kWave);
  const dim3 grid((a.max_pages + per_block - 1) / per_block, rows);
  if (pw == 64) hipLaunchKernelGGL((gemv_int4_kernel<QDT, HAS_SEL, 64>), grid, blk, 0, st, a);
  else if (pw == 16) hipLaunchKernelGGL((gemv_int4_kernel<QDT, HAS_SEL, 16>), grid, blk, 0, st, a);
  else hipLaunchKernelGGL((gemv_int4_kernel<QDT, HAS_SEL, 8>), grid, blk, 0, st, a);
}

}  // namespace twl

extern "C" int twl_gemv_int4(const void* q, int q_dtype, float* out, uint32_t out_stride,
                             int32_t* out_count, const void* k_int4, const int32_t* sel_pages,
                             const int32_t* sel_count, uint32_t sel_stride,
                             const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                             const int32_t* kv_last_page_len, uint32_t batch,
                             uint32_t num_q_heads, uint32_t num_kv_heads,
                             uint32_t max_pages_per_row, float sm_scale, void* stream) {
  if (!q || !out || !k_int4 || !kv_page_indices || !kv_page_indptr || !kv_last_page_len)
    return TWL_ENULL;
  if (sel_count && !sel_pages) return TWL_ENULL;
  if (q_dtype != TWL_F16 && q_dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (max_pages_per_row == 0 || (uint64_t)max_pages_per_row * TWL_PAGE > out_stride)
    return TWL_EINVAL;
  if (sel_pages && sel_stride < max_pages_per_row) return TWL_EINVAL;
  if ((uint64_t)batch * num_q_heads > 65535u) return TWL_EINVAL;
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k_int4) & 15u) || (((uintptr_t)out) & 3u))
    return TWL_EALIGN;
  twl::GemvArgs a{};
  a.q = q; a.out = out; a.out_stride = out_stride; a.out_count = out_count;
  a.k_int4 = (const uint8_t*)k_int4; a.sel_pages = sel_pages; a.sel_count = sel_count;
  a.sel_stride = sel_stride; a.kv_page_indices = kv_page_indices; a.kv_page_indptr = kv_page_indptr;
  a.kv_last_page_len = kv_last_page_len; a.num_q_heads = num_q_heads;
  a.num_kv_heads = num_kv_heads; a.max_pages = max_pages_per_row; a.sm_scale = sm_scale;
  const uint32_t rows = batch * num_q_heads;
  hipStream_t st = (hipStream_t)stream;
  // enough wavefronts to give every SIMD of the chip two: shorter runs when the batch is small
  const uint64_t row_pages = (uint64_t)rows * max_pages_per_row;
  int cus = 256;
  (void)twl::device_cu_count(&cus);
  const uint64_t want_waves = 8ull * (uint64_t)cus;
  // about one row per compute unit and a row of scores that fits LDS: a workgroup per row
  // (measured at 256 rows: 2048 pages per row 122.7 -> 114.2 us, 512 pages per row no change)
  if (max_pages_per_row > 512u && max_pages_per_row <= 2048u && 2u * rows >= (uint32_t)cus &&
      rows <= 2u * (uint32_t)cus) {
    const int wide = ((((uintptr_t)out) & 15u) == 0 && (out_stride & 3u) == 0) ? 1 : 0;
    const size_t lds = (size_t)max_pages_per_row * TWL_PAGE * sizeof(float);
    const dim3 grid_r(rows), blk_r(twl::kGemvRowThreads);
#define TWL_GEMV_ROWS(DT, SEL)                                                              \
  do {                                                                                        \
    if (lds > 48 * 1024)                                                                      \
      (void)hipFuncSetAttribute((const void*)twl::gemv_int4_rows_kernel<DT, SEL>,             \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);        \
    hipLaunchKernelGGL((twl::gemv_int4_rows_kernel<DT, SEL>), grid_r, blk_r, lds, st, a, wide); \
  } while (0)
    if (q_dtype == TWL_F16) {
      if (sel_pages) TWL_GEMV_ROWS(TWL_F16, true);
      else TWL_GEMV_ROWS(TWL_F16, false);
    } else {
      if (sel_pages) TWL_GEMV_ROWS(TWL_BF16, true);
      else TWL_GEMV_ROWS(TWL_BF16, false);
    }
#undef TWL_GEMV_ROWS
    return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
  }
  const int pw = row_pages / 64 >= want_waves ? 64 : (row_pages / 16 >= want_waves ? 16 : 8);
  if (q_dtype == TWL_F16) {
    if (sel_pages) twl::launch_gemv<TWL_F16, true>(a, rows, pw, st);
    else twl::launch_gemv<TWL_F16, false>(a, rows, pw, st);
  } else {
    if (sel_pages) twl::launch_gemv<TWL_BF16, true>(a, rows, pw, st);
    else twl::launch_gemv<TWL_BF16, false>(a, rows, pw, st);
  }
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}


extern "C" int twl_gemv_int4_group(const void* q, int q_dtype, float* out, uint32_t out_stride,
                                   int32_t* out_count, const void* k_int4,
                                   const int32_t* sel_pages, const int32_t* sel_count,
                                   uint32_t sel_stride, const int32_t* kv_page_indices,
                                   const int32_t* kv_page_indptr, const int32_t* kv_last_page_len,
                                   uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                                   uint32_t max_pages_per_row, float sm_scale, void* stream) {
  if (!q || !out || !k_int4 || !sel_pages || !kv_page_indices || !kv_page_indptr ||
      !kv_last_page_len)
    return TWL_ENULL;
  if (q_dtype != TWL_F16 && q_dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  const uint32_t group = num_q_heads / num_kv_heads;
  if (group != 2 && group != 4 && group != 8) return TWL_EINVAL;
  if (max_pages_per_row == 0 || (uint64_t)max_pages_per_row * TWL_PAGE > out_stride)
    return TWL_EINVAL;
  if (sel_stride < max_pages_per_row) return TWL_EINVAL;
  if ((uint64_t)batch * num_q_heads > 65535u) return TWL_EINVAL;
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k_int4) & 15u) || (((uintptr_t)out) & 3u))
    return TWL_EALIGN;
  twl::GemvArgs a{};
  a.q = q; a.out = out; a.out_stride = out_stride; a.out_count = out_count;
  a.k_int4 = (const uint8_t*)k_int4; a.sel_pages = sel_pages; a.sel_count = sel_count;
  a.sel_stride = sel_stride; a.kv_page_indices = kv_page_indices; a.kv_page_indptr = kv_page_indptr;
  a.kv_last_page_len = kv_last_page_len; a.num_q_heads = num_q_heads;
  a.num_kv_heads = num_kv_heads; a.max_pages = max_pages_per_row; a.sm_scale = sm_scale;
  hipStream_t st = (hipStream_t)stream;
  // 16 pages per wavefront, 4 in flight (measured at 8 x 8 kv heads x 512 pages: 16 / 4 12.1 us,
  // 8 / 4 12.3, 16 / 8 12.3, 8 / 8 12.0, 4 / 4 13.9: the launch is about as long as its fixed
  // phases, launch, page-table and query round trips, the write-out, plus 50 MB at HBM speed)
#define TWL_GEMV_GROUP2(DT, PW_, U_)                                                              \
  do {                                                                                            \
    const uint32_t per_block = PW_ * (twl::kGemvThreads / twl::kWave);                            \
    const dim3 grid((max_pages_per_row + per_block - 1) / per_block, batch * num_kv_heads);       \
    const dim3 blk(twl::kGemvThreads);                                                            \
    if (group == 2) hipLaunchKernelGGL((twl::gemv_int4_group_kernel<DT, 2, PW_, U_>), grid, blk, 0, st, a); \
    else if (group == 4) hipLaunchKernelGGL((twl::gemv_int4_group_kernel<DT, 4, PW_, U_>), grid, blk, 0, st, a); \
    else hipLaunchKernelGGL((twl::gemv_int4_group_kernel<DT, 8, PW_, U_>), grid, blk, 0, st, a);   \
  } while (0)
#define TWL_GEMV_GROUP(DT) TWL_GEMV_GROUP2(DT, 16, 4)
  if (q_dtype == TWL_F16) TWL_GEMV_GROUP(TWL_F16);
  else TWL_GEMV_GROUP(TWL_BF16);
#undef TWL_GEMV_GROUP2
#undef TWL_GEMV_GROUP
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
