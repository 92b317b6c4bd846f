// Estimator + pruner of ONE row inside a workgroup: INT4 score GEMV over the row's page list with
// the scores kept in registers, fp32 softmax, top-p bisection and ordered compaction. Shared by
// the kernel that takes the page list from memory (fused_row.hip) and the one-launch select +
// estimate + prune kernel (layer_row.hip), which hands the list over in registers.
//
// Restates twilight/pyimpl/attention.py:252-255 followed by twilight/pyimpl/top_p.py:10-15 and the
// mask combine attention.py:280-281.
//
// Layout: the row's candidate pages are dealt to the wavefronts in consecutive runs of 4*VPT pages;
// a wavefront streams its run four pages at a time exactly like gemv_int4_kernel (lane = token
// l/4, quantisation group l%4, quad reduction), and lane l keeps, of each group of four pages, the
// score of page l%4, token l/4. So thread registers x[g] hold candidate
//     position = 16 * (wave*4*VPT + 4*g + l%4) + l/4
// and the softmax / bisection (top_p_core.h) run on them in place. Compaction walks positions in
// (wave, g, l%4, l/4) order with wave ballots.
#ifndef TWL_FUSED_ROW_CORE_H_
#define TWL_FUSED_ROW_CORE_H_

#include "top_p_core.h"

namespace twl {


struct FusedArgs {
  const void* q;
  const uint8_t* k_int4;
  const int32_t* sel_pages;
  const int32_t* sel_count;
  uint32_t sel_stride;
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  const int32_t* kv_last_page_len;
  uint32_t num_q_heads, num_kv_heads;
  uint32_t max_pages;
  float sm_scale;
  const float* p_arr;
  float p;
  int high_mode;
  int32_t* idx;
  uint32_t idx_stride;
  int32_t* count;
  float* scores_out;   // nullable
  uint32_t score_stride;
  int32_t* cand_count; // nullable
  float* low_out;      // nullable
  float* surv_probs;   // nullable [rows, idx_stride]: estimated probability of survivor j beside idx
};

// 8 nibbles of one dword against 8 q values held as 4 half2 pairs (n0,n4),(n1,n5),(n2,n6),(n3,n7);
// a nibble at mantissa bits 4..7 of an fp16 with exponent 0 is exactly 1 + n/64 (see gemv_int4.hip)
__device__ __forceinline__ float fused_dot8(uint32_t w, const half2_t* qp, float acc) {
  const uint32_t m = 0x00F000F0u, one = 0x3C003C00u;
  acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w << 4, m, one)), qp[0], acc, false);
  acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w, m, one)), qp[1], acc, false);
  acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w >> 4, m, one)), qp[2], acc, false);
  acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, and_or(w >> 8, m, one)), qp[3], acc, false);
  return acc;
}

struct FusedSmem {
  float red[2][2][16];
  int wave_tot[16];
  float first;
  BisectSmem bis;
};

// the 64 bytes of q this lane multiplies with (dims 32*(l%4) .. +32), requested as 4 x 16 B
__device__ __forceinline__ void fused_load_q(const void* q, uint32_t row, int g4, u32x4 (&qraw)[4]) {
  const uint16_t* qrow = (const uint16_t*)q + (size_t)row * TWL_HEAD_DIM + 32 * g4;
#pragma unroll
  for (int i = 0; i < 4; ++i) qraw[i] = *(const u32x4*)(qrow + 8 * i);
}

// `my_logical[r]`: lane l holds the logical page of list entry wave*4*VPT + 64*r + l (anything for
// entries >= sel_n). Every thread of the workgroup must call, with the same row arguments.
template <int QDT, int THREADS, int VPT>
__device__ __forceinline__ void estimate_prune_row(const FusedArgs& a, FusedSmem& fsm, uint32_t row,
                                                   uint32_t kvh, int pg_begin, int req_pages,
                                                   int last_len, int sel_n,
                                                   int (&my_logical)[(4 * VPT + 63) / 64],
                                                   const u32x4 (&qraw)[4]) {
  constexpr int NWAVES = THREADS / kWave;
  constexpr int PW = 4 * VPT;            // pages per wavefront
  constexpr int RUNS = (PW + 63) / 64;   // page ids are held one per lane, 64 at a time
  float (&red)[2][2][16] = fsm.red;
  int (&wave_tot)[16] = fsm.wave_tot;
  float& first = fsm.first;
  const int tx = threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tx / kWave);
  const int e0 = wave * PW;  // first list entry of this wavefront
  const int g4 = lane & 3;   // quantisation group while streaming, page-of-four afterwards
  const int t = lane >> 2;   // token of the page
  int n_pages = min(max(sel_n, 0), (int)a.max_pages);
  if (req_pages <= 0) n_pages = 0;
  if (tx == 0 && a.cand_count) a.cand_count[row] = n_pages * TWL_PAGE;

  int my_phys[RUNS];
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    my_logical[r] = min(max(my_logical[r], 0), max(req_pages - 1, 0));
    my_phys[r] = (e0 + 64 * r + lane < n_pages && 64 * r + lane < PW)
                     ? a.kv_page_indices[pg_begin + my_logical[r]] : 0;
  }

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

  // ---- stream the run: scores into x[] --------------------------------------------------------
  const size_t rec_stride = (size_t)a.num_kv_heads * TWL_INT4_RECORD_BYTES;
  // record address = (wave-uniform pointer) + (lane offset): the uniform half is computed on the
  // scalar unit and a load needs one 32-bit vector register for its address instead of two per
  // page in flight
  const uint8_t* sbase = a.k_int4 + (size_t)kvh * TWL_INT4_RECORD_BYTES;
  const uint32_t nib_off = 16u * (uint32_t)lane;
  const uint32_t sz_off = 1024u + 4u * (uint32_t)lane;
  const float ninf = -__builtin_inff();
  float x[VPT];
#pragma unroll
  for (int g = 0; g < VPT; ++g) x[g] = ninf;
#pragma unroll
  for (int g = 0; g < VPT; ++g) {
    const int i0 = e0 + 4 * g;          // first list entry of this group of four pages
    if (i0 < n_pages) {                 // uniform over the wavefront
      const int r = g / 16;             // which 64-entry run the group belongs to (compile time)
      u32x4 nib[4];
      uint32_t sz[4];
      int logical[4];
      // (the empty asm keeps the widening of the lane offsets inside this block, next to the
      // loads, which is what lets them take the scalar base + 32-bit vector offset form)
      uint32_t o16 = nib_off, o4 = sz_off;
      asm volatile("" : "+v"(o16), "+v"(o4));
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        // entries past the list reuse the group's first entry: a valid address, result discarded
        const int src = (i0 + u < n_pages) ? (4 * (g % 16) + u) : (4 * (g % 16));
        const int phys = __builtin_amdgcn_readlane(my_phys[r], src);
        logical[u] = __builtin_amdgcn_readlane(my_logical[r], src);
        const uint8_t* rec = sbase + (size_t)(uint32_t)phys * rec_stride;   // wave-uniform
        nib[u] = __builtin_nontemporal_load((const u32x4*)(rec + o16));
        sz[u] = __builtin_nontemporal_load((const uint32_t*)(rec + o4));
      }
      float mine = ninf;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        float acc = 0.0f;
        acc = fused_dot8(nib[u].x, qp + 0, acc);
        acc = fused_dot8(nib[u].y, qp + 4, acc);
        acc = fused_dot8(nib[u].z, qp + 8, acc);
        acc = fused_dot8(nib[u].w, qp + 12, acc);
        const float scale64 = f16_bits_to_f32(sz[u] & 0xFFFFu) * 64.0f;
        const float zero = f16_bits_to_f32(sz[u] >> 16);
        const float part = quad_allreduce<OpSum>(fmaf(scale64, acc - qsum, zero * qsum));
        const int valid = (i0 + u < n_pages) ? ((logical[u] == req_pages - 1) ? last_len : TWL_PAGE) : 0;
        const float val = (t < valid) ? part * a.sm_scale : ninf;
        mine = (g4 == u) ? val : mine;
      }
      x[g] = mine;
    }
  }
  if (a.scores_out) {
    float* orow = a.scores_out + (size_t)row * a.score_stride;
#pragma unroll
    for (int g = 0; g < VPT; ++g) {
      const int pg = e0 + 4 * g + g4;
      if (pg < n_pages) orow[pg * TWL_PAGE + t] = x[g];
    }
  }

  // ---- softmax + bisection in place (top_p_core.h) ---------------------------------------------
  int buf = 0;
  const float max_prob = softmax_regs<THREADS, VPT>(x, red, buf);
  const float p = a.p_arr ? a.p_arr[row] : a.p;
  float high;
  if (a.high_mode == TWL_HIGH_FIRST) {
    // csrc/include/sampling.cuh:156-159 reads probs[row, 0], the probability of TOKEN 0 of the
    // context, on a full-length row in which tokens outside the selection have probability 0
    // (attention.py:255,274-278). Candidate 0 (wave 0, lane 0, group 0) is token 0 exactly when
    // logical page 0 heads the ascending page list; otherwise the bound is 0, the loop ends at
    // once and every candidate with a positive probability is kept.
    if (tx == 0) first = (n_pages > 0 && my_logical[0] == 0) ? x[0] : 0.0f;
    __syncthreads();
    high = first;
  } else {
    high = max_prob;  // the row maximum, without another reduction
  }
  int iters = 0;
  const float low = bisect_regs<TWL_F32, THREADS, VPT>(x, p, high, red, buf, iters, fsm.bis,
                                                      a.high_mode != TWL_HIGH_FIRST);
  if (tx == 0 && a.low_out) a.low_out[row] = low;

  // ---- ordered compaction ------------------------------------------------------------------------
  // positions ascend in (wave, g, l%4, l/4) order: inside a (wave, g) slice lane l comes after the
  // lanes with a smaller l%4 and after those with the same l%4 and a smaller l/4
  const uint64_t pat = 0x1111111111111111ull;
  uint64_t before_mask = (pat << g4) & ((1ull << lane) - 1ull);
  if (g4 > 0) before_mask |= pat;
  if (g4 > 1) before_mask |= pat << 1;
  if (g4 > 2) before_mask |= pat << 2;
  int wcount = 0;
#pragma unroll
  for (int g = 0; g < VPT; ++g) wcount += __builtin_popcountll(__ballot(x[g] > low));
  if (NWAVES > 1) {
    if (lane == 0) wave_tot[wave] = wcount;
    __syncthreads();
  }
  int pos = 0, total = wcount;
  if (NWAVES > 1) {
    total = 0;
#pragma unroll
    for (int w = 0; w < NWAVES; ++w) {
      const int c = wave_tot[w];
      pos += (w < wave) ? c : 0;
      total += c;
    }
  }
  int32_t* dst = a.idx + (size_t)row * a.idx_stride;
  float* wdst = a.surv_probs ? a.surv_probs + (size_t)row * a.idx_stride : nullptr;
#pragma unroll
  for (int g = 0; g < VPT; ++g) {
    const bool keep = x[g] > low;
    const uint64_t bal = __ballot(keep);
    if (bal) {  // uniform
      const int r = g / 16;
      // logical page of list entry e0 + 4g + l%4 lives in lane 4*(g%16) + l%4 of my_logical[r]
      const int lp = __builtin_amdgcn_ds_bpermute(4 * (4 * (g % 16) + g4), my_logical[r]);
      if (keep) {
        const int at = pos + __builtin_popcountll(bal & before_mask);
        dst[at] = lp * TWL_PAGE + t;
        if (wdst) wdst[at] = x[g];
      }
      pos += __builtin_popcountll(bal);
    }
  }
  if (tx == 0) a.count[row] = total;
}

}  // namespace twl
#endif  // TWL_FUSED_ROW_CORE_H_
