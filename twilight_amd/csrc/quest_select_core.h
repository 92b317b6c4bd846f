// Top-k page selection of one row inside a workgroup (MSB-first radix select on order-preserving
// keys held in registers, ascending emission), shared by the stand-alone selector kernel and the
// one-launch select + estimate + prune kernel. Restates the topk of twilight/pyimpl/quest.py:93-99.
#ifndef TWL_QUEST_SELECT_CORE_H_
#define TWL_QUEST_SELECT_CORE_H_

#include "twl_common.h"

namespace twl {

// pages to keep for a token budget (quest.py:93-98), before clamping to the request's page count
__device__ __forceinline__ int quest_budget_pages(uint32_t token_budget) {
  return max(1, (int)(token_budget / TWL_PAGE)) + ((token_budget % TWL_PAGE) ? 1 : 0);
}

struct SelSmem {
  int hist[4][256];  // one histogram per radix pass (at most 4 x 8 bits), zeroed by select_smem_init
  int pick[4][3];    // per pass: chosen digit, remaining k, keys in the chosen bin
  int scr[32];       // per-wave key maxima / minima
  int wave_tot[16];
};

// Zero the histograms. Every thread of the workgroup calls it, and a barrier must lie between this
// call and select_row_topk (any barrier of the caller will do: the select itself then needs no
// barrier for clearing).
template <int THREADS>
__device__ __forceinline__ void select_smem_init(SelSmem& sm) {
  for (int i = threadIdx.x; i < 4 * 256; i += THREADS) (&sm.hist[0][0])[i] = 0;
}

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = as_u32(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// The k best of the n_pages scores at `src` (global or LDS; 0 < k <= n_pages <= THREADS*VPT), by
// all THREADS threads of the workgroup (every thread must call, with the same arguments); thread t
// holds pages [t*VPT, (t+1)*VPT). The chosen page numbers are written in ascending order to `dst`
// (skipped when NULL) and, when `dst_lds` is given, to that LDS array as well (valid for the whole
// workgroup after its next barrier).
template <int THREADS, int VPT>
__device__ __forceinline__ void select_row_topk(const float* src, int n_pages, int k, int32_t* dst,
                                                int32_t* dst_lds, SelSmem& sm) {
  constexpr int NWAVES = THREADS / kWave;
  const int tx = threadIdx.x;
  const int lane = lane_id();
  const int wave = tx / kWave;
  if (k == n_pages) {  // everything is selected
    for (int i = tx; i < n_pages; i += THREADS) {
      if (dst) dst[i] = i;
      if (dst_lds) dst_lds[i] = i;
    }
    return;
  }

  uint32_t key[VPT];
  {
    // all loads are issued before any is consumed (index clamped instead of predicated)
    float v[VPT];
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int e = min(tx * VPT + j, n_pages - 1);
      v[j] = src[e];
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j) key[j] = (tx * VPT + j < n_pages) ? order_key(v[j]) : 0u;
  }

  // ---- radix select of the k-th largest key ------------------------------------------------
  // Page scores of a row share their sign and most of their exponent, so a pass over the top
  // byte would pile every key into one or two LDS bins (serialised atomics). The bits that are
  // common to the row's largest and smallest key are skipped: the first digit starts at the
  // highest bit in which two keys differ.
  uint32_t kmax = 0u, kmin = 0xFFFFFFFFu;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    kmax = max(kmax, key[j]);
    kmin = min(kmin, key[j] ? key[j] : 0xFFFFFFFFu);
  }
#pragma unroll
  for (int ctrl_step = 0; ctrl_step < 1; ++ctrl_step) {
    kmax = max(kmax, (uint32_t)dpp<kDppXor1>(0, (int)kmax));
    kmin = min(kmin, (uint32_t)dpp<kDppXor1>((int)0xFFFFFFFF, (int)kmin));
    kmax = max(kmax, (uint32_t)dpp<kDppXor2>(0, (int)kmax));
    kmin = min(kmin, (uint32_t)dpp<kDppXor2>((int)0xFFFFFFFF, (int)kmin));
    kmax = max(kmax, (uint32_t)dpp<kDppHalfMirror>(0, (int)kmax));
    kmin = min(kmin, (uint32_t)dpp<kDppHalfMirror>((int)0xFFFFFFFF, (int)kmin));
    kmax = max(kmax, (uint32_t)dpp<kDppMirror>(0, (int)kmax));
    kmin = min(kmin, (uint32_t)dpp<kDppMirror>((int)0xFFFFFFFF, (int)kmin));
    kmax = max(kmax, (uint32_t)dpp<kDppBcast15, 0xA>(0, (int)kmax));
    kmin = min(kmin, (uint32_t)dpp<kDppBcast15, 0xA>((int)0xFFFFFFFF, (int)kmin));
    kmax = max(kmax, (uint32_t)dpp<kDppBcast31, 0xC>(0, (int)kmax));
    kmin = min(kmin, (uint32_t)dpp<kDppBcast31, 0xC>((int)0xFFFFFFFF, (int)kmin));
  }
  if (lane == kWave - 1) {
    sm.scr[wave] = (int)kmax;
    sm.scr[16 + wave] = (int)kmin;
  }
  __syncthreads();
  kmax = 0u; kmin = 0xFFFFFFFFu;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) {
    kmax = max(kmax, (uint32_t)sm.scr[w]);
    kmin = min(kmin, (uint32_t)sm.scr[16 + w]);
  }
  const uint32_t diff = kmax ^ kmin;
  int top = diff ? 32 - __builtin_clz(diff) : 0;  // low bits in which keys of the row may differ
  uint32_t prefix_mask = top >= 32 ? 0u : ~((1u << top) - 1u);
  uint32_t prefix = kmax & prefix_mask;
  int k_rem = k;
  int pass = 0;
  while (top > 0) {
    const int bits = min(8, top);
    const int shift = top - bits;
    const uint32_t dmask = (1u << bits) - 1u;
    int (&hist)[256] = sm.hist[pass];  // zeroed by select_smem_init
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      if ((key[j] & prefix_mask) == prefix && key[j] != 0u)
        atomicAdd(&hist[(key[j] >> shift) & dmask], 1);
    }
    __syncthreads();
    if (wave == 0) {
      // lane l owns digits 255-4l .. 252-4l (descending)
      int hcnt[4];
      int mine = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        hcnt[j] = hist[255 - 4 * lane - j];
        mine += hcnt[j];
      }
      const int incl = wave_inclusive_scan(mine);
      int run = incl - mine;  // keys with a larger digit than this lane's first
      if (run < k_rem && k_rem <= incl) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (run < k_rem && k_rem <= run + hcnt[j]) {
            sm.pick[pass][0] = 255 - 4 * lane - j;
            sm.pick[pass][1] = k_rem - run;
            sm.pick[pass][2] = hcnt[j];
          }
          run += hcnt[j];
        }
      }
    }
    __syncthreads();
    prefix |= (uint32_t)sm.pick[pass][0] << shift;
    prefix_mask |= dmask << shift;
    k_rem = sm.pick[pass][1];
    top = shift;
    if (k_rem == sm.pick[pass][2] && top > 0 && prefix != 0u) {
      // every key of the chosen bin is taken: the remaining digits need not be resolved (after
      // two passes a bin mostly holds one or two keys). Keys >= prefix are the selection.
      prefix -= 1u;
      k_rem = 0;
      break;
    }
    ++pass;
  }
  const uint32_t T = prefix;  // keys > T are taken, and k_rem of the keys equal to T

  // ---- ordered compaction ------------------------------------------------------------------
  int packed = 0;  // (count of key > T) << 16 | (count of key == T)
#pragma unroll
  for (int j = 0; j < VPT; ++j) packed += (key[j] > T ? 0x10000 : 0) + (key[j] == T ? 1 : 0);
  const int incl = wave_inclusive_scan(packed);
  const int wtot = __builtin_amdgcn_readlane(incl, 63);
  if (lane == 0) sm.wave_tot[wave] = wtot;
  __syncthreads();
  int before = incl - packed;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) before += (w < wave) ? sm.wave_tot[w] : 0;
  int gt_before = before >> 16, eq_before = before & 0xFFFF;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int e = tx * VPT + j;
    if (key[j] > T) {
      const int o = gt_before + min(eq_before, k_rem);
      if (dst) dst[o] = e;
      if (dst_lds) dst_lds[o] = e;
      ++gt_before;
    } else if (key[j] == T) {
      if (eq_before < k_rem) {
        if (dst) dst[gt_before + eq_before] = e;
        if (dst_lds) dst_lds[gt_before + eq_before] = e;
      }
      ++eq_before;
    }
  }
}

}  // namespace twl
#endif  // TWL_QUEST_SELECT_CORE_H_
