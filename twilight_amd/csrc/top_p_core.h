// Register-resident softmax and top-p bisection shared by the stand-alone top-p kernels and the
// fused GEMV + top-p kernel. A row is spread over the THREADS threads of one workgroup, VPT values
// per thread (which value sits where does not matter here); `red` is float[2][2][16] in LDS and
// `buf` alternates between its halves so that consecutive block reductions need one barrier each.
#ifndef TWL_TOP_P_CORE_H_
#define TWL_TOP_P_CORE_H_

#include "twl_common.h"

namespace twl {

// x <- softmax(x) in fp32 (twilight/pyimpl/top_p.py:11-13); -inf entries get probability 0.
// Returns the largest probability of the row: the element(s) equal to the row maximum get
// exp2(0) = 1 exactly and no correction, i.e. 1 * (1 / sum); every other element multiplies the
// same 1 / sum by a factor <= 1. An empty row returns 0.
template <int THREADS, int VPT>
__device__ __forceinline__ float softmax_regs(float (&x)[VPT], float (*red)[2][16], int& buf) {
  constexpr int NWAVES = THREADS / kWave;
  float row_max_prob = 0.0f;
    float m = -__builtin_inff();
#pragma unroll
    for (int k = 0; k < VPT; ++k) m = fmaxf(m, x[k]);
    m = block_allreduce<OpMax, NWAVES>(m, red[buf][0]);
    buf ^= 1;
    float z = 0.0f;
    if (m == -__builtin_inff()) {
      // empty row or all candidates masked: every probability is 0
#pragma unroll
      for (int k = 0; k < VPT; ++k) x[k] = 0.0f;
    } else {
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        // exp(d) = 2^(d*log2e): hardware exp2 on the rounded product, corrected by the product's
        // rounding error (about 1 ulp overall). exp2(-inf) == 0 for masked / out-of-row slots.
        const float dlt = x[k] - m;
        const float t = dlt * 1.4426950408889634f;
        float err = fmaf(dlt, 1.4426950408889634f, -t);
        err = fmaf(dlt, 1.925963033500453e-08f, err);
        const float r = __builtin_amdgcn_exp2f(t);
        x[k] = (dlt == -__builtin_inff()) ? 0.0f : fmaf(r, err * 0.6931471805599453f, r);
        z += x[k];
      }
      z = block_allreduce<OpSum, NWAVES>(z, red[buf][0]);
      buf ^= 1;
      const float rz = 1.0f / z;
#pragma unroll
      for (int k = 0; k < VPT; ++k) x[k] *= rz;
      row_max_prob = rz;
    }
    return row_max_prob;
}

// Maximum of the (non-negative) row, in every thread.
template <int THREADS, int VPT>
__device__ __forceinline__ float row_max_regs(const float (&x)[VPT], float (*red)[2][16],
                                              int& buf) {
  constexpr int NWAVES = THREADS / kWave;
  float m = 0.0f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) m = fmaxf(m, x[k]);
  m = block_allreduce<OpMax, NWAVES>(m, red[buf][0]);
  buf ^= 1;
  return m;
}

// LDS of the bisection's single-wavefront phase (see bisect_regs)
constexpr int kHeavyPerLane = 4;   // list slots per lane of the single-wavefront phase
constexpr int kHeavyShift = 8;     // tau = high / 2^kHeavyShift
constexpr int kHeavyCap = kWave * kHeavyPerLane;
struct BisectSmem {
  float hlist[kHeavyCap];
  uint32_t wcnt[16], wmax[16], wmin[16];
  uint32_t state[8];
};

// The bisection of csrc/include/sampling.cuh:156-217 on probabilities held in registers, starting
// from the bracket (0, high]. Returns the final `low` (keep x > low); x is clamped to >= 0.
// `high_is_row_max` (the same in every thread): `high` is the row's maximum, row_max_regs.
//
// Attention rows are peaked: while the pivot is above tau = high / 256, an iteration only
// distinguishes between the few elements above tau (the sum over x > pivot, the smallest element
// above `low` once `low` has moved, the largest element below `high`); everything else enters
// through two numbers, the largest element <= tau and the smallest positive element. Those
// iterations (about 8 of 15 on decode rows) are run by ONE wavefront on a list of the elements
// above tau, without workgroup barriers, while the other wavefronts wait; the loop then goes on
// over the whole row from the state that wavefront leaves. Same iterations, same decisions; the
// sums of the first phase add the same numbers in another order. Rows with more than kHeavyCap
// elements above tau skip the phase.
template <int DT, int THREADS, int VPT>
__device__ __forceinline__ float bisect_regs(float (&x)[VPT], float p, float high,
                                             float (*red)[2][16], int& buf, int& iters,
                                             BisectSmem& bs, bool high_is_row_max) {
  constexpr int NWAVES = THREADS / kWave;
  constexpr bool HEAVY = NWAVES > 1 && THREADS * VPT >= 2048;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  float low = 0.0f;
  const float eps = round_to<DT>(1e-5f);
  // Probabilities are non-negative, so their bit patterns order like unsigned integers; anything
  // else (negative, -0, NaN) is treated as 0.
  uint32_t xb[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    x[k] = (x[k] > 0.0f) ? x[k] : 0.0f;
    xb[k] = as_u32(x[k]);
  }
  // A = min{x > low} and B = max{x <= high} as bit patterns, without the reference's caps (it
  // starts the two searches from `high` and `low`, sampling.cuh:174-175; the caps are applied
  // where the values are used). One search pattern serves both:
  //   key = x - c            (c = bits(low) + 1)   smallest key  -> A = c + key
  //   key = c - x            (c = bits(high))      smallest key  -> B = c - key
  // in wrapping unsigned arithmetic, where elements on the wrong side of the bound wrap to keys
  // >= 2^31. A only moves when `low` moves and B only when `high` moves, so an iteration runs the
  // search for whichever bound the previous iteration changed.
  constexpr uint32_t kInfBits = 0x7F800000u;
  uint32_t A_bits = kInfBits, B_bits = 0u;
  // `below` (search max{x <= c} instead of min{x >= c}) is the same in every thread of the
  // workgroup, so it is branched on rather than blended: 1.5 vector ops per value instead of 3.5
  auto block_min_key = [&](uint32_t c, bool below) -> uint32_t {
    uint32_t kmin = 0xFFFFFFFFu;
    if (__builtin_amdgcn_readfirstlane((int)below)) {
#pragma unroll
      for (int k = 0; k < VPT; ++k) kmin = min(kmin, c - xb[k]);
    } else {
#pragma unroll
      for (int k = 0; k < VPT; ++k) kmin = min(kmin, xb[k] - c);
    }
    return kmin;
  };
  auto wave_min_u32 = [&](uint32_t v) -> uint32_t {  // total ends up in lanes 48..63
    v = min(v, (uint32_t)dpp<kDppXor1>((int)0xFFFFFFFF, (int)v));
    v = min(v, (uint32_t)dpp<kDppXor2>((int)0xFFFFFFFF, (int)v));
    v = min(v, (uint32_t)dpp<kDppHalfMirror>((int)0xFFFFFFFF, (int)v));
    v = min(v, (uint32_t)dpp<kDppMirror>((int)0xFFFFFFFF, (int)v));
    v = min(v, (uint32_t)dpp<kDppBcast15, 0xA>((int)0xFFFFFFFF, (int)v));
    v = min(v, (uint32_t)dpp<kDppBcast31, 0xC>((int)0xFFFFFFFF, (int)v));
    return v;
  };
  auto wave_sum_f32 = [&](float v) -> float {  // total ends up in lanes 48..63
    v = row16_allreduce<OpSum>(v);
    v += dpp<kDppBcast15, 0xA>(0.0f, v);
    v += dpp<kDppBcast31, 0xC>(0.0f, v);
    return v;
  };
  // cross-wave step: lane 63 of every wave publishes, everybody folds the NWAVES partials
  auto block_fold = [&](float& sv, uint32_t& kv) {
    if (NWAVES == 1) {
      sv = as_f32(__builtin_amdgcn_readlane(as_i32(sv), 63));
      kv = (uint32_t)__builtin_amdgcn_readlane((int)kv, 63);
      return;
    }
    if (lane == kWave - 1) {
      red[buf][0][wave] = sv;
      red[buf][1][wave] = as_f32(kv);
    }
    __syncthreads();
    float ts = red[buf][0][lane & (NWAVES - 1)];
    uint32_t tk = as_u32(red[buf][1][lane & (NWAVES - 1)]);
    if (NWAVES >= 2) {
      ts += dpp<kDppXor1>(0.0f, ts);
      tk = min(tk, (uint32_t)dpp<kDppXor1>((int)0xFFFFFFFF, (int)tk));
    }
    if (NWAVES >= 4) {
      ts += dpp<kDppXor2>(0.0f, ts);
      tk = min(tk, (uint32_t)dpp<kDppXor2>((int)0xFFFFFFFF, (int)tk));
    }
    if (NWAVES >= 8) {
      ts += dpp<kDppHalfMirror>(0.0f, ts);
      tk = min(tk, (uint32_t)dpp<kDppHalfMirror>((int)0xFFFFFFFF, (int)tk));
    }
    if (NWAVES >= 16) {
      ts += dpp<kDppMirror>(0.0f, ts);
      tk = min(tk, (uint32_t)dpp<kDppMirror>((int)0xFFFFFFFF, (int)tk));
    }
    sv = ts;
    kv = tk;
    buf ^= 1;
  };
  if (high_is_row_max) {
    B_bits = as_u32(high);  // the largest element <= the row's maximum is that maximum
  } else {  // B for the initial `high`
    const uint32_t c = as_u32(high);
    float dummy = 0.0f;
    uint32_t k = wave_min_u32(block_min_key(c, true));
    block_fold(dummy, k);
    B_bits = (k < 0x80000000u) ? c - k : 0u;
  }
  bool sel_a = true;
  bool more = true;
  iters = 0;
  // one iteration's bookkeeping, given the sum over x > mid and the smallest search key
  auto update = [&](float mid, uint32_t c, float s, uint32_t kmin) {
    const bool found = kmin < 0x80000000u;
    if (sel_a) A_bits = found ? c + kmin : kInfBits;
    else B_bits = found ? c - kmin : 0u;
    const float min_gt_low = fminf(high, as_f32(A_bits));   // sampling.cuh:174,184-186,196-197
    const float max_le_high = fmaxf(low, as_f32(B_bits));   // sampling.cuh:175,187-189,199-201
    const bool accept = s >= p;                             // sampling.cuh:211-216
    low = accept ? mid : low;
    high = accept ? high : fminf(mid, max_le_high);
    sel_a = accept;
    ++iters;
    more = round_to<DT>(max_le_high - min_gt_low) > eps && iters < 4096;
  };

  if constexpr (HEAVY) {
    const float tau = high * (1.0f / (float)(1 << kHeavyShift));
    const uint32_t tau_b = as_u32(tau);
    // ---- census: elements above tau per wavefront, largest element <= tau, smallest positive
    uint32_t cnt = 0, mx = 0u, mn1 = 0xFFFFFFFFu;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const bool h = xb[k] > tau_b;
      cnt += (uint32_t)__builtin_popcountll(__ballot(h));
      mx = max(mx, h ? 0u : xb[k]);
      mn1 = min(mn1, xb[k] - 1u);  // 0 wraps to the largest key
    }
    mn1 = wave_min_u32(mn1);
    mx = ~wave_min_u32(~mx);
    if (lane == kWave - 1) {
      bs.wcnt[wave] = cnt;
      bs.wmax[wave] = mx;
      bs.wmin[wave] = mn1;
    }
    __syncthreads();
    uint32_t tot = bs.wcnt[lane & (NWAVES - 1)];
    uint32_t gmx = bs.wmax[lane & (NWAVES - 1)];
    uint32_t gmn = bs.wmin[lane & (NWAVES - 1)];
    const int incl = wave_inclusive_scan((lane < NWAVES) ? (int)tot : 0);
    const uint32_t my_off =
        (wave == 0) ? 0u : (uint32_t)__builtin_amdgcn_readlane(incl, wave - 1);
    const uint32_t n_heavy = (uint32_t)__builtin_amdgcn_readlane(incl, NWAVES - 1);
    if (NWAVES >= 2) {
      gmx = max(gmx, (uint32_t)dpp<kDppXor1>(0, (int)gmx));
      gmn = min(gmn, (uint32_t)dpp<kDppXor1>((int)0xFFFFFFFF, (int)gmn));
    }
    if (NWAVES >= 4) {
      gmx = max(gmx, (uint32_t)dpp<kDppXor2>(0, (int)gmx));
      gmn = min(gmn, (uint32_t)dpp<kDppXor2>((int)0xFFFFFFFF, (int)gmn));
    }
    if (NWAVES >= 8) {
      gmx = max(gmx, (uint32_t)dpp<kDppHalfMirror>(0, (int)gmx));
      gmn = min(gmn, (uint32_t)dpp<kDppHalfMirror>((int)0xFFFFFFFF, (int)gmn));
    }
    if (NWAVES >= 16) {
      gmx = max(gmx, (uint32_t)dpp<kDppMirror>(0, (int)gmx));
      gmn = min(gmn, (uint32_t)dpp<kDppMirror>((int)0xFFFFFFFF, (int)gmn));
    }
    const uint32_t max_light_bits = (uint32_t)__builtin_amdgcn_readfirstlane((int)gmx);
    const uint32_t min_pos_key = (uint32_t)__builtin_amdgcn_readfirstlane((int)gmn);  // bits - 1
    // the phase needs tau > 0 (so that `low` is either 0 or above tau) and a list that fits
    const bool heavy = n_heavy <= (uint32_t)kHeavyCap && high > 1e-30f;
    if (heavy) {
      // ---- the list, in (wavefront, slot, lane) order: the same on every run
      uint32_t off = my_off;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        const bool h = xb[k] > tau_b;
        const uint64_t m = __ballot(h);
        const uint32_t rank = __builtin_amdgcn_mbcnt_hi(
            (uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        if (h) bs.hlist[off + rank] = x[k];
        off += (uint32_t)__builtin_popcountll(m);
      }
      __syncthreads();
      if (wave == 0) {
        float hv[kHeavyPerLane];
        uint32_t hb[kHeavyPerLane];
        bool hvalid[kHeavyPerLane];
#pragma unroll
        for (int j = 0; j < kHeavyPerLane; ++j) {
          const uint32_t i = (uint32_t)lane + kWave * j;
          hvalid[j] = i < n_heavy;
          hv[j] = hvalid[j] ? bs.hlist[i] : 0.0f;
          hb[j] = as_u32(hv[j]);
        }
        auto lane63_f = [](float v) { return as_f32(__builtin_amdgcn_readlane(as_i32(v), 63)); };
        auto lane63_u = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readlane((int)v, 63); };
        while (more) {
          const float mid = round_to<DT>((low + high) * 0.5f);
          if (!(mid >= tau)) break;  // below tau the rest of the row matters: whole-row phase
          float s = 0.0f, s_odd = 0.0f;
#pragma unroll
          for (int j = 0; j < kHeavyPerLane; ++j) {
            const float v = (hv[j] > mid) ? hv[j] : 0.0f;
            if (j & 1) s_odd += v;
            else s += v;
          }
          s = lane63_f(wave_sum_f32(s + s_odd));
          const uint32_t c = sel_a ? as_u32(low) + 1u : as_u32(high);
          uint32_t kmin = 0xFFFFFFFFu;
          if (!sel_a) {
            // largest element <= high: on the list, else the largest element <= tau (<= high
            // because high >= mid >= tau); no such element and an element equal to 0 both give 0
#pragma unroll
            for (int j = 0; j < kHeavyPerLane; ++j)
              kmin = min(kmin, hvalid[j] ? c - hb[j] : 0xFFFFFFFFu);
            kmin = lane63_u(wave_min_u32(kmin));
            if (kmin >= 0x80000000u) kmin = c - max_light_bits;
          } else if (low == 0.0f) {
            kmin = min_pos_key;  // c == 1: smallest positive element of the row, as bits - c
          } else {
            // smallest element > low >= tau: it is on the list or does not exist
#pragma unroll
            for (int j = 0; j < kHeavyPerLane; ++j)
              kmin = min(kmin, hvalid[j] ? hb[j] - c : 0xFFFFFFFFu);
            kmin = lane63_u(wave_min_u32(kmin));
          }
          update(mid, c, s, kmin);
        }
        if (lane == 0) {
          bs.state[0] = as_u32(low);
          bs.state[1] = as_u32(high);
          bs.state[2] = A_bits;
          bs.state[3] = B_bits;
          bs.state[4] = sel_a ? 1u : 0u;
          bs.state[5] = (uint32_t)iters;
          bs.state[6] = more ? 1u : 0u;
        }
      }
      __syncthreads();
      low = as_f32(bs.state[0]);
      high = as_f32(bs.state[1]);
      A_bits = bs.state[2];
      B_bits = bs.state[3];
      sel_a = bs.state[4] != 0u;
      iters = (int)bs.state[5];
      more = bs.state[6] != 0u;
    }
  }

  while (more) {
    const float mid = round_to<DT>((low + high) * 0.5f);
    // two interleaved partial sums (even / odd slots): a fixed order, half the dependent chain
    float s = 0.0f, s_odd = 0.0f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const float v = (x[k] > mid) ? x[k] : 0.0f;
      if (k & 1) s_odd += v;
      else s += v;
    }
    s += s_odd;
    const uint32_t c = sel_a ? as_u32(low) + 1u : as_u32(high);
    uint32_t kmin = wave_min_u32(block_min_key(c, !sel_a));
    s = wave_sum_f32(s);
    block_fold(s, kmin);
    update(mid, c, s, kmin);
  }

  return low;
}

}  // namespace twl
#endif  // TWL_TOP_P_CORE_H_
