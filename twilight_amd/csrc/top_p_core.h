// Register-resident softmax and top-p bisection shared by the stand-alone top-p kernels and the
// fused GEMV + top-p kernel. A row is spread over the THREADS threads of one workgroup, VPT values
// per thread (which value sits where does not matter here); `red` is float[2][2][16] in LDS and
// `buf` alternates between its halves so that consecutive block reductions need one barrier each.
#ifndef TWL_TOP_P_CORE_H_
#define TWL_TOP_P_CORE_H_

#include "twl_common.h"

namespace twl {

// x <- softmax(x) in fp32 (twilight/pyimpl/top_p.py:11-13); -inf entries get probability 0.
template <int THREADS, int VPT>
__device__ __forceinline__ void softmax_regs(float (&x)[VPT], float (*red)[2][16], int& buf) {
  constexpr int NWAVES = THREADS / kWave;
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
    }
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

// The bisection of csrc/include/sampling.cuh:156-217 on probabilities held in registers, starting
// from the bracket (0, high]. Returns the final `low` (keep x > low); x is clamped to >= 0.
template <int DT, int THREADS, int VPT>
__device__ __forceinline__ float bisect_regs(float (&x)[VPT], float p, float high,
                                             float (*red)[2][16], int& buf, int& iters) {
  constexpr int NWAVES = THREADS / kWave;
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
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
  {  // B for the initial `high`
    const uint32_t c = as_u32(high);
    float dummy = 0.0f;
    uint32_t k = wave_min_u32(block_min_key(c, true));
    block_fold(dummy, k);
    B_bits = (k < 0x80000000u) ? c - k : 0u;
  }
  bool sel_a = true;
  float min_gt_low, max_le_high;
  iters = 0;
  do {
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
    const bool found = kmin < 0x80000000u;
    if (sel_a) A_bits = found ? c + kmin : kInfBits;
    else B_bits = found ? c - kmin : 0u;
    min_gt_low = fminf(high, as_f32(A_bits));   // sampling.cuh:174,184-186,196-197
    max_le_high = fmaxf(low, as_f32(B_bits));   // sampling.cuh:175,187-189,199-201
    const bool accept = s >= p;                 // sampling.cuh:211-216
    low = accept ? mid : low;
    high = accept ? high : fminf(mid, max_le_high);
    sel_a = accept;
    ++iters;
  } while (round_to<DT>(max_le_high - min_gt_low) > eps && iters < 4096);

  return low;
}

}  // namespace twl
#endif  // TWL_TOP_P_CORE_H_
