/*
 * twl_oracle.c — TEST INFRASTRUCTURE ONLY. CPU restatement (plain C, scalar, one thread) of the
 * loop-heavy parts of Twilight's Select-then-Prune decode path. Nothing in the shipped library or
 * package may link or call this file; tests, the smoke check and the CPU-baseline leg of the
 * benchmark use it as the checker.
 *
 * What is restated, and from where:
 *   twl_oracle_top_p_f32   csrc/include/sampling.cuh:156-231 (TopPReturnMaskKernel after its dead
 *                          max pass :135-155), rows/cols as csrc/src/sampling.cu:51-60
 *   twl_oracle_top_p_cub   the same kernel with every operation in its element type (half,
 *                          nv_bfloat16 or float: sampling.cu:22-63) and the additions in the
 *                          order of cub::BlockReduce<.., BLOCK_REDUCE_WARP_REDUCTIONS>
 *                          (sampling.cuh:54); see the comment above the function
 *   twl_oracle_nucleus     textbook nucleus set (sort descending, cumulative sum in fp64):
 *                          the mathematical definition the bisection approximates
 *   twl_oracle_int4_quant  twilight/pyimpl/quantize.py:4-13 applied per group, with the fp16
 *                          rounding of scale / zero that the storage format of this build adds
 *   twl_oracle_int4_dequant  nibble * scale + zero, one fp32 rounding
 *
 * Pinning (see tests/test_oracle_*.py): top-p against twl_oracle_nucleus + brute force over all
 * subsets for d <= 12 + degenerate rows; twl_oracle_top_p_cub against rows followed in exact
 * rational arithmetic with explicit round-to-nearest-even (tests/golden "top_p_cub_order": sums
 * whose order decides, midpoints and widths that are not representable, a subnormal halving;
 * each row is checked to come out differently under fp32 sums, a left-to-right sum and an
 * unrounded midpoint), and its fp32 form against twl_oracle_top_p_f32 wherever the margin allows; quant against the known-answer vector of
 * twilight/pyimpl/quantize.py:30-48 evaluated by hand, min/max reproduction and |err| <= scale/2.
 *
 * Block sums of twl_oracle_top_p_f32: the reference adds fp32 values in the order of
 * cub::BlockReduce; this function accumulates in fp64 and rounds once, which is within an ulp or
 * two of every order, and reports how close each decision came (margin). twl_oracle_top_p_cub
 * follows CUB's order itself.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- IEEE binary16 / bfloat16 helpers (round to nearest even) -------------------------------- */
static uint16_t f32_to_f16_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7FFFFFFFu;
  if (absx >= 0x7F800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x0200u : 0));
  }
  if (absx >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7C00u);
  }
  if (absx < 0x33000001u) { /* below half of the smallest subnormal (2^-25) -> 0 */
    return (uint16_t)sign;
  }
  int32_t exp = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
  int shift;                                     /* bits to drop */
  uint32_t base;
  if (exp < -14) { /* subnormal half: value = man * 2^(exp-23), unit 2^-24 */
    shift = -exp - 1; /* 13 + (-14 - exp) */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(exp + 15) << 10;
    man &= 0x7FFFFFu;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q += 1; /* may carry into the exponent: fine */
  return (uint16_t)(sign | (base + q));
}

static float f16_bits_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t x;
  if (exp == 0) {
    if (man == 0) {
      x = sign;
    } else {
      float v = (float)man * 5.9604644775390625e-08f; /* 2^-24 */
      memcpy(&x, &v, 4);
      x |= sign;
    }
  } else if (exp == 31) {
    x = sign | 0x7F800000u | (man << 13);
  } else {
    x = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

static uint16_t f32_to_bf16_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7FFFu + lsb;
  return (uint16_t)(x >> 16);
}

static float bf16_bits_to_f32(uint16_t h) {
  uint32_t x = (uint32_t)h << 16;
  float f;
  memcpy(&f, &x, 4);
  return f;
}

/* exported so that the Python side can cross-check them against numpy's float16 */
uint16_t twl_oracle_f32_to_f16(float f) { return f32_to_f16_bits(f); }
float twl_oracle_f16_to_f32(uint16_t h) { return f16_bits_to_f32(h); }
uint16_t twl_oracle_f32_to_bf16(float f) { return f32_to_bf16_bits(f); }

/* ---- top-p bisection ------------------------------------------------------------------------- */
/* One fp32 row of csrc/include/sampling.cuh:156-231. */
static void top_p_row(const float* x, uint32_t d, float p_in, int high_mode,
                      uint8_t* mask, float* low_out, int32_t* iters_out, float* margin_out) {
  float p = p_in;                  /* DType p = DType(top_p...)            sampling.cuh:125 */
  float low = 0.0f;                /*                                       sampling.cuh:159 */
  float high;
  if (high_mode == 0) {
    high = x[0];                   /* "load attention sink"                 sampling.cuh:156-159 */
  } else {
    high = 0.0f;                   /* paper Algorithm 1: r = max(W) */
    for (uint32_t j = 0; j < d; ++j) high = x[j] > high ? x[j] : high;
  }
  const float eps = 1e-5f;                  /*                              sampling.cuh:162 */
  float min_gt_low, max_le_high;
  int32_t iters = 0;
  double margin = 1e30; /* smallest |S - p| met: how close a decision came to a rounding flip */
  do {                                       /*                             sampling.cuh:171 */
    float mid = (low + high) / 2.0f;                  /*                    sampling.cuh:173 */
    min_gt_low = high;                       /*                             sampling.cuh:174 */
    max_le_high = low;                       /*                             sampling.cuh:175 */
    double sum = 0.0;
    for (uint32_t j = 0; j < d; ++j) {
      float v = x[j];
      if (v > mid) sum += (double)v;                         /* :183,191-193 */
      if (v > low && v < min_gt_low) min_gt_low = v;          /* :184-186 */
      if (v <= high && v > max_le_high) max_le_high = v;      /* :187-189 */
    }
    float s = (float)sum;
    if (fabs(sum - (double)p) < margin) margin = fabs(sum - (double)p);
    if (s >= p) {                            /*                             sampling.cuh:211-213 */
      low = mid;
    } else {                                 /*                             sampling.cuh:214-216 */
      high = mid < max_le_high ? mid : max_le_high;
    }
    ++iters;
    if (iters > 4096) break; /* cannot happen for finite input; guards a NaN row */
  } while (max_le_high - min_gt_low > eps);                 /*             sampling.cuh:217 */
  if (mask) {
    for (uint32_t j = 0; j < d; ++j) mask[j] = x[j] > low ? 1 : 0; /*       sampling.cuh:219-230 */
  }
  if (low_out) *low_out = low;
  if (iters_out) *iters_out = iters;
  if (margin_out) *margin_out = (float)margin;
}

void twl_oracle_top_p_f32(const float* probs, uint8_t* mask, const float* p_arr, float p,
                          uint32_t rows, uint32_t d, int high_mode, float* low_out,
                          int32_t* iters_out, float* margin_out) {
  for (uint32_t r = 0; r < rows; ++r) {
    top_p_row(probs + (size_t)r * d, d, p_arr ? p_arr[r] : p, high_mode,
              mask ? mask + (size_t)r * d : NULL, low_out ? low_out + r : NULL,
              iters_out ? iters_out + r : NULL, margin_out ? margin_out + r : NULL);
  }
}

/* ---- the same kernel with every operation in its element type and CUB's summation order ------
 *
 * TopPReturnMaskKernel<1024, BLOCK_REDUCE_WARP_REDUCTIONS, VEC, DType> (csrc/include/sampling.cuh:
 * 119-231, instantiated for half / nv_bfloat16 at csrc/src/sampling.cu:22-43 and for float at
 * :45-63) keeps p, low, high, mid, eps, the running sum and every partial sum in DType. With a
 * 16-bit DType the order of the additions decides the result, so it is restated here as CUB
 * publishes it (cub/block/specializations/block_reduce_warp_reductions.cuh,
 * cub/warp/specializations/warp_reduce_shfl.cuh, cub/thread/thread_reduce.cuh; the form of CUB
 * 1.x .. 2.4, which covers the CUDA 11.8 - 12.4 toolkits that torch 2.5.0, requirements.txt:1, is
 * built for; CUB is a dependency of the reference that is absent from its tree):
 *   - thread t of 1024 owns, in chunk i, the VEC = gcd(16 / sizeof(DType), d) elements starting at
 *     (i * 1024 + t) * VEC (sampling.cuh:176-181,239-243), zero-filled past d;
 *   - BlockReduce::Sum<VEC>(items): ThreadReduce folds a thread's items left to right starting
 *     from item 0; each warp of 32 then runs five shuffle-down steps with offsets 1, 2, 4, 8, 16,
 *     lane l adding lane l + offset's value when l + offset <= 31; lane 0 of every warp stores
 *     its aggregate and thread 0 adds the aggregates of warps 1 .. 31 to its own, in that order;
 *   - the kernel adds each chunk's block sum to threadlocal_sum (sampling.cuh:191-193).
 * Every addition rounds to nearest even in DType (__hadd for half and nv_bfloat16, one rounding).
 * mid = (low + high) / DType(2): the sum rounds, then the halving rounds (it only can for a
 * subnormal half). max_le_high - min_gt_low rounds too; minima, maxima and comparisons are exact.
 * high_mode 1 (the row maximum) is this build's variant of :156-159; everything else is the same.
 *
 * A DType value is carried as a double (every fp16 / bf16 / fp32 value is one exactly). a + b of
 * two such values is computed in double and rounded to DType: exact-then-round for fp16, and for
 * bf16 / fp32 a double rounding that cannot change the result (53 >= 2 * 24 + 2 bits).
 */
typedef struct { int mant; int emin; double maxv; } fmt_t; /* significand bits incl. the hidden one */
static const fmt_t kFmt[3] = {
  {11, -14, 65504.0},                          /* IEEE binary16 */
  {8, -126, 3.3895313892515355e38},            /* bfloat16 */
  {24, -126, 3.4028234663852886e38},           /* IEEE binary32 */
};

static double dt_round(double x, int dtype) {
  if (x == 0.0 || isnan(x) || isinf(x)) return x;
  const fmt_t* f = &kFmt[dtype];
  int e;
  (void)frexp(fabs(x), &e);      /* |x| in [2^(e-1), 2^e) */
  int ex = e - 1;
  if (ex < f->emin) ex = f->emin; /* subnormal: the spacing stops shrinking */
  const double quantum = ldexp(1.0, ex - (f->mant - 1));
  const double y = nearbyint(x / quantum) * quantum; /* the division is an exact scaling; RNE */
  if (fabs(y) > f->maxv) return x > 0 ? INFINITY : -INFINITY;
  return y;
}
static double dt_add(double a, double b, int dtype) {
  if (b == 0.0) return a; /* exact, and by far the commonest case in a masked sum */
  if (a == 0.0) return b;
  return dt_round(a + b, dtype);
}

#define CUB_BLOCK 1024u
#define CUB_WARP 32u

static uint32_t gcd_u32(uint32_t a, uint32_t b) { while (b) { uint32_t t = a % b; a = b; b = t; } return a; }

/* cub::BlockReduce<DType, 1024, BLOCK_REDUCE_WARP_REDUCTIONS>::Sum of one value per thread */
static double cub_block_sum(double* v /* [1024], destroyed */, int dtype) {
  for (uint32_t off = 1; off < CUB_WARP; off <<= 1)          /* WarpReduceShfl::ReduceStep */
    for (uint32_t w = 0; w < CUB_BLOCK; w += CUB_WARP)
      for (uint32_t l = 0; l + off < CUB_WARP; ++l)           /* l + off <= last_lane */
        v[w + l] = dt_add(v[w + l], v[w + l + off], dtype);   /* lane l + off is still this step's input */
  double agg = v[0];                                          /* ApplyWarpAggregates, thread 0 */
  for (uint32_t w = 1; w < CUB_BLOCK / CUB_WARP; ++w) agg = dt_add(agg, v[w * CUB_WARP], dtype);
  return agg;
}

static void top_p_row_cub(const double* x, uint32_t d, float p_in, int high_mode, int dtype,
                          uint8_t* mask, float* low_out, int32_t* iters_out) {
  const uint32_t vec = gcd_u32(dtype == 2 ? 4u : 8u, d);                 /* sampling.cuh:239 */
  const uint32_t chunks = (d + CUB_BLOCK * vec - 1) / (CUB_BLOCK * vec); /* sampling.cuh:176 */
  const double p = dt_round((double)p_in, dtype);                        /* sampling.cuh:125 */
  double low = 0.0, high;                                                /* sampling.cuh:159 */
  if (high_mode == 0) {
    high = x[0];                                                         /* sampling.cuh:156-159 */
  } else {
    high = 0.0;
    for (uint32_t j = 0; j < d; ++j) high = x[j] > high ? x[j] : high;
  }
  const double eps = dt_round(1e-5, dtype);                              /* sampling.cuh:162 */
  double min_gt_low, max_le_high;
  double part[CUB_BLOCK];
  int32_t iters = 0;
  do {                                                                   /* sampling.cuh:171 */
    double threadlocal_sum = 0.0;                                        /* :172 */
    const double mid = dt_round(dt_round(low + high, dtype) / 2.0, dtype); /* :173 */
    min_gt_low = high;                                                   /* :174 */
    max_le_high = low;                                                   /* :175 */
    for (uint32_t i = 0; i < chunks; ++i) {                              /* :176 */
      for (uint32_t t = 0; t < CUB_BLOCK; ++t) {
        const uint64_t e0 = ((uint64_t)i * CUB_BLOCK + t) * vec;
        double acc = 0.0;
        for (uint32_t j = 0; j < vec; ++j) {
          const double v = (e0 + j < d) ? x[e0 + j] : 0.0;               /* fill(0), :177-180 */
          const double g = (v > mid) ? v : 0.0;                          /* :183 */
          acc = (j == 0) ? g : dt_add(acc, g, dtype);                    /* ThreadReduce */
          if (e0 + j < d) {
            if (v > low && v < min_gt_low) min_gt_low = v;               /* :184-186 */
            if (v <= high && v > max_le_high) max_le_high = v;           /* :187-189 */
          }
        }
        part[t] = acc;
      }
      threadlocal_sum = dt_add(threadlocal_sum, cub_block_sum(part, dtype), dtype); /* :191-193 */
    }
    if (threadlocal_sum >= p) {                                          /* :211-213 */
      low = mid;
    } else {                                                             /* :214-216 */
      high = mid < max_le_high ? mid : max_le_high;
    }
    ++iters;
    if (iters > 4096) break; /* cannot happen for finite input; guards a NaN row */
  } while (dt_round(max_le_high - min_gt_low, dtype) > eps);             /* :217 */
  if (mask)
    for (uint32_t j = 0; j < d; ++j) mask[j] = x[j] > low ? 1 : 0;       /* :219-230 */
  if (low_out) *low_out = (float)low;
  if (iters_out) *iters_out = iters;
}

/* probs: 16-bit patterns (dtype 0 = fp16, 1 = bf16) or floats (dtype 2), [rows, d] */
void twl_oracle_top_p_cub(const void* probs, int dtype, uint8_t* mask, const float* p_arr, float p,
                          uint32_t rows, uint32_t d, int high_mode, float* low_out,
                          int32_t* iters_out) {
  double* x = (double*)malloc(sizeof(double) * (size_t)d);
  for (uint32_t r = 0; r < rows; ++r) {
    for (uint32_t j = 0; j < d; ++j) {
      if (dtype == 2) {
        x[j] = (double)((const float*)probs)[(size_t)r * d + j];
      } else {
        const uint16_t b = ((const uint16_t*)probs)[(size_t)r * d + j];
        x[j] = (double)(dtype == 0 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b));
      }
    }
    top_p_row_cub(x, d, p_arr ? p_arr[r] : p, high_mode, dtype, mask ? mask + (size_t)r * d : NULL,
                  low_out ? low_out + r : NULL, iters_out ? iters_out + r : NULL);
  }
  free(x);
}

/* one addition / one rounding in the element type, exported so that tests can pin them */
double twl_oracle_dt_add(double a, double b, int dtype) { return dt_add(a, b, dtype); }
double twl_oracle_dt_round(double x, int dtype) { return dt_round(x, dtype); }

/* ---- textbook nucleus set -------------------------------------------------------------------- */
typedef struct { float v; uint32_t i; } vi_t;
static int cmp_desc(const void* a, const void* b) {
  const vi_t* x = (const vi_t*)a;
  const vi_t* y = (const vi_t*)b;
  if (x->v > y->v) return -1;
  if (x->v < y->v) return 1;
  return (x->i > y->i) - (x->i < y->i);
}
/* Smallest prefix of the descending order whose fp64 mass is >= p, closed under ties with its
 * last element. Writes the 0/1 mask, the pivot value (smallest kept probability) and the kept
 * mass; returns the number kept. */
uint32_t twl_oracle_nucleus(const float* probs, uint32_t d, double p, uint8_t* mask,
                            float* pivot_out, double* mass_out) {
  vi_t* s = (vi_t*)malloc(sizeof(vi_t) * (size_t)d);
  for (uint32_t j = 0; j < d; ++j) { s[j].v = probs[j]; s[j].i = j; }
  qsort(s, d, sizeof(vi_t), cmp_desc);
  double acc = 0.0;
  uint32_t k = 0;
  while (k < d) {
    acc += (double)s[k].v;
    ++k;
    if (acc >= p) break;
  }
  while (k < d && s[k].v == s[k - 1].v && s[k].v > 0.0f) { acc += (double)s[k].v; ++k; }
  memset(mask, 0, d);
  for (uint32_t j = 0; j < k; ++j) mask[s[j].i] = 1;
  if (pivot_out) *pivot_out = k ? s[k - 1].v : 0.0f;
  if (mass_out) *mass_out = acc;
  free(s);
  return k;
}

/* ---- INT4 group quantisation ----------------------------------------------------------------- */
/* k: [n_groups, group] fp32. Per group (twilight/pyimpl/quantize.py:4-13 with kv.view(.., group)):
 *   scale = clamp(max - min, 1e-9) / 15 ; zeros = -min ; code = clamp(round((kv + zeros)/scale),0,15)
 * with the storage rounding of this build: scale_h = fp16(scale) floored at the smallest normal
 * fp16 (2^-14) and capped at 65504, zero_h = fp16(min) (finite), code computed in fp32 from the
 * ROUNDED scale_h / zero_h with one IEEE division and rint (half to even, like torch.round). */
void twl_oracle_int4_quant(const float* k, uint32_t n_groups, uint32_t group, uint8_t* codes,
                           uint16_t* scale_h, uint16_t* zero_h) {
  for (uint32_t g = 0; g < n_groups; ++g) {
    const float* x = k + (size_t)g * group;
    float mn = x[0], mx = x[0];
    for (uint32_t j = 1; j < group; ++j) {
      mn = x[j] < mn ? x[j] : mn;
      mx = x[j] > mx ? x[j] : mx;
    }
    float range = mx - mn;
    if (range < 1e-9f) range = 1e-9f;
    float scale = range / 15.0f;
    float sh = f16_bits_to_f32(f32_to_f16_bits(scale));
    if (sh < 6.103515625e-05f) sh = 6.103515625e-05f;
    if (sh > 65504.0f) sh = 65504.0f;
    float zh = f16_bits_to_f32(f32_to_f16_bits(mn));
    if (zh > 65504.0f) zh = 65504.0f;
    if (zh < -65504.0f) zh = -65504.0f;
    scale_h[g] = f32_to_f16_bits(sh);
    zero_h[g] = f32_to_f16_bits(zh);
    for (uint32_t j = 0; j < group; ++j) {
      float c = rintf((x[j] - zh) / sh);
      if (c < 0.0f) c = 0.0f;
      if (c > 15.0f) c = 15.0f;
      codes[(size_t)g * group + j] = (uint8_t)c;
    }
  }
}

void twl_oracle_int4_dequant(const uint8_t* codes, const uint16_t* scale_h, const uint16_t* zero_h,
                             uint32_t n_groups, uint32_t group, float* out) {
  for (uint32_t g = 0; g < n_groups; ++g) {
    float s = f16_bits_to_f32(scale_h[g]);
    float z = f16_bits_to_f32(zero_h[g]);
    for (uint32_t j = 0; j < group; ++j)
      out[(size_t)g * group + j] = (float)codes[(size_t)g * group + j] * s + z;
  }
}
