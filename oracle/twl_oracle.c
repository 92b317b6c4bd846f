/*
 * twl_oracle.c — TEST INFRASTRUCTURE ONLY. CPU restatement (plain C, scalar, one thread) of the
 * loop-heavy parts of Twilight's Select-then-Prune decode path. Nothing in the shipped library or
 * package may link or call this file; tests, the smoke check and the CPU-baseline leg of the
 * benchmark use it as the checker.
 *
 * What is restated, and from where:
 *   twl_oracle_top_p_f32   csrc/include/sampling.cuh:156-231 (TopPReturnMaskKernel after its dead
 *                          max pass :135-155), rows/cols as csrc/src/sampling.cu:51-60
 *   twl_oracle_top_p_f16   the same kernel instantiated with a 16-bit DType (sampling.cu:22-43);
 *                          pivots live in the 16-bit type, the partial sums are kept in fp32
 *                          (the reference sums in the 16-bit type, in an order fixed by CUB's
 *                          block reduction, which a sequential restatement cannot reproduce:
 *                          PARITY UNPINNED for the 16-bit entry, except on rows whose sums and
 *                          midpoints are exact in every width, tests/golden "top_p_dyadic")
 *   twl_oracle_nucleus     textbook nucleus set (sort descending, cumulative sum in fp64):
 *                          the mathematical definition the bisection approximates
 *   twl_oracle_int4_quant  twilight/pyimpl/quantize.py:4-13 applied per group, with the fp16
 *                          rounding of scale / zero that the storage format of this build adds
 *   twl_oracle_int4_dequant  nibble * scale + zero, one fp32 rounding
 *
 * Pinning (see tests/test_oracle_*.py): top-p against twl_oracle_nucleus + brute force over all
 * subsets for d <= 12 + degenerate rows; quant against the known-answer vector of
 * twilight/pyimpl/quantize.py:30-48 evaluated by hand, min/max reproduction and |err| <= scale/2.
 *
 * Block sums: the reference adds fp32 values in a tree order chosen by cub::BlockReduce. Any
 * order is a valid fp32 evaluation of the same sum; this file accumulates in fp64 and rounds once,
 * which is within an ulp or two of every such order.
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

/* round a float to the value set of the 16-bit type: 0 = fp16, 1 = bf16, 2 = none (fp32) */
static float round_to(float v, int dtype) {
  if (dtype == 0) return f16_bits_to_f32(f32_to_f16_bits(v));
  if (dtype == 1) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  return v;
}

/* ---- top-p bisection ------------------------------------------------------------------------- */
/* One row of csrc/include/sampling.cuh:156-231. x[] already holds the row as floats (for 16-bit
 * inputs: the exact values of the 16-bit numbers). dtype selects the arithmetic of the pivots. */
static void top_p_row(const float* x, uint32_t d, float p_in, int high_mode, int dtype,
                      uint8_t* mask, float* low_out, int32_t* iters_out, float* margin_out) {
  float p = round_to(p_in, dtype); /* DType p = DType(top_p...)            sampling.cuh:125 */
  float low = 0.0f;                /*                                       sampling.cuh:159 */
  float high;
  if (high_mode == 0) {
    high = x[0];                   /* "load attention sink"                 sampling.cuh:156-159 */
  } else {
    high = 0.0f;                   /* paper Algorithm 1: r = max(W) */
    for (uint32_t j = 0; j < d; ++j) high = x[j] > high ? x[j] : high;
  }
  const float eps = round_to(1e-5f, dtype); /*                              sampling.cuh:162 */
  float min_gt_low, max_le_high;
  int32_t iters = 0;
  double margin = 1e30; /* smallest |S - p| met: how close a decision came to a rounding flip */
  do {                                       /*                             sampling.cuh:171 */
    float mid = round_to((low + high) / 2.0f, dtype); /*                    sampling.cuh:173 */
    min_gt_low = high;                       /*                             sampling.cuh:174 */
    max_le_high = low;                       /*                             sampling.cuh:175 */
    double sum = 0.0;
    for (uint32_t j = 0; j < d; ++j) {
      float v = x[j];
      if (v > mid) sum += (double)v;                         /* :183,191-193 */
      if (v > low && v < min_gt_low) min_gt_low = v;          /* :184-186 */
      if (v <= high && v > max_le_high) max_le_high = v;      /* :187-189 */
    }
    float s = (float)sum; /* fp32 partial sums for every dtype */
    if (fabs(sum - (double)p) < margin) margin = fabs(sum - (double)p);
    if (s >= p) {                            /*                             sampling.cuh:211-213 */
      low = mid;
    } else {                                 /*                             sampling.cuh:214-216 */
      high = mid < max_le_high ? mid : max_le_high;
    }
    ++iters;
    if (iters > 4096) break; /* cannot happen for finite input; guards a NaN row */
  } while (round_to(max_le_high - min_gt_low, dtype) > eps); /*             sampling.cuh:217 */
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
    top_p_row(probs + (size_t)r * d, d, p_arr ? p_arr[r] : p, high_mode, 2,
              mask ? mask + (size_t)r * d : NULL, low_out ? low_out + r : NULL,
              iters_out ? iters_out + r : NULL, margin_out ? margin_out + r : NULL);
  }
}

/* probs: 16-bit patterns, dtype 0 = fp16, 1 = bf16 */
void twl_oracle_top_p_f16(const uint16_t* probs, int dtype, uint8_t* mask, const float* p_arr,
                          float p, uint32_t rows, uint32_t d, int high_mode, float* low_out,
                          int32_t* iters_out, float* margin_out) {
  float* x = (float*)malloc(sizeof(float) * (size_t)d);
  for (uint32_t r = 0; r < rows; ++r) {
    const uint16_t* src = probs + (size_t)r * d;
    for (uint32_t j = 0; j < d; ++j)
      x[j] = dtype == 0 ? f16_bits_to_f32(src[j]) : bf16_bits_to_f32(src[j]);
    top_p_row(x, d, p_arr ? p_arr[r] : p, high_mode, dtype, mask ? mask + (size_t)r * d : NULL,
              low_out ? low_out + r : NULL, iters_out ? iters_out + r : NULL,
              margin_out ? margin_out + r : NULL);
  }
  free(x);
}

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
