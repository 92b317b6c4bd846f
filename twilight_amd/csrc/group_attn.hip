// Paged decode attention in which the q heads of a kv head share ONE token list: either every
// token of the request (dense decode: the layers a configuration leaves dense,
// twilight/pyimpl/attention.py:199-201, and the dense baseline) or a list per (request, kv head)
// such as the union of the group's survivor sets. K and V of a token are fetched once and used
// for all G = num_q_heads / num_kv_heads query heads.
//
// Same arithmetic as the masked softmax.V of twilight/pyimpl/attention.py:188-190,299-306 over the
// listed tokens: logits = sm_scale * q.K in fp32, fp32 softmax, fp32 accumulation of p.V, output
// rounded to the q dtype. The weights are not rounded to the q dtype before the V product
// (attention.py:302-304 does): the sums are carried in fp32 flash-decoding style, which differs
// from that rounding by less than the rounding of the output.
//
// Work split: workgroup (chunk, request, head block) owns `chunk` consecutive list positions of
// `hb` kv heads. 16 lanes share a token (a lane owns 8 of the 128 head dims = one 16-byte load of
// K and one of V), so the 256 threads are 16 lane groups = hb kv heads x 16/hb token slots. With
// hb = min(kv heads, 16) in dense mode a load instruction of the workgroup covers whole tokens
// with all their heads: contiguous 4 KB of an NHD cache. Every lane group carries its own running
// (max, sum, acc) over its tokens (no LDS, no barrier in the loop) and leaves it in the workspace;
// a second kernel merges the partial results of a row.
#include "twl_common.h"

namespace twl {

struct GroupAttnArgs {
  const void* q;
  void* out;
  const void* k_cache;
  const void* v_cache;
  uint64_t page_stride, token_stride, head_stride;
  const int32_t* idx;       // [batch, kv heads, idx_stride] or NULL (every token)
  uint32_t idx_stride;
  const int32_t* count;     // [batch, kv heads] (with idx)
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  const int32_t* kv_last_page_len;
  uint32_t batch, num_q_heads, num_kv_heads;
  uint32_t hb_log2;         // kv heads per workgroup = 1 << hb_log2 (<= 16)
  uint32_t chunk;           // list positions per workgroup and kv head (multiple of 64)
  uint32_t max_chunks;
  uint32_t max_tokens;      // dense form: requests are read up to this many tokens
  float scale_log2;         // sm_scale * log2(e)
  float* lse_out;
  float* partials;          // [batch, kv heads, max_chunks, 16 >> hb_log2, G, kGrpPartial]
};

constexpr int kGrpThreads = 256;
constexpr int kGrpPartial = TWL_HEAD_DIM + 4; // m (log2 units), l, 2 unused, acc[128]: 16-byte rows
constexpr int kGrpMaxChunk = 512;
constexpr float kGrpNoMax = -3.0e38f;         // finite stand-in for "no token seen yet"

struct GroupPlan {
  uint32_t hb_log2, chunk, max_chunks;
};

// The launch shape as a function of the call's sizes only (the workspace size follows from it).
inline GroupPlan group_plan(uint32_t batch, uint32_t num_kv_heads, uint32_t max_tokens, bool list) {
  GroupPlan p{};
  if (!list)
    while (p.hb_log2 < 4 && num_kv_heads % (2u << p.hb_log2) == 0) ++p.hb_log2;
  p.chunk = list ? 128 : kGrpMaxChunk;
  const uint64_t groups = (uint64_t)batch * (num_kv_heads >> p.hb_log2);
  if (!list)
    while (p.chunk > 64 && groups * ((max_tokens + p.chunk - 1) / p.chunk) < 512) p.chunk >>= 1;
  p.max_chunks = (max_tokens + p.chunk - 1) / p.chunk;
  if (p.max_chunks == 0) p.max_chunks = 1;
  return p;
}

// tokens of request b / list length of (b, kvh)
__device__ __forceinline__ int group_list_len(const GroupAttnArgs& a, uint32_t b, uint32_t kvh) {
  if (a.idx) return min(max(a.count[b * a.num_kv_heads + kvh], 0), (int)a.idx_stride);
  const int npg = a.kv_page_indptr[b + 1] - a.kv_page_indptr[b];
  if (npg <= 0) return 0;
  return min((npg - 1) * TWL_PAGE + min(max(a.kv_last_page_len[b], 0), TWL_PAGE), (int)a.max_tokens);
}

template <int DT, int G>
__global__ __launch_bounds__(kGrpThreads) void group_attn_partial_kernel(GroupAttnArgs a) {
  // tokens per lane group whose K and V loads are issued together (16 loads of 16 bytes per
  // lane; half of that with 8 q heads per kv head, whose accumulators need the registers)
  constexpr int kGrpUnroll = G >= 8 ? 4 : 8;
  __shared__ int slot_id[kGrpMaxChunk];   // physical token slot = page * 16 + slot in page
  const int tx = threadIdx.x;
  const uint32_t hb = 1u << a.hb_log2, ts = 16u >> a.hb_log2;
  const uint32_t hblocks = a.num_kv_heads >> a.hb_log2;
  const uint32_t b = blockIdx.y / hblocks, hblk = blockIdx.y - b * hblocks;
  const int gid = tx >> 4, sub = tx & 15;
  const uint32_t kvh = hblk * hb + (gid & (hb - 1));
  const int tsel = gid >> a.hb_log2;
  // with a list a workgroup serves one kv head (hb == 1), without one every head has the same
  // length: n is uniform over the workgroup
  const int n = group_list_len(a, b, kvh);
  // dense form: one chunk per workgroup; with lists (mostly far shorter than their stride) the
  // grid holds a few chunks per kv head and a workgroup walks the chunks of a long list
  for (uint32_t ch = blockIdx.x; (int)(ch * a.chunk) < n; ch += gridDim.x) {
    const int j0 = ch * a.chunk;
    const int cn = min((int)a.chunk, n - j0);

    // ---- resolve the chunk's token addresses once --------------------------------------------
    const int pbase = a.kv_page_indptr[b];
    const int plast = max(a.kv_page_indptr[b + 1] - pbase - 1, 0);
    for (int i = tx; i < cn; i += kGrpThreads) {
      const int tok =
          a.idx ? a.idx[((size_t)b * a.num_kv_heads + kvh) * a.idx_stride + j0 + i] : j0 + i;
      // a position outside the request (a corrupt list) is folded onto its last page rather than
      // read past the page table
      slot_id[i] = a.kv_page_indices[pbase + min(max(tok >> 4, 0), plast)] * TWL_PAGE + (tok & 15);
    }
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const u32x4 v = *(const u32x4*)((const uint16_t*)a.q +
                                      ((size_t)b * a.num_q_heads + kvh * G + g) * TWL_HEAD_DIM + 8 * sub);
      unpack8<DT>(v, qf[g]);
#pragma unroll
      for (int d = 0; d < 8; ++d) qf[g][d] *= a.scale_log2;
    }
    __syncthreads();

    const size_t head_off = (size_t)kvh * a.head_stride + 8 * sub;
    const uint16_t* kc = (const uint16_t*)a.k_cache;
    const uint16_t* vc = (const uint16_t*)a.v_cache;
    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      m[g] = kGrpNoMax;
      l[g] = 0.0f;
#pragma unroll
      for (int d = 0; d < 8; ++d) acc[g][d] = 0.0f;
    }

    const int steps = (cn + (int)ts - 1) / (int)ts;   // list positions tsel + ts * s, s < steps
    for (int s0 = 0; s0 < steps; s0 += kGrpUnroll) {
      u32x4 kreg[kGrpUnroll], vreg[kGrpUnroll];
      bool valid[kGrpUnroll];
      size_t off[kGrpUnroll];
#pragma unroll
      for (int u = 0; u < kGrpUnroll; ++u) {
        const int t = tsel + (int)ts * (s0 + u);
        valid[u] = t < cn;
        const int sid = slot_id[min(t, cn - 1)];
        off[u] = (size_t)(sid >> 4) * a.page_stride + (size_t)(sid & 15) * a.token_stride + head_off;
        kreg[u] = __builtin_nontemporal_load((const u32x4*)(kc + off[u]));
      }
#pragma unroll
      for (int u = 0; u < kGrpUnroll; ++u)
        vreg[u] = __builtin_nontemporal_load((const u32x4*)(vc + off[u]));

      float sc[kGrpUnroll][G];
#pragma unroll
      for (int u = 0; u < kGrpUnroll; ++u) {
        float kf[8];
        unpack8<DT>(kreg[u], kf);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          float d0 = 0.0f;
#pragma unroll
          for (int d = 0; d < 8; ++d) d0 = fmaf(qf[g][d], kf[d], d0);
          d0 = row16_allreduce<OpSum>(d0);
          sc[u][g] = valid[u] ? d0 : -__builtin_inff();
        }
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float mn = m[g];
#pragma unroll
        for (int u = 0; u < kGrpUnroll; ++u) mn = fmaxf(mn, sc[u][g]);
        const float f = __builtin_amdgcn_exp2f(m[g] - mn);
        m[g] = mn;
        float ps = 0.0f;
#pragma unroll
        for (int u = 0; u < kGrpUnroll; ++u) {
          sc[u][g] = __builtin_amdgcn_exp2f(sc[u][g] - mn);   // now the weight
          ps += sc[u][g];
        }
        l[g] = fmaf(l[g], f, ps);
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[g][d] *= f;
      }
#pragma unroll
      for (int u = 0; u < kGrpUnroll; ++u) {
        float vf[8];
        unpack8<DT>(vreg[u], vf);
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int d = 0; d < 8; ++d) acc[g][d] = fmaf(sc[u][g], vf[d], acc[g][d]);
      }
    }

    // ---- leave the lane group's partial result -------------------------------------------------
    float* part = a.partials +
                  ((((size_t)b * a.num_kv_heads + kvh) * a.max_chunks + ch) * ts + tsel) *
                      (size_t)(G * kGrpPartial);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float* pg = part + g * kGrpPartial;
      if (sub == 0) {
        pg[0] = m[g];
        pg[1] = l[g];
      }
      f32x4* dst = (f32x4*)(pg + 4 + 8 * sub);
      dst[0] = f32x4{acc[g][0], acc[g][1], acc[g][2], acc[g][3]};
      dst[1] = f32x4{acc[g][4], acc[g][5], acc[g][6], acc[g][7]};
    }
    __syncthreads();   // slot_id is rewritten by the next chunk
  }
}

// One workgroup per (request, q head) merges the row's partial results: 16 slices of 32 threads,
// a thread folds 4 of the 128 dims over every 16th partial with a running maximum, and the slices
// are folded through LDS.
constexpr int kMergeThreads = 512;
constexpr int kMergeSlices = kMergeThreads / 32;

template <int DT>
__global__ __launch_bounds__(kMergeThreads) void group_attn_merge_kernel(GroupAttnArgs a) {
  __shared__ float sm_m[kMergeSlices], sm_l[kMergeSlices];
  __shared__ f32x4 sm_o[kMergeSlices][32];
  const uint32_t row = blockIdx.x;
  const uint32_t b = row / a.num_q_heads, h = row - b * a.num_q_heads;
  const uint32_t G = a.num_q_heads / a.num_kv_heads;
  const uint32_t kvh = h / G, g = h - kvh * G;
  const uint32_t ts = 16u >> a.hb_log2;
  const int tx = threadIdx.x, dq = tx & 31, slice = tx >> 5;
  uint16_t* orow = (uint16_t*)a.out + (size_t)row * TWL_HEAD_DIM;
  const int n = group_list_len(a, b, kvh);
  if (n == 0) {
    if (tx < TWL_HEAD_DIM) orow[tx] = 0;
    if (tx == 0 && a.lse_out) a.lse_out[row] = -__builtin_inff();
    return;
  }
  const int nparts = ((n + (int)a.chunk - 1) / (int)a.chunk) * (int)ts;
  const size_t pstride = (size_t)G * kGrpPartial;
  const float* base = a.partials + ((size_t)b * a.num_kv_heads + kvh) * a.max_chunks * ts * pstride +
                      (size_t)g * kGrpPartial;
  float m = kGrpNoMax, l = 0.0f;
  f32x4 o = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int p0 = slice; p0 < nparts; p0 += 4 * kMergeSlices) {
    u32x2 ml[4];
    f32x4 pa[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float* r = base + (size_t)min(p0 + u * kMergeSlices, nparts - 1) * pstride;
      ml[u] = *(const u32x2*)r;
      pa[u] = *(const f32x4*)(r + 4 + 4 * dq);
    }
    float pm[4], mn = m;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      pm[u] = (p0 + u * kMergeSlices < nparts) ? as_f32(ml[u].x) : kGrpNoMax;
      mn = fmaxf(mn, pm[u]);
    }
    const float f0 = __builtin_amdgcn_exp2f(m - mn);
    l *= f0;
    o *= f0;
    m = mn;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float f = (p0 + u * kMergeSlices < nparts) ? __builtin_amdgcn_exp2f(pm[u] - mn) : 0.0f;
      l = fmaf(as_f32(ml[u].y), f, l);
      o += pa[u] * f;
    }
  }
  if (dq == 0) {
    sm_m[slice] = m;
    sm_l[slice] = l;
  }
  sm_o[slice][dq] = o;
  __syncthreads();
  if (tx >= 32) return;
  float gm = kGrpNoMax;
#pragma unroll
  for (int s = 0; s < kMergeSlices; ++s) gm = fmaxf(gm, sm_m[s]);
  float gl = 0.0f;
  f32x4 go = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int s = 0; s < kMergeSlices; ++s) {
    const float f = __builtin_amdgcn_exp2f(sm_m[s] - gm);
    gl = fmaf(sm_l[s], f, gl);
    go += sm_o[s][dq] * f;
  }
  const float inv = 1.0f / gl;
  u32x2 packed;
  packed.x = f32_to_bits16<DT>(go.x * inv) | (f32_to_bits16<DT>(go.y * inv) << 16);
  packed.y = f32_to_bits16<DT>(go.z * inv) | (f32_to_bits16<DT>(go.w * inv) << 16);
  *(u32x2*)(orow + 4 * dq) = packed;
  // m is in log2 units (the logits were scaled by log2 e): back to natural logarithms
  if (tx == 0 && a.lse_out) a.lse_out[row] = (gm + log2f(gl)) * 0.6931471805599453f;
}

template <int DT>
static int launch_group_attn(const GroupAttnArgs& a, hipStream_t stream) {
  const uint32_t G = a.num_q_heads / a.num_kv_heads;
  dim3 grid(a.idx ? (a.max_chunks < 16u ? a.max_chunks : 16u) : a.max_chunks,
            a.batch * (a.num_kv_heads >> a.hb_log2));
  dim3 block(kGrpThreads);
  switch (G) {
    case 1: hipLaunchKernelGGL((group_attn_partial_kernel<DT, 1>), grid, block, 0, stream, a); break;
    case 2: hipLaunchKernelGGL((group_attn_partial_kernel<DT, 2>), grid, block, 0, stream, a); break;
    case 4: hipLaunchKernelGGL((group_attn_partial_kernel<DT, 4>), grid, block, 0, stream, a); break;
    case 8: hipLaunchKernelGGL((group_attn_partial_kernel<DT, 8>), grid, block, 0, stream, a); break;
    default: return TWL_EINVAL;
  }
  if (hipGetLastError() != hipSuccess) return TWL_ELAUNCH;
  hipLaunchKernelGGL((group_attn_merge_kernel<DT>), dim3(a.batch * a.num_q_heads),
                     dim3(kMergeThreads), 0, stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

// ---- union of the survivor lists of a kv head's q heads ----------------------------------------
// One workgroup per (request, kv head): the G ascending lists are marked in an LDS bitmap over the
// token positions and the set bits are written back in ascending order.
struct GroupUnionArgs {
  const int32_t* idx;      // [batch, q heads, idx_stride]
  uint32_t idx_stride;
  const int32_t* count;    // [batch, q heads]
  uint32_t num_q_heads, num_kv_heads;
  uint32_t max_tokens;     // token positions are < max_tokens
  int32_t* group_idx;      // [batch, kv heads, group_stride]
  uint32_t group_stride;
  int32_t* group_count;    // [batch, kv heads]
};

constexpr int kUnionThreads = 1024;
constexpr int kUnionWaves = kUnionThreads / kWave;

__global__ __launch_bounds__(kUnionThreads) void group_union_kernel(GroupUnionArgs a) {
  extern __shared__ uint32_t bits[];   // ceil(max_tokens / 32) words
  __shared__ int wave_tot[kUnionWaves];
  __shared__ int running;
  const int tx = threadIdx.x;
  const uint32_t b = blockIdx.x / a.num_kv_heads, kvh = blockIdx.x - b * a.num_kv_heads;
  const uint32_t G = a.num_q_heads / a.num_kv_heads;
  const int words = (int)((a.max_tokens + 31) / 32);
  const size_t row0 = (size_t)b * a.num_q_heads + kvh * G;
  // the G lists as one run of items: item t belongs to list g with cum[g] <= t < cum[g + 1]
  int cum[9];
  cum[0] = 0;
  for (uint32_t g = 0; g < 8; ++g)
    cum[g + 1] = cum[g] + (g < G ? min(max(a.count[row0 + g], 0), (int)a.idx_stride) : 0);
  for (int w = tx; w < words; w += kUnionThreads) bits[w] = 0;
  if (tx == 0) running = 0;
  __syncthreads();
  for (int t = tx; t < cum[8]; t += kUnionThreads) {
    int g = 0;
#pragma unroll
    for (int x = 1; x < 8; ++x) g += (t >= cum[x]) ? 1 : 0;
    const int tok = a.idx[(row0 + g) * a.idx_stride + (t - cum[g])];
    if (tok >= 0 && (uint32_t)tok < a.max_tokens) atomicOr(&bits[tok >> 5], 1u << (tok & 31));
  }
  __syncthreads();
  int32_t* dst = a.group_idx + (size_t)blockIdx.x * a.group_stride;
  const int lane = lane_id(), wave = tx / kWave;
  for (int w0 = 0; w0 < words; w0 += kUnionThreads) {
    const int w = w0 + tx;
    uint32_t v = (w < words) ? bits[w] : 0u;
    const int c = __builtin_popcount(v);
    const int incl = wave_inclusive_scan(c);
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int before = running;
#pragma unroll
    for (int wv = 0; wv < kUnionWaves; ++wv) before += (wv < wave) ? wave_tot[wv] : 0;
    int pos = before + incl - c;
    while (v) {
      const int bit = __builtin_ctz(v);
      v &= v - 1;
      if ((uint32_t)pos < a.group_stride) dst[pos] = w * 32 + bit;
      ++pos;
    }
    __syncthreads();
    if (tx == kUnionThreads - 1) running = before + incl;
    __syncthreads();
  }
  if (tx == 0) a.group_count[blockIdx.x] = min(running, (int)a.group_stride);
}

}  // namespace twl

extern "C" uint64_t twl_group_attn_workspace_bytes(uint32_t batch, uint32_t num_q_heads,
                                                   uint32_t num_kv_heads, uint32_t max_tokens,
                                                   int with_list) {
  if (batch == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0) return 0;
  const twl::GroupPlan p = twl::group_plan(batch, num_kv_heads, max_tokens, with_list != 0);
  const uint64_t parts = (uint64_t)batch * num_kv_heads * p.max_chunks * (16u >> p.hb_log2);
  return parts * (num_q_heads / num_kv_heads) * twl::kGrpPartial * sizeof(float);
}

extern "C" int twl_group_attn(const void* q, void* out, int dtype, const void* k_cache,
                              const void* v_cache, uint64_t page_stride, uint64_t token_stride,
                              uint64_t head_stride, const int32_t* group_idx, uint32_t idx_stride,
                              const int32_t* group_count, uint32_t max_tokens,
                              const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                              const int32_t* kv_last_page_len, uint32_t batch,
                              uint32_t num_q_heads, uint32_t num_kv_heads, float sm_scale,
                              float* lse_out, void* workspace, uint64_t workspace_bytes,
                              void* stream) {
  if (!q || !out || !k_cache || !v_cache || !kv_page_indices || !kv_page_indptr || !workspace)
    return TWL_ENULL;
  const bool list = group_idx != nullptr;
  if (list ? !group_count : !kv_last_page_len) return TWL_ENULL;
  if (dtype != TWL_F16 && dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  const uint32_t G = num_q_heads / num_kv_heads;
  if (G != 1 && G != 2 && G != 4 && G != 8) return TWL_EINVAL;
  if (list) {
    if (idx_stride == 0) return TWL_EINVAL;
    max_tokens = idx_stride;
  }
  if (max_tokens == 0 || max_tokens > (1u << 24)) return TWL_EINVAL;
  if ((uint64_t)batch * num_q_heads > 65535u) return TWL_EINVAL;
  if (workspace_bytes <
      twl_group_attn_workspace_bytes(batch, num_q_heads, num_kv_heads, max_tokens, list))
    return TWL_EINVAL;
  if ((page_stride | token_stride | head_stride) & 7u) return TWL_EALIGN;  // 16-byte loads
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k_cache) & 15u) || (((uintptr_t)v_cache) & 15u) ||
      (((uintptr_t)out) & 7u) || (((uintptr_t)workspace) & 15u))
    return TWL_EALIGN;
  const twl::GroupPlan p = twl::group_plan(batch, num_kv_heads, max_tokens, list);
  if ((uint64_t)batch * (num_kv_heads >> p.hb_log2) > 65535u) return TWL_EINVAL;
  twl::GroupAttnArgs a{};
  a.q = q; a.out = out; a.k_cache = k_cache; a.v_cache = v_cache; a.page_stride = page_stride;
  a.token_stride = token_stride; a.head_stride = head_stride; a.idx = group_idx;
  a.idx_stride = idx_stride; a.count = group_count; a.kv_page_indices = kv_page_indices;
  a.kv_page_indptr = kv_page_indptr; a.kv_last_page_len = kv_last_page_len; a.batch = batch;
  a.num_q_heads = num_q_heads; a.num_kv_heads = num_kv_heads; a.hb_log2 = p.hb_log2;
  a.chunk = p.chunk; a.max_chunks = p.max_chunks; a.max_tokens = max_tokens;
  a.scale_log2 = sm_scale * 1.4426950408889634f;
  a.lse_out = lse_out; a.partials = (float*)workspace;
  return dtype == TWL_F16 ? twl::launch_group_attn<TWL_F16>(a, (hipStream_t)stream)
                          : twl::launch_group_attn<TWL_BF16>(a, (hipStream_t)stream);
}

extern "C" int twl_group_union(const int32_t* idx, uint32_t idx_stride, const int32_t* count,
                               uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                               uint32_t max_tokens, int32_t* group_idx, uint32_t group_stride,
                               int32_t* group_count, void* stream) {
  if (!idx || !count || !group_idx || !group_count) return TWL_ENULL;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0 ||
      idx_stride == 0 || group_stride == 0)
    return TWL_EINVAL;
  if (num_q_heads / num_kv_heads > 8) return TWL_EINVAL;
  if (max_tokens == 0 || max_tokens > 256u * 1024u) return TWL_EINVAL;   // 32 KB bitmap in LDS
  if ((uint64_t)batch * num_kv_heads > 0x7FFFFFFFull) return TWL_EINVAL;
  twl::GroupUnionArgs a{};
  a.idx = idx; a.idx_stride = idx_stride; a.count = count; a.num_q_heads = num_q_heads;
  a.num_kv_heads = num_kv_heads; a.max_tokens = max_tokens; a.group_idx = group_idx;
  a.group_stride = group_stride; a.group_count = group_count;
  const size_t lds = (size_t)((max_tokens + 31) / 32) * sizeof(uint32_t);
  hipLaunchKernelGGL(twl::group_union_kernel, dim3(batch * num_kv_heads),
                     dim3(twl::kUnionThreads), lds, (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
