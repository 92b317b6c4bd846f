// Sparse paged decode attention over per-row survivor lists.
//
// Restates the masked softmax.V of twilight/pyimpl/attention.py:188-190,299-306 restricted to the
// surviving tokens: logits = sm_scale * q.K in fp32, fp32 softmax over the survivors,
// probabilities rounded to the q dtype (attention.py:302-304), fp32 accumulation of p.V, output
// rounded to the q dtype.
//
// One workgroup (4 wavefronts) per (batch, head) row — after pruning a row keeps tens to a few
// hundred tokens, so rows are short and many. 16 lanes share a token: each lane owns 8 of the
// 128 head dims (one 16-byte load from K, one from V), a wavefront covers 4 tokens per step and
// the workgroup 16. Logits are staged in LDS so that the softmax normaliser is known before any
// probability is rounded, exactly as the reference does.
#include "twl_common.h"

namespace twl {

struct AttnArgs {
  const void* q;
  void* out;
  const void* k_cache;
  const void* v_cache;
  uint64_t page_stride, token_stride, head_stride;
  const int32_t* idx;
  uint32_t idx_stride;
  const int32_t* count;
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  uint32_t num_q_heads, num_kv_heads;
  float sm_scale;
  float* lse_out;
  uint32_t lds_tokens;  // capacity of the logit staging area
};

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / kWave;
constexpr int kAttnTokPerStep = 4 * kAttnWaves;  // 16
constexpr int kAttnUnroll = 4;

template <int DT>
__device__ __forceinline__ void unpack8(const u32x4& v, float* f) {
  const uint32_t ws[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = bits16_to_f32<DT>(ws[j] & 0xFFFFu);
    f[2 * j + 1] = bits16_to_f32<DT>(ws[j] >> 16);
  }
}

template <int DT>
__global__ __launch_bounds__(kAttnThreads) void sparse_attn_kernel(AttnArgs a) {
  extern __shared__ float lds[];  // [lds_tokens] logits, then probabilities
  __shared__ float red[2][16];
  __shared__ float oacc[kAttnWaves][TWL_HEAD_DIM];

  const uint32_t row = blockIdx.x;
  const uint32_t b = row / a.num_q_heads;
  const uint32_t h = row - b * a.num_q_heads;
  const uint32_t kvh = h / (a.num_q_heads / a.num_kv_heads);
  const int tx = threadIdx.x;
  const int lane = lane_id();
  const int wave = tx / kWave;
  const int sub = lane & 15;   // which 8 dims
  const int slot = lane >> 4;  // which of the wave's 4 tokens
  const int n = min(max(a.count[row], 0), (int)min(a.idx_stride, a.lds_tokens));
  uint16_t* orow = (uint16_t*)a.out + (size_t)row * TWL_HEAD_DIM;

  if (n == 0) {
    if (tx < TWL_HEAD_DIM) orow[tx] = 0;
    if (tx == 0 && a.lse_out) a.lse_out[row] = -__builtin_inff();
    return;
  }

  float qf[8];
  {
    u32x4 v = *(const u32x4*)((const uint16_t*)a.q + (size_t)row * TWL_HEAD_DIM + 8 * sub);
    unpack8<DT>(v, qf);
  }
  const int32_t* irow = a.idx + (size_t)row * a.idx_stride;
  const int32_t* ptab = a.kv_page_indices + a.kv_page_indptr[b];
  const size_t head_off = (size_t)kvh * a.head_stride + 8 * sub;
  const uint16_t* kc = (const uint16_t*)a.k_cache;
  const uint16_t* vc = (const uint16_t*)a.v_cache;

  // ---- phase 1: logits -> LDS -------------------------------------------------------------
  float wmax = -__builtin_inff();
  for (int j0 = 0; j0 < n; j0 += kAttnTokPerStep * kAttnUnroll) {
    u32x4 kv[kAttnUnroll];
    int jj[kAttnUnroll];
#pragma unroll
    for (int u = 0; u < kAttnUnroll; ++u) {
      const int j = j0 + u * kAttnTokPerStep + wave * 4 + slot;
      jj[u] = j;
      const int tok = irow[min(j, n - 1)];
      const size_t off = (size_t)ptab[tok >> 4] * a.page_stride +
                         (size_t)(tok & 15) * a.token_stride + head_off;
      kv[u] = *(const u32x4*)(kc + off);
    }
#pragma unroll
    for (int u = 0; u < kAttnUnroll; ++u) {
      float kf[8];
      unpack8<DT>(kv[u], kf);
      float acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc = fmaf(qf[i], kf[i], acc);
      acc = row16_allreduce<OpSum>(acc) * a.sm_scale;
      if (jj[u] < n) {
        wmax = fmaxf(wmax, acc);
        if (sub == 0) lds[jj[u]] = acc;
      }
    }
  }
  const float m = block_allreduce<OpMax, kAttnWaves>(wmax, red[0]);  // barrier inside: LDS visible

  // ---- phase 2: normaliser, probabilities rounded to the q dtype ---------------------------
  float z = 0.0f;
  for (int j = tx; j < n; j += kAttnThreads) {
    const float e = expf(lds[j] - m);
    lds[j] = e;
    z += e;
  }
  z = block_allreduce<OpSum, kAttnWaves>(z, red[1]);
  if (tx == 0 && a.lse_out) a.lse_out[row] = m + logf(z);
  for (int j = tx; j < n; j += kAttnThreads) lds[j] = round_to<DT>(lds[j] / z);
  __syncthreads();

  // ---- phase 3: out = sum_j p_j * V_j -------------------------------------------------------
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
  for (int j0 = 0; j0 < n; j0 += kAttnTokPerStep * kAttnUnroll) {
    u32x4 vv[kAttnUnroll];
    float pj[kAttnUnroll];
#pragma unroll
    for (int u = 0; u < kAttnUnroll; ++u) {
      const int j = j0 + u * kAttnTokPerStep + wave * 4 + slot;
      const int jc = min(j, n - 1);
      const int tok = irow[jc];
      const size_t off = (size_t)ptab[tok >> 4] * a.page_stride +
                         (size_t)(tok & 15) * a.token_stride + head_off;
      vv[u] = *(const u32x4*)(vc + off);
      pj[u] = (j < n) ? lds[jc] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < kAttnUnroll; ++u) {
      float vf[8];
      unpack8<DT>(vv[u], vf);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(pj[u], vf[i], acc[i]);
    }
  }
  // fold the 4 token slots of the wave (lanes l, l^16, l^32, l^48), then the 4 waves
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float v = acc[i];
    v += __shfl_xor(v, 16, kWave);
    v += __shfl_xor(v, 32, kWave);
    acc[i] = v;
  }
  if (slot == 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) oacc[wave][8 * sub + i] = acc[i];
  }
  __syncthreads();
  if (tx < TWL_HEAD_DIM) {
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) v += oacc[w][tx];
    orow[tx] = (uint16_t)f32_to_bits16<DT>(v);
  }
}

}  // namespace twl

extern "C" int twl_sparse_attn(const void* q, void* out, int dtype, const void* k_cache,
                               const void* v_cache, uint64_t page_stride, uint64_t token_stride,
                               uint64_t head_stride, const int32_t* idx, uint32_t idx_stride,
                               const int32_t* count, const int32_t* kv_page_indices,
                               const int32_t* kv_page_indptr, uint32_t batch,
                               uint32_t num_q_heads, uint32_t num_kv_heads, float sm_scale,
                               float* lse_out, void* stream) {
  if (!q || !out || !k_cache || !v_cache || !idx || !count || !kv_page_indices || !kv_page_indptr)
    return TWL_ENULL;
  if (dtype != TWL_F16 && dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (idx_stride == 0 || idx_stride > TWL_MAX_CANDIDATES) return TWL_EINVAL;
  if ((page_stride | token_stride | head_stride) & 7u) return TWL_EALIGN;  // 16-byte loads
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k_cache) & 15u) || (((uintptr_t)v_cache) & 15u) ||
      (((uintptr_t)out) & 1u))
    return TWL_EALIGN;
  twl::AttnArgs a{};
  a.q = q; a.out = out; a.k_cache = k_cache; a.v_cache = v_cache; a.page_stride = page_stride;
  a.token_stride = token_stride; a.head_stride = head_stride; a.idx = idx;
  a.idx_stride = idx_stride; a.count = count; a.kv_page_indices = kv_page_indices;
  a.kv_page_indptr = kv_page_indptr; a.num_q_heads = num_q_heads; a.num_kv_heads = num_kv_heads;
  a.sm_scale = sm_scale; a.lse_out = lse_out; a.lds_tokens = idx_stride;
  const size_t lds_bytes = (size_t)idx_stride * sizeof(float);
  dim3 grid(batch * num_q_heads);
  if (dtype == TWL_F16) {
    if (lds_bytes > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)twl::sparse_attn_kernel<TWL_F16>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    hipLaunchKernelGGL((twl::sparse_attn_kernel<TWL_F16>), grid, dim3(twl::kAttnThreads),
                       lds_bytes, (hipStream_t)stream, a);
  } else {
    if (lds_bytes > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)twl::sparse_attn_kernel<TWL_BF16>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    hipLaunchKernelGGL((twl::sparse_attn_kernel<TWL_BF16>), grid, dim3(twl::kAttnThreads),
                       lds_bytes, (hipStream_t)stream, a);
  }
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
