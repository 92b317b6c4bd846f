// Log-sum-exp of per-block-quantised int8 Q.K^T on the int8 matrix cores.
//
// Restates qk_int8_per_block, twilight/kernel/triton/qk_int8_per_block.py:22-143: for every query
// row m the base-2 log-sum-exp over all keys n of
//     s[m][n] = float(sum_d q[m][d] * k[n][d]) * q_scale[m / 128] * k_scale[n / 64]
// (q_scale / k_scale are per 128-row query block and per 64-row key block, :73-74,38-39; they carry
// the softmax scale and log2(e), so the result is in base 2, :107-109). The reference never adds V
// (its accumulator stays 0, :30-49), so its first output is all zeros and only `lse` carries
// information. Keys past kv_len inside the last 64-block are loaded as zeros by the reference
// (masked tl.load, :36-37) and therefore count as s = 0; the same is done here.
//
// Tiling: a workgroup of 4 wavefronts takes 128 query rows (the q_scale block), a wavefront 32 of
// them; the key tile of a block goes through LDS once for all four. Products run on v_mfma_i32_32x32x32_i8 with the KEY tile as the A operand (rows of the
// product) and the wave's 32 queries as the B operand (columns), so a lane's 16 accumulators all
// belong to ONE query (column = lane % 32) and the running (max, sum) of the online softmax lives
// per lane without any cross-lane traffic; the two lane halves of a query are merged once at the
// end. A and B use the same lane -> k-slice assignment (lane / 32 picks 16 of the 32 depth
// bytes), and integer accumulation is exact, so the product does not depend on which slice the
// hardware pairs with which.
#include "twl_common.h"

namespace twl {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct QkArgs {
  const int8_t* q;
  const int8_t* k;
  const float* q_scale;
  const float* k_scale;
  float* lse;
  int64_t sq_b, sq_h, sq_n;  // byte (= element) strides of q: batch, head, row
  int64_t sk_b, sk_h, sk_n;
  uint32_t H, Hkv, qo_len, kv_len;
};

constexpr int kQkBlockM = 128;
constexpr int kQkBlockN = 64;

template <int HEAD_DIM>
__global__ __launch_bounds__(256) void qk_int8_lse_kernel(QkArgs a) {
  constexpr int KC = HEAD_DIM / 32;  // depth chunks of one matrix instruction
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t mblk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const uint32_t kvh = h / (a.H / a.Hkv);
  const uint32_t m_blocks = (a.qo_len + kQkBlockM - 1) / kQkBlockM;
  const uint32_t n_blocks = (a.kv_len + kQkBlockN - 1) / kQkBlockN;
  const int c = lane & 31;    // query (B operand column) / key row (A operand row) of this lane
  const int g = lane >> 5;    // which 16 depth bytes of a 32-byte chunk
  const uint32_t m = mblk * kQkBlockM + wave * 32 + c;

  const float qs = a.q_scale[((size_t)b * a.H + h) * m_blocks + mblk];
  const float* ks = a.k_scale + ((size_t)b * a.Hkv + kvh) * n_blocks;

  v4i qb[KC];
  {
    const int8_t* qrow = a.q + b * a.sq_b + h * a.sq_h + (int64_t)m * a.sq_n + 16 * g;
#pragma unroll
    for (int kc = 0; kc < KC; ++kc)
      qb[kc] = (m < a.qo_len) ? *(const v4i*)(qrow + 32 * kc) : v4i{0, 0, 0, 0};
  }
  // The key tile of a block (64 keys x HEAD_DIM bytes) is fetched once per workgroup and shared by
  // its four wavefronts through LDS, double-buffered: the next tile is requested before this one
  // is multiplied and stored after, one barrier per block. (Every wavefront fetching the tile for
  // itself made the kernel wait on the L2: 4x the traffic.) Rows are padded by 16 bytes so that
  // the 32 rows an operand load touches spread over the banks.
  constexpr int ROW = HEAD_DIM + 16;
  constexpr int PPK = HEAD_DIM / 16;               // 16-byte pieces per key
  constexpr int PPT = kQkBlockN * PPK / 256;       // pieces per thread and tile (1 or 2)
  __shared__ __align__(16) int8_t ktile[2][kQkBlockN][ROW];
  const int8_t* kbase = a.k + b * a.sk_b + kvh * a.sk_h;
  v4i stage[PPT];
  auto fetch = [&](uint32_t nb) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const uint32_t p = threadIdx.x + 256 * i;
      const uint32_t key = p / PPK, part = p % PPK;
      const uint32_t n = nb * kQkBlockN + key;
      stage[i] = (n < a.kv_len) ? *(const v4i*)(kbase + (int64_t)n * a.sk_n + 16 * part)
                                : v4i{0, 0, 0, 0};
    }
  };
  auto park = [&](int buf) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const uint32_t p = threadIdx.x + 256 * i;
      *(v4i*)&ktile[buf][p / PPK][16 * (p % PPK)] = stage[i];
    }
  };
  fetch(0);
  park(0);
  __syncthreads();

  float run_m = -__builtin_inff(), run_l = 1.0f;  // qk_int8_per_block.py:79-80
  for (uint32_t nb = 0; nb < n_blocks; ++nb) {
    const int buf = nb & 1;
    if (nb + 1 < n_blocks) fetch(nb + 1);
    const float sc = ks[nb];
    v16i acc[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      v4i ka[KC];
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) ka[kc] = *(const v4i*)&ktile[buf][32 * s + c][32 * kc + 16 * g];
      v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int kc = 0; kc < KC; ++kc)
        z = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[kc], qb[kc], z, 0, 0, 0);
      acc[s] = z;
    }
    // online softmax of this lane's 32 scores (qk_int8_per_block.py:39-48). The kernel is bound by
    // this part, not by the matrix cores (8 matrix instructions against 32 exponentials per lane
    // and key block), so it is kept to one integer max, one convert, one fma and one exp2 per
    // score: the block's largest score is the scale times the largest (smallest, for a negative
    // scale) integer product.
    const float s2 = qs * sc;
    int imax = acc[0][0], imin = acc[0][0];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        imax = max(imax, acc[s][v]);
        imin = min(imin, acc[s][v]);
      }
    const float tmax = fmaxf(run_m, fmaxf((float)imax * s2, (float)imin * s2));
    float add = 0.0f, add2 = 0.0f;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float e = __builtin_amdgcn_exp2f(fmaf((float)acc[s][v], s2, -tmax));
        if (v & 1) add2 += e;
        else add += e;
      }
    run_l = run_l * __builtin_amdgcn_exp2f(run_m - tmax) + (add + add2);
    run_m = tmax;
    if (nb + 1 < n_blocks) park(buf ^ 1);  // last read two barriers ago
    __syncthreads();
  }
  // merge the two lane halves of a query: lane c and lane c + 32
  const float om = as_f32(__builtin_amdgcn_ds_bpermute(4 * (lane ^ 32), as_i32(run_m)));
  const float ol = as_f32(__builtin_amdgcn_ds_bpermute(4 * (lane ^ 32), as_i32(run_l)));
  const float mm = fmaxf(run_m, om);
  const float ll = run_l * __builtin_amdgcn_exp2f(run_m - mm) + ol * __builtin_amdgcn_exp2f(om - mm);
  if (g == 0 && m < a.qo_len)
    a.lse[((size_t)b * a.H + h) * a.qo_len + m] = __builtin_log2f(ll) + mm;  // :107-109
}

}  // namespace twl

extern "C" int twl_qk_int8_lse(const int8_t* q, const int8_t* k, const float* q_scale,
                               const float* k_scale, float* lse, uint32_t batch,
                               uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t qo_len,
                               uint32_t kv_len, uint32_t head_dim, int64_t sq_b, int64_t sq_h,
                               int64_t sq_n, int64_t sk_b, int64_t sk_h, int64_t sk_n,
                               void* stream) {
  if (!q || !k || !q_scale || !k_scale || !lse) return TWL_ENULL;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (qo_len == 0 || kv_len == 0) return TWL_EINVAL;
  if (head_dim != 64 && head_dim != 128) return TWL_EINVAL;
  if (num_q_heads > 65535u || batch > 65535u) return TWL_EINVAL;
  // 16-byte vector loads of int8 rows
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k) & 15u) || (((uintptr_t)lse) & 3u)) return TWL_EALIGN;
  const int64_t strides[6] = {sq_b, sq_h, sq_n, sk_b, sk_h, sk_n};
  for (int i = 0; i < 6; ++i)
    if (strides[i] < 0 || (strides[i] & 15)) return TWL_EALIGN;
  twl::QkArgs a{};
  a.q = q; a.k = k; a.q_scale = q_scale; a.k_scale = k_scale; a.lse = lse;
  a.sq_b = sq_b; a.sq_h = sq_h; a.sq_n = sq_n; a.sk_b = sk_b; a.sk_h = sk_h; a.sk_n = sk_n;
  a.H = num_q_heads; a.Hkv = num_kv_heads; a.qo_len = qo_len; a.kv_len = kv_len;
  const dim3 grid((qo_len + twl::kQkBlockM - 1) / twl::kQkBlockM, num_q_heads, batch);
  hipStream_t s = (hipStream_t)stream;
  if (head_dim == 128) hipLaunchKernelGGL((twl::qk_int8_lse_kernel<128>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((twl::qk_int8_lse_kernel<64>), grid, dim3(256), 0, s, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
