// KV-append side of the path: INT4 shadow records and Quest min/max metadata from paged K.
//
// The quantiser restates twilight/pyimpl/quantize.py:4-13 (asymmetric min/max, 4 bits) per group
// of 32 channels, storing scale and zero (= group minimum) as fp16 and computing the code from the
// ROUNDED scale / zero so that code * scale + zero is what the GEMV will see. The reference
// re-quantises all of K on every decode step (twilight/pyimpl/attention.py:247-251); here it runs
// once per page when the page is written. The metadata is the channel-wise min / max over the
// page's valid tokens, the stored form of the per-chunk amax of twilight/pyimpl/quest.py:68-74.
//
// One wavefront per (page, kv head): lane l = token l/4, group l%4 reads its 32 channels
// (4 x 16 B), quantises them in registers and writes 16 B of nibbles + one (scale, zero) pair;
// the page tile is staged through LDS once for the per-channel min / max.
#include "twl_common.h"

namespace twl {

struct ShadowArgs {
  const void* k_cache;
  uint64_t page_stride, token_stride, head_stride;
  const int32_t* page_ids;
  const int32_t* valid_len;
  uint32_t num_pages, num_kv_heads;
  uint8_t* k_int4;
  uint8_t* meta;
};

constexpr int kShThreads = 256;
constexpr int kShWaves = kShThreads / kWave;

template <int DT>
__global__ __launch_bounds__(kShThreads) void kv_shadow_kernel(ShadowArgs a) {
  __shared__ float tile[kShWaves][TWL_PAGE][TWL_HEAD_DIM + 4];
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  const uint32_t item = blockIdx.x * kShWaves + wave;
  const bool active = item < a.num_pages * a.num_kv_heads;  // wave-uniform
  const uint32_t pi = active ? item / a.num_kv_heads : 0;
  const uint32_t kvh = active ? item - pi * a.num_kv_heads : 0;
  const int page = a.page_ids ? a.page_ids[pi] : (int)pi;
  const int valid = a.valid_len ? min(max(a.valid_len[pi], 0), TWL_PAGE) : TWL_PAGE;
  const int t = lane >> 2, g = lane & 3;

  float x[32];
  if (active) {
    const uint16_t* src = (const uint16_t*)a.k_cache + (size_t)page * a.page_stride +
                          (size_t)t * a.token_stride + (size_t)kvh * a.head_stride + 32 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      u32x4 v = *(const u32x4*)(src + 8 * i);
      const uint32_t ws[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[8 * i + 2 * j] = bits16_to_f32<DT>(ws[j] & 0xFFFFu);
        x[8 * i + 2 * j + 1] = bits16_to_f32<DT>(ws[j] >> 16);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = 0.0f;
  }

  if (active && a.k_int4) {
    uint8_t* rec = a.k_int4 + ((size_t)page * a.num_kv_heads + kvh) * TWL_INT4_RECORD_BYTES;
    u32x4 packed = {0u, 0u, 0u, 0u};
    uint32_t sz = 0;
    if (t < valid) {
      float mn = x[0], mx = x[0];
#pragma unroll
      for (int i = 1; i < 32; ++i) {
        mn = fminf(mn, x[i]);
        mx = fmaxf(mx, x[i]);
      }
      const float range = fmaxf(mx - mn, 1e-9f);
      float sh = round_to<TWL_F16>(range / 15.0f);
      sh = fminf(fmaxf(sh, 6.103515625e-05f), 65504.0f);
      float zh = round_to<TWL_F16>(mn);
      zh = fminf(fmaxf(zh, -65504.0f), 65504.0f);
      uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        float c = rintf((x[i] - zh) / sh);
        c = fminf(fmaxf(c, 0.0f), 15.0f);
        w[i >> 3] |= (uint32_t)c << (4 * (i & 7));
      }
      packed.x = w[0]; packed.y = w[1]; packed.z = w[2]; packed.w = w[3];
      sz = f32_to_f16_bits(sh) | (f32_to_f16_bits(zh) << 16);
    }
    *(u32x4*)(rec + 16 * lane) = packed;
    *(uint32_t*)(rec + 1024 + 4 * lane) = sz;
  }

  if (a.meta) {  // uniform across the block: barriers below are reached by every thread
#pragma unroll
    for (int i = 0; i < 32; ++i) tile[wave][t][32 * g + i] = x[i];
    __syncthreads();
    if (active) {
      // lane l reduces channels 2l and 2l+1 over the valid tokens
      float mn0 = __builtin_inff(), mn1 = __builtin_inff();
      float mx0 = -__builtin_inff(), mx1 = -__builtin_inff();
      for (int tt = 0; tt < valid; ++tt) {
        const float v0 = tile[wave][tt][2 * lane], v1 = tile[wave][tt][2 * lane + 1];
        mn0 = fminf(mn0, v0); mx0 = fmaxf(mx0, v0);
        mn1 = fminf(mn1, v1); mx1 = fmaxf(mx1, v1);
      }
      if (valid == 0) { mn0 = mn1 = mx0 = mx1 = 0.0f; }
      uint8_t* rec = a.meta + ((size_t)page * a.num_kv_heads + kvh) * TWL_META_RECORD_BYTES;
      const int c = lane >> 1, o = (lane & 1) * 4;
      *(uint32_t*)(rec + 16 * c + o) = f32_to_bits16<DT>(mn0) | (f32_to_bits16<DT>(mn1) << 16);
      *(uint32_t*)(rec + 16 * c + 8 + o) = f32_to_bits16<DT>(mx0) | (f32_to_bits16<DT>(mx1) << 16);
    }
  }
}

// Decode append: one new token per request goes into slot kv_last_page_len[b] of the request's
// last page (the host has made sure that page exists and, when it is a fresh page, has set the
// length to 0), K and V rows are stored, the token's part of the INT4 record is quantised, the
// page's min / max metadata is folded with the new row, and the length is advanced. One workgroup
// per request; its wavefronts share the kv heads.
struct AppendArgs {
  const void* k_new;
  const void* v_new;
  uint64_t new_batch_stride, new_head_stride;
  void* k_cache;
  void* v_cache;
  uint64_t page_stride, token_stride, head_stride;
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  int32_t* kv_last_page_len;
  uint32_t num_kv_heads;
  uint8_t* k_int4;
  uint8_t* meta;
  uint16_t* planes;     // nullable: metadata in plane layout (meta_planes.hip)
  uint32_t plane_cap;
  const int32_t* plane_slots;  // nullable: plane slot of each batch position
  uint32_t plane_num_slots;
};

// 16 wavefronts per request: a kv head is a chain of two or three dependent memory round trips
// (row in, records / runs in, results out), so heads run side by side rather than one after the
// other (4 wavefronts: 55 us per call at 32 kv heads; one workgroup per request is kept because
// the request's length is read by every wavefront and advanced once at the end)
constexpr int kAppendThreads = 1024;
constexpr int kAppendWaves = kAppendThreads / kWave;

template <int DT>
__global__ __launch_bounds__(kAppendThreads) void kv_append_kernel(AppendArgs a) {
  const uint32_t b = blockIdx.x;
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  const int pg_end = a.kv_page_indptr[b + 1];
  const int n_pages = pg_end - a.kv_page_indptr[b];
  const int slot = a.kv_last_page_len[b];
  __syncthreads();  // every wave has read the length before it is advanced below
  if (n_pages <= 0 || slot < 0 || slot >= TWL_PAGE) return;  // nothing sane to do; length untouched
  const int page = a.kv_page_indices[pg_end - 1];
  const bool use_planes = a.planes && n_pages <= (int)a.plane_cap;
  const uint32_t pslot = use_planes ? plane_slot(a.plane_slots, a.plane_num_slots, b) : 0u;
  constexpr int HU = 2;  // heads in flight per wavefront: their loads overlap
  for (uint32_t kvh0 = wave; kvh0 < a.num_kv_heads; kvh0 += HU * kAppendWaves) {
    uint32_t kw[HU], vw[HU], om[HU], ox[HU];
    const int mc = lane >> 1, mo = (lane & 1) * 4;
    // ---- every load first: the stores below may alias them as far as the compiler knows, and a
    // load issued after a store waits for a memory round trip of its own -------------------------
#pragma unroll
    for (int u = 0; u < HU; ++u) {
      const uint32_t kvh = kvh0 + u * kAppendWaves;
      kw[u] = vw[u] = om[u] = ox[u] = 0u;
      if (kvh < a.num_kv_heads) {
        const size_t src_off = (size_t)b * a.new_batch_stride + (size_t)kvh * a.new_head_stride;
        kw[u] = *((const uint32_t*)((const uint16_t*)a.k_new + src_off) + lane);  // 2 channels per lane
        vw[u] = *((const uint32_t*)((const uint16_t*)a.v_new + src_off) + lane);
        if (a.meta && slot > 0) {
          const uint8_t* mrec = a.meta + ((size_t)page * a.num_kv_heads + kvh) * TWL_META_RECORD_BYTES;
          om[u] = *(const uint32_t*)(mrec + 16 * mc + mo);
          ox[u] = *(const uint32_t*)(mrec + 16 * mc + 8 + mo);
        }
      }
    }
    // ---- stores ------------------------------------------------------------------------------
#pragma unroll
    for (int u = 0; u < HU; ++u) {
      const uint32_t kvh = kvh0 + u * kAppendWaves;
      if (kvh >= a.num_kv_heads) continue;  // wave-uniform
      const size_t dst_off = (size_t)page * a.page_stride + (size_t)slot * a.token_stride +
                             (size_t)kvh * a.head_stride;
      const float k0 = bits16_to_f32<DT>(kw[u] & 0xFFFFu), k1 = bits16_to_f32<DT>(kw[u] >> 16);
      *((uint32_t*)((uint16_t*)a.k_cache + dst_off) + lane) = kw[u];
      *((uint32_t*)((uint16_t*)a.v_cache + dst_off) + lane) = vw[u];
      if (a.k_int4) {
        uint8_t* rec = a.k_int4 + ((size_t)page * a.num_kv_heads + kvh) * TWL_INT4_RECORD_BYTES;
        if (slot == 0) {  // a fresh page: the other 15 tokens' parts read as "not written"
          *(u32x4*)(rec + 16 * lane) = u32x4{0u, 0u, 0u, 0u};
          *(uint32_t*)(rec + 1024 + 4 * lane) = 0u;
        }
        // The new row's 4 groups of 32 channels, 16 lanes per group, 2 channels per lane: the
        // same arithmetic per element as kv_shadow_kernel (min / max are order-independent), two
        // divisions per lane instead of 32 in a row on four lanes.
        const float mn = row16_allreduce<OpMin>(fminf(k0, k1));
        const float mx = row16_allreduce<OpMax>(fmaxf(k0, k1));
        const float range = fmaxf(mx - mn, 1e-9f);
        float sh = round_to<TWL_F16>(range / 15.0f);
        sh = fminf(fmaxf(sh, 6.103515625e-05f), 65504.0f);
        float zh = round_to<TWL_F16>(mn);
        zh = fminf(fmaxf(zh, -65504.0f), 65504.0f);
        float c0 = rintf((k0 - zh) / sh), c1 = rintf((k1 - zh) / sh);
        c0 = fminf(fmaxf(c0, 0.0f), 15.0f);
        c1 = fminf(fmaxf(c1, 0.0f), 15.0f);
        // channels 2r, 2r+1 (r = lane % 16) are byte r % 4 of dword r / 4 of the group's 16 bytes
        int wv = (int)(((uint32_t)c0 | ((uint32_t)c1 << 4)) << (8 * (lane & 3)));
        wv |= dpp<kDppXor1>(0, wv);
        wv |= dpp<kDppXor2>(0, wv);
        const int li = 4 * slot + (lane >> 4);  // the record's (token, group) index
        if ((lane & 3) == 0) *(uint32_t*)(rec + 16 * li + 4 * ((lane & 15) >> 2)) = (uint32_t)wv;
        if ((lane & 15) == 0)
          *(uint32_t*)(rec + 1024 + 4 * li) = f32_to_f16_bits(sh) | (f32_to_f16_bits(zh) << 16);
      }
      if (a.meta) {  // lane l folds channels 2l, 2l+1 into the page's min / max
        uint8_t* mrec = a.meta + ((size_t)page * a.num_kv_heads + kvh) * TWL_META_RECORD_BYTES;
        float mn0 = k0, mn1 = k1, mx0 = k0, mx1 = k1;
        if (slot > 0) {
          mn0 = fminf(mn0, bits16_to_f32<DT>(om[u] & 0xFFFFu));
          mn1 = fminf(mn1, bits16_to_f32<DT>(om[u] >> 16));
          mx0 = fmaxf(mx0, bits16_to_f32<DT>(ox[u] & 0xFFFFu));
          mx1 = fmaxf(mx1, bits16_to_f32<DT>(ox[u] >> 16));
        }
        const uint32_t bmn0 = f32_to_bits16<DT>(mn0), bmn1 = f32_to_bits16<DT>(mn1);
        const uint32_t bmx0 = f32_to_bits16<DT>(mx0), bmx1 = f32_to_bits16<DT>(mx1);
        *(uint32_t*)(mrec + 16 * mc + mo) = bmn0 | (bmn1 << 16);
        *(uint32_t*)(mrec + 16 * mc + 8 + mo) = bmx0 | (bmx1 << 16);
        if (use_planes && slot == TWL_PAGE - 1) {
          // This token completes the page: its min / max go to the plane layout (runs
          // [d][min|max][logical page] of the request's slot), 256 scattered 2-byte stores per
          // head, once per 16 tokens. Until then the scoring passes take a request's last page
          // from the record above, so the planes are not touched on the other 15 steps (folding
          // them every step cost 8 of 15 us per call at 8 requests x 32 kv heads).
          uint16_t* pl = a.planes +
                         ((size_t)pslot * a.num_kv_heads + kvh) * (TWL_HEAD_DIM * 2) * a.plane_cap +
                         (n_pages - 1);
          pl[(size_t)(4 * lane + 0) * a.plane_cap] = (uint16_t)bmn0;
          pl[(size_t)(4 * lane + 1) * a.plane_cap] = (uint16_t)bmx0;
          pl[(size_t)(4 * lane + 2) * a.plane_cap] = (uint16_t)bmn1;
          pl[(size_t)(4 * lane + 3) * a.plane_cap] = (uint16_t)bmx1;
        }
      }
    }
  }
  if (threadIdx.x == 0) a.kv_last_page_len[b] = slot + 1;
}

// one thread per (record, token, group): 32 outputs
__global__ __launch_bounds__(256) void dequant_int4_kernel(const uint8_t* k_int4,
                                                           uint32_t num_records, float* out) {
  const uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  const uint64_t rec_i = gid >> 6;
  if (rec_i >= num_records) return;
  const int l = (int)(gid & 63);
  const uint8_t* rec = k_int4 + rec_i * TWL_INT4_RECORD_BYTES;
  u32x4 v = *(const u32x4*)(rec + 16 * l);
  const uint32_t sz = *(const uint32_t*)(rec + 1024 + 4 * l);
  const float scale = f16_bits_to_f32(sz & 0xFFFFu), zero = f16_bits_to_f32(sz >> 16);
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  float* dst = out + rec_i * (TWL_PAGE * TWL_HEAD_DIM) + 32 * l;  // token l/4, group l%4
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const float c = (float)((w[i >> 3] >> (4 * (i & 7))) & 0xFu);
    dst[i] = fmaf(c, scale, zero);
  }
}

}  // namespace twl

extern "C" int twl_kv_shadow_build(const void* k_cache, int kv_dtype, uint64_t page_stride,
                                   uint64_t token_stride, uint64_t head_stride,
                                   const int32_t* page_ids, const int32_t* valid_len,
                                   uint32_t num_pages, uint32_t num_kv_heads, void* k_int4,
                                   void* meta, void* stream) {
  if (!k_cache || (!k_int4 && !meta)) return TWL_ENULL;
  if (kv_dtype != TWL_F16 && kv_dtype != TWL_BF16) return TWL_EDTYPE;
  if (num_pages == 0 || num_kv_heads == 0) return TWL_EINVAL;
  if ((uint64_t)num_pages * num_kv_heads > 0x7FFFFFFFull) return TWL_EINVAL;
  if ((page_stride | token_stride | head_stride) & 7u) return TWL_EALIGN;
  if ((((uintptr_t)k_cache) & 15u) || (((uintptr_t)k_int4) & 15u) || (((uintptr_t)meta) & 15u))
    return TWL_EALIGN;
  twl::ShadowArgs a{};
  a.k_cache = k_cache; a.page_stride = page_stride; a.token_stride = token_stride;
  a.head_stride = head_stride; a.page_ids = page_ids; a.valid_len = valid_len;
  a.num_pages = num_pages; a.num_kv_heads = num_kv_heads; a.k_int4 = (uint8_t*)k_int4;
  a.meta = (uint8_t*)meta;
  const uint32_t items = num_pages * num_kv_heads;
  dim3 grid((items + twl::kShWaves - 1) / twl::kShWaves);
  if (kv_dtype == TWL_F16)
    hipLaunchKernelGGL((twl::kv_shadow_kernel<TWL_F16>), grid, dim3(twl::kShThreads), 0,
                       (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL((twl::kv_shadow_kernel<TWL_BF16>), grid, dim3(twl::kShThreads), 0,
                       (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_dequant_int4(const void* k_int4, uint32_t num_records, float* out,
                                void* stream) {
  if (!k_int4 || !out) return TWL_ENULL;
  if (num_records == 0 || num_records > (1u << 25)) return TWL_EINVAL;
  if ((((uintptr_t)k_int4) & 15u) || (((uintptr_t)out) & 3u)) return TWL_EALIGN;
  const uint64_t threads = (uint64_t)num_records * 64;
  hipLaunchKernelGGL(twl::dequant_int4_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256),
                     0, (hipStream_t)stream, (const uint8_t*)k_int4, num_records, out);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

extern "C" int twl_kv_append(const void* k_new, const void* v_new, int kv_dtype,
                             uint64_t new_batch_stride, uint64_t new_head_stride, void* k_cache,
                             void* v_cache, uint64_t page_stride, uint64_t token_stride,
                             uint64_t head_stride, const int32_t* kv_page_indices,
                             const int32_t* kv_page_indptr, int32_t* kv_last_page_len,
                             uint32_t batch, uint32_t num_kv_heads, void* k_int4, void* meta,
                             void* meta_planes, uint32_t plane_cap_pages,
                             const int32_t* plane_slots, uint32_t plane_num_slots, void* stream) {
  if (!k_new || !v_new || !k_cache || !v_cache || !kv_page_indices || !kv_page_indptr ||
      !kv_last_page_len)
    return TWL_ENULL;
  if (kv_dtype != TWL_F16 && kv_dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_kv_heads == 0) return TWL_EINVAL;
  if ((page_stride | token_stride | head_stride | new_batch_stride | new_head_stride) & 7u)
    return TWL_EALIGN;
  if ((((uintptr_t)k_new) & 15u) || (((uintptr_t)v_new) & 15u) || (((uintptr_t)k_cache) & 15u) ||
      (((uintptr_t)v_cache) & 15u) || (((uintptr_t)k_int4) & 15u) || (((uintptr_t)meta) & 15u) ||
      (((uintptr_t)meta_planes) & 15u))
    return TWL_EALIGN;
  if (meta_planes && (plane_cap_pages == 0 || (plane_cap_pages & 7u))) return TWL_EINVAL;
  if (meta_planes && plane_slots && plane_num_slots == 0) return TWL_EINVAL;
  if (meta_planes && !meta) return TWL_ENULL;  // the planes are written from the folded record
  twl::AppendArgs a{};
  a.k_new = k_new; a.v_new = v_new; a.new_batch_stride = new_batch_stride;
  a.new_head_stride = new_head_stride; a.k_cache = k_cache; a.v_cache = v_cache;
  a.page_stride = page_stride; a.token_stride = token_stride; a.head_stride = head_stride;
  a.kv_page_indices = kv_page_indices; a.kv_page_indptr = kv_page_indptr;
  a.kv_last_page_len = kv_last_page_len; a.num_kv_heads = num_kv_heads;
  a.k_int4 = (uint8_t*)k_int4; a.meta = (uint8_t*)meta;
  a.planes = (uint16_t*)meta_planes; a.plane_cap = plane_cap_pages;
  a.plane_slots = plane_slots; a.plane_num_slots = plane_num_slots;
  if (kv_dtype == TWL_F16)
    hipLaunchKernelGGL((twl::kv_append_kernel<TWL_F16>), dim3(batch), dim3(twl::kAppendThreads), 0,
                       (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL((twl::kv_append_kernel<TWL_BF16>), dim3(batch), dim3(twl::kAppendThreads), 0,
                       (hipStream_t)stream, a);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}
