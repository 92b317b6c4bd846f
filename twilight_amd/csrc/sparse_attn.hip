// Sparse paged decode attention over per-row survivor lists.
//
// Restates the masked softmax.V of twilight/pyimpl/attention.py:188-190,299-306 restricted to the
// surviving tokens: logits = sm_scale * q.K in fp32, fp32 softmax over the survivors, fp32
// accumulation of p.V, output rounded to the q dtype.
//
// After pruning a row keeps tens to a few hundred tokens, with a long tail of rows that keep
// thousands, so the work is split by tokens, not by rows: workgroup (s, row) owns survivors
// [128 s, 128 s + 128) of its row and exits at once when the row is shorter (split-K across CUs).
// Inside a workgroup (4 wavefronts) 16 lanes share a token: each lane owns 8 of the 128 head dims,
// i.e. one 16-byte load from K and one from V; token addresses are resolved once into LDS and then
// all K and V loads of the chunk are issued before any arithmetic, so a chunk costs about one HBM
// round trip.
//   - A row that fits one chunk is finished in place: probabilities are normalised and rounded to
//     the q dtype before the V product, exactly as attention.py:302-304 does.
//   - A longer row leaves (max, sum, unnormalised acc[128]) per chunk in the workspace; the chunk
//     that finishes last (ticket counter) merges them FlashDecoding-style. There the weights
//     stay in fp32 (no intermediate rounding to the q dtype): the difference is below the output
//     rounding.
#include <atomic>
#include <chrono>

#include "twl_common.h"

#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "the split-row merge relies on how gfx950 orders device-scope write-through stores"
#endif

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
  uint64_t* tickets;  // [rows]: (tag << 16) | chunks finished
  float* partials;    // [rows, max_splits, kAttnPartial]
  uint32_t max_splits;
  uint32_t rows;
  uint32_t pool;      // workgroups that serve chunks 1.. of long rows
  uint64_t epoch;     // 48 bits, never 0, different in every call: tag of this call's ticket words
  const float* weights;  // USE_W kernels only: [rows, idx_stride] weight of survivor j (q, K unused)
};

constexpr int kAttnSteps = 8;                          // tokens per lane group (16 lanes)
constexpr int kAttnPartial = TWL_HEAD_DIM + 2;         // m, l, acc[128]

// A workgroup of THREADS threads owns a chunk of THREADS / 2 survivors: 16 lanes share a token,
// a lane group takes kAttnSteps tokens.
template <int THREADS>
struct AttnSmem {
  static constexpr int kWaves = THREADS / kWave;
  static constexpr int kChunk = THREADS / 16 * kAttnSteps;
  static constexpr int kGroups = 4 * kWaves;
  int slot_id[kChunk];          // physical token slot = page * 16 + slot
  float w[kChunk];              // logits, then weights
  float red[2][16];
  float oacc[kGroups][TWL_HEAD_DIM];
  int is_last;
};

// Thread 0 of every chunk of a split row, before the chunk's loads are waited for: make the row's
// ticket word carry this call's tag. A word with another tag (zero included) is a leftover and is
// replaced by (tag << 16); when the exchange fails somebody else has just done the same. The
// word is requested ahead of the chunk's K / V loads (`seen`) and looked at after the logits, so
// the round trip hides behind them; the fetch_add at the end of the chunk, the one on the critical
// path, stays a single operation.
__device__ __forceinline__ void tag_ticket(uint64_t* tk, uint64_t seen, uint64_t epoch) {
  while ((seen >> 16) != epoch) {
    if (__hip_atomic_compare_exchange_strong(tk, &seen, epoch << 16, __ATOMIC_RELAXED,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      break;
  }
}

// One chunk (survivors [128*split, 128*split+128) of `row`, which has n > 128*split survivors).
// Called by all threads of the workgroup.
// `tok_pre` (chunk 0 only, HAVE_TOK): the chunk's survivor index of this thread, already loaded.
// USE_W: the logits are not computed from q and K; survivor j of the row carries the non-negative
// weight a.weights[row, j] (the estimator's probability, attention.py:295-296) and the output is
// sum_j w_j V_j / sum_j w_j. No K is read; as a partial result the chunk has maximum 0 and sum
// sum_j w_j, which the merge below handles unchanged.
template <int DT, bool HAVE_TOK, bool USE_W, int THREADS>
__device__ __forceinline__ void attn_chunk(const AttnArgs& a, AttnSmem<THREADS>& sm, uint32_t row,
                                           int split, int n, int tok_pre) {
  constexpr int kAttnThreads = THREADS;
  constexpr int kAttnWaves = AttnSmem<THREADS>::kWaves;
  constexpr int kAttnChunk = AttnSmem<THREADS>::kChunk;
  constexpr int kGroups = AttnSmem<THREADS>::kGroups;
  int (&slot_id)[kAttnChunk] = sm.slot_id;
  float (&w)[kAttnChunk] = sm.w;
  float (&red)[2][16] = sm.red;
  float (&oacc)[kGroups][TWL_HEAD_DIM] = sm.oacc;
  int& is_last = sm.is_last;
  const int j0 = split * kAttnChunk;
  const int tx = threadIdx.x;
  uint16_t* orow = (uint16_t*)a.out + (size_t)row * TWL_HEAD_DIM;
  const int cn = min(kAttnChunk, n - j0);            // survivors of this chunk
  const int n_splits = (n + kAttnChunk - 1) / kAttnChunk;

  const uint32_t b = row / a.num_q_heads;
  const uint32_t h = row - b * a.num_q_heads;
  const uint32_t kvh = h / (a.num_q_heads / a.num_kv_heads);
  const int lane = lane_id();
  const int wave = tx / kWave;
  const int sub = lane & 15;   // which 8 dims
  const int grp = lane >> 4;   // which of the wave's 4 concurrent tokens

  // ---- resolve token addresses once ---------------------------------------------------------
  const int pg_lo = a.kv_page_indptr[b], pg_hi = a.kv_page_indptr[b + 1];
  if (tx < kAttnChunk) {
    int sid = 0;
    if (tx < cn) {
      const int tok = HAVE_TOK ? tok_pre : a.idx[(size_t)row * a.idx_stride + j0 + tx];
      // a position outside the request (a corrupt list) is folded onto its last page rather than
      // read past the page table
      const int pg = min(max(tok >> 4, 0), max(pg_hi - pg_lo - 1, 0));
      sid = a.kv_page_indices[pg_lo + pg] * TWL_PAGE + (tok & 15);
    }
    slot_id[tx] = sid;
  }
  float qf[8];
  float e_pre = 0.0f;
  if (USE_W) {
    if (tx < cn) e_pre = fmaxf(a.weights[(size_t)row * a.idx_stride + j0 + tx], 0.0f);
  } else {
    u32x4 v = *(const u32x4*)((const uint16_t*)a.q + (size_t)row * TWL_HEAD_DIM + 8 * sub);
    unpack8<DT>(v, qf);
  }
  __syncthreads();

  uint64_t ticket_seen = 0;
  if (n_splits > 1 && tx == 0)
    ticket_seen = __hip_atomic_load(&a.tickets[row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // ---- issue every K and V load of the chunk -------------------------------------------------
  const size_t head_off = (size_t)kvh * a.head_stride + 8 * sub;
  const uint16_t* kc = (const uint16_t*)a.k_cache;
  const uint16_t* vc = (const uint16_t*)a.v_cache;
  u32x4 kreg[kAttnSteps], vreg[kAttnSteps];
  int tloc[kAttnSteps];
#pragma unroll
  for (int i = 0; i < kAttnSteps; ++i) {
    const int t = i * (4 * kAttnWaves) + wave * 4 + grp;  // local token of this lane group
    tloc[i] = t;
    kreg[i] = u32x4{0u, 0u, 0u, 0u};
    if (!USE_W && t < cn) {   // lane groups past the chunk's end request nothing
      const int sid = slot_id[t];
      const size_t off = (size_t)(sid >> 4) * a.page_stride + (size_t)(sid & 15) * a.token_stride +
                         head_off;
      kreg[i] = *(const u32x4*)(kc + off);
    }
  }
#pragma unroll
  for (int i = 0; i < kAttnSteps; ++i) {
    vreg[i] = u32x4{0u, 0u, 0u, 0u};
    if (tloc[i] < cn) {
      const int sid = slot_id[tloc[i]];
      const size_t off = (size_t)(sid >> 4) * a.page_stride + (size_t)(sid & 15) * a.token_stride +
                         head_off;
      vreg[i] = *(const u32x4*)(vc + off);
    }
  }

  // ---- logits -------------------------------------------------------------------------------
  float m = 0.0f;
  float z = 0.0f;
  float e = 0.0f;
  if (USE_W) {
    if (n_splits > 1 && tx == 0) tag_ticket(&a.tickets[row], ticket_seen, a.epoch);
    e = e_pre;
    z = e;
  } else {
    float wmax = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < kAttnSteps; ++i) {
      float kf[8];
      unpack8<DT>(kreg[i], kf);
      float acc = 0.0f;
#pragma unroll
      for (int d = 0; d < 8; ++d) acc = fmaf(qf[d], kf[d], acc);
      acc = row16_allreduce<OpSum>(acc) * a.sm_scale;
      if (tloc[i] < cn) {
        wmax = fmaxf(wmax, acc);
        if (sub == 0) w[tloc[i]] = acc;
      }
    }
    if (n_splits > 1 && tx == 0) tag_ticket(&a.tickets[row], ticket_seen, a.epoch);
    m = block_allreduce<OpMax, kAttnWaves>(wmax, red[0]);  // barrier: w[] visible

    // ---- weights ----------------------------------------------------------------------------
    if (tx < cn) {
      e = expf(w[tx] - m);
      z = e;
    }
  }
  z = block_allreduce<OpSum, kAttnWaves>(z, red[1]);
  const bool single = (n_splits == 1);
  if (tx < cn) w[tx] = single ? round_to<DT>(e / z) : e;
  __syncthreads();

  // ---- acc = sum_t w_t * V_t ----------------------------------------------------------------
  float acc[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) acc[d] = 0.0f;
#pragma unroll
  for (int i = 0; i < kAttnSteps; ++i) {
    const float wt = (tloc[i] < cn) ? w[tloc[i]] : 0.0f;
    float vf[8];
    unpack8<DT>(vreg[i], vf);
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[d] = fmaf(wt, vf[d], acc[d]);
  }
  // fold the lane groups (4 per wave) through LDS: every thread adds the groups of its residue
  // class, then the first 128 threads add the classes
  constexpr int kParts = kAttnThreads / TWL_HEAD_DIM;
  // (two 16-byte stores per lane: the 16 lanes of a token cover 512 contiguous bytes; eight
  // 4-byte stores at a stride of 32 bytes were 16-way bank conflicts)
  *(f32x4*)&oacc[wave * 4 + grp][8 * sub] = f32x4{acc[0], acc[1], acc[2], acc[3]};
  *(f32x4*)&oacc[wave * 4 + grp][8 * sub + 4] = f32x4{acc[4], acc[5], acc[6], acc[7]};
  __syncthreads();
  float o = 0.0f;
  {
    const int dd = tx & (TWL_HEAD_DIM - 1), part = tx / TWL_HEAD_DIM;
#pragma unroll
    for (int gi = 0; gi < kGroups / kParts; ++gi) o += oacc[gi * kParts + part][dd];
    __syncthreads();
    oacc[part][dd] = o;
    __syncthreads();
    o = 0.0f;
    if (tx < TWL_HEAD_DIM) {
#pragma unroll
      for (int pp = 0; pp < kParts; ++pp) o += oacc[pp][tx];
    }
  }

  if (single) {
    if (tx < TWL_HEAD_DIM) orow[tx] = (uint16_t)f32_to_bits16<DT>(o);
    if (tx == 0 && a.lse_out) a.lse_out[row] = m + logf(z);
    return;
  }

  // ---- split row: publish the partial, the last chunk to finish merges -------------------------
  // The chunks of a row run on different XCDs, whose L2 caches are not coherent with each other
  // inside a kernel. What the memory model offers for that, a release at device scope on the
  // ticket and an acquire by the merging chunk, writes back and invalidates a whole L2 per split
  // row: measured, it takes this kernel from 9.4 to 27.1 us at the benchmark's 256 rows. The
  // ordering below is therefore built from what gfx950 guarantees for single operations (the file
  // refuses to compile for another target):
  //   - the partial travels as device-scope relaxed atomic stores: write-through, never left
  //     dirty in this XCD's L2;
  //   - s_waitcnt with every counter at zero returns when those stores have been acknowledged at
  //     device scope; the workgroup barrier after it therefore has every thread's partial in
  //     place before thread 0 touches the ticket;
  //   - the ticket is a device-scope read-modify-write, performed where all XCDs see it;
  //   - the chunk that draws the last ticket reads the partials with device-scope relaxed atomic
  //     loads, which bypass its own caches.
  // Towards the compiler the order is pinned by the barriers and compiler-level fences.
  // The ticket word is (tag << 16) | chunks finished, with the tag of this call (`epoch`, never
  // 0, different from call to call). Every chunk of a split row made sure at its start that the
  // word carries this call's tag (tag_ticket below), so a word left behind by a call that never
  // finished, or never initialised, counts as zero instead of making the row merge early or
  // never. The merging chunk leaves the word zero.
  float* part = a.partials + ((size_t)row * a.max_splits + split) * kAttnPartial;
  if (tx < TWL_HEAD_DIM)
    __hip_atomic_store(part + 2 + tx, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tx == 0) {
    __hip_atomic_store(part + 0, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(part + 1, z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(0);  // every counter to zero: this thread's stores have been acknowledged
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __syncthreads();
  if (tx == 0) {
    const uint64_t before = __hip_atomic_fetch_add(&a.tickets[row], (uint64_t)1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
    is_last = ((uint32_t)(before & 0xFFFFu) == (uint32_t)(n_splits - 1));
  }
  __syncthreads();
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  if (!is_last) return;
  // The partials are read back with device-scope loads that bypass this XCD's caches.
  const float* prow = a.partials + (size_t)row * a.max_splits * kAttnPartial;
  float* fm = &oacc[0][0];   // [n_splits <= 256] chunk maxima, then rescale factors
  float* fl = &oacc[2][0];   // [n_splits] chunk sums
  float lm = -__builtin_inff();
  for (int s = tx; s < n_splits; s += kAttnThreads) {
    const float ms = __hip_atomic_load(prow + (size_t)s * kAttnPartial, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    const float ls = __hip_atomic_load(prow + (size_t)s * kAttnPartial + 1, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    fm[s] = ms;
    fl[s] = ls;
    lm = fmaxf(lm, ms);
  }
  const float gm = block_allreduce<OpMax, kAttnWaves>(lm, red[0]);
  float lsum = 0.0f;
  for (int s = tx; s < n_splits; s += kAttnThreads) {
    const float f = expf(fm[s] - gm);
    fm[s] = f;
    lsum = fmaf(fl[s], f, lsum);
  }
  const float gl = block_allreduce<OpSum, kAttnWaves>(lsum, red[1]);  // barrier: factors visible
  const int d = tx & (TWL_HEAD_DIM - 1), cls = tx / TWL_HEAD_DIM;
  constexpr int kInFlight = 32 / kParts;            // loads in flight per thread
  float go = 0.0f;
  for (int s0 = cls; s0 < n_splits; s0 += 32) {
    float pv[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int s = min(s0 + kParts * u, n_splits - 1);
      pv[u] = __hip_atomic_load(prow + (size_t)s * kAttnPartial + 2 + d, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int s = s0 + kParts * u;
      go = fmaf(pv[u], (s < n_splits) ? fm[s] : 0.0f, go);
    }
  }
  // fm / fl live in rows 0..3 of oacc: the classes meet in rows 8..
  oacc[8 + cls][d] = go;
  __syncthreads();
  if (tx < TWL_HEAD_DIM) {
    go = 0.0f;
#pragma unroll
    for (int pp = 0; pp < kParts; ++pp) go += oacc[8 + pp][tx];
    orow[tx] = (uint16_t)f32_to_bits16<DT>(go / gl);
  }
  if (tx == 0) {
    if (a.lse_out) a.lse_out[row] = gm + logf(gl);
    // ready for the next call
    __hip_atomic_store(&a.tickets[row], (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Workgroup g < rows serves chunk 0 of row g. The remaining `pool` workgroups serve the chunks
// 1.. of rows with more than 128 survivors: pool workgroup j takes overflow chunks j, j+pool, ...
// in row-major order, locating each with a block-wide prefix sum over the rows' chunk counts
// (a few KB from L2), so a launch never contains more than rows + pool workgroups however long
// the longest row is.
template <int DT, bool USE_W, int THREADS>
__global__ __launch_bounds__(THREADS) void sparse_attn_kernel(AttnArgs a) {
  constexpr int kAttnThreads = THREADS;
  constexpr int kAttnWaves = AttnSmem<THREADS>::kWaves;
  constexpr int kAttnChunk = AttnSmem<THREADS>::kChunk;
  __shared__ AttnSmem<THREADS> sm;
  __shared__ int wave_tot[kAttnWaves];
  __shared__ int found[3];  // row, split, n
  const int tx = threadIdx.x;
  if (blockIdx.x < a.rows) {
    const uint32_t row = blockIdx.x;
    // the first survivors are requested together with the count they depend on
    const int tok_pre = ((uint32_t)tx < min((uint32_t)kAttnChunk, a.idx_stride))
                            ? a.idx[(size_t)row * a.idx_stride + tx] : 0;
    const int n = min(max(a.count[row], 0), (int)a.idx_stride);
    if (n == 0) {
      if (tx < TWL_HEAD_DIM) ((uint16_t*)a.out)[(size_t)row * TWL_HEAD_DIM + tx] = 0;
      if (tx == 0 && a.lse_out) a.lse_out[row] = -__builtin_inff();
    } else {
      attn_chunk<DT, true, USE_W, THREADS>(a, sm, row, 0, n, tok_pre);
    }
    return;
  }
  const int lane = lane_id();
  const int wave = tx / kWave;
  // j only grows, so the search for the row that owns overflow chunk j goes on from the tile of
  // rows where the previous one was found (`tile0`, with `base` overflow chunks before it)
  uint32_t tile0 = 0;
  int base = 0;
  for (int j = (int)(blockIdx.x - a.rows);; j += (int)a.pool) {
    bool hit = false;
    while (tile0 < a.rows) {
      const uint32_t r = tile0 + tx;
      int n = 0, ov = 0;
      if (r < a.rows) {
        n = min(max(a.count[r], 0), (int)a.idx_stride);
        ov = max((n + kAttnChunk - 1) / kAttnChunk - 1, 0);
      }
      const int incl = wave_inclusive_scan(ov);
      if (lane == kWave - 1) wave_tot[wave] = incl;
      __syncthreads();
      int before = base, total = base;
#pragma unroll
      for (int wv = 0; wv < kAttnWaves; ++wv) {
        before += (wv < wave) ? wave_tot[wv] : 0;
        total += wave_tot[wv];
      }
      const int lo = before + incl - ov;  // first overflow chunk index owned by row r
      if (ov > 0 && j >= lo && j < lo + ov) {
        found[0] = (int)r; found[1] = j - lo + 1; found[2] = n;
      }
      hit = (j < total);
      __syncthreads();
      if (hit) break;        // the next j starts from this tile again
      base = total;
      tile0 += kAttnThreads;
    }
    if (!hit) return;  // j is past the last overflow chunk: nothing left for this workgroup
    attn_chunk<DT, false, USE_W, THREADS>(a, sm, (uint32_t)found[0], found[1], found[2], 0);
    __syncthreads();
  }
}

}  // namespace twl

// The workspace is sized for the smallest chunk any launch configuration uses.
constexpr int kAttnMinChunk = 128;

extern "C" uint64_t twl_sparse_attn_workspace_bytes(uint32_t rows, uint32_t idx_stride) {
  const uint64_t splits = (idx_stride + kAttnMinChunk - 1) / kAttnMinChunk;
  uint64_t tickets = ((uint64_t)rows * sizeof(uint64_t) + 255) & ~255ull;
  return tickets + (uint64_t)rows * splits * twl::kAttnPartial * sizeof(float);
}

namespace twl {
// Tag of a call's ticket words: 48 bits that start from a per-process random value and advance
// by an odd constant, never 0. A ticket word that this call did not write (another call's, or
// memory that was never cleared) carries this tag with probability 2^-48.
static uint64_t next_epoch() {
  static std::atomic<uint64_t> state{0};
  uint64_t s = state.load(std::memory_order_relaxed);
  if (s == 0) {
    uint64_t seed = (uint64_t)std::chrono::steady_clock::now().time_since_epoch().count();
    seed ^= (uint64_t)(uintptr_t)&state * 0x9E3779B97F4A7C15ull;
    seed ^= seed >> 29;
    seed |= 1;
    uint64_t expected = 0;
    state.compare_exchange_strong(expected, seed, std::memory_order_relaxed);
  }
  for (;;) {
    const uint64_t v = state.fetch_add(0x9E3779B97F4A7C15ull, std::memory_order_relaxed);
    const uint64_t tag = (v ^ (v >> 23)) & 0xFFFFFFFFFFFFull;
    if (tag) return tag;
  }
}

template <int THREADS>
static void launch_attn_threads(const AttnArgs& a0, int dtype, bool weighted, hipStream_t stream) {
  AttnArgs a = a0;
  constexpr int chunk = AttnSmem<THREADS>::kChunk;
  a.max_splits = (a.idx_stride + chunk - 1) / chunk;
  const uint64_t overflow_max = (uint64_t)a.rows * (a.max_splits - 1);
  a.pool = (uint32_t)(overflow_max < 1024 ? overflow_max : 1024);
  dim3 grid(a.rows + a.pool), block(THREADS);
  if (weighted) {
    if (dtype == TWL_F16)
      hipLaunchKernelGGL((sparse_attn_kernel<TWL_F16, true, THREADS>), grid, block, 0, stream, a);
    else
      hipLaunchKernelGGL((sparse_attn_kernel<TWL_BF16, true, THREADS>), grid, block, 0, stream, a);
  } else if (dtype == TWL_F16) {
    hipLaunchKernelGGL((sparse_attn_kernel<TWL_F16, false, THREADS>), grid, block, 0, stream, a);
  } else {
    hipLaunchKernelGGL((sparse_attn_kernel<TWL_BF16, false, THREADS>), grid, block, 0, stream, a);
  }
}
}  // namespace twl

// Validation and launch shared by the two entry points; `workspace` holds
// twl_sparse_attn_workspace_bytes(rows, idx_stride) bytes (any contents).
static int launch_sparse_attn(const void* q, void* out, int dtype, const void* k_cache,
                              const void* v_cache, uint64_t page_stride, uint64_t token_stride,
                              uint64_t head_stride, const int32_t* idx, uint32_t idx_stride,
                              const int32_t* count, const int32_t* kv_page_indices,
                              const int32_t* kv_page_indptr, uint32_t rows, uint32_t num_q_heads,
                              uint32_t num_kv_heads, float sm_scale, float* lse_out,
                              void* workspace, hipStream_t stream,
                              const float* weights = nullptr) {
  twl::AttnArgs a{};
  a.weights = weights;
  a.q = q; a.out = out; a.k_cache = k_cache; a.v_cache = v_cache; a.page_stride = page_stride;
  a.token_stride = token_stride; a.head_stride = head_stride; a.idx = idx;
  a.idx_stride = idx_stride; a.count = count; a.kv_page_indices = kv_page_indices;
  a.kv_page_indptr = kv_page_indptr; a.num_q_heads = num_q_heads; a.num_kv_heads = num_kv_heads;
  a.sm_scale = sm_scale; a.lse_out = lse_out;
  a.tickets = (uint64_t*)workspace;
  a.partials = (float*)((uint8_t*)workspace + (((uint64_t)rows * sizeof(uint64_t) + 255) & ~255ull));
  a.rows = rows;
  a.epoch = twl::next_epoch();
  // Workgroup size, measured on rows of 100-400 survivors (256 rows: 13.1 us) and on rows of
  // mostly 1-2 survivors with a few of thousands (9.9 us): 512 threads, rows up to 256 survivors
  // finished in place, 13.4 / 11.4 us; 1024 threads, up to 512 in place, 17.2 / 18.1 us (one
  // 16-wavefront workgroup per compute unit: the pool workgroups queue behind the rows).
  twl::launch_attn_threads<256>(a, dtype, weights != nullptr, stream);
  return hipGetLastError() == hipSuccess ? TWL_OK : TWL_ELAUNCH;
}

// Everything of the argument check that does not concern the workspace. Sets *rows_out.
static int check_sparse_attn(const void* q, const void* out, int dtype, const void* k_cache,
                             const void* v_cache, uint64_t page_stride, uint64_t token_stride,
                             uint64_t head_stride, const int32_t* idx, uint32_t idx_stride,
                             const int32_t* count, const int32_t* kv_page_indices,
                             const int32_t* kv_page_indptr, uint32_t batch, uint32_t num_q_heads,
                             uint32_t num_kv_heads, uint32_t* rows_out) {
  if (!q || !out || !k_cache || !v_cache || !idx || !count || !kv_page_indices || !kv_page_indptr)
    return TWL_ENULL;
  if (dtype != TWL_F16 && dtype != TWL_BF16) return TWL_EDTYPE;
  if (batch == 0 || num_q_heads == 0 || num_kv_heads == 0 || num_q_heads % num_kv_heads != 0)
    return TWL_EINVAL;
  if (idx_stride == 0 || idx_stride > TWL_MAX_CANDIDATES) return TWL_EINVAL;
  const uint64_t rows64 = (uint64_t)batch * num_q_heads;
  if (rows64 > 65535u) return TWL_EINVAL;
  if ((page_stride | token_stride | head_stride) & 7u) return TWL_EALIGN;  // 16-byte loads
  if ((((uintptr_t)q) & 15u) || (((uintptr_t)k_cache) & 15u) || (((uintptr_t)v_cache) & 15u) ||
      (((uintptr_t)out) & 1u))
    return TWL_EALIGN;
  *rows_out = (uint32_t)rows64;
  return TWL_OK;
}

extern "C" int twl_sparse_attn(const void* q, void* out, int dtype, const void* k_cache,
                               const void* v_cache, uint64_t page_stride, uint64_t token_stride,
                               uint64_t head_stride, const int32_t* idx, uint32_t idx_stride,
                               const int32_t* count, const int32_t* kv_page_indices,
                               const int32_t* kv_page_indptr, uint32_t batch,
                               uint32_t num_q_heads, uint32_t num_kv_heads, float sm_scale,
                               float* lse_out, void* workspace, uint64_t workspace_bytes,
                               void* stream) {
  if (!workspace) return TWL_ENULL;
  uint32_t rows = 0;
  const int rc = check_sparse_attn(q, out, dtype, k_cache, v_cache, page_stride, token_stride,
                                   head_stride, idx, idx_stride, count, kv_page_indices,
                                   kv_page_indptr, batch, num_q_heads, num_kv_heads, &rows);
  if (rc != TWL_OK) return rc;
  if (workspace_bytes < twl_sparse_attn_workspace_bytes(rows, idx_stride)) return TWL_EINVAL;
  if (((uintptr_t)workspace) & 255u) return TWL_EALIGN;
  return launch_sparse_attn(q, out, dtype, k_cache, v_cache, page_stride, token_stride,
                            head_stride, idx, idx_stride, count, kv_page_indices, kv_page_indptr,
                            rows, num_q_heads, num_kv_heads, sm_scale, lse_out, workspace,
                            (hipStream_t)stream);
}

// Attention with given weights instead of q.K logits (attention.py:295-296 followed by :299-306):
// out[row] = sum_j w_j V[idx_j] / sum_j w_j. K and q are not read.
extern "C" int twl_sparse_attn_weighted(void* out, int dtype, const void* v_cache,
                                        uint64_t page_stride, uint64_t token_stride,
                                        uint64_t head_stride, const int32_t* idx,
                                        uint32_t idx_stride, const int32_t* count,
                                        const float* weights, const int32_t* kv_page_indices,
                                        const int32_t* kv_page_indptr, uint32_t batch,
                                        uint32_t num_q_heads, uint32_t num_kv_heads,
                                        float* lse_out, void* workspace,
                                        uint64_t workspace_bytes, void* stream) {
  if (!workspace || !weights) return TWL_ENULL;
  if (((uintptr_t)weights) & 3u) return TWL_EALIGN;
  uint32_t rows = 0;
  // q and K take no part; the shared check sees V in their place
  const int rc = check_sparse_attn(v_cache, out, dtype, v_cache, v_cache, page_stride,
                                   token_stride, head_stride, idx, idx_stride, count,
                                   kv_page_indices, kv_page_indptr, batch, num_q_heads,
                                   num_kv_heads, &rows);
  if (rc != TWL_OK) return rc;
  if (workspace_bytes < twl_sparse_attn_workspace_bytes(rows, idx_stride)) return TWL_EINVAL;
  if (((uintptr_t)workspace) & 255u) return TWL_EALIGN;
  return launch_sparse_attn(nullptr, out, dtype, nullptr, v_cache, page_stride, token_stride,
                            head_stride, idx, idx_stride, count, kv_page_indices, kv_page_indptr,
                            rows, num_q_heads, num_kv_heads, 1.0f, lse_out, workspace,
                            (hipStream_t)stream, weights);
}

// ---- the same call without a workspace argument -------------------------------------------------
// The split-row partials and tickets live in an array that is part of the library's device image,
// so the call allocates nothing. Every GPU holds its own copy of the array at its own address;
// host code may not use the array's name as an address (it is a host-side stand-in), so the device
// address is looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[TWL_STATIC_SCRATCH_BYTES];

namespace twl {
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

}  // namespace twl

extern "C" int twl_sparse_attn_static(const void* q, void* out, int dtype, const void* k_cache,
                                      const void* v_cache, uint64_t page_stride,
                                      uint64_t token_stride, uint64_t head_stride,
                                      const int32_t* idx, uint32_t idx_stride,
                                      const int32_t* count, const int32_t* kv_page_indices,
                                      const int32_t* kv_page_indptr, uint32_t batch,
                                      uint32_t num_q_heads, uint32_t num_kv_heads, float sm_scale,
                                      float* lse_out, void* stream) {
  uint32_t rows = 0;
  const int rc = check_sparse_attn(q, out, dtype, k_cache, v_cache, page_stride, token_stride,
                                   head_stride, idx, idx_stride, count, kv_page_indices,
                                   kv_page_indptr, batch, num_q_heads, num_kv_heads, &rows);
  if (rc != TWL_OK) return rc;
  // rows * ceil(idx_stride / 128) partial results of 520 bytes must fit the array
  if (twl_sparse_attn_workspace_bytes(rows, idx_stride) > (uint64_t)TWL_STATIC_SCRATCH_BYTES)
    return TWL_ETOOBIG;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return TWL_ENODEVICE;
  if (dev < 0 || dev >= twl::kMaxDevices) return TWL_EINVAL;
  // The array used is the current device's copy: q must live on that device (a caller whose
  // current device is another GPU would otherwise hand its kernel a foreign address).
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, q) != hipSuccess) {
    (void)hipGetLastError();
    return TWL_EINVAL;
  }
  if (attr.device != dev) return TWL_EINVAL;
  void* ws = twl::g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ws) {
    // first call on this device: look up the array's address on THIS GPU. Not under stream
    // capture, where the lookup could end the capture with an error of its own.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cap) != hipSuccess) {
      (void)hipGetLastError();
      return TWL_EINVAL;
    }
    if (cap != hipStreamCaptureStatusNone) return TWL_EINVAL;
    void* p = nullptr;
    if (hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)) != hipSuccess || !p)
      return TWL_ELAUNCH;
    twl::g_scratch_ptr[dev].store(p, std::memory_order_release);
    ws = p;
  }
  // The array keeps what the last call left; nothing in it has to be cleared: the ticket words
  // are tagged per call (tag_ticket) and the partial results are written before they are read.
  return launch_sparse_attn(q, out, dtype, k_cache, v_cache, page_stride, token_stride,
                            head_stride, idx, idx_stride, count, kv_page_indices, kv_page_indptr,
                            rows, num_q_heads, num_kv_heads, sm_scale, lse_out, ws,
                            (hipStream_t)stream);
}
