/*
 * twilight_hip.h — C ABI of libtwilight_hip.so: the Select-then-Prune decode hot path of
 * Twilight (Quest page selector -> INT4-K score GEMV -> softmax + top-p prune -> sparse paged
 * decode attention) as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers unless the name ends in _host. The library never
 *     allocates, frees or synchronises: outputs and workspaces are caller-owned, kernels are
 *     enqueued on `stream` (a hipStream_t passed as void*; NULL = the default stream).
 *   - Return value: TWL_OK (0) or a negative TWL_E* code; twl_strerror() names it. Arguments are
 *     validated on the host before anything touches the GPU, so TWL_EINVAL/TWL_ENULL/... are
 *     returned even on a machine without a GPU.
 *   - rows = batch * num_q_heads, row r = b * num_q_heads + h. KV head of q head h is
 *     h / (num_q_heads / num_kv_heads). head_dim is 128, page size is 16 tokens (TWL_PAGE).
 *   - Page tables are FlashInfer-style CSR: request b owns logical pages
 *     kv_page_indices[kv_page_indptr[b] .. kv_page_indptr[b+1]) (values = physical page ids);
 *     its last logical page holds kv_last_page_len[b] (1..16) valid tokens.
 *   - A "page list" is per row: sel_pages[r * sel_stride + i], i < sel_count[r], holds LOGICAL
 *     page numbers of request b in ascending order. Candidate c of a row is token (c % 16) of
 *     its (c / 16)-th listed page. sel_pages == NULL means "all pages of the request".
 *   - A "survivor list" is per row: idx[r * idx_stride + j], j < count[r], holds LOGICAL token
 *     positions (page * 16 + slot) in ascending order.
 *
 * Storage formats defined by this library (nothing in the reference pins them)
 *   - INT4 K shadow: one 1280-byte record per (physical page, kv head), records ordered
 *     [page][kv_head]. Bytes [0,1024): token t (0..15) occupies bytes [64t, 64t+64); element d
 *     (0..127) of that token is the low (d even) or high (d odd) nibble of byte d/2. Bytes
 *     [1024,1280): 64 pairs of IEEE fp16 (scale, zero), pair index t*4 + g for quantisation group
 *     g = d/32. Dequantised value = float(nibble) * float(scale) + float(zero), one fp32 rounding.
 *   - Quest page metadata: one 512-byte record per (physical page, kv head), ordered
 *     [page][kv_head]: 32 chunks of 16 bytes; chunk c holds fp16 min[4c..4c+3] then fp16
 *     max[4c..4c+3] over the valid tokens of the page ("fp16" = the cache dtype, fp16 or bf16).
 *   - Quest page metadata, plane layout (optional second copy, see twl_meta_planes_build):
 *     planes[slot][kv_head][d][0 = min, 1 = max][logical page], 16-bit values in the cache dtype,
 *     plane_cap_pages pages per run (a multiple of 8; a multiple of 128 keeps every run 256-byte
 *     aligned, which the scoring passes reward: 71 -> 64 us at 2032 pages per run against 2048),
 *     slot = position of the request in the batch or, with a slot table (plane_slots [batch],
 *     entries in [0, plane_num_slots)), the table's entry. A scoring pass reads a request's
 *     pages from the planes except its last page (whose plane entries are written when it is
 *     complete) and, where the request is at most 128 pages longer than a multiple of 2048, the
 *     pages beyond that multiple: those come from the records.
 *   - Paged K / V caches: fp16 or bf16, addressed with explicit element strides
 *     (page, token, kv head); head_dim is contiguous.
 */
#ifndef TWILIGHT_HIP_H_
#define TWILIGHT_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TWL_PAGE 16          /* tokens per KV page */
#define TWL_HEAD_DIM 128     /* head dimension */
#define TWL_QGROUP 32        /* INT4 quantisation group along head_dim */
#define TWL_INT4_RECORD_BYTES 1280
#define TWL_META_RECORD_BYTES 512
#define TWL_MAX_CANDIDATES 32768 /* longest row twl_top_p_* / twl_softmax_top_p_f32 accept */

enum twl_status {
  TWL_OK = 0,
  TWL_ENULL = -1,    /* a required pointer is NULL */
  TWL_EINVAL = -2,   /* a size / stride / mode argument is out of range */
  TWL_EDTYPE = -3,   /* unsupported element type code */
  TWL_EALIGN = -4,   /* a pointer or stride breaks the alignment the kernel needs */
  TWL_ELAUNCH = -5,  /* the HIP runtime rejected the launch (hipGetLastError != hipSuccess) */
  TWL_ENODEVICE = -6, /* no usable HIP device */
  TWL_ETOOBIG = -7    /* the problem does not fit a fixed-size buffer of the library */
};

enum twl_dtype { TWL_F16 = 0, TWL_BF16 = 1, TWL_F32 = 2 };

/* how the top-p bisection initialises its upper bound */
enum twl_top_p_high {
  TWL_HIGH_FIRST = 0, /* probs[row][0], as csrc/include/sampling.cuh:156-159 does: the
                       * probability of token 0 of the context. Entry points that prune a
                       * candidate list (page lists: twl_softmax_top_p_f32 with sel_pages,
                       * twl_gemv_top_p, twl_select_estimate_prune, twl_decode_layer) take the
                       * first candidate's probability when logical page 0 heads the list and
                       * 0 otherwise (a token outside the selection has probability 0 on the
                       * reference's full-length row): the search then ends at once and every
                       * candidate with a positive probability is kept */
  TWL_HIGH_MAX = 1    /* the row maximum (paper Algorithm 1) */
};

const char* twl_strerror(int status);
/* ABI version of this header; bumps when a signature changes. twl_abi_version() returns the
 * version the library was built with: a caller compares the two before anything else. */
#define TWL_ABI_VERSION 10
int twl_abi_version(void);
/* Number of HIP devices visible, or a negative twl_status. */
int twl_device_count(void);

/* ---------------------------------------------------------------------------------------------
 * Top-p pruner on normalised probabilities.
 * Replaces: top_p_fp32_return_mask / top_p_fp16_return_mask, csrc/src/sampling.cu:22-63, and the
 * kernel they launch, TopPReturnMaskKernel, csrc/include/sampling.cuh:119-231 (launcher :233-250).
 * probs is [rows, d] contiguous (the reference's [B,H,1,N] tensor with rows = B*H, d = N).
 * p_arr (nullable) holds one p per row and overrides p, as top_p_arr does (sampling.cuh:125).
 * Outputs, each nullable (at least one must be given):
 *   mask  uint8 [rows, d]: 1 where probs > low at the end of the bisection (sampling.cuh:219-230)
 *   idx   int32 [rows, idx_stride] + count int32 [rows]: the positions where mask is 1, ascending.
 * low_out (nullable) float [rows]: the final lower pivot; iters_out (nullable) int32 [rows]: the
 * number of bisection iterations executed.
 * d must be in [1, TWL_MAX_CANDIDATES]; idx_stride >= d when idx is given. p is not range-checked,
 * as in the reference (only NaN is refused): p >= 1 lets no sum reach it, the search ends with
 * low = 0 and every positive probability is kept; p <= 0 is reached by every sum. The entry
 * points that are not the reference's (twl_softmax_top_p_f32, twl_gemv_top_p,
 * twl_select_estimate_prune, twl_decode_layer) require 0 < p <= 1.
 * ------------------------------------------------------------------------------------------- */
int twl_top_p_f32(const float* probs, uint8_t* mask, int32_t* idx, int32_t* count,
                  const float* p_arr, float p, uint32_t rows, uint32_t d, uint32_t idx_stride,
                  int high_mode, float* low_out, int32_t* iters_out, void* stream);
/* Same for fp16 (dtype = TWL_F16) or bf16 (TWL_BF16) probabilities, with the arithmetic of the
 * reference's DType = half / nv_bfloat16 instantiation (csrc/src/sampling.cu:22-43): p, low, high,
 * mid, the tolerance 1e-5, the bracket width and every partial sum are values of the 16-bit type
 * (each operation rounds to nearest even), and the additions run in the order of
 * cub::BlockReduce<DType, 1024, BLOCK_REDUCE_WARP_REDUCTIONS> (sampling.cuh:54,171-217: a thread
 * folds its VEC = gcd(8, d) items left to right, warps of 32 add pairwise, the 32 warp results
 * are added in warp order, chunks of 1024 * VEC elements in chunk order; CUB 1.x - 2.4). Masks,
 * low_out and iters_out therefore equal the reference kernel's bit for bit. TWL_HIGH_MAX is this
 * library's variant of the upper bound; everything else is unchanged by it. */
int twl_top_p_f16(const void* probs, int dtype, uint8_t* mask, int32_t* idx, int32_t* count,
                  const float* p_arr, float p, uint32_t rows, uint32_t d, uint32_t idx_stride,
                  int high_mode, float* low_out, int32_t* iters_out, void* stream);
/* twl_top_p_f32 with the additions of the reference's DType = float instantiation
 * (csrc/src/sampling.cu:45-63) in the order of cub::BlockReduce<float, 1024,
 * BLOCK_REDUCE_WARP_REDUCTIONS> (sampling.cuh:54; VEC = gcd(4, d)), as twl_top_p_f16 has them for
 * the 16-bit types: masks, low_out and iters_out equal the reference kernel's on every row, also
 * where a partial sum meets p within a rounding error (there twl_top_p_f32, which adds in an
 * order of its own and is about three times faster, may decide an iteration the other way and
 * keep a set that differs by tokens within 1e-5 of the pivot). Same arguments as twl_top_p_f32. */
int twl_top_p_f32_exact(const float* probs, uint8_t* mask, int32_t* idx, int32_t* count,
                        const float* p_arr, float p, uint32_t rows, uint32_t d,
                        uint32_t idx_stride, int high_mode, float* low_out, int32_t* iters_out,
                        void* stream);

/* ---------------------------------------------------------------------------------------------
 * Fused softmax + top-p + stream compaction over raw (un-normalised) scores.
 * Replaces: top_p_unnormalized, twilight/pyimpl/top_p.py:10-15 (softmax in fp32 then the mask
 * kernel) and the mask combine twilight/pyimpl/attention.py:280-281 in index-list form.
 * scores is [rows, score_stride] fp32; row r has lens[r] candidates (lens == NULL: every row has
 * d). -inf scores are legal and get probability 0. Survivors are emitted as
 *   idx[r*idx_stride + j] = token_of(position) ascending, count[r],
 * where token_of(c) = sel_pages[r*sel_stride + c/16]*16 + c%16 when sel_pages != NULL, else c.
 * probs_out (nullable) float [rows, score_stride] receives the softmax for inspection.
 * ------------------------------------------------------------------------------------------- */
int twl_softmax_top_p_f32(const float* scores, uint32_t score_stride, const int32_t* lens,
                          uint32_t rows, uint32_t d, const float* p_arr, float p, int high_mode,
                          const int32_t* sel_pages, uint32_t sel_stride, int32_t* idx,
                          uint32_t idx_stride, int32_t* count, float* probs_out, float* low_out,
                          void* stream);

/* ---------------------------------------------------------------------------------------------
 * Estimator and pruner in one launch: twl_gemv_int4 over a row's page list followed by
 * twl_softmax_top_p_f32 on those scores, the scores staying in registers.
 * Replaces: twilight/pyimpl/attention.py:252-255 (estimate) + twilight/pyimpl/top_p.py:10-15
 * (softmax, mask kernel) + attention.py:280-281 (combine), in index-list form.
 * Arguments as in twl_gemv_int4 and twl_softmax_top_p_f32; sel_pages is required and
 * max_pages_per_row * 16 <= TWL_MAX_CANDIDATES. scores_out (nullable) float [rows, score_stride]
 * receives the raw scaled scores (candidate order, -inf past the last page's length) for
 * inspection; cand_count (nullable) int32 [rows] the candidate count; low_out (nullable) the final
 * lower pivot. The survivor list idx / count is identical to the two-call sequence: the same
 * arithmetic runs on the same values, only the summation order of the softmax denominator and of
 * the bisection sums differs (fp32, the order inside a sum is unspecified in both).
 * ------------------------------------------------------------------------------------------- */
int twl_gemv_top_p(const void* q, int q_dtype, const void* k_int4, const int32_t* sel_pages,
                   const int32_t* sel_count, uint32_t sel_stride, const int32_t* kv_page_indices,
                   const int32_t* kv_page_indptr, const int32_t* kv_last_page_len, uint32_t batch,
                   uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t max_pages_per_row,
                   float sm_scale, const float* p_arr, float p, int high_mode, int32_t* idx,
                   uint32_t idx_stride, int32_t* count, float* scores_out, uint32_t score_stride,
                   int32_t* cand_count, float* low_out, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Selector + estimator + pruner in one launch, one workgroup per (batch, head) row:
 * twl_quest_page_scores, twl_quest_topk_pages and twl_gemv_top_p with the page scores and the
 * page list kept on chip. Replaces: twilight/pyimpl/quest.py:17-122 + attention.py:252-255 +
 * top_p.py:10-15 + attention.py:280-281. Outputs as those three calls give them: sel_pages /
 * sel_count (ascending logical pages, ties at the k-th score to the lower page), idx / count,
 * optionally page_scores_out [rows, page_score_stride], scores_out [rows, score_stride] and
 * cand_count. max_pages_per_req <= 8192. With meta_planes (plane layout, see
 * twl_meta_planes_build; meta is still needed: a request's last page is scored from its record)
 * the page scores are accumulated channel by channel
 * in ascending order from the sign-selected runs; they can differ from twl_quest_page_scores in
 * the last bits (other summation order). Meant for about one row per compute unit (decode at
 * moderate batch). With GQA every q-head row reads its kv head's metadata; the rows of a group
 * are placed on one XCD so that all but the first read find it in that L2 (ahead of the
 * three-call form with meta_planes, level with it on records).
 * ------------------------------------------------------------------------------------------- */
int twl_select_estimate_prune(const void* q, int dtype, const void* meta, const void* k_int4,
                              const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                              const int32_t* kv_last_page_len, uint32_t batch,
                              uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t token_budget,
                              uint32_t max_pages_per_req, float sm_scale, const float* p_arr,
                              float p, int high_mode, int32_t* sel_pages, uint32_t sel_stride,
                              int32_t* sel_count, int32_t* idx, uint32_t idx_stride,
                              int32_t* count, float* page_scores_out, uint32_t page_score_stride,
                              float* scores_out, uint32_t score_stride, int32_t* cand_count,
                              const void* meta_planes, uint32_t plane_cap_pages,
                              const int32_t* plane_slots, uint32_t plane_num_slots,
                              void* stream);

/* ---------------------------------------------------------------------------------------------
 * INT4-K score GEMV over candidate pages: out[r, c] = sm_scale * sum_d q[r,d] * dequant(K[c,d]).
 * Replaces: the estimator matmul twilight/pyimpl/attention.py:252-255 and the absent
 * ftka.cuda_ops.gemv.batched_sparse_gemv_int4_k whose call site is
 * benchmark/efficiency/bench_gemv.py:445-454.
 * q [batch, num_q_heads, 128] in q_dtype (TWL_F16 or TWL_BF16); k_int4 = the INT4 shadow records.
 * The dot products run on fp16 pairs with fp32 accumulation, so a bf16 q is converted to fp16
 * first (here, in twl_gemv_top_p, twl_select_estimate_prune and twl_decode_layer's estimator):
 * exact for 2^-17 <= |q| <= 65504, rounded to a multiple of 2^-24 below, saturated to +-65504
 * above. Accepted range of q for results within the 1e-3 score tolerance: |q| <= 65504.
 * out fp32 [rows, out_stride]; candidates past the request's length get -inf. sel_count (nullable
 * with sel_pages) gives pages per row; out_count (nullable) int32 [rows] receives the number of
 * candidate slots written (pages * 16).
 * ------------------------------------------------------------------------------------------- */
int twl_gemv_int4(const void* q, int q_dtype, float* out, uint32_t out_stride, int32_t* out_count,
                  const void* k_int4, const int32_t* sel_pages, const int32_t* sel_count,
                  uint32_t sel_stride, const int32_t* kv_page_indices,
                  const int32_t* kv_page_indptr, const int32_t* kv_last_page_len, uint32_t batch,
                  uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t max_pages_per_row,
                  float sm_scale, void* stream);

/* twl_gemv_int4 for q heads that share kv heads AND one page list per kv head: the list of a
 * group's first q head (sel_pages / sel_count row b * num_q_heads + kvh * G, required) serves the
 * G = num_q_heads / num_kv_heads heads of the group (G in {2, 4, 8}), every INT4 record is
 * fetched once per group and out / out_count are written for every q head. The group's
 * products run on the matrix cores (v_mfma_f32_16x16x32_f16 on the exact fp16 values of the
 * nibbles, fp32 accumulation): a head's scores equal twl_gemv_int4's over the same list up to
 * the fp32 rounding of sums taken in another order (within 2e-5 of the row's typical score in
 * the tests), not bit for bit.
 * Replaces: the same estimator matmul (attention.py:252-255) when the candidate set is chosen per
 * kv head (the reference repeats K per q head, attention.py:124-126, and selects per q head; see
 * twl_layer_args.group_select). */
int twl_gemv_int4_group(const void* q, int q_dtype, float* out, uint32_t out_stride,
                        int32_t* out_count, const void* k_int4, const int32_t* sel_pages,
                        const int32_t* sel_count, uint32_t sel_stride,
                        const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                        const int32_t* kv_last_page_len, uint32_t batch, uint32_t num_q_heads,
                        uint32_t num_kv_heads, uint32_t max_pages_per_row, float sm_scale,
                        void* stream);

/* ---------------------------------------------------------------------------------------------
 * Token-granular paged score GEMVs in the tensor layouts (and call shapes) of the absent
 * ftka.cuda_ops.gemv module, as used by benchmark/efficiency/bench_gemv.py. K cache
 * [max_pages, page_size, num_heads, 128 elements]; q fp16 [batch, num_heads, 128]; o fp16
 * [batch, num_heads, o_stride] written in place for n < request length; one page list per request
 * shared by all heads.
 *   twl_gemv_int4_nhd  batched_sparse_gemv_int4_k, bench_gemv.py:445-454: k_u8 [.., 64] uint8 (low
 *                      nibble = even element), scales / zeros fp16 [max_pages, page_size, heads],
 *                      dequant k*scale + zero (:181)
 *   twl_gemv_int8_nhd  batched_sparse_gemv_int8_k, bench_gemv.py:135-144: k_u8 [.., 128] uint8 =
 *                      int8 value + 128 (:78,93), same scales / zeros
 *   twl_gemv_f16_nhd   batched_sparse_gemv, bench_gemv.py:234-241: fp16 K cache
 *   twl_gemv_f16_single  single_sparse_gemv, bench_gemv.py:33: q [heads,128], k [seq,heads,128],
 *                      o [heads, seq]
 * ------------------------------------------------------------------------------------------- */
int twl_gemv_int4_nhd(const void* q, void* o, uint32_t o_stride, const uint8_t* k_u8,
                      const void* scales, const void* zeros, const int32_t* kv_page_indices,
                      const int32_t* kv_page_indptr, const int32_t* kv_last_page_len,
                      uint32_t batch, uint32_t num_heads, uint32_t page_size,
                      uint32_t max_pages_per_req, float sm_scale, void* stream);
int twl_gemv_int8_nhd(const void* q, void* o, uint32_t o_stride, const uint8_t* k_u8,
                      const void* scales, const void* zeros, const int32_t* kv_page_indices,
                      const int32_t* kv_page_indptr, const int32_t* kv_last_page_len,
                      uint32_t batch, uint32_t num_heads, uint32_t page_size,
                      uint32_t max_pages_per_req, float sm_scale, void* stream);
int twl_gemv_f16_nhd(const void* q, void* o, uint32_t o_stride, const void* k_cache,
                     const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                     const int32_t* kv_last_page_len, uint32_t batch, uint32_t num_heads,
                     uint32_t page_size, uint32_t max_pages_per_req, float sm_scale, void* stream);
int twl_gemv_f16_single(const void* q, void* o, const void* k, uint32_t num_heads,
                        uint32_t seq_len, float sm_scale, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Sparse paged decode attention over survivor lists.
 * Replaces: the masked softmax.V of twilight/pyimpl/attention.py:188-190,299-306 restricted to
 * the surviving tokens. logits = sm_scale * q.K (fp32), softmax in fp32, probabilities rounded to
 * the q dtype before the V product (attention.py:302-304), fp32 accumulation, output in the q
 * dtype [batch, num_q_heads, 128]. Rows with count 0 produce zeros. lse_out (nullable) float
 * [rows] receives log(sum exp(logit)) of the row.
 * k_cache / v_cache: element type kv_dtype (TWL_F16 / TWL_BF16, must equal q's type); element
 * (page, token, kv_head, d) lives at page*page_stride + token*token_stride + kv_head*head_stride + d.
 * Rows longer than 128 survivors are split over several workgroups that meet in `workspace`
 * (256-byte aligned, at least twl_sparse_attn_workspace_bytes(rows, idx_stride) bytes, no initial
 * contents required: its first rows*8 bytes are 64-bit ticket words that carry a 48-bit tag of
 * the call, drawn from a per-process random sequence, so a word left by a call that never
 * finished, or memory that was never cleared, counts as zero unless it happens to hold the
 * call's tag, a 2^-48 event per split row; a finished call leaves the words zero).
 * Two calls that share a workspace must not overlap in time. In a split row the
 * softmax weights are not rounded to the q dtype before the V product (the partial sums are
 * merged in fp32); a row of at most 128 survivors follows the reference rounding exactly.
 * ------------------------------------------------------------------------------------------- */
uint64_t twl_sparse_attn_workspace_bytes(uint32_t rows, uint32_t idx_stride);
int twl_sparse_attn(const void* q, void* out, int dtype, const void* k_cache, const void* v_cache,
                    uint64_t page_stride, uint64_t token_stride, uint64_t head_stride,
                    const int32_t* idx, uint32_t idx_stride, const int32_t* count,
                    const int32_t* kv_page_indices, const int32_t* kv_page_indptr, uint32_t batch,
                    uint32_t num_q_heads, uint32_t num_kv_heads, float sm_scale, float* lse_out,
                    void* workspace, uint64_t workspace_bytes, void* stream);
/* twl_sparse_attn for callers that cannot allocate (code under HIP graph capture, serving loops
 * and harnesses that forbid hipMalloc, callers with no workspace to bring). It has no counterpart
 * in the reference. Same arguments and results as twl_sparse_attn without the workspace: the
 * split-row partial results and tickets live in an array of TWL_STATIC_SCRATCH_BYTES bytes that is
 * part of the library's device image (every GPU the library runs on holds it until the process
 * ends). The call allocates and frees nothing. Returns TWL_ETOOBIG when
 * twl_sparse_attn_workspace_bytes(batch * num_q_heads, idx_stride) exceeds that size (24 MiB hold
 * 512 rows of up to 8192 survivors). The array used is the current device's: TWL_EINVAL when q
 * does not live on the current device. The first call on a device looks up the array's address
 * there and must happen outside stream capture (TWL_EINVAL on a capturing stream; later calls
 * may be captured). All calls on one GPU share the array: calls that
 * overlap in time on one GPU (two streams, two threads) race. Nothing in the array has to be
 * cleared between calls (the ticket words are tagged per call), so the call is one launch. */
#define TWL_STATIC_SCRATCH_BYTES (24u << 20)
int twl_sparse_attn_static(const void* q, void* out, int dtype, const void* k_cache,
                           const void* v_cache, uint64_t page_stride, uint64_t token_stride,
                           uint64_t head_stride, const int32_t* idx, uint32_t idx_stride,
                           const int32_t* count, const int32_t* kv_page_indices,
                           const int32_t* kv_page_indptr, uint32_t batch, uint32_t num_q_heads,
                           uint32_t num_kv_heads, float sm_scale, float* lse_out, void* stream);

/* Attention over the survivor lists with GIVEN weights in place of the q.K logits.
 * Replaces: twilight/pyimpl/attention.py:295-296 (use_estimated_weights_in_attn: the estimator's
 * logits stand in for the exact ones) followed by the masked softmax.V of :299-306. The softmax
 * over the survivors of the estimator's logits equals the estimator's candidate probabilities
 * renormalised over the survivors, so the weights are those probabilities:
 *   out[row] = sum_j w[row, j] * V[idx[row, j]] / sum_j w[row, j],   j < count[row]
 * weights: float [batch * num_q_heads, idx_stride], entry j beside idx[row, j]; negative values
 * count as zero; a row whose weights sum to zero gives NaN, as a softmax over nothing does.
 * Neither q nor K is read. Rounding as in twl_sparse_attn: in a row of at most 128 survivors the
 * normalised weights are rounded to `dtype` before the V product (attention.py:302-304), longer
 * rows keep fp32. lse_out (nullable) receives log(sum_j w[row, j]). Workspace as twl_sparse_attn. */
int twl_sparse_attn_weighted(void* out, int dtype, const void* v_cache, uint64_t page_stride,
                             uint64_t token_stride, uint64_t head_stride, const int32_t* idx,
                             uint32_t idx_stride, const int32_t* count, const float* weights,
                             const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                             uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                             float* lse_out, void* workspace, uint64_t workspace_bytes,
                             void* stream);

/* ---------------------------------------------------------------------------------------------
 * Paged decode attention with ONE token list per (request, kv head), shared by the kv head's
 * G = num_q_heads / num_kv_heads query heads (G in {1, 2, 4, 8}): K and V of a token are fetched
 * once for the group.
 * Replaces: the same masked softmax.V of twilight/pyimpl/attention.py:188-190,299-306, (a) over
 * every token of the request (group_idx == NULL; kv_last_page_len gives the length): the dense
 * decode of the layers a configuration leaves dense (attention.py:199-201, config default :413)
 * and the dense baseline; (b) over group_idx int32 [batch, num_kv_heads, idx_stride] ascending
 * token positions with group_count int32 [batch, num_kv_heads], e.g. the union of the group's
 * survivor sets (twl_group_union): the "top-p per kv-head group" reading of GQA, where the
 * reference itself repeats K / V per q head (attention.py:124-126).
 * max_tokens: upper bound of the request lengths (dense form: tokens of a request beyond it are
 * not attended to; ignored with a list, whose bound is idx_stride). out [batch, num_q_heads, 128] in dtype, lse_out (nullable) float
 * [batch, num_q_heads]; an empty list gives a zero row and lse -inf. workspace: at least
 * twl_group_attn_workspace_bytes(...) bytes, 16-byte aligned, no initial contents required; two
 * calls that share it must not overlap in time. The softmax weights stay in fp32 (they are not
 * rounded to dtype before the V product as attention.py:302-304 does; the difference is below
 * the rounding of the output).
 * ------------------------------------------------------------------------------------------- */
uint64_t twl_group_attn_workspace_bytes(uint32_t batch, uint32_t num_q_heads,
                                        uint32_t num_kv_heads, uint32_t max_tokens, int with_list);
int twl_group_attn(const void* q, void* out, int dtype, const void* k_cache, const void* v_cache,
                   uint64_t page_stride, uint64_t token_stride, uint64_t head_stride,
                   const int32_t* group_idx, uint32_t idx_stride, const int32_t* group_count,
                   uint32_t max_tokens, const int32_t* kv_page_indices,
                   const int32_t* kv_page_indptr, const int32_t* kv_last_page_len, uint32_t batch,
                   uint32_t num_q_heads, uint32_t num_kv_heads, float sm_scale, float* lse_out,
                   void* workspace, uint64_t workspace_bytes, void* stream);
/* Union of the survivor lists of each kv head's q heads (mask OR over the group; the per-head
 * lists are those of twl_top_p_* / twl_decode_layer: idx int32 [batch, num_q_heads, idx_stride],
 * count int32 [batch, num_q_heads]; at most 8 q heads per kv head). Token positions must be
 * < max_tokens (<= 262144). Output:
 * group_idx int32 [batch, num_kv_heads, group_stride] ascending, group_count int32
 * [batch, num_kv_heads]; a union longer than group_stride is cut to its first group_stride
 * positions (group_stride >= min(max_tokens, G * idx_stride) never cuts). */
int twl_group_union(const int32_t* idx, uint32_t idx_stride, const int32_t* count, uint32_t batch,
                    uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t max_tokens,
                    int32_t* group_idx, uint32_t group_stride, int32_t* group_count, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Quest page selector: page score + top-k pages per row.
 * Replaces: quest_selector, twilight/pyimpl/quest.py:17-122, in its page-metadata form:
 * score(page) = sum_d max(q_d * max_d, q_d * min_d) (== (q*sign) . amax(K*sign), quest.py:37-84),
 * k = min(pages of the request, max(1, budget/16) + (budget%16 != 0)) (quest.py:93-98), top-k by
 * score with ties resolved toward the lower page number. Output: sel_pages [rows, sel_stride]
 * ascending logical page numbers, sel_count [rows]. page_scores (nullable) float
 * [rows, score_stride] receives the raw page scores (required: it is also the staging area).
 * ------------------------------------------------------------------------------------------- */
int twl_quest_select(const void* q, int q_dtype, const void* meta, const int32_t* kv_page_indices,
                     const int32_t* kv_page_indptr, uint32_t batch, uint32_t num_q_heads,
                     uint32_t num_kv_heads, uint32_t token_budget, uint32_t max_pages_per_req,
                     int32_t* sel_pages, uint32_t sel_stride, int32_t* sel_count,
                     float* page_scores, uint32_t score_stride, void* stream);
/* The two kernels of twl_quest_select as separate calls: page scores only (quest.py:36-84), and
 * top-k page selection over given scores (quest.py:93-122). */
int twl_quest_page_scores(const void* q, int q_dtype, const void* meta,
                          const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                          uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                          uint32_t max_pages_per_req, float* page_scores, uint32_t score_stride,
                          void* stream);
int twl_quest_topk_pages(const float* page_scores, uint32_t score_stride,
                         const int32_t* kv_page_indptr, uint32_t batch, uint32_t num_q_heads,
                         uint32_t token_budget, uint32_t max_pages_per_req, int32_t* sel_pages,
                         uint32_t sel_stride, int32_t* sel_count, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Rotary position embedding of one decode token, in place: q [batch, num_q_heads, 128] and
 * k [batch, num_kv_heads, 128] in dtype, cos / sin [batch, 128] in dtype (the values of the
 * request's position).
 * Replaces: apply_rotary_pos_emb as called at twilight/pyimpl/attention.py:118-123 (half-split
 * convention: out = x * cos + rotate_half(x) * sin, rotate_half(x) = (-x[64:], x[:64])), with
 * the roundings of its chain of element-wise tensor operations (each product and the sum rounded
 * to dtype), so the result is bit-identical to the unfused form; one launch instead of about ten.
 * ------------------------------------------------------------------------------------------- */
int twl_rope_qk(void* q, void* k, const void* cos, const void* sin, int dtype, uint32_t batch,
                uint32_t num_q_heads, uint32_t num_kv_heads, void* stream);

/* ---------------------------------------------------------------------------------------------
 * KV-append side: build the INT4 shadow and the Quest metadata of whole pages from the paged K.
 * Replaces: min_max_per_token_quant_kv, twilight/pyimpl/quantize.py:4-13 (applied per group of 32
 * with fp16 scale / zero storage) and the per-chunk amax of twilight/pyimpl/quest.py:68-74.
 * Processes physical pages page_ids[0..num_pages) (page_ids == NULL: pages 0..num_pages-1);
 * valid_len (nullable) int32 [num_pages] gives the valid tokens of each page (default 16): the
 * metadata covers only valid tokens, nibbles of invalid tokens are written as 0 with scale 0.
 * k_int4 and/or meta may be NULL to skip that output.
 * ------------------------------------------------------------------------------------------- */
int twl_kv_shadow_build(const void* k_cache, int kv_dtype, uint64_t page_stride,
                        uint64_t token_stride, uint64_t head_stride, const int32_t* page_ids,
                        const int32_t* valid_len, uint32_t num_pages, uint32_t num_kv_heads,
                        void* k_int4, void* meta, void* stream);

/* Decode append of one token per request in one launch (the per-step form of the row above;
 * twilight/pyimpl/attention.py:138-141 appends to the HF cache and :247-251 re-quantises all of K
 * instead). k_new / v_new are [batch, num_kv_heads, 128] with element strides (batch, head). For
 * request b the token goes to slot s = kv_last_page_len[b] (0..15) of its LAST listed page; the
 * caller has appended a fresh page to the table and set the length to 0 when the previous page was
 * full. Writes the K / V rows, the token's INT4 codes and (scale, zero) pairs (a fresh page's
 * other tokens are zeroed), folds the row into the page's min / max metadata (records and, when
 * meta_planes is given, the plane layout below), and stores s + 1 to kv_last_page_len[b].
 * k_int4 / meta / meta_planes may be NULL. Records are identical to what
 * twl_kv_shadow_build gives for the same page contents. */
int twl_kv_append(const void* k_new, const void* v_new, int kv_dtype, uint64_t new_batch_stride,
                  uint64_t new_head_stride, void* k_cache, void* v_cache, uint64_t page_stride,
                  uint64_t token_stride, uint64_t head_stride, const int32_t* kv_page_indices,
                  const int32_t* kv_page_indptr, int32_t* kv_last_page_len, uint32_t batch,
                  uint32_t num_kv_heads, void* k_int4, void* meta, void* meta_planes,
                  uint32_t plane_cap_pages, const int32_t* plane_slots, uint32_t plane_num_slots,
                  void* stream);

/* Quest metadata in PLANE layout: planes[slot][kv_head][d][0 = min, 1 = max][logical page], 16-bit
 * values in the cache dtype, plane_cap_pages (a multiple of 8) pages per run, slot = position of
 * the request in the batch. For one query only the run selected by the sign of q_d is read
 * (score = sum_d q_d * (q_d > 0 ? max_d : min_d), twilight/pyimpl/quest.py:37-84), so the scoring
 * pass of twl_select_estimate_prune touches half the bytes of the record layout. Nothing in the
 * reference corresponds to it (it recomputes the chunk maxima from K every step, quest.py:68-74).
 * twl_meta_planes_build fills the planes of the pages of the current page table from the metadata
 * records of twl_kv_shadow_build. A request's LAST page is always scored from its record, not from
 * the planes: twl_kv_append (given meta_planes) folds a new token into the record at every step
 * and writes the page's plane entries once, when the token completes the page. The plane entries
 * of a last page may therefore be stale; every kernel here ignores them.
 * plane_slots (nullable, device, [batch]) names the slot of every batch position, so that a
 * request keeps its planes when its position in the batch changes (continuous batching: a request
 * leaves and the others move up); plane_num_slots is the number of slots the buffer holds, and
 * entries outside [0, plane_num_slots) are clamped. NULL: slot = batch position. Two positions of
 * one batch must not name the same slot. */
int twl_meta_planes_build(const void* meta, const int32_t* kv_page_indices,
                          const int32_t* kv_page_indptr, uint32_t batch, uint32_t num_kv_heads,
                          uint32_t max_pages_per_req, void* meta_planes, uint32_t plane_cap_pages,
                          const int32_t* plane_slots, uint32_t plane_num_slots, void* stream);
/* twl_quest_page_scores from the plane layout (one q head per row reads the runs its signs
 * select: half the bytes of the record form; with GQA the q heads of a group do not share reads
 * here, the record form does). Scores are accumulated channel by channel in ascending order. */
int twl_quest_page_scores_planes(const void* q, int q_dtype, const void* meta_planes,
                                 uint32_t plane_cap_pages, const int32_t* plane_slots,
                                 uint32_t plane_num_slots, const void* meta,
                                 const int32_t* kv_page_indices, const int32_t* kv_page_indptr,
                                 uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                                 uint32_t max_pages_per_req, float* page_scores,
                                 uint32_t score_stride, void* stream);

/* Unpack INT4 shadow records to fp32: out [num_pages, num_kv_heads, 16, 128] (record order).
 * Exists so that tests can compare dequantised values bit for bit. */
int twl_dequant_int4(const void* k_int4, uint32_t num_records, float* out, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Double-Sparse label ops (strides are in elements).
 * twl_get_label_tensor replaces get_label_tensor, twilight/kernel/triton/channel.py:11-79:
 *   out[l,h,c] = x[l,h,channel[h,c]], elements of elem_bytes (2 or 4) bytes, channel int64.
 * twl_bgemv_int8 replaces bgemv_int8, twilight/kernel/triton/bgemv_int8.py:12-75:
 *   out[b,h,n] = (sum_c q[b,h,c] * k[b*n_ctx+n,h,c]) * scale[b*n_ctx+n,h]; q / scale / out fp16,
 *   k int8, fp32 accumulation.
 * ------------------------------------------------------------------------------------------- */
int twl_get_label_tensor(const void* x, const int64_t* channel, void* out, uint32_t elem_bytes,
                         uint32_t L, uint32_t H, uint32_t r, int64_t sx_l, int64_t sx_h,
                         int64_t sx_d, int64_t sc_h, int64_t sc_c, int64_t so_l, int64_t so_h,
                         int64_t so_c, void* stream);
int twl_bgemv_int8(const void* q_label, const int8_t* k_label, const void* k_scales, void* out,
                   uint32_t B, uint32_t H, uint32_t r, uint32_t n_ctx, int64_t sq_b, int64_t sq_h,
                   int64_t sq_d, int64_t sk_t, int64_t sk_h, int64_t sk_d, int64_t ss_t,
                   int64_t ss_h, int64_t so_b, int64_t so_h, int64_t so_n, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Base-2 log-sum-exp of per-block-quantised int8 Q.K^T (int8 matrix cores).
 * Replaces: qk_int8_per_block, twilight/kernel/triton/qk_int8_per_block.py:22-143 (its `lse`
 * output, :105-109; its first output is identically zero because V is never accumulated).
 *   lse[b,h,m] = log2 sum_n 2^( float(q[b,h,m,:] . k[b,h/group,n,:]) * q_scale[b,h,m/128]
 *                                                                  * k_scale[b,h/group,n/64] )
 * over n < 64*ceil(kv_len/64); keys in [kv_len, 64*ceil(kv_len/64)) count as all-zero rows, as the
 * reference's masked loads make them (:36-37). q / k int8 with byte strides (batch, head, row) and
 * contiguous head_dim (64 or 128); pointers and strides must be multiples of 16. q_scale fp32
 * [batch, num_q_heads, ceil(qo_len/128)], k_scale fp32 [batch, num_kv_heads, ceil(kv_len/64)],
 * lse fp32 [batch, num_q_heads, qo_len].
 * ------------------------------------------------------------------------------------------- */
int twl_qk_int8_lse(const int8_t* q, const int8_t* k, const float* q_scale, const float* k_scale,
                    float* lse, uint32_t batch, uint32_t num_q_heads, uint32_t num_kv_heads,
                    uint32_t qo_len, uint32_t kv_len, uint32_t head_dim, int64_t sq_b,
                    int64_t sq_h, int64_t sq_n, int64_t sk_b, int64_t sk_h, int64_t sk_n,
                    void* stream);

/* ---------------------------------------------------------------------------------------------
 * The whole decode layer on one stream: quest select -> INT4 GEMV -> softmax + top-p -> sparse
 * attention (twilight/pyimpl/attention.py:188-306 for q_len == 1). Every intermediate is a
 * caller-provided buffer (see the field comments); no host synchronisation happens inside.
 * ------------------------------------------------------------------------------------------- */
typedef struct twl_layer_args {
  /* inputs */
  const void* q;            /* [batch, num_q_heads, 128], dtype */
  int dtype;                /* TWL_F16 or TWL_BF16: type of q, K, V and out */
  const void* k_cache;      /* paged K */
  const void* v_cache;      /* paged V */
  uint64_t page_stride, token_stride, head_stride; /* element strides of both caches */
  const void* k_int4;       /* INT4 shadow records */
  const void* meta;         /* Quest metadata records */
  const void* meta_planes;  /* the same in plane layout (nullable), see twl_meta_planes_build */
  uint32_t plane_cap_pages;
  const int32_t* plane_slots; /* nullable: plane slot of each batch position */
  uint32_t plane_num_slots;
  const int32_t* kv_page_indices;
  const int32_t* kv_page_indptr;
  const int32_t* kv_last_page_len;
  uint32_t batch, num_q_heads, num_kv_heads;
  uint32_t max_pages_per_req; /* >= the longest request's page count */
  uint32_t token_budget;      /* Quest budget in tokens (selector: token_budget) */
  float top_p;                /* pruner threshold */
  int high_mode;              /* twl_top_p_high */
  float sm_scale;             /* 1/sqrt(128) in the reference */
  /* workspaces / intermediate outputs, all caller-owned */
  int32_t* sel_pages;  uint32_t sel_stride;  /* [rows, sel_stride], sel_stride >= selected pages */
  int32_t* sel_count;                        /* [rows] */
  float* page_scores;  uint32_t page_score_stride; /* [rows, >= max_pages_per_req]; NULL: the
                                                      head of `scores` is used as staging and
                                                      score_stride must be >= max_pages_per_req */
  float* scores;       uint32_t score_stride;/* [rows, score_stride], >= 16 * selected pages */
  int32_t* cand_count;                       /* [rows] */
  int32_t* idx;        uint32_t idx_stride;  /* [rows, idx_stride], >= 16 * selected pages */
  int32_t* count;                            /* [rows] */
  void* attn_workspace; uint64_t attn_workspace_bytes; /* see twl_sparse_attn */
  /* output */
  void* out;                /* [batch, num_q_heads, 128], dtype */
  /* 0 = let the library choose by batch shape: with one q head per kv head, between half a row
   * and two rows per compute unit and <= 8192 pages per request the selector, estimator and
   * pruner are ONE launch (twl_select_estimate_prune); with fewer rows than half the compute
   * units every stage is its own launch (the estimator needs more workgroups than rows);
   * otherwise twl_quest_select + twl_gemv_top_p. 1 = always every stage its own launch
   * (twl_quest_select, twl_gemv_int4, twl_softmax_top_p_f32). The results are the same either
   * way; with 0, `scores` and `page_scores` are guaranteed filled only when keep_scores != 0. */
  int split_estimator;
  int keep_scores;
  /* Group attention (optional; group_idx == NULL: every q head attends over its own survivor
   * list, as the reference's repeated K / V does, attention.py:124-126). With group_idx the q
   * heads of a kv head attend over the UNION of their survivor lists (twl_group_union, then
   * twl_group_attn): group_idx int32 [batch, num_kv_heads, group_idx_stride] and group_count
   * int32 [batch, num_kv_heads] receive the unions; group_idx_stride >= min(16 *
   * max_pages_per_req, G * 16 * k) never cuts one. group_workspace: at least
   * twl_group_attn_workspace_bytes(batch, num_q_heads, num_kv_heads, group_idx_stride, 1) bytes.
   * Needs 16 * max_pages_per_req <= 262144 and G in {1, 2, 4, 8}. */
  int32_t* group_idx; uint32_t group_idx_stride;
  int32_t* group_count;
  void* group_workspace; uint64_t group_workspace_bytes;
  /* use_estimated_weights != 0: the attention takes the estimator's weights instead of exact q.K
   * logits (use_estimated_weights_in_attn, attention.py:295-296; see twl_sparse_attn_weighted).
   * surv_probs: float [rows, idx_stride], required then; it receives the estimator's probability
   * of every survivor beside idx. Whenever surv_probs is given it is filled, whatever the flag.
   * Not available together with group_idx. */
  float* surv_probs;
  int use_estimated_weights;
  /* group_select != 0 (G = num_q_heads / num_kv_heads in {2, 4, 8}): the Quest selection is made
   * per kv head — a page's score is the largest of its group's q-head scores — so the q heads of
   * a group share one candidate list, the metadata and the INT4 records are read once per kv head
   * (twl_quest_page_scores per group, twl_quest_topk_pages, twl_gemv_int4_group,
   * twl_softmax_top_p_f32), and every q head still prunes and attends on its own scores. Not the
   * reference's per-q-head selection (attention.py:124-126 repeats K per q head): an option, as
   * group_idx is. sel_pages / sel_count hold the group's list in each of its q-head rows;
   * `scores`, `cand_count` and `page_scores` (all required: TWL_ENULL before anything is
   * launched) are always written. */
  int group_select;
} twl_layer_args;

int twl_decode_layer(const twl_layer_args* args, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TWILIGHT_HIP_H_ */
