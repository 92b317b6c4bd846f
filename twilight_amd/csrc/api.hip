// Library-level entry points: status strings, version, and the whole decode layer as one call
// that enqueues the kernels of the path back to back on the caller's stream.
#include "twl_common.h"

extern "C" const char* twl_strerror(int status) {
  switch (status) {
    case TWL_OK: return "ok";
    case TWL_ENULL: return "a required pointer is NULL";
    case TWL_EINVAL: return "a size, stride or mode argument is out of range";
    case TWL_EDTYPE: return "unsupported element type";
    case TWL_EALIGN: return "pointer or stride alignment not supported";
    case TWL_ELAUNCH: return "HIP kernel launch failed";
    case TWL_ENODEVICE: return "no usable HIP device";
    case TWL_ETOOBIG: return "the problem does not fit a fixed-size buffer of the library";
    default: return "unknown twl_status";
  }
}

extern "C" int twl_abi_version(void) { return TWL_ABI_VERSION; }

extern "C" int twl_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return TWL_ENODEVICE;
  }
  return n;
}

namespace twl {
int layer_attention(const twl_layer_args* a, void* stream);
}

// twilight/pyimpl/attention.py:188-306 for q_len == 1: selector -> estimator -> pruner -> attention.
extern "C" int twl_decode_layer(const twl_layer_args* a, void* stream) {
  if (!a) return TWL_ENULL;
  if (!a->sel_pages || !a->sel_count || !a->scores || !a->cand_count || !a->idx || !a->count ||
      !a->out)
    return TWL_ENULL;
  if (a->group_idx && (!a->group_count || !a->group_workspace)) return TWL_ENULL;
  if (a->use_estimated_weights && !a->surv_probs) return TWL_ENULL;
  if (a->use_estimated_weights && a->group_idx) return TWL_EINVAL;
  if (a->batch == 0 || a->num_q_heads == 0) return TWL_EINVAL;
  const uint32_t rows = a->batch * a->num_q_heads;
  uint32_t k = (a->token_budget / TWL_PAGE ? a->token_budget / TWL_PAGE : 1) +
               (a->token_budget % TWL_PAGE ? 1 : 0);
  if (k > a->max_pages_per_req) k = a->max_pages_per_req;
  if (a->sel_stride < k || a->score_stride < k * TWL_PAGE || a->idx_stride < k * TWL_PAGE)
    return TWL_EINVAL;
  float* page_scores = a->page_scores ? a->page_scores : a->scores;
  const uint32_t ps_stride = a->page_scores ? a->page_score_stride : a->score_stride;
  if (ps_stride < a->max_pages_per_req) return TWL_EINVAL;
  if (k * TWL_PAGE > TWL_MAX_CANDIDATES) return TWL_EINVAL;

  int rc;
  if (a->group_select && a->num_q_heads != a->num_kv_heads) {
    // one candidate list per kv head: scores (group maximum) -> top-k -> group GEMV -> pruner.
    // Everything the four launches need is checked before the first one: the score matrix and
    // the candidate counts travel through memory between them (requests shorter than the budget
    // leave score slots unwritten, which only cand_count tells the pruner).
    if (!a->page_scores || !a->meta || !a->k_int4 || !a->scores || !a->cand_count ||
        !a->sel_pages || !a->sel_count || !a->q || !a->kv_page_indices || !a->kv_page_indptr ||
        !a->kv_last_page_len)
      return TWL_ENULL;
    {
      const uint32_t g = a->num_kv_heads ? a->num_q_heads / a->num_kv_heads : 0;
      if (a->num_kv_heads == 0 || a->num_q_heads % a->num_kv_heads != 0 ||
          (g != 2 && g != 4 && g != 8))
        return TWL_EINVAL;
    }
    rc = twl::quest_page_scores_ex(a->q, a->dtype, a->meta, a->kv_page_indices,
                                   a->kv_page_indptr, a->batch, a->num_q_heads, a->num_kv_heads,
                                   a->max_pages_per_req, a->page_scores, a->page_score_stride, 1,
                                   stream);
    if (rc != TWL_OK) return rc;
    rc = twl_quest_topk_pages(a->page_scores, a->page_score_stride, a->kv_page_indptr, a->batch,
                              a->num_q_heads, a->token_budget, a->max_pages_per_req,
                              a->sel_pages, a->sel_stride, a->sel_count, stream);
    if (rc != TWL_OK) return rc;
    rc = twl_gemv_int4_group(a->q, a->dtype, a->scores, a->score_stride, a->cand_count, a->k_int4,
                             a->sel_pages, a->sel_count, a->sel_stride, a->kv_page_indices,
                             a->kv_page_indptr, a->kv_last_page_len, a->batch, a->num_q_heads,
                             a->num_kv_heads, k, a->sm_scale, stream);
    if (rc != TWL_OK) return rc;
    rc = twl::softmax_top_p_ex(a->scores, a->score_stride, a->cand_count, rows, k * TWL_PAGE,
                               nullptr, a->top_p, a->high_mode, a->sel_pages, a->sel_stride,
                               a->idx, a->idx_stride, a->count, nullptr, nullptr, a->surv_probs,
                               stream);
    if (rc != TWL_OK) return rc;
    return twl::layer_attention(a, stream);
  }
  int cus = 0;
  const bool have_cus = twl::device_cu_count(&cus) == TWL_OK;
  // Fewer rows than half the compute units: a workgroup per row leaves most of the chip idle while
  // each row streams its pages one memory round trip after the other, so the estimator runs as a
  // GEMV over many short wavefronts and the pruner as a launch of its own (measured at 32 q heads,
  // 32768 tokens: 57 -> 43 us at batch 1, 63 -> 56 us at batch 3, equal at batch 4).
  // (With q heads sharing kv heads the separate launches are still ahead at exactly half a row
  // per unit: 56.6 against 59.7 us.)
  const bool gqa = a->num_q_heads != a->num_kv_heads;
  const bool split = a->split_estimator ||
                     (have_cus && (2u * rows < (uint32_t)cus || (gqa && 2u * rows == (uint32_t)cus)));
  // one workgroup per row from the metadata to the survivor list pays off while there are about
  // as many rows as compute units (measured: ahead from half a row per unit on; with the record
  // layout up to two rows per unit, with the plane layout at every larger batch tried). With
  // q heads sharing kv heads it needs the plane layout to be ahead of the grouped scoring kernel
  // (which reads each record once per group): 56 us against 64 us, with records 65 us.
  const bool planes_fit = a->meta_planes && a->plane_cap_pages >= a->max_pages_per_req;
  const bool row_kernel = !split && (a->num_q_heads == a->num_kv_heads || planes_fit) &&
                          a->max_pages_per_req <= 8192 && have_cus &&
                          2u * rows >= (uint32_t)cus && (planes_fit || rows <= 2u * (uint32_t)cus);
  if (row_kernel) {
    // 1+2+3. page scores, top-k pages, INT4 estimate, softmax, top-p, compaction: one launch
    rc = twl::select_estimate_prune_ex(
        a->q, a->dtype, a->meta, a->k_int4, a->kv_page_indices, a->kv_page_indptr,
        a->kv_last_page_len, a->batch, a->num_q_heads, a->num_kv_heads, a->token_budget,
        a->max_pages_per_req, a->sm_scale, nullptr, a->top_p, a->high_mode, a->sel_pages,
        a->sel_stride, a->sel_count, a->idx, a->idx_stride, a->count,
        a->keep_scores ? a->page_scores : nullptr, a->page_score_stride,
        a->keep_scores ? a->scores : nullptr, a->score_stride, a->cand_count, a->meta_planes,
        a->plane_cap_pages, a->plane_slots, a->plane_num_slots, a->surv_probs, stream);
    if (rc != TWL_OK) return rc;
  } else {
    // 1. Quest page scores + top-k pages; without GQA sharing the plane layout halves the read
    if (k == a->max_pages_per_req && !a->keep_scores) {
      // no request is longer than the budget: every page is kept, no metadata is read (the
      // selection does not look at the scores when it keeps everything)
      rc = twl_quest_topk_pages(page_scores, ps_stride, a->kv_page_indptr, a->batch,
                                a->num_q_heads, a->token_budget, a->max_pages_per_req,
                                a->sel_pages, a->sel_stride, a->sel_count, stream);
    } else if (a->meta_planes && a->num_q_heads == a->num_kv_heads &&
               a->plane_cap_pages >= a->max_pages_per_req) {
      rc = twl_quest_page_scores_planes(a->q, a->dtype, a->meta_planes, a->plane_cap_pages,
                                        a->plane_slots, a->plane_num_slots, a->meta,
                                        a->kv_page_indices, a->kv_page_indptr, a->batch, a->num_q_heads,
                                        a->num_kv_heads, a->max_pages_per_req, page_scores,
                                        ps_stride, stream);
      if (rc != TWL_OK) return rc;
      rc = twl_quest_topk_pages(page_scores, ps_stride, a->kv_page_indptr, a->batch,
                                a->num_q_heads, a->token_budget, a->max_pages_per_req,
                                a->sel_pages, a->sel_stride, a->sel_count, stream);
    } else {
      rc = twl_quest_select(a->q, a->dtype, a->meta, a->kv_page_indices, a->kv_page_indptr,
                            a->batch, a->num_q_heads, a->num_kv_heads, a->token_budget,
                            a->max_pages_per_req, a->sel_pages, a->sel_stride, a->sel_count,
                            page_scores, ps_stride, stream);
    }
    if (rc != TWL_OK) return rc;
    if (!split) {
      // 2+3. INT4 estimate, softmax, top-p and compaction in one launch
      rc = twl::gemv_top_p_ex(a->q, a->dtype, a->k_int4, a->sel_pages, a->sel_count, a->sel_stride,
                          a->kv_page_indices, a->kv_page_indptr, a->kv_last_page_len, a->batch,
                          a->num_q_heads, a->num_kv_heads, k, a->sm_scale, nullptr, a->top_p,
                          a->high_mode, a->idx, a->idx_stride, a->count,
                          a->keep_scores ? a->scores : nullptr, a->score_stride, a->cand_count,
                          nullptr, a->surv_probs, stream);
      if (rc != TWL_OK) return rc;
    } else {
      // 2. INT4 estimate over the selected pages
      rc = twl_gemv_int4(a->q, a->dtype, a->scores, a->score_stride, a->cand_count, a->k_int4,
                         a->sel_pages, a->sel_count, a->sel_stride, a->kv_page_indices,
                         a->kv_page_indptr, a->kv_last_page_len, a->batch, a->num_q_heads,
                         a->num_kv_heads, k, a->sm_scale, stream);
      if (rc != TWL_OK) return rc;
      // 3. softmax + top-p + compaction to token positions
      rc = twl::softmax_top_p_ex(a->scores, a->score_stride, a->cand_count, rows, k * TWL_PAGE,
                                 nullptr, a->top_p, a->high_mode, a->sel_pages, a->sel_stride,
                                 a->idx, a->idx_stride, a->count, nullptr, nullptr,
                                 a->surv_probs, stream);
      if (rc != TWL_OK) return rc;
    }
  }
  return twl::layer_attention(a, stream);
}

// 4. exact attention over the survivors: per q head, or per kv head over the group's union
int twl::layer_attention(const twl_layer_args* a, void* stream) {
  int rc;
  if (a->group_idx) {
    if (!a->group_count || !a->group_workspace) return TWL_ENULL;
    rc = twl_group_union(a->idx, a->idx_stride, a->count, a->batch, a->num_q_heads,
                         a->num_kv_heads, a->max_pages_per_req * TWL_PAGE, a->group_idx,
                         a->group_idx_stride, a->group_count, stream);
    if (rc != TWL_OK) return rc;
    return twl_group_attn(a->q, a->out, a->dtype, a->k_cache, a->v_cache, a->page_stride,
                          a->token_stride, a->head_stride, a->group_idx, a->group_idx_stride,
                          a->group_count, 0, a->kv_page_indices, a->kv_page_indptr,
                          a->kv_last_page_len, a->batch, a->num_q_heads, a->num_kv_heads,
                          a->sm_scale, nullptr, a->group_workspace, a->group_workspace_bytes,
                          stream);
  }
  if (a->use_estimated_weights)
    return twl_sparse_attn_weighted(a->out, a->dtype, a->v_cache, a->page_stride, a->token_stride,
                                    a->head_stride, a->idx, a->idx_stride, a->count, a->surv_probs,
                                    a->kv_page_indices, a->kv_page_indptr, a->batch,
                                    a->num_q_heads, a->num_kv_heads, nullptr, a->attn_workspace,
                                    a->attn_workspace_bytes, stream);
  return twl_sparse_attn(a->q, a->out, a->dtype, a->k_cache, a->v_cache, a->page_stride,
                         a->token_stride, a->head_stride, a->idx, a->idx_stride, a->count,
                         a->kv_page_indices, a->kv_page_indptr, a->batch, a->num_q_heads,
                         a->num_kv_heads, a->sm_scale, nullptr, a->attn_workspace,
                         a->attn_workspace_bytes, stream);
}
