"""Op surface of the Select-then-Prune decode path.

``top_p_fp16_return_mask``, ``top_p_fp32_return_mask``, ``get_label_tensor``, ``bgemv_int8`` and
``qk_int8_per_block`` are the reference's own names (twilight/kernel/__init__.py:1-3,
twilight/kernel/triton/__init__.py:3-6); the rest are the
index-list / paged forms the decode layer needs, including the call shape of the INT4 GEMV the
reference benchmarks (benchmark/efficiency/bench_gemv.py:445-454).
"""
from .sampling import (top_p_fp16_return_mask, top_p_fp32_return_mask, top_p_select,
                       softmax_top_p)
from .gemv import (batched_sparse_gemv, batched_sparse_gemv_int4_k, batched_sparse_gemv_int8_k,
                   single_sparse_gemv, sparse_gemv_int4, sparse_gemv_int4_top_p,
                   quest_gemv_int4_top_p)
from .attention import (attention_workspace_bytes, group_attention_workspace_bytes,
                        group_paged_decode_attention, group_union_lists, rope_qk_,
                        sparse_paged_decode_attention, weighted_paged_decode_attention)
from .quest import quest_num_pages, quest_select
from .kv_shadow import dequant_int4, kv_append, kv_shadow_build, meta_planes_build
from .label_ops import bgemv_int8, get_label_tensor, qk_int8_per_block

__all__ = [
    "top_p_fp16_return_mask", "top_p_fp32_return_mask", "top_p_select", "softmax_top_p",
    "batched_sparse_gemv", "batched_sparse_gemv_int4_k", "batched_sparse_gemv_int8_k",
    "single_sparse_gemv", "sparse_gemv_int4", "sparse_gemv_int4_top_p", "quest_gemv_int4_top_p",
    "sparse_paged_decode_attention", "weighted_paged_decode_attention",
    "attention_workspace_bytes", "group_paged_decode_attention", "group_union_lists",
    "group_attention_workspace_bytes", "rope_qk_",
    "quest_num_pages", "quest_select", "dequant_int4", "kv_shadow_build", "kv_append", "meta_planes_build",
    "get_label_tensor", "bgemv_int8", "qk_int8_per_block",
]
