"""Quest page selector op (twilight/pyimpl/quest.py:17-122 in page-metadata form)."""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ._check import (check_dim, check_dtype, check_input, check_same_device, dtype_code, ptr,
                     stream_of)


def quest_num_pages(token_budget: int, pages_in_request: int) -> int:
    """Pages kept for a budget: twilight/pyimpl/quest.py:93-98 with chunk_size 16."""
    k = max(1, token_budget // _lib.PAGE) + (1 if token_budget % _lib.PAGE else 0)
    return min(k, pages_in_request)


def quest_select(q: torch.Tensor, meta: torch.Tensor, kv_page_indices: torch.Tensor,
                 kv_page_indptr: torch.Tensor, token_budget: int, max_pages_per_req: int,
                 sel_pages: Optional[torch.Tensor] = None,
                 sel_count: Optional[torch.Tensor] = None,
                 page_scores: Optional[torch.Tensor] = None):
    """Per (batch, head) row: score every page of the request and keep the top pages.

    ``q`` [B,H,128] fp16/bf16; ``meta`` uint8 [pages, Hkv, 512] Quest min/max records in q's
    dtype. Returns ``(sel_pages int32 [B,H,k] ascending logical pages, sel_count int32 [B,H],
    page_scores fp32 [B,H,max_pages_per_req])``; ties at the k-th score keep the lower page.
    """
    check_input(q, "q"); check_dim(3, q, "q")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM:
        raise RuntimeError(f"head_dim must be {_lib.HEAD_DIM}, got {D}")
    check_input(meta, "meta"); check_dtype(meta, torch.uint8, "meta")
    if meta.dim() != 3 or meta.size(2) != _lib.META_RECORD_BYTES:
        raise RuntimeError("meta must be uint8 [pages, kv_heads, 512]")
    Hkv = meta.size(1)
    if H % Hkv != 0:
        raise RuntimeError(f"num_q_heads {H} must be a multiple of num_kv_heads {Hkv}")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr)):
        check_input(t, name); check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1:
        raise RuntimeError("kv_page_indptr must have B+1 elements")
    if token_budget <= 0 or max_pages_per_req <= 0:
        raise RuntimeError("token_budget and max_pages_per_req must be positive")
    check_same_device(q, ("meta", meta), ("kv_page_indices", kv_page_indices),
                      ("kv_page_indptr", kv_page_indptr))
    k = quest_num_pages(token_budget, max_pages_per_req)
    dev = q.device
    with torch.cuda.device(dev):
        if sel_pages is None:
            sel_pages = torch.empty((B, H, k), dtype=torch.int32, device=dev)
        if sel_count is None:
            sel_count = torch.empty((B, H), dtype=torch.int32, device=dev)
        if page_scores is None:
            page_scores = torch.empty((B, H, max_pages_per_req), dtype=torch.float32, device=dev)
        for name, t in (("sel_pages", sel_pages), ("sel_count", sel_count)):
            check_input(t, name); check_dtype(t, torch.int32, name)
        check_input(page_scores, "page_scores"); check_dtype(page_scores, torch.float32, "page_scores")
        rc = _lib.lib().twl_quest_select(
            ptr(q), dtype_code(q.dtype, "q"), ptr(meta), ptr(kv_page_indices), ptr(kv_page_indptr),
            B, H, Hkv, token_budget, max_pages_per_req, ptr(sel_pages), sel_pages.size(-1),
            ptr(sel_count), ptr(page_scores), page_scores.size(-1), stream_of(q))
    _lib.check(rc, "QuestSelect")
    return sel_pages, sel_count, page_scores
