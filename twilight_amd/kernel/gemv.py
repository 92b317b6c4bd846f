"""INT4-K score GEMV ops (estimator of twilight/pyimpl/attention.py:252-255)."""
from __future__ import annotations

import math
from typing import Optional

import torch

from .. import _lib
from ._check import (check_dim, check_dtype, check_input, check_same_device, dtype_code, ptr,
                     stream_of)


def sparse_gemv_int4(q: torch.Tensor, k_int4: torch.Tensor, kv_page_indices: torch.Tensor,
                     kv_page_indptr: torch.Tensor, kv_last_page_len: torch.Tensor,
                     sel_pages: Optional[torch.Tensor] = None,
                     sel_count: Optional[torch.Tensor] = None,
                     max_pages: Optional[int] = None, sm_scale: Optional[float] = None,
                     out: Optional[torch.Tensor] = None, out_count: Optional[torch.Tensor] = None,
                     group_lists: bool = False):
    """``scores[b,h,c] = sm_scale * q[b,h,:] . dequant(K_int4[candidate c])`` in fp32.

    ``q`` [B,H,128] fp16/bf16; ``k_int4`` uint8 [pages, Hkv, 1280] INT4 shadow records;
    the CSR page table of the batch; ``sel_pages`` int32 [B,H,S] per-row ascending logical page
    lists with ``sel_count`` int32 [B,H] (both None: every page of the request, ``max_pages``
    = the longest request's page count). Candidate slots past a request's length are ``-inf``.
    ``group_lists``: the q heads of a kv head share the page list of the group's first q head
    (``twl_gemv_int4_group``: every record fetched once per kv head; 2, 4 or 8 q heads per kv head).
    Returns ``(scores fp32 [B,H,16*max_pages], cand_count int32 [B,H])``.
    """
    check_input(q, "q")
    check_dim(3, q, "q")
    B, H, D = q.shape
    if group_lists and sel_pages is None:
        raise RuntimeError("group_lists needs sel_pages")
    if D != _lib.HEAD_DIM:
        raise RuntimeError(f"head_dim must be {_lib.HEAD_DIM}, got {D}")
    check_input(k_int4, "k_int4")
    check_dtype(k_int4, torch.uint8, "k_int4")
    if k_int4.dim() != 3 or k_int4.size(2) != _lib.INT4_RECORD_BYTES:
        raise RuntimeError("k_int4 must be uint8 [pages, kv_heads, 1280]")
    Hkv = k_int4.size(1)
    if H % Hkv != 0:
        raise RuntimeError(f"num_q_heads {H} must be a multiple of num_kv_heads {Hkv}")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                    ("kv_last_page_len", kv_last_page_len)):
        check_input(t, name)
        check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1 or kv_last_page_len.numel() != B:
        raise RuntimeError("kv_page_indptr must have B+1 and kv_last_page_len B elements")
    sel_stride = 0
    if sel_pages is not None:
        check_input(sel_pages, "sel_pages")
        check_dtype(sel_pages, torch.int32, "sel_pages")
        if sel_pages.dim() != 3 or sel_pages.size(0) != B or sel_pages.size(1) != H:
            raise RuntimeError("sel_pages must be int32 [B, H, S]")
        sel_stride = sel_pages.size(2)
        if max_pages is None:
            max_pages = sel_stride
        if sel_count is not None:
            check_input(sel_count, "sel_count")
            check_dtype(sel_count, torch.int32, "sel_count")
            if sel_count.numel() != B * H:
                raise RuntimeError("sel_count must have B*H elements")
    elif sel_count is not None:
        raise RuntimeError("sel_count given without sel_pages")
    if max_pages is None:
        raise RuntimeError("max_pages is required when sel_pages is None")
    check_same_device(q, ("k_int4", k_int4), ("kv_page_indices", kv_page_indices),
                      ("kv_page_indptr", kv_page_indptr), ("kv_last_page_len", kv_last_page_len),
                      ("sel_pages", sel_pages), ("sel_count", sel_count))
    dev = q.device
    M = max_pages * _lib.PAGE
    with torch.cuda.device(dev):
        if out is None:
            out = torch.empty((B, H, M), dtype=torch.float32, device=dev)
        else:
            check_input(out, "out")
            check_dtype(out, torch.float32, "out")
            if out.dim() != 3 or out.size(0) != B or out.size(1) != H or out.size(2) < M:
                raise RuntimeError("out must be fp32 [B, H, >= 16*max_pages]")
        if out_count is None:
            out_count = torch.empty((B, H), dtype=torch.int32, device=dev)
        scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
        entry = _lib.lib().twl_gemv_int4_group if group_lists else _lib.lib().twl_gemv_int4
        rc = entry(
            ptr(q), dtype_code(q.dtype, "q"), ptr(out), out.size(2), ptr(out_count), ptr(k_int4),
            ptr(sel_pages), ptr(sel_count), sel_stride, ptr(kv_page_indices), ptr(kv_page_indptr),
            ptr(kv_last_page_len), B, H, Hkv, max_pages, scale, stream_of(q))
    _lib.check(rc, "SparseGemvInt4")
    return out, out_count


def sparse_gemv_int4_top_p(q: torch.Tensor, k_int4: torch.Tensor, kv_page_indices: torch.Tensor,
                           kv_page_indptr: torch.Tensor, kv_last_page_len: torch.Tensor,
                           sel_pages: torch.Tensor, sel_count: Optional[torch.Tensor],
                           top_p, high: str = "max", max_pages: Optional[int] = None,
                           sm_scale: Optional[float] = None, return_scores: bool = False,
                           return_low: bool = False):
    """Estimator + pruner in one launch: :func:`sparse_gemv_int4` over the rows' page lists, then
    fp32 softmax, top-p bisection and compaction (twilight/pyimpl/attention.py:252-255,
    twilight/pyimpl/top_p.py:10-15, attention.py:280-281) without materialising the scores.

    Arguments as :func:`sparse_gemv_int4` (``sel_pages`` is required) and
    :func:`twilight_amd.kernel.softmax_top_p`. Returns ``(idx int32 [B,H,16*max_pages], count
    int32 [B,H], cand_count int32 [B,H])`` plus the raw scores and / or the final pivot when asked.
    """
    from .sampling import _check_p, _high_mode
    check_input(q, "q")
    check_dim(3, q, "q")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM:
        raise RuntimeError(f"head_dim must be {_lib.HEAD_DIM}, got {D}")
    check_input(k_int4, "k_int4")
    check_dtype(k_int4, torch.uint8, "k_int4")
    if k_int4.dim() != 3 or k_int4.size(2) != _lib.INT4_RECORD_BYTES:
        raise RuntimeError("k_int4 must be uint8 [pages, kv_heads, 1280]")
    Hkv = k_int4.size(1)
    if H % Hkv != 0:
        raise RuntimeError(f"num_q_heads {H} must be a multiple of num_kv_heads {Hkv}")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                    ("kv_last_page_len", kv_last_page_len), ("sel_pages", sel_pages)):
        check_input(t, name)
        check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1 or kv_last_page_len.numel() != B:
        raise RuntimeError("kv_page_indptr must have B+1 and kv_last_page_len B elements")
    if sel_pages.dim() != 3 or sel_pages.size(0) != B or sel_pages.size(1) != H:
        raise RuntimeError("sel_pages must be int32 [B, H, S]")
    sel_stride = sel_pages.size(2)
    if max_pages is None:
        max_pages = sel_stride
    if max_pages * _lib.PAGE > _lib.MAX_CANDIDATES:
        raise RuntimeError(f"{max_pages * _lib.PAGE} candidates exceed the supported maximum "
                           f"{_lib.MAX_CANDIDATES}")
    if sel_count is not None:
        check_input(sel_count, "sel_count")
        check_dtype(sel_count, torch.int32, "sel_count")
        if sel_count.numel() != B * H:
            raise RuntimeError("sel_count must have B*H elements")
    p_arr, p_val = _check_p(top_p, B * H, q)
    check_same_device(q, ("k_int4", k_int4), ("kv_page_indices", kv_page_indices),
                      ("kv_page_indptr", kv_page_indptr), ("kv_last_page_len", kv_last_page_len),
                      ("sel_pages", sel_pages), ("sel_count", sel_count))
    dev = q.device
    M = max_pages * _lib.PAGE
    with torch.cuda.device(dev):
        idx = torch.empty((B, H, M), dtype=torch.int32, device=dev)
        count = torch.empty((B, H), dtype=torch.int32, device=dev)
        cand = torch.empty((B, H), dtype=torch.int32, device=dev)
        scores = (torch.full((B, H, M), float("-inf"), dtype=torch.float32, device=dev)
                  if return_scores else None)
        low = torch.empty((B, H), dtype=torch.float32, device=dev) if return_low else None
        scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
        rc = _lib.lib().twl_gemv_top_p(
            ptr(q), dtype_code(q.dtype, "q"), ptr(k_int4), ptr(sel_pages), ptr(sel_count),
            sel_stride, ptr(kv_page_indices), ptr(kv_page_indptr), ptr(kv_last_page_len), B, H,
            Hkv, max_pages, scale, ptr(p_arr), p_val, _high_mode(high), ptr(idx), M, ptr(count),
            ptr(scores), M, ptr(cand), ptr(low), stream_of(q))
    _lib.check(rc, "SparseGemvInt4TopP")
    out = [idx, count, cand]
    if return_scores:
        out.append(scores)
    if return_low:
        out.append(low)
    return tuple(out)


def quest_gemv_int4_top_p(q: torch.Tensor, meta: torch.Tensor, k_int4: torch.Tensor,
                          kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                          kv_last_page_len: torch.Tensor, token_budget: int,
                          max_pages_per_req: int, top_p, high: str = "max",
                          sm_scale: Optional[float] = None, return_scores: bool = False,
                          meta_planes: Optional[torch.Tensor] = None,
                          plane_slots: Optional[torch.Tensor] = None):
    """Selector + estimator + pruner in one launch, one workgroup per (batch, head) row:
    :func:`twilight_amd.kernel.quest_select` followed by :func:`sparse_gemv_int4_top_p`
    (twilight/pyimpl/quest.py:17-122, attention.py:252-255, top_p.py:10-15, attention.py:280-281)
    with the page scores and the page list kept on chip.

    ``meta_planes`` [slots,Hkv,128,2,cap] (:func:`twilight_amd.kernel.meta_planes_build`) makes
    the page-score pass read the plane layout (half the bytes; scores may differ from the record
    form in the last bits); ``plane_slots`` int32 [B] names each request's slot (default: its
    position in the batch).

    Returns ``(sel_pages int32 [B,H,k], sel_count int32 [B,H], idx int32 [B,H,16k], count int32
    [B,H], cand_count int32 [B,H])``, k = budget pages clamped to ``max_pages_per_req``; with
    ``return_scores`` also ``page_scores`` fp32 [B,H,max_pages_per_req] and ``scores`` fp32
    [B,H,16k].
    """
    from .quest import quest_num_pages
    from .sampling import _check_p, _high_mode
    check_input(q, "q")
    check_dim(3, q, "q")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM:
        raise RuntimeError(f"head_dim must be {_lib.HEAD_DIM}, got {D}")
    check_input(k_int4, "k_int4")
    check_dtype(k_int4, torch.uint8, "k_int4")
    if k_int4.dim() != 3 or k_int4.size(2) != _lib.INT4_RECORD_BYTES:
        raise RuntimeError("k_int4 must be uint8 [pages, kv_heads, 1280]")
    Hkv = k_int4.size(1)
    check_input(meta, "meta")
    check_dtype(meta, torch.uint8, "meta")
    if meta.dim() != 3 or meta.size(1) != Hkv or meta.size(2) != _lib.META_RECORD_BYTES \
            or meta.size(0) != k_int4.size(0):
        raise RuntimeError("meta must be uint8 [pages, kv_heads, 512] like k_int4")
    if H % Hkv != 0:
        raise RuntimeError(f"num_q_heads {H} must be a multiple of num_kv_heads {Hkv}")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                    ("kv_last_page_len", kv_last_page_len)):
        check_input(t, name)
        check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1 or kv_last_page_len.numel() != B:
        raise RuntimeError("kv_page_indptr must have B+1 and kv_last_page_len B elements")
    if token_budget <= 0 or max_pages_per_req <= 0 or max_pages_per_req > 8192:
        raise RuntimeError("token_budget must be positive and max_pages_per_req in [1, 8192]")
    k = quest_num_pages(token_budget, max_pages_per_req)
    M = k * _lib.PAGE
    if M > _lib.MAX_CANDIDATES:
        raise RuntimeError(f"{M} candidates exceed the supported maximum {_lib.MAX_CANDIDATES}")
    p_arr, p_val = _check_p(top_p, B * H, q)
    cap = 0
    if meta_planes is not None:
        from .kv_shadow import _check_planes
        cap = _check_planes(meta_planes, B, Hkv, q.dtype, plane_slots)
        if cap < max_pages_per_req:
            raise RuntimeError("meta_planes holds fewer pages per request than max_pages_per_req")
    elif plane_slots is not None:
        raise RuntimeError("plane_slots given without meta_planes")
    check_same_device(q, ("k_int4", k_int4), ("meta", meta), ("kv_page_indices", kv_page_indices),
                      ("kv_page_indptr", kv_page_indptr), ("kv_last_page_len", kv_last_page_len),
                      ("meta_planes", meta_planes), ("plane_slots", plane_slots))
    dev = q.device
    with torch.cuda.device(dev):
        sel = torch.zeros((B, H, k), dtype=torch.int32, device=dev)
        selc = torch.empty((B, H), dtype=torch.int32, device=dev)
        idx = torch.empty((B, H, M), dtype=torch.int32, device=dev)
        count = torch.empty((B, H), dtype=torch.int32, device=dev)
        cand = torch.empty((B, H), dtype=torch.int32, device=dev)
        ps = (torch.zeros((B, H, max_pages_per_req), dtype=torch.float32, device=dev)
              if return_scores else None)
        scores = (torch.full((B, H, M), float("-inf"), dtype=torch.float32, device=dev)
                  if return_scores else None)
        scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
        rc = _lib.lib().twl_select_estimate_prune(
            ptr(q), dtype_code(q.dtype, "q"), ptr(meta), ptr(k_int4), ptr(kv_page_indices),
            ptr(kv_page_indptr), ptr(kv_last_page_len), B, H, Hkv, int(token_budget),
            int(max_pages_per_req), scale, ptr(p_arr), p_val, _high_mode(high), ptr(sel), k,
            ptr(selc), ptr(idx), M, ptr(count), ptr(ps), max_pages_per_req, ptr(scores), M,
            ptr(cand), ptr(meta_planes), cap, ptr(plane_slots),
            0 if meta_planes is None else meta_planes.size(0), stream_of(q))
    _lib.check(rc, "SelectEstimatePrune")
    out = [sel, selc, idx, count, cand]
    if return_scores:
        out += [ps, scores]
    return tuple(out)


def batched_sparse_gemv_int4_k(q: torch.Tensor, o: torch.Tensor, k_u8: torch.Tensor,
                               quant_scales: torch.Tensor, quant_zeros: torch.Tensor,
                               kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                               kv_last_page_len: torch.Tensor,
                               sm_scale: float = 1.0) -> None:
    """Same call shape as ``ftka.cuda_ops.gemv.batched_sparse_gemv_int4_k`` at
    benchmark/efficiency/bench_gemv.py:445-454 (tensors built at :390-443).

    ``q`` fp16 [B,H,128]; ``o`` fp16 [B,H,N] filled in place; ``k_u8`` uint8
    [max_pages, page_size, H, 64] (low nibble = even element); ``quant_scales`` / ``quant_zeros``
    fp16 [max_pages, page_size, H] with dequant ``k*scale + zero`` (bench_gemv.py:181); one page
    list per request shared by all heads. ``sm_scale`` defaults to 1 (the bench compares against
    a plain ``q @ k``, bench_gemv.py:491).
    """
    check_input(q, "q"); check_dim(3, q, "q"); check_dtype(q, torch.float16, "q")
    check_input(o, "o"); check_dim(3, o, "o"); check_dtype(o, torch.float16, "o")
    check_input(k_u8, "k_cache"); check_dim(4, k_u8, "k_cache"); check_dtype(k_u8, torch.uint8, "k_cache")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM or k_u8.size(3) != D // 2 or k_u8.size(2) != H:
        raise RuntimeError("k_cache must be uint8 [max_pages, page_size, num_heads, 64]")
    page_size = k_u8.size(1)
    for name, t in (("quant_scales", quant_scales), ("quant_zeros", quant_zeros)):
        check_input(t, name); check_dtype(t, torch.float16, name)
        if tuple(t.shape) != tuple(k_u8.shape[:3]):
            raise RuntimeError(f"{name} must be fp16 [max_pages, page_size, num_heads]")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                    ("kv_last_page_len", kv_last_page_len)):
        check_input(t, name); check_dtype(t, torch.int32, name)
    if o.size(0) != B or o.size(1) != H:
        raise RuntimeError("o must be fp16 [B, H, N]")
    if kv_page_indptr.numel() != B + 1 or kv_last_page_len.numel() != B:
        raise RuntimeError("kv_page_indptr must have B+1 and kv_last_page_len B elements")
    check_same_device(q, ("o", o), ("k_cache", k_u8), ("quant_scales", quant_scales),
                      ("quant_zeros", quant_zeros), ("kv_page_indices", kv_page_indices),
                      ("kv_page_indptr", kv_page_indptr), ("kv_last_page_len", kv_last_page_len))
    max_pages_per_req = o.size(2) // page_size
    if max_pages_per_req == 0:
        raise RuntimeError("o is shorter than one page")
    with torch.cuda.device(q.device):
        rc = _lib.lib().twl_gemv_int4_nhd(
            ptr(q), ptr(o), o.size(2), ptr(k_u8), ptr(quant_scales), ptr(quant_zeros),
            ptr(kv_page_indices), ptr(kv_page_indptr), ptr(kv_last_page_len), B, H, page_size,
            max_pages_per_req, float(sm_scale), stream_of(q))
    _lib.check(rc, "BatchedSparseGemvInt4K")


def _check_nhd_common(q, o, k_cache, last_dim, kv_page_indices, kv_page_indptr, kv_last_page_len,
                      o_dims):
    check_input(q, "q"); check_dim(3, q, "q"); check_dtype(q, torch.float16, "q")
    check_input(o, "o"); check_dim(o_dims, o, "o"); check_dtype(o, torch.float16, "o")
    check_input(k_cache, "k_cache"); check_dim(4, k_cache, "k_cache")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM or k_cache.size(3) != last_dim or k_cache.size(2) != H:
        raise RuntimeError(f"k_cache must be [max_pages, page_size, num_heads, {last_dim}]")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                    ("kv_last_page_len", kv_last_page_len)):
        check_input(t, name); check_dtype(t, torch.int32, name)
    if o.size(0) != B or o.size(1) != H:
        raise RuntimeError("o must be fp16 [B, H, (1,) N]")
    if kv_page_indptr.numel() != B + 1 or kv_last_page_len.numel() != B:
        raise RuntimeError("kv_page_indptr must have B+1 and kv_last_page_len B elements")
    check_same_device(q, ("o", o), ("k_cache", k_cache), ("kv_page_indices", kv_page_indices),
                      ("kv_page_indptr", kv_page_indptr), ("kv_last_page_len", kv_last_page_len))
    page_size = k_cache.size(1)
    n_out = o.size(-1)
    if n_out // page_size == 0:
        raise RuntimeError("o is shorter than one page")
    return B, H, page_size, n_out


def batched_sparse_gemv(q: torch.Tensor, o: torch.Tensor, k_cache: torch.Tensor,
                        kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                        kv_last_page_len: torch.Tensor, sm_scale: float = 1.0) -> None:
    """Call shape of ``ftka.cuda_ops.gemv.batched_sparse_gemv`` at
    benchmark/efficiency/bench_gemv.py:234-241: ``o[b,h,0,n] = q[b,h,:] . k_cache[token n of b]``.

    ``q`` fp16 [B,H,128]; ``o`` fp16 [B,H,1,N] written in place; ``k_cache`` fp16
    [max_pages, page_size, H, 128]; CSR page list per request.
    """
    B, H, page_size, n_out = _check_nhd_common(q, o, k_cache, _lib.HEAD_DIM, kv_page_indices,
                                               kv_page_indptr, kv_last_page_len, 4)
    check_dtype(k_cache, torch.float16, "k_cache")
    if o.size(2) != 1:
        raise RuntimeError("o must be fp16 [B, H, 1, N]")
    with torch.cuda.device(q.device):
        rc = _lib.lib().twl_gemv_f16_nhd(ptr(q), ptr(o), n_out, ptr(k_cache), ptr(kv_page_indices),
                                         ptr(kv_page_indptr), ptr(kv_last_page_len), B, H,
                                         page_size, n_out // page_size, float(sm_scale),
                                         stream_of(q))
    _lib.check(rc, "BatchedSparseGemv")


def batched_sparse_gemv_int8_k(q: torch.Tensor, o: torch.Tensor, k_u8: torch.Tensor,
                               quant_scales: torch.Tensor, quant_zeros: torch.Tensor,
                               kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                               kv_last_page_len: torch.Tensor, sm_scale: float = 1.0) -> None:
    """Call shape of ``ftka.cuda_ops.gemv.batched_sparse_gemv_int8_k`` at
    benchmark/efficiency/bench_gemv.py:135-144: ``k_u8`` uint8 [max_pages, page_size, H, 128] holds
    ``int8 value + 128`` (:78,93); dequant ``(k_u8 - 128) * scale + zero`` with per-token fp16
    ``quant_scales`` / ``quant_zeros`` [max_pages, page_size, H] (:181); ``o`` fp16 [B,H,N]."""
    B, H, page_size, n_out = _check_nhd_common(q, o, k_u8, _lib.HEAD_DIM, kv_page_indices,
                                               kv_page_indptr, kv_last_page_len, 3)
    check_dtype(k_u8, torch.uint8, "k_cache")
    for name, t in (("quant_scales", quant_scales), ("quant_zeros", quant_zeros)):
        check_input(t, name); check_dtype(t, torch.float16, name)
        if tuple(t.shape) != tuple(k_u8.shape[:3]):
            raise RuntimeError(f"{name} must be fp16 [max_pages, page_size, num_heads]")
    check_same_device(q, ("quant_scales", quant_scales), ("quant_zeros", quant_zeros))
    with torch.cuda.device(q.device):
        rc = _lib.lib().twl_gemv_int8_nhd(ptr(q), ptr(o), n_out, ptr(k_u8), ptr(quant_scales),
                                          ptr(quant_zeros), ptr(kv_page_indices),
                                          ptr(kv_page_indptr), ptr(kv_last_page_len), B, H,
                                          page_size, n_out // page_size, float(sm_scale),
                                          stream_of(q))
    _lib.check(rc, "BatchedSparseGemvInt8K")


def single_sparse_gemv(q: torch.Tensor, o: torch.Tensor, k: torch.Tensor,
                       sm_scale: float = 1.0) -> None:
    """Call shape of ``ftka.cuda_ops.gemv.single_sparse_gemv`` at
    benchmark/efficiency/bench_gemv.py:33: ``o[h,n] = q[h,:] . k[n,h,:]`` for one request;
    ``q`` fp16 [H,128], ``k`` fp16 [N,H,128], ``o`` fp16 [H,N] written in place."""
    check_input(q, "q"); check_dim(2, q, "q"); check_dtype(q, torch.float16, "q")
    check_input(k, "k"); check_dim(3, k, "k"); check_dtype(k, torch.float16, "k")
    check_input(o, "o"); check_dim(2, o, "o"); check_dtype(o, torch.float16, "o")
    H, D = q.shape
    N = k.size(0)
    if D != _lib.HEAD_DIM or k.size(1) != H or k.size(2) != D or tuple(o.shape) != (H, N) or N == 0:
        raise RuntimeError("shapes must be q [H,128], k [N,H,128], o [H,N]")
    check_same_device(q, ("k", k), ("o", o))
    with torch.cuda.device(q.device):
        rc = _lib.lib().twl_gemv_f16_single(ptr(q), ptr(o), ptr(k), H, N, float(sm_scale),
                                            stream_of(q))
    _lib.check(rc, "SingleSparseGemv")
