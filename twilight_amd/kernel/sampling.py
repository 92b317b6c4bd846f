"""Top-p pruner ops.

``top_p_fp32_return_mask`` / ``top_p_fp16_return_mask`` keep the names, argument order and
return type of twilight/kernel/cuda/sampling.py:118-133. ``top_p_select`` and ``softmax_top_p``
are the index-list forms the decode layer uses.
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch

from .. import _lib
from ._check import (check_dim, check_dtype, check_input, check_same_device, dtype_code, ptr,
                     stream_of)

_HIGH = {"first": _lib.TWL_HIGH_FIRST, "max": _lib.TWL_HIGH_MAX}


def _high_mode(high: str) -> int:
    try:
        return _HIGH[high]
    except KeyError:
        raise RuntimeError(f"high must be 'first' or 'max', got {high!r}") from None


def _to_tensor_scalar_tuple(x):
    # kernel/cuda/sampling.py:111-115
    if isinstance(x, torch.Tensor):
        return (x, 0.0)
    return (None, float(x))


def _check_probs(probs: torch.Tensor, lists: bool = False) -> Tuple[int, int]:
    check_input(probs, "probs")          # csrc/src/sampling.cu:25,48
    check_dim(4, probs, "probs")         # csrc/src/sampling.cu:27,50 (batch, heads, qo_len, kv_len)
    if lists and probs.size(2) != 1:
        raise RuntimeError("probs must have qo_len == 1 (shape [batch, heads, 1, kv_len])")
    # The mask ops do what csrc/src/sampling.cu:51-60 does with qo_len != 1: dim 2 is ignored, the
    # kernel gets batch * heads rows of kv_len, i.e. the FIRST batch * heads rows of the contiguous
    # buffer, and the rest of the mask stays False. Only decode (qo_len == 1) is meaningful.
    rows, d = probs.size(0) * probs.size(1), probs.size(3)
    if rows == 0 or d == 0:
        raise RuntimeError("probs must not be empty")
    if d > _lib.MAX_CANDIDATES:
        raise RuntimeError(f"kv_len {d} exceeds the supported maximum {_lib.MAX_CANDIDATES}")
    return rows, d


def _check_p(top_p, rows: int, ref: torch.Tensor, any_p: bool = False):
    """``any_p``: the reference's ops do not look at the value of a scalar ``top_p``
    (kernel/cuda/sampling.py:111-133); the drop-in ops follow (only NaN raises)."""
    p_arr, p_val = _to_tensor_scalar_tuple(top_p)
    if p_arr is not None:
        check_input(p_arr, "top_p")
        check_dtype(p_arr, torch.float32, "top_p")
        check_same_device(ref, ("top_p", p_arr))
        if p_arr.numel() != rows:
            raise RuntimeError(f"top_p tensor must have batch*heads = {rows} elements")
    elif p_val != p_val or (not any_p and not (0.0 < p_val <= 1.0)):
        raise RuntimeError(f"top_p must be in (0, 1], got {p_val}")
    return p_arr, p_val


def _run_top_p(probs, top_p, high, want_mask, want_idx, want_stats=False, exact=False):
    rows, d = _check_probs(probs, lists=want_idx)
    p_arr, p_val = _check_p(top_p, rows, probs, any_p=True)
    mode = _high_mode(high)
    dev = probs.device
    with torch.cuda.device(dev):
        # the caller (Python) owns every output, as kernel/cuda/sampling.py:72,92 does
        mask = torch.zeros_like(probs, dtype=torch.bool) if want_mask else None
        idx = torch.empty((probs.size(0), probs.size(1), d), dtype=torch.int32, device=dev) \
            if want_idx else None
        count = torch.empty((probs.size(0), probs.size(1)), dtype=torch.int32, device=dev) \
            if want_idx else None
        low = torch.empty(rows, dtype=torch.float32, device=dev) if want_stats else None
        iters = torch.empty(rows, dtype=torch.int32, device=dev) if want_stats else None
        L = _lib.lib()
        if probs.dtype == torch.float32:
            fn = L.twl_top_p_f32_exact if exact else L.twl_top_p_f32
            rc = fn(ptr(probs), ptr(mask), ptr(idx), ptr(count), ptr(p_arr), p_val,
                    rows, d, d, mode, ptr(low), ptr(iters), stream_of(probs))
        else:
            rc = L.twl_top_p_f16(ptr(probs), dtype_code(probs.dtype, "probs"), ptr(mask), ptr(idx),
                                 ptr(count), ptr(p_arr), p_val, rows, d, d, mode, ptr(low),
                                 ptr(iters), stream_of(probs))
    _lib.check(rc, "TopPReturnMask")
    return mask, idx, count, low, iters


def top_p_fp32_return_mask(probs: torch.Tensor, top_p: Union[torch.Tensor, float],
                           high: str = "first", exact: bool = False) -> torch.Tensor:
    """Drop-in for twilight/kernel/cuda/sampling.py:127-133.

    ``probs`` fp32 [B,H,1,N] normalised probabilities; ``top_p`` a float or a float32 tensor of
    B*H per-row values. Returns a bool mask of the same shape: ``probs > low`` after the
    bisection of csrc/include/sampling.cuh:156-231. ``high="first"`` initialises the upper pivot
    to ``probs[...,0]`` exactly as the reference does; ``high="max"`` uses the row maximum.
    ``exact=True`` adds the partial sums in the order of the reference's cub::BlockReduce
    (csrc/include/sampling.cuh:54 with DType = float, csrc/src/sampling.cu:45-63), so that the
    mask is the reference kernel's on every row, also where a sum meets ``top_p`` within a
    rounding error; the default kernel adds in its own order and is about three times faster.
    """
    check_input(probs, "probs")
    check_dtype(probs, torch.float32, "probs")
    return _run_top_p(probs, top_p, high, True, False, exact=exact)[0]


def top_p_fp16_return_mask(probs: torch.Tensor, top_p: Union[torch.Tensor, float],
                           high: str = "first") -> torch.Tensor:
    """Drop-in for twilight/kernel/cuda/sampling.py:118-124 (fp16 or bf16 probabilities,
    csrc/src/sampling.cu:22-43). Like that instantiation of the kernel, p, the pivots, the
    tolerance and every partial sum are values of the 16-bit type, and the additions run in the
    order of the reference's cub::BlockReduce (csrc/include/sampling.cuh:54), so the mask is the
    one the reference's arithmetic gives, bit for bit. Note what that arithmetic does: a sum of
    many small probabilities stalls in 16 bits, so the kept mass can differ visibly from the fp32
    entry's on the same row."""
    check_input(probs, "probs")
    if probs.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"probs must be float16 or bfloat16, got {probs.dtype}")
    return _run_top_p(probs, top_p, high, True, False)[0]


def top_p_select(probs: torch.Tensor, top_p: Union[torch.Tensor, float], high: str = "first",
                 return_mask: bool = False, return_stats: bool = False, exact: bool = False):
    """Index-list form: ``(idx int32 [B,H,N], count int32 [B,H])`` with ``idx[b,h,:count[b,h]]``
    the ascending positions where the mask of :func:`top_p_fp32_return_mask` is set (entries past
    ``count`` are unspecified). Optionally also the mask and ``(low, iters)`` per row."""
    mask, idx, count, low, iters = _run_top_p(probs, top_p, high, return_mask, True, return_stats,
                                              exact=exact)
    out = [idx, count]
    if return_mask:
        out.append(mask)
    if return_stats:
        out += [low, iters]
    return tuple(out)


def softmax_top_p(scores: torch.Tensor, top_p: Union[torch.Tensor, float],
                  lens: Optional[torch.Tensor] = None, sel_pages: Optional[torch.Tensor] = None,
                  high: str = "max", return_probs: bool = False, return_low: bool = False):
    """Fused form of twilight/pyimpl/top_p.py:10-15 over candidate scores.

    ``scores`` fp32 [B,H,M] raw estimator scores (``-inf`` = not a candidate); ``lens`` int32
    [B,H] candidates per row (default M); ``sel_pages`` int32 [B,H,S] page list that maps
    candidate c to token ``sel_pages[c//16]*16 + c%16``. Returns ``(idx [B,H,M], count [B,H])``
    plus the softmax and / or the final pivot when asked.
    """
    check_input(scores, "scores")
    check_dim(3, scores, "scores")
    check_dtype(scores, torch.float32, "scores")
    B, H, M = scores.shape
    rows = B * H
    if rows == 0 or M == 0:
        raise RuntimeError("scores must not be empty")
    if M > _lib.MAX_CANDIDATES:
        raise RuntimeError(f"{M} candidates exceed the supported maximum {_lib.MAX_CANDIDATES}")
    p_arr, p_val = _check_p(top_p, rows, scores)
    if lens is not None:
        check_input(lens, "lens")
        check_dtype(lens, torch.int32, "lens")
        if lens.numel() != rows:
            raise RuntimeError(f"lens must have {rows} elements")
    sel_stride = 0
    if sel_pages is not None:
        check_input(sel_pages, "sel_pages")
        check_dtype(sel_pages, torch.int32, "sel_pages")
        check_dim(3, sel_pages, "sel_pages")
        sel_stride = sel_pages.size(2)
        if sel_pages.size(0) * sel_pages.size(1) != rows or sel_stride * _lib.PAGE < M:
            raise RuntimeError("sel_pages must be [B, H, >= M/16]")
    check_same_device(scores, ("lens", lens), ("sel_pages", sel_pages))
    dev = scores.device
    with torch.cuda.device(dev):
        idx = torch.empty((B, H, M), dtype=torch.int32, device=dev)
        count = torch.empty((B, H), dtype=torch.int32, device=dev)
        probs = torch.zeros_like(scores) if return_probs else None
        low = torch.empty((B, H), dtype=torch.float32, device=dev) if return_low else None
        rc = _lib.lib().twl_softmax_top_p_f32(
            ptr(scores), M, ptr(lens), rows, M, ptr(p_arr), p_val, _high_mode(high),
            ptr(sel_pages), sel_stride, ptr(idx), M, ptr(count), ptr(probs), ptr(low),
            stream_of(scores))
    _lib.check(rc, "SoftmaxTopP")
    out = [idx, count]
    if return_probs:
        out.append(probs)
    if return_low:
        out.append(low)
    return tuple(out)
