"""Sparse paged decode attention op (twilight/pyimpl/attention.py:188-190,299-306 over survivors)."""
from __future__ import annotations

import math
from typing import Optional

import torch

from .. import _lib
from ._check import (check_cuda, check_dim, check_dtype, check_input, check_same_device,
                     dtype_code, ptr, stream_of)


def _cache_strides(cache: torch.Tensor, name: str):
    """``cache`` is a 4-D view [pages, 16, Hkv, 128] with a contiguous last dim (any page /
    token / head strides: both NHD and HND storage work)."""
    check_cuda(cache, name)
    check_dim(4, cache, name)
    if cache.size(1) != _lib.PAGE or cache.size(3) != _lib.HEAD_DIM:
        raise RuntimeError(f"{name} must be viewed as [pages, 16, kv_heads, 128]")
    if cache.stride(3) != 1:
        raise RuntimeError(f"{name}: head_dim must be contiguous")
    return cache.stride(0), cache.stride(1), cache.stride(2)


def attention_workspace_bytes(rows: int, idx_stride: int) -> int:
    """Bytes of scratch :func:`sparse_paged_decode_attention` needs for ``rows`` = B*H rows of at
    most ``idx_stride`` survivors."""
    return int(_lib.lib().twl_sparse_attn_workspace_bytes(rows, idx_stride))


def weighted_paged_decode_attention(weights: torch.Tensor, v_cache: torch.Tensor,
                                    idx: torch.Tensor, count: torch.Tensor,
                                    kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                                    return_lse: bool = False, out: Optional[torch.Tensor] = None,
                                    workspace: Optional[torch.Tensor] = None):
    """Attention over per-row survivor lists with given weights in place of q.K logits
    (``use_estimated_weights_in_attn``, attention.py:295-296, then :299-306).

    ``weights`` fp32 [B,H,S]: entry j weighs token ``idx[b,h,j]`` (j < ``count[b,h]``);
    ``v_cache`` [pages,16,Hkv,128] fp16/bf16. Returns ``out`` [B,H,128] in the cache dtype:
    sum_j w_j V_j / sum_j w_j (and, when asked, log sum_j w_j as ``lse``).
    """
    check_input(weights, "weights"); check_dtype(weights, torch.float32, "weights")
    check_dim(3, weights, "weights")
    B, H, S = weights.shape
    vs = _cache_strides(v_cache, "v_cache")
    Hkv = v_cache.size(2)
    if v_cache.size(3) != _lib.HEAD_DIM:
        raise RuntimeError(f"head_dim must be {_lib.HEAD_DIM}, got {v_cache.size(3)}")
    if H % Hkv != 0:
        raise RuntimeError(f"num_q_heads {H} must be a multiple of num_kv_heads {Hkv}")
    check_input(idx, "idx"); check_dtype(idx, torch.int32, "idx"); check_dim(3, idx, "idx")
    check_input(count, "count"); check_dtype(count, torch.int32, "count")
    if tuple(idx.shape) != (B, H, S) or count.numel() != B * H:
        raise RuntimeError("idx must be [B,H,S] like weights and count [B,H]")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr)):
        check_input(t, name); check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1:
        raise RuntimeError("kv_page_indptr must have B+1 elements")
    check_same_device(weights, ("v_cache", v_cache), ("idx", idx), ("count", count),
                      ("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr))
    dev = weights.device
    with torch.cuda.device(dev):
        if out is None:
            out = torch.empty((B, H, _lib.HEAD_DIM), dtype=v_cache.dtype, device=dev)
        else:
            check_input(out, "out")
            if tuple(out.shape) != (B, H, _lib.HEAD_DIM) or out.dtype != v_cache.dtype:
                raise RuntimeError("out must be [B,H,128] of the cache dtype")
        lse = torch.empty((B, H), dtype=torch.float32, device=dev) if return_lse else None
        need = attention_workspace_bytes(B * H, S)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=dev)
        else:
            check_input(workspace, "workspace"); check_dtype(workspace, torch.uint8, "workspace")
            if workspace.numel() < need or workspace.device != dev:
                raise RuntimeError(f"workspace must hold {need} bytes on {dev}")
        rc = _lib.lib().twl_sparse_attn_weighted(
            ptr(out), dtype_code(v_cache.dtype, "v_cache"), ptr(v_cache), vs[0], vs[1], vs[2],
            ptr(idx), S, ptr(count), ptr(weights), ptr(kv_page_indices), ptr(kv_page_indptr),
            B, H, Hkv, ptr(lse), ptr(workspace), workspace.numel(), stream_of(weights))
    _lib.check(rc, "WeightedPagedDecodeAttention")
    return (out, lse) if return_lse else out


def sparse_paged_decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                  idx: torch.Tensor, count: torch.Tensor,
                                  kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                                  sm_scale: Optional[float] = None, return_lse: bool = False,
                                  out: Optional[torch.Tensor] = None,
                                  workspace: Optional[torch.Tensor] = None,
                                  static_scratch: bool = False):
    """Exact softmax attention of one decode token restricted to per-row survivor lists.

    ``q`` [B,H,128] fp16/bf16; ``k_cache`` / ``v_cache`` [pages,16,Hkv,128] of the same dtype;
    ``idx`` int32 [B,H,S] ascending logical token positions, ``count`` int32 [B,H]. Returns
    ``out`` [B,H,128] in q's dtype (and ``lse`` fp32 [B,H] when asked). Probabilities are rounded
    to q's dtype before the V product as at attention.py:302-304 (rows of more than 128 survivors
    are split over workgroups and merged in fp32 instead). ``workspace`` is a
    uint8 tensor of :func:`attention_workspace_bytes` bytes that calls on one stream may share;
    by default a fresh one is allocated. With ``static_scratch`` (and ``out`` given, ``return_lse``
    off) the call allocates nothing: the split rows meet in a buffer inside the library
    (``twl_sparse_attn_static``), shared by every such call on the GPU, so those calls must not
    overlap in time; shapes beyond its 24 MiB raise.
    """
    check_input(q, "q")
    check_dim(3, q, "q")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM:
        raise RuntimeError(f"head_dim must be {_lib.HEAD_DIM}, got {D}")
    ks = _cache_strides(k_cache, "k_cache")
    vs = _cache_strides(v_cache, "v_cache")
    if ks != vs or k_cache.shape != v_cache.shape:
        raise RuntimeError("k_cache and v_cache must share shape and strides")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise RuntimeError("q, k_cache and v_cache must share one dtype (float16 or bfloat16)")
    Hkv = k_cache.size(2)
    if H % Hkv != 0:
        raise RuntimeError(f"num_q_heads {H} must be a multiple of num_kv_heads {Hkv}")
    check_input(idx, "idx"); check_dtype(idx, torch.int32, "idx"); check_dim(3, idx, "idx")
    check_input(count, "count"); check_dtype(count, torch.int32, "count")
    if idx.size(0) != B or idx.size(1) != H or count.numel() != B * H:
        raise RuntimeError("idx must be [B,H,S] and count [B,H]")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr)):
        check_input(t, name); check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1:
        raise RuntimeError("kv_page_indptr must have B+1 elements")
    check_same_device(q, ("k_cache", k_cache), ("v_cache", v_cache), ("idx", idx),
                      ("count", count), ("kv_page_indices", kv_page_indices),
                      ("kv_page_indptr", kv_page_indptr))
    dev = q.device
    with torch.cuda.device(dev):
        if out is None:
            out = torch.empty_like(q)
        else:
            check_input(out, "out")
            if out.shape != q.shape or out.dtype != q.dtype:
                raise RuntimeError("out must match q")
        lse = torch.empty((B, H), dtype=torch.float32, device=dev) if return_lse else None
        scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
        if static_scratch:
            if workspace is not None:
                raise RuntimeError("static_scratch and workspace exclude each other")
            rc = _lib.lib().twl_sparse_attn_static(
                ptr(q), ptr(out), dtype_code(q.dtype, "q"), ptr(k_cache), ptr(v_cache), ks[0],
                ks[1], ks[2], ptr(idx), idx.size(2), ptr(count), ptr(kv_page_indices),
                ptr(kv_page_indptr), B, H, Hkv, scale, ptr(lse), stream_of(q))
            _lib.check(rc, "SparsePagedDecodeAttention")
            return (out, lse) if return_lse else out
        need = attention_workspace_bytes(B * H, idx.size(2))
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=dev)
        else:
            check_input(workspace, "workspace"); check_dtype(workspace, torch.uint8, "workspace")
            if workspace.numel() < need or workspace.device != dev:
                raise RuntimeError(f"workspace must hold {need} bytes on {dev}")
        rc = _lib.lib().twl_sparse_attn(
            ptr(q), ptr(out), dtype_code(q.dtype, "q"), ptr(k_cache), ptr(v_cache), ks[0], ks[1],
            ks[2], ptr(idx), idx.size(2), ptr(count), ptr(kv_page_indices), ptr(kv_page_indptr),
            B, H, Hkv, scale, ptr(lse), ptr(workspace), workspace.numel(), stream_of(q))
    _lib.check(rc, "SparsePagedDecodeAttention")
    return (out, lse) if return_lse else out


def group_attention_workspace_bytes(batch: int, num_q_heads: int, num_kv_heads: int,
                                    max_tokens: int, with_list: bool) -> int:
    """Bytes of scratch :func:`group_paged_decode_attention` needs (``max_tokens``: the longest
    request, or the stride of the group lists)."""
    return int(_lib.lib().twl_group_attn_workspace_bytes(batch, num_q_heads, num_kv_heads,
                                                         max_tokens, int(with_list)))


def group_paged_decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                 kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                                 kv_last_page_len: Optional[torch.Tensor] = None,
                                 max_tokens: Optional[int] = None,
                                 group_idx: Optional[torch.Tensor] = None,
                                 group_count: Optional[torch.Tensor] = None,
                                 sm_scale: Optional[float] = None, return_lse: bool = False,
                                 out: Optional[torch.Tensor] = None,
                                 workspace: Optional[torch.Tensor] = None):
    """Softmax attention of one decode token in which the q heads of a kv head share one token
    list, so K / V are read once per kv head (twilight/pyimpl/attention.py:188-190,299-306 over the
    listed tokens; the reference repeats K / V per q head, attention.py:124-126).

    Without ``group_idx``: dense decode over every token of each request (``kv_last_page_len``
    int32 [B] and ``max_tokens`` >= the longest request are needed) — what the reference runs in
    the layers its configuration leaves dense (attention.py:199-201). With ``group_idx`` int32
    [B,Hkv,S] (ascending token positions) and ``group_count`` int32 [B,Hkv]: attention of every q
    head over its group's list, e.g. the union from :func:`group_union_lists`. ``q`` [B,H,128]
    fp16/bf16 with H/Hkv in {1,2,4,8}; returns ``out`` [B,H,128] (and ``lse`` fp32 [B,H])."""
    check_input(q, "q")
    check_dim(3, q, "q")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM:
        raise RuntimeError(f"head_dim must be {_lib.HEAD_DIM}, got {D}")
    ks = _cache_strides(k_cache, "k_cache")
    vs = _cache_strides(v_cache, "v_cache")
    if ks != vs or k_cache.shape != v_cache.shape:
        raise RuntimeError("k_cache and v_cache must share shape and strides")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise RuntimeError("q, k_cache and v_cache must share one dtype (float16 or bfloat16)")
    Hkv = k_cache.size(2)
    if H % Hkv != 0 or H // Hkv not in (1, 2, 4, 8):
        raise RuntimeError(f"num_q_heads {H} must be 1, 2, 4 or 8 times num_kv_heads {Hkv}")
    others = [("k_cache", k_cache), ("v_cache", v_cache), ("kv_page_indices", kv_page_indices),
              ("kv_page_indptr", kv_page_indptr)]
    for name, t in others[2:]:
        check_input(t, name); check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1:
        raise RuntimeError("kv_page_indptr must have B+1 elements")
    with_list = group_idx is not None
    if with_list:
        if group_count is None:
            raise RuntimeError("group_count is needed with group_idx")
        check_input(group_idx, "group_idx"); check_dtype(group_idx, torch.int32, "group_idx")
        check_dim(3, group_idx, "group_idx")
        check_input(group_count, "group_count"); check_dtype(group_count, torch.int32, "group_count")
        if group_idx.size(0) != B or group_idx.size(1) != Hkv or group_count.numel() != B * Hkv:
            raise RuntimeError("group_idx must be [B,Hkv,S] and group_count [B,Hkv]")
        others += [("group_idx", group_idx), ("group_count", group_count)]
        bound = group_idx.size(2)
    else:
        if kv_last_page_len is None or max_tokens is None:
            raise RuntimeError("dense decode needs kv_last_page_len and max_tokens")
        check_input(kv_last_page_len, "kv_last_page_len")
        check_dtype(kv_last_page_len, torch.int32, "kv_last_page_len")
        if kv_last_page_len.numel() != B:
            raise RuntimeError("kv_last_page_len must have B elements")
        others.append(("kv_last_page_len", kv_last_page_len))
        bound = int(max_tokens)
        if bound <= 0:
            raise RuntimeError("max_tokens must be positive")
    check_same_device(q, *others)
    dev = q.device
    with torch.cuda.device(dev):
        if out is None:
            out = torch.empty_like(q)
        else:
            check_input(out, "out")
            if out.shape != q.shape or out.dtype != q.dtype:
                raise RuntimeError("out must match q")
        lse = torch.empty((B, H), dtype=torch.float32, device=dev) if return_lse else None
        scale = 1.0 / math.sqrt(D) if sm_scale is None else float(sm_scale)
        need = group_attention_workspace_bytes(B, H, Hkv, bound, with_list)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=dev)
        else:
            check_input(workspace, "workspace"); check_dtype(workspace, torch.uint8, "workspace")
            if workspace.numel() < need or workspace.device != dev:
                raise RuntimeError(f"workspace must hold {need} bytes on {dev}")
        rc = _lib.lib().twl_group_attn(
            ptr(q), ptr(out), dtype_code(q.dtype, "q"), ptr(k_cache), ptr(v_cache), ks[0], ks[1],
            ks[2], ptr(group_idx), group_idx.size(2) if with_list else 0, ptr(group_count), bound,
            ptr(kv_page_indices), ptr(kv_page_indptr), ptr(kv_last_page_len), B, H, Hkv, scale,
            ptr(lse), ptr(workspace), workspace.numel(), stream_of(q))
    _lib.check(rc, "GroupPagedDecodeAttention")
    return (out, lse) if return_lse else out


def group_union_lists(idx: torch.Tensor, count: torch.Tensor, num_kv_heads: int, max_tokens: int,
                      group_stride: Optional[int] = None):
    """Union of the survivor lists of each kv head's q heads: ``idx`` int32 [B,H,S] ascending,
    ``count`` int32 [B,H] -> ``(group_idx int32 [B,Hkv,group_stride] ascending, group_count int32
    [B,Hkv])``. Token positions must be < ``max_tokens`` (<= 262144). The default
    ``group_stride`` = min(max_tokens, (H/Hkv)·S) holds every possible union."""
    check_input(idx, "idx"); check_dtype(idx, torch.int32, "idx"); check_dim(3, idx, "idx")
    check_input(count, "count"); check_dtype(count, torch.int32, "count")
    B, H, S = idx.shape
    if count.numel() != B * H:
        raise RuntimeError("count must be [B,H]")
    if num_kv_heads <= 0 or H % num_kv_heads != 0:
        raise RuntimeError(f"num_q_heads {H} must be a multiple of num_kv_heads {num_kv_heads}")
    check_same_device(idx, ("count", count))
    if group_stride is None:
        group_stride = min(int(max_tokens), (H // num_kv_heads) * S)
    dev = idx.device
    with torch.cuda.device(dev):
        gidx = torch.empty((B, num_kv_heads, group_stride), dtype=torch.int32, device=dev)
        gcnt = torch.empty((B, num_kv_heads), dtype=torch.int32, device=dev)
        rc = _lib.lib().twl_group_union(ptr(idx), S, ptr(count), B, H, num_kv_heads, int(max_tokens),
                                        ptr(gidx), group_stride, ptr(gcnt), stream_of(idx))
    _lib.check(rc, "GroupUnionLists")
    return gidx, gcnt


def rope_qk_(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    """Rotary position embedding of one decode token in place: ``q`` [B,H,128], ``k`` [B,Hkv,128],
    ``cos`` / ``sin`` [B,128], all contiguous in one dtype (fp16 / bf16). Same values, bit for bit,
    as ``apply_rotary_pos_emb`` on tensors of that dtype (twilight/pyimpl/attention.py:118-123)."""
    for name, t in (("q", q), ("k", k), ("cos", cos), ("sin", sin)):
        check_input(t, name)
        if t.dtype != q.dtype:
            raise RuntimeError("q, k, cos and sin must share one dtype")
    check_dim(3, q, "q"); check_dim(3, k, "k"); check_dim(2, cos, "cos"); check_dim(2, sin, "sin")
    B, H, D = q.shape
    if D != _lib.HEAD_DIM or k.size(2) != D or k.size(0) != B:
        raise RuntimeError("q must be [B,H,128] and k [B,Hkv,128]")
    if tuple(cos.shape) != (B, D) or tuple(sin.shape) != (B, D):
        raise RuntimeError("cos and sin must be [B,128]")
    check_same_device(q, ("k", k), ("cos", cos), ("sin", sin))
    with torch.cuda.device(q.device):
        rc = _lib.lib().twl_rope_qk(ptr(q), ptr(k), ptr(cos), ptr(sin), dtype_code(q.dtype, "q"), B, H,
                                    k.size(1), stream_of(q))
    _lib.check(rc, "RopeQK")
