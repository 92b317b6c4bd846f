"""KV-append ops: INT4 shadow + Quest metadata builder, and the INT4 unpacker used by tests."""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ._check import check_dtype, check_input, check_same_device, dtype_code, ptr, stream_of
from .attention import _cache_strides


def kv_shadow_build(k_cache: torch.Tensor, k_int4: Optional[torch.Tensor],
                    meta: Optional[torch.Tensor], page_ids: Optional[torch.Tensor] = None,
                    valid_len: Optional[torch.Tensor] = None) -> None:
    """Quantise whole pages of ``k_cache`` [pages,16,Hkv,128] into ``k_int4`` uint8
    [pages,Hkv,1280] (twilight/pyimpl/quantize.py:4-13 per group of 32, fp16 scale/zero) and
    write their channel-wise min/max into ``meta`` uint8 [pages,Hkv,512]
    (twilight/pyimpl/quest.py:68-74). ``page_ids`` int32 selects physical pages (default all);
    ``valid_len`` int32 gives the valid tokens of each listed page (default 16)."""
    ps, ts, hs = _cache_strides(k_cache, "k_cache")
    Hkv = k_cache.size(2)
    if k_int4 is None and meta is None:
        raise RuntimeError("at least one of k_int4 / meta is required")
    if k_int4 is not None:
        check_input(k_int4, "k_int4"); check_dtype(k_int4, torch.uint8, "k_int4")
        if k_int4.dim() != 3 or k_int4.size(1) != Hkv or k_int4.size(2) != _lib.INT4_RECORD_BYTES \
                or k_int4.size(0) != k_cache.size(0):
            raise RuntimeError("k_int4 must be uint8 [pages, kv_heads, 1280]")
    if meta is not None:
        check_input(meta, "meta"); check_dtype(meta, torch.uint8, "meta")
        if meta.dim() != 3 or meta.size(1) != Hkv or meta.size(2) != _lib.META_RECORD_BYTES \
                or meta.size(0) != k_cache.size(0):
            raise RuntimeError("meta must be uint8 [pages, kv_heads, 512]")
    n = k_cache.size(0)
    if page_ids is not None:
        check_input(page_ids, "page_ids"); check_dtype(page_ids, torch.int32, "page_ids")
        n = page_ids.numel()
    if valid_len is not None:
        check_input(valid_len, "valid_len"); check_dtype(valid_len, torch.int32, "valid_len")
        if valid_len.numel() != n:
            raise RuntimeError("valid_len must have one entry per processed page")
    check_same_device(k_cache, ("k_int4", k_int4), ("meta", meta), ("page_ids", page_ids),
                      ("valid_len", valid_len))
    if n == 0:
        return
    with torch.cuda.device(k_cache.device):
        rc = _lib.lib().twl_kv_shadow_build(
            ptr(k_cache), dtype_code(k_cache.dtype, "k_cache"), ps, ts, hs, ptr(page_ids),
            ptr(valid_len), n, Hkv, ptr(k_int4), ptr(meta), stream_of(k_cache))
    _lib.check(rc, "KvShadowBuild")


def kv_append(k_new: torch.Tensor, v_new: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
              kv_last_page_len: torch.Tensor, k_int4: Optional[torch.Tensor] = None,
              meta: Optional[torch.Tensor] = None,
              meta_planes: Optional[torch.Tensor] = None,
              plane_slots: Optional[torch.Tensor] = None) -> None:
    """Decode append of one token per request in one launch. ``k_new`` / ``v_new`` [B,Hkv,128]
    (head_dim contiguous) go to slot ``kv_last_page_len[b]`` of each request's last listed page;
    the token's INT4 codes and the page's min/max metadata are updated and ``kv_last_page_len`` is
    advanced in place. The caller extends the page table (and sets the length to 0) beforehand
    when a request's last page is full. ``meta_planes`` [slots,Hkv,128,2,cap] (plane-layout
    metadata, :func:`meta_planes_build`) is kept current too when given; ``plane_slots`` int32 [B]
    names the slot of each request (default: its position in the batch)."""
    ps, ts, hs = _cache_strides(k_cache, "k_cache")
    if _cache_strides(v_cache, "v_cache") != (ps, ts, hs) or v_cache.dtype != k_cache.dtype:
        raise RuntimeError("k_cache and v_cache must share dtype and strides")
    Hkv = k_cache.size(2)
    for name, t in (("k_new", k_new), ("v_new", v_new)):
        if not t.is_cuda or t.dim() != 3 or t.size(1) != Hkv or t.size(2) != _lib.HEAD_DIM \
                or t.stride(2) != 1 or t.dtype != k_cache.dtype:
            raise RuntimeError(f"{name} must be a CUDA [B, {Hkv}, {_lib.HEAD_DIM}] tensor of "
                               f"{k_cache.dtype} with contiguous head_dim")
    B = k_new.size(0)
    if v_new.size(0) != B or v_new.stride() != k_new.stride():
        raise RuntimeError("k_new and v_new must share shape and strides")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                    ("kv_last_page_len", kv_last_page_len)):
        check_input(t, name); check_dtype(t, torch.int32, name)
    if kv_page_indptr.numel() != B + 1 or kv_last_page_len.numel() != B:
        raise RuntimeError("kv_page_indptr must have B+1 and kv_last_page_len B elements")
    for name, t, nb in (("k_int4", k_int4, _lib.INT4_RECORD_BYTES), ("meta", meta, _lib.META_RECORD_BYTES)):
        if t is not None:
            check_input(t, name); check_dtype(t, torch.uint8, name)
            if t.dim() != 3 or t.size(0) != k_cache.size(0) or t.size(1) != Hkv or t.size(2) != nb:
                raise RuntimeError(f"{name} must be uint8 [pages, kv_heads, {nb}]")
    cap = 0
    if meta_planes is not None:
        cap = _check_planes(meta_planes, B, Hkv, k_cache.dtype, plane_slots)
    elif plane_slots is not None:
        raise RuntimeError("plane_slots given without meta_planes")
    check_same_device(k_cache, ("v_cache", v_cache), ("k_new", k_new), ("v_new", v_new),
                      ("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                      ("kv_last_page_len", kv_last_page_len), ("k_int4", k_int4), ("meta", meta),
                      ("meta_planes", meta_planes), ("plane_slots", plane_slots))
    if B == 0:
        return
    with torch.cuda.device(k_cache.device):
        rc = _lib.lib().twl_kv_append(
            ptr(k_new), ptr(v_new), dtype_code(k_cache.dtype, "k_cache"), k_new.stride(0),
            k_new.stride(1), ptr(k_cache), ptr(v_cache), ps, ts, hs, ptr(kv_page_indices),
            ptr(kv_page_indptr), ptr(kv_last_page_len), B, Hkv, ptr(k_int4), ptr(meta),
            ptr(meta_planes), cap, ptr(plane_slots),
            0 if meta_planes is None else meta_planes.size(0), stream_of(k_cache))
    _lib.check(rc, "KvAppend")


def _check_planes(meta_planes: torch.Tensor, B: int, Hkv: int, dtype: torch.dtype,
                  plane_slots: Optional[torch.Tensor] = None) -> int:
    """Shape checks of the plane buffer (and of the slot table, whose VALUES stay on the device:
    the kernels clamp them into the buffer). Returns the pages per run."""
    check_input(meta_planes, "meta_planes")
    if meta_planes.dtype != dtype:
        raise RuntimeError(f"meta_planes must have the cache dtype {dtype}")
    if meta_planes.dim() != 5 or meta_planes.size(0) == 0 or meta_planes.size(1) != Hkv \
            or meta_planes.size(2) != _lib.HEAD_DIM or meta_planes.size(3) != 2 \
            or meta_planes.size(4) % 8 != 0 or meta_planes.size(4) == 0:
        raise RuntimeError("meta_planes must be [slots, kv_heads, 128, 2, cap] with cap a multiple of 8")
    if plane_slots is None:
        if meta_planes.size(0) < B:
            raise RuntimeError("meta_planes must hold a slot per request of the batch "
                               "(or pass plane_slots)")
    else:
        check_input(plane_slots, "plane_slots")
        check_dtype(plane_slots, torch.int32, "plane_slots")
        if plane_slots.numel() != B:
            raise RuntimeError("plane_slots must have one entry per request of the batch")
    return meta_planes.size(4)


def meta_planes_build(meta: torch.Tensor, kv_page_indices: torch.Tensor,
                      kv_page_indptr: torch.Tensor, max_pages_per_req: int,
                      meta_planes: torch.Tensor,
                      plane_slots: Optional[torch.Tensor] = None) -> None:
    """Fill the plane-layout metadata ``meta_planes`` [B,Hkv,128,2,cap] (cache dtype; per request
    slot, kv head and channel the minima of all logical pages contiguously, then the maxima) from
    the 512-byte records ``meta`` uint8 [pages,Hkv,512] for the pages of the page table. The
    selector then reads only the run the sign of q_d selects: half the bytes. ``plane_slots``
    int32 [B]: the slot of each request (default: its position in the batch); a page table of a
    few requests with their slots refills just those."""
    check_input(meta, "meta"); check_dtype(meta, torch.uint8, "meta")
    if meta.dim() != 3 or meta.size(2) != _lib.META_RECORD_BYTES:
        raise RuntimeError("meta must be uint8 [pages, kv_heads, 512]")
    for name, t in (("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr)):
        check_input(t, name); check_dtype(t, torch.int32, name)
    B = kv_page_indptr.numel() - 1
    cap = _check_planes(meta_planes, B, meta.size(1), meta_planes.dtype, plane_slots)
    if meta_planes.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("meta_planes must be float16 or bfloat16")
    if max_pages_per_req <= 0 or max_pages_per_req > cap:
        raise RuntimeError("max_pages_per_req must be in [1, cap]")
    check_same_device(meta, ("kv_page_indices", kv_page_indices), ("kv_page_indptr", kv_page_indptr),
                      ("meta_planes", meta_planes), ("plane_slots", plane_slots))
    if B == 0:
        return
    with torch.cuda.device(meta.device):
        rc = _lib.lib().twl_meta_planes_build(ptr(meta), ptr(kv_page_indices), ptr(kv_page_indptr),
                                              B, meta.size(1), int(max_pages_per_req),
                                              ptr(meta_planes), cap, ptr(plane_slots),
                                              meta_planes.size(0), stream_of(meta))
    _lib.check(rc, "MetaPlanesBuild")


def dequant_int4(k_int4: torch.Tensor) -> torch.Tensor:
    """uint8 [pages,Hkv,1280] records -> fp32 [pages,Hkv,16,128] (nibble*scale + zero)."""
    check_input(k_int4, "k_int4"); check_dtype(k_int4, torch.uint8, "k_int4")
    if k_int4.dim() != 3 or k_int4.size(2) != _lib.INT4_RECORD_BYTES:
        raise RuntimeError("k_int4 must be uint8 [pages, kv_heads, 1280]")
    P, Hkv, _ = k_int4.shape
    with torch.cuda.device(k_int4.device):
        out = torch.empty((P, Hkv, _lib.PAGE, _lib.HEAD_DIM), dtype=torch.float32,
                          device=k_int4.device)
        rc = _lib.lib().twl_dequant_int4(ptr(k_int4), P * Hkv, ptr(out), stream_of(k_int4))
    _lib.check(rc, "DequantInt4")
    return out
