"""ctypes binding of ``libtwilight_hip.so`` (declared in ``include/twilight_hip.h``).

There is no fallback: if the library is missing, :func:`lib` raises, and every op of
``twilight_amd.kernel`` fails with it.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_uint8, c_uint32,
                    c_uint64, c_void_p)

from .build import LIB_PATH

TWL_OK = 0
TWL_F16, TWL_BF16, TWL_F32 = 0, 1, 2
ABI_VERSION = 10  # TWL_ABI_VERSION of include/twilight_hip.h, checked when the library is loaded
TWL_HIGH_FIRST, TWL_HIGH_MAX = 0, 1
PAGE = 16
HEAD_DIM = 128
INT4_RECORD_BYTES = 1280
META_RECORD_BYTES = 512
MAX_CANDIDATES = 32768
STATIC_SCRATCH_BYTES = 24 << 20

# every symbol include/twilight_hip.h declares
EXPORTS = (
    "twl_strerror", "twl_abi_version", "twl_device_count", "twl_top_p_f32", "twl_top_p_f16", "twl_top_p_f32_exact",
    "twl_softmax_top_p_f32", "twl_gemv_top_p", "twl_select_estimate_prune", "twl_gemv_int4", "twl_gemv_int4_nhd",
    "twl_gemv_int8_nhd", "twl_gemv_f16_nhd", "twl_gemv_f16_single", "twl_sparse_attn",
    "twl_sparse_attn_workspace_bytes", "twl_sparse_attn_static", "twl_sparse_attn_weighted", "twl_gemv_int4_group",
    "twl_group_attn",
    "twl_group_attn_workspace_bytes",
    "twl_group_union", "twl_rope_qk", "twl_quest_select",
    "twl_quest_page_scores", "twl_quest_topk_pages", "twl_kv_shadow_build", "twl_kv_append", "twl_meta_planes_build", "twl_quest_page_scores_planes", "twl_dequant_int4",
    "twl_decode_layer", "twl_get_label_tensor", "twl_bgemv_int8", "twl_qk_int8_lse",
)


class LayerArgs(ctypes.Structure):
    """Mirror of ``struct twl_layer_args``."""
    _fields_ = [
        ("q", c_void_p), ("dtype", c_int), ("k_cache", c_void_p), ("v_cache", c_void_p),
        ("page_stride", c_uint64), ("token_stride", c_uint64), ("head_stride", c_uint64),
        ("k_int4", c_void_p), ("meta", c_void_p),
        ("meta_planes", c_void_p), ("plane_cap_pages", c_uint32),
        ("plane_slots", c_void_p), ("plane_num_slots", c_uint32),
        ("kv_page_indices", c_void_p), ("kv_page_indptr", c_void_p), ("kv_last_page_len", c_void_p),
        ("batch", c_uint32), ("num_q_heads", c_uint32), ("num_kv_heads", c_uint32),
        ("max_pages_per_req", c_uint32), ("token_budget", c_uint32),
        ("top_p", c_float), ("high_mode", c_int), ("sm_scale", c_float),
        ("sel_pages", c_void_p), ("sel_stride", c_uint32),
        ("sel_count", c_void_p),
        ("page_scores", c_void_p), ("page_score_stride", c_uint32),
        ("scores", c_void_p), ("score_stride", c_uint32),
        ("cand_count", c_void_p),
        ("idx", c_void_p), ("idx_stride", c_uint32),
        ("count", c_void_p),
        ("attn_workspace", c_void_p), ("attn_workspace_bytes", c_uint64),
        ("out", c_void_p),
        ("split_estimator", c_int), ("keep_scores", c_int),
        ("group_idx", c_void_p), ("group_idx_stride", c_uint32),
        ("group_count", c_void_p),
        ("group_workspace", c_void_p), ("group_workspace_bytes", c_uint64),
        ("surv_probs", c_void_p), ("use_estimated_weights", c_int),
        ("group_select", c_int),
    ]


_lib = None


def lib() -> ctypes.CDLL:
    """Load the library once. Raises ``RuntimeError`` when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m twilight_amd.build` "
            "(hipcc --offload-arch=gfx950); twilight_amd has no CPU or PyTorch fallback")
    L = ctypes.CDLL(LIB_PATH)
    vp, u32, u64, f32, i32 = c_void_p, c_uint32, c_uint64, c_float, c_int
    L.twl_strerror.argtypes = [c_int]
    L.twl_strerror.restype = c_char_p
    L.twl_abi_version.argtypes = []
    L.twl_abi_version.restype = c_int
    if L.twl_abi_version() != ABI_VERSION:
        raise RuntimeError(
            f"{LIB_PATH} has ABI version {L.twl_abi_version()}, this package binds version "
            f"{ABI_VERSION}: rebuild it with `python -m twilight_amd.build`")
    L.twl_device_count.argtypes = []
    L.twl_top_p_f32.argtypes = [vp, vp, vp, vp, vp, f32, u32, u32, u32, i32, vp, vp, vp]
    L.twl_top_p_f32_exact.argtypes = L.twl_top_p_f32.argtypes
    L.twl_top_p_f16.argtypes = [vp, i32, vp, vp, vp, vp, f32, u32, u32, u32, i32, vp, vp, vp]
    L.twl_softmax_top_p_f32.argtypes = [vp, u32, vp, u32, u32, vp, f32, i32, vp, u32, vp, u32, vp,
                                        vp, vp, vp]
    L.twl_gemv_top_p.argtypes = [vp, i32, vp, vp, vp, u32, vp, vp, vp, u32, u32, u32, u32, f32, vp,
                                 f32, i32, vp, u32, vp, vp, u32, vp, vp, vp]
    L.twl_select_estimate_prune.argtypes = [vp, i32, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32,
                                            f32, vp, f32, i32, vp, u32, vp, vp, u32, vp, vp, u32,
                                            vp, u32, vp, vp, u32, vp, u32, vp]
    L.twl_gemv_int4.argtypes = [vp, i32, vp, u32, vp, vp, vp, vp, u32, vp, vp, vp, u32, u32, u32,
                                u32, f32, vp]
    L.twl_gemv_int4_group.argtypes = L.twl_gemv_int4.argtypes
    L.twl_gemv_int4_nhd.argtypes = [vp, vp, u32, vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, f32, vp]
    L.twl_gemv_int8_nhd.argtypes = L.twl_gemv_int4_nhd.argtypes
    L.twl_gemv_f16_nhd.argtypes = [vp, vp, u32, vp, vp, vp, vp, u32, u32, u32, u32, f32, vp]
    L.twl_gemv_f16_single.argtypes = [vp, vp, vp, u32, u32, f32, vp]
    L.twl_sparse_attn.argtypes = [vp, vp, i32, vp, vp, u64, u64, u64, vp, u32, vp, vp, vp, u32, u32,
                                  u32, f32, vp, vp, u64, vp]
    L.twl_sparse_attn_workspace_bytes.argtypes = [u32, u32]
    L.twl_sparse_attn_static.argtypes = [vp, vp, i32, vp, vp, u64, u64, u64, vp, u32, vp, vp, vp, u32,
                                         u32, u32, f32, vp, vp]
    L.twl_sparse_attn_weighted.argtypes = [vp, i32, vp, u64, u64, u64, vp, u32, vp, vp, vp, vp, u32,
                                           u32, u32, vp, vp, u64, vp]
    L.twl_group_attn_workspace_bytes.argtypes = [u32, u32, u32, u32, i32]
    L.twl_group_attn.argtypes = [vp, vp, i32, vp, vp, u64, u64, u64, vp, u32, vp, u32, vp, vp, vp,
                                 u32, u32, u32, f32, vp, vp, u64, vp]
    L.twl_group_union.argtypes = [vp, u32, vp, u32, u32, u32, u32, vp, u32, vp, vp]
    L.twl_rope_qk.argtypes = [vp, vp, vp, vp, i32, u32, u32, u32, vp]
    L.twl_quest_select.argtypes = [vp, i32, vp, vp, vp, u32, u32, u32, u32, u32, vp, u32, vp, vp,
                                   u32, vp]
    L.twl_quest_page_scores.argtypes = [vp, i32, vp, vp, vp, u32, u32, u32, u32, vp, u32, vp]
    L.twl_quest_topk_pages.argtypes = [vp, u32, vp, u32, u32, u32, u32, vp, u32, vp, vp]
    L.twl_kv_shadow_build.argtypes = [vp, i32, u64, u64, u64, vp, vp, u32, u32, vp, vp, vp]
    L.twl_dequant_int4.argtypes = [vp, u32, vp, vp]
    L.twl_decode_layer.argtypes = [POINTER(LayerArgs), vp]
    L.twl_get_label_tensor.argtypes = [vp, vp, vp, u32, u32, u32, u32] + [c_int64] * 8 + [vp]
    L.twl_bgemv_int8.argtypes = [vp, vp, vp, vp, u32, u32, u32, u32] + [c_int64] * 11 + [vp]
    L.twl_kv_append.argtypes = [vp, vp, i32, u64, u64, vp, vp, u64, u64, u64, vp, vp, vp, u32, u32,
                                vp, vp, vp, u32, vp, u32, vp]
    L.twl_meta_planes_build.argtypes = [vp, vp, vp, u32, u32, u32, vp, u32, vp, u32, vp]
    L.twl_quest_page_scores_planes.argtypes = [vp, i32, vp, u32, vp, u32, vp, vp, vp, u32, u32, u32,
                                               u32, vp, u32, vp]
    i64 = ctypes.c_int64
    L.twl_qk_int8_lse.argtypes = [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, i64, i64, i64,
                                  i64, i64, i64, vp]
    for name in EXPORTS:
        if name not in ("twl_strerror", "twl_sparse_attn_workspace_bytes",
                        "twl_group_attn_workspace_bytes"):
            getattr(L, name).restype = c_int
    L.twl_sparse_attn_workspace_bytes.restype = c_uint64
    L.twl_group_attn_workspace_bytes.restype = c_uint64
    _lib = L
    return L


def strerror(rc: int) -> str:
    return lib().twl_strerror(rc).decode()


def check(rc: int, what: str) -> None:
    """Raise ``RuntimeError`` for a non-zero status, as the reference's TORCH_CHECK does
    (csrc/src/sampling.cu:39-40,61-62)."""
    if rc != TWL_OK:
        raise RuntimeError(f"{what} failed with error code {rc}: {strerror(rc)}")
