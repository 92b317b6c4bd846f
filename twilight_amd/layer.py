"""Host-side driver of one Select-then-Prune decode layer.

Mirrors the decode branch of twilight/pyimpl/attention.py:188-306 (selector -> weight estimator
-> weight pruner -> attention) with the configuration keys of benchmark/configs/*.json:
``selector: {type: quest, token_budget, chunk_size}``, ``weight_estimator: {type: min_max_quant,
quant_bit: 4}``, ``weight_pruner: {type: top_p, threshold}``, and the optional ``selector.sparsity_rate``
(quest.py:45-46) and ``use_estimated_weights_in_attn`` (attention.py:295-296). All buffers are allocated once; a
step is a single call into ``twl_decode_layer`` which enqueues the kernels on the current stream.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional

import torch

from . import _lib
from .cache import PagedKVCache
from .kernel._check import check_dim, check_input, dtype_code, ptr, stream_of
from .kernel.quest import quest_num_pages


def parse_sparse_config(cfg: dict) -> dict:
    """Validate a reference-style algorithm config (twilight/pyimpl/attention.py:360-400) and
    return the parameters of the path this package implements."""
    sel = dict(cfg.get("selector", {}))
    est = dict(cfg.get("weight_estimator", {}))
    prn = dict(cfg.get("weight_pruner", {}))
    if sel.get("type", "quest") != "quest":
        raise RuntimeError(f"selector type {sel.get('type')!r} is not supported (only 'quest')")
    if sel.get("chunk_size", _lib.PAGE) != _lib.PAGE:
        raise RuntimeError(f"quest chunk_size must equal the page size {_lib.PAGE}")
    if est.get("type", "min_max_quant") != "min_max_quant" or est.get("quant_bit", 4) != 4:
        raise RuntimeError("weight_estimator must be {type: min_max_quant, quant_bit: 4}")
    if prn.get("type", "top_p") != "top_p":
        raise RuntimeError(f"weight_pruner type {prn.get('type')!r} is not supported (only 'top_p')")
    rate = float(sel.get("sparsity_rate", -1))
    if rate != -1 and not (0.0 <= rate <= 1.0):
        raise RuntimeError(f"selector sparsity_rate must be -1 (off) or in [0, 1], got {rate}")
    return dict(token_budget=int(sel.get("token_budget", 8192)),
                top_p=float(prn.get("threshold", 0.85)), sparsity_rate=rate,
                use_estimated_weights=bool(cfg.get("use_estimated_weights_in_attn", False)))


class TwilightDecodeLayer:
    """One attention layer's decode step over a :class:`PagedKVCache`."""

    def __init__(self, cache: PagedKVCache, num_q_heads: int, token_budget: int = 8192,
                 top_p: float = 0.85, high: str = "max", sm_scale: Optional[float] = None,
                 fused_estimator: bool = True, keep_scores: bool = False,
                 reserve_pages: int = 0, group_union: bool = False,
                 sparsity_rate: float = -1, use_estimated_weights: bool = False,
                 group_select: bool = False):
        if num_q_heads % cache.num_kv_heads != 0:
            raise RuntimeError("num_q_heads must be a multiple of the cache's kv heads")
        if not (0.0 < top_p <= 1.0):
            raise RuntimeError(f"top_p must be in (0, 1], got {top_p}")
        if high not in ("first", "max"):
            raise RuntimeError("high must be 'first' or 'max'")
        self.cache, self.H = cache, num_q_heads
        self.token_budget, self.top_p = int(token_budget), float(top_p)
        self.high_mode = _lib.TWL_HIGH_FIRST if high == "first" else _lib.TWL_HIGH_MAX
        self.sm_scale = 1.0 / math.sqrt(_lib.HEAD_DIM) if sm_scale is None else float(sm_scale)
        # fused_estimator: estimate + prune in one launch; the estimator scores are then written
        # to ``self.scores`` only when keep_scores is set (the split path always writes them)
        self.fused_estimator, self.keep_scores = bool(fused_estimator), bool(keep_scores)
        # work buffers are sized for requests of up to reserve_pages pages, so a context that grows
        # during decode does not reallocate them every time a request takes a new page
        self.reserve_pages = int(reserve_pages)
        # group_union: the q heads of a kv head attend over the union of their survivor lists
        # (``group_idx`` / ``group_count``) instead of each over its own; ``count`` / ``idx`` still
        # hold the per-head results of the pruner
        self.group_union = bool(group_union)
        if self.group_union and num_q_heads // cache.num_kv_heads not in (1, 2, 4, 8):
            raise RuntimeError("group_union needs 1, 2, 4 or 8 q heads per kv head")
        # sparsity_rate != -1 replaces token_budget every step by int(longest request * rate), as
        # quest.py:45-46 does with the sequence length of its padded batch
        self.sparsity_rate = float(sparsity_rate)
        if self.sparsity_rate != -1 and not (0.0 <= self.sparsity_rate <= 1.0):
            raise RuntimeError("sparsity_rate must be -1 (off) or in [0, 1]")
        # use_estimated_weights: the attention weighs V with the estimator's probabilities of the
        # survivors (``surv_probs``) instead of computing exact logits from K
        self.use_estimated_weights = bool(use_estimated_weights)
        if self.use_estimated_weights and self.group_union:
            raise RuntimeError("use_estimated_weights and group_union exclude each other")
        # group_select: one candidate list per kv head (a page scores the largest of its group's
        # q-head scores), metadata and INT4 records read once per kv head; every q head still
        # prunes and attends on its own scores. Not the reference's per-q-head selection.
        self.group_select = bool(group_select) and num_q_heads != cache.num_kv_heads
        if self.group_select and num_q_heads // cache.num_kv_heads not in (2, 4, 8):
            raise RuntimeError("group_select needs 2, 4 or 8 q heads per kv head")
        self._alloc()

    @classmethod
    def from_config(cls, cache: PagedKVCache, num_q_heads: int, cfg: dict, **kw):
        return cls(cache, num_q_heads, **parse_sparse_config(cfg), **kw)

    def _alloc(self) -> None:
        c = self.cache
        B, H, dev = c.batch, self.H, c.device
        cap = max(c.max_pages_per_req, self.reserve_pages)
        self.k_pages = quest_num_pages(self._budget(cap * _lib.PAGE), cap)
        M = self.k_pages * _lib.PAGE
        if M > _lib.MAX_CANDIDATES:
            raise RuntimeError(f"token budget {M} exceeds the supported maximum {_lib.MAX_CANDIDATES}")
        i32, f32 = torch.int32, torch.float32
        self.sel_pages = torch.zeros((B, H, self.k_pages), dtype=i32, device=dev)
        self.sel_count = torch.zeros((B, H), dtype=i32, device=dev)
        self.page_scores = torch.zeros((B, H, cap), dtype=f32, device=dev)
        self.scores = torch.zeros((B, H, M), dtype=f32, device=dev)
        self.cand_count = torch.zeros((B, H), dtype=i32, device=dev)
        self.idx = torch.zeros((B, H, M), dtype=i32, device=dev)
        self.count = torch.zeros((B, H), dtype=i32, device=dev)
        self.out = torch.zeros((B, H, _lib.HEAD_DIM), dtype=c.dtype, device=dev)
        ws = int(_lib.lib().twl_sparse_attn_workspace_bytes(B * H, M))
        self.attn_workspace = torch.zeros(ws, dtype=torch.uint8, device=dev)
        self.surv_probs = torch.zeros((B, H, M), dtype=f32, device=dev) \
            if self.use_estimated_weights else None
        self.group_idx = self.group_count = self.group_workspace = None
        if self.group_union:
            Hkv = c.num_kv_heads
            gs = min(cap * _lib.PAGE, (H // Hkv) * M)
            self.group_idx = torch.zeros((B, Hkv, gs), dtype=i32, device=dev)
            self.group_count = torch.zeros((B, Hkv), dtype=i32, device=dev)
            gws = int(_lib.lib().twl_group_attn_workspace_bytes(B, H, Hkv, gs, 1))
            self.group_workspace = torch.empty(gws, dtype=torch.uint8, device=dev)
        self._shape = (B, cap)
        self._args, self._args_key = None, None

    def _budget(self, seq_len: int) -> int:
        """Token budget of a step whose longest request holds ``seq_len`` tokens."""
        if self.sparsity_rate == -1:
            return self.token_budget
        # quest.py:45-46, then :91-93: a budget of 0 still keeps one chunk, which is what a budget
        # of one whole chunk asks for
        budget = int(seq_len * self.sparsity_rate)
        return budget if budget > 0 else _lib.PAGE

    def _build_args(self, q: torch.Tensor) -> "_lib.LayerArgs":
        c = self.cache
        ks = c.k_cache.stride()
        a = _lib.LayerArgs()
        a.q, a.dtype = ptr(q), dtype_code(q.dtype, "q")
        a.k_cache, a.v_cache = ptr(c.k_cache), ptr(c.v_cache)
        a.page_stride, a.token_stride, a.head_stride = ks[0], ks[1], ks[2]
        a.k_int4, a.meta = ptr(c.k_int4), ptr(c.meta)
        planes = getattr(c, "meta_planes", None)
        slots = getattr(c, "plane_slots", None)
        fits = planes is not None and planes.size(4) >= c.max_pages_per_req and \
            (planes.size(0) >= c.batch if slots is None else slots.numel() == c.batch)
        if fits:
            a.meta_planes, a.plane_cap_pages = ptr(planes), planes.size(4)
            a.plane_slots, a.plane_num_slots = ptr(slots), planes.size(0)
        else:
            a.meta_planes, a.plane_cap_pages = None, 0
            a.plane_slots, a.plane_num_slots = None, 0
        a.kv_page_indices, a.kv_page_indptr = ptr(c.kv_page_indices), ptr(c.kv_page_indptr)
        a.kv_last_page_len = ptr(c.kv_last_page_len)
        a.batch, a.num_q_heads, a.num_kv_heads = c.batch, self.H, c.num_kv_heads
        a.max_pages_per_req, a.token_budget = c.max_pages_per_req, self._budget(c.max_seq_len)
        a.top_p, a.high_mode, a.sm_scale = self.top_p, self.high_mode, self.sm_scale
        a.sel_pages, a.sel_stride = ptr(self.sel_pages), self.sel_pages.size(2)
        a.sel_count = ptr(self.sel_count)
        a.page_scores, a.page_score_stride = ptr(self.page_scores), self.page_scores.size(2)
        a.scores, a.score_stride = ptr(self.scores), self.scores.size(2)
        a.cand_count = ptr(self.cand_count)
        a.idx, a.idx_stride = ptr(self.idx), self.idx.size(2)
        a.count = ptr(self.count)
        a.attn_workspace, a.attn_workspace_bytes = ptr(self.attn_workspace), self.attn_workspace.numel()
        a.out = ptr(self.out)
        a.split_estimator = 0 if self.fused_estimator else 1
        a.keep_scores = 1 if self.keep_scores else 0
        if self.group_union:
            a.group_idx, a.group_idx_stride = ptr(self.group_idx), self.group_idx.size(2)
            a.group_count = ptr(self.group_count)
            a.group_workspace = ptr(self.group_workspace)
            a.group_workspace_bytes = self.group_workspace.numel()
        if self.use_estimated_weights:
            a.surv_probs, a.use_estimated_weights = ptr(self.surv_probs), 1
        a.group_select = 1 if self.group_select else 0
        return a

    def forward(self, q: torch.Tensor) -> torch.Tensor:
        """``q`` [B, H, 128] in the cache dtype -> attention output [B, H, 128] (same buffer every
        call). Intermediates stay readable as ``sel_pages/sel_count/idx/count`` (and ``scores``
        with ``keep_scores`` or the split estimator)."""
        c = self.cache
        check_input(q, "q")
        check_dim(3, q, "q")
        if c.batch != self._shape[0] or c.max_pages_per_req > self._shape[1]:
            self._alloc()
        if tuple(q.shape) != (c.batch, self.H, _lib.HEAD_DIM) or q.dtype != c.dtype:
            raise RuntimeError(f"q must be [{c.batch}, {self.H}, {_lib.HEAD_DIM}] of {c.dtype}")
        if q.device != c.device:
            raise RuntimeError(f"q must be on {c.device}")
        key = (q.data_ptr(), c.k_cache.data_ptr(), c.v_cache.data_ptr(), c.k_int4.data_ptr(),
               c.meta.data_ptr(), c.kv_page_indices.data_ptr(), c.kv_page_indptr.data_ptr(),
               c.kv_last_page_len.data_ptr(), c.max_pages_per_req,
               0 if c.meta_planes is None else c.meta_planes.data_ptr(),
               0 if c.plane_slots is None else c.plane_slots.data_ptr())
        if self._args_key != key:
            self._args, self._args_key = self._build_args(q), key
        a = self._args
        if self.sparsity_rate != -1:
            a.token_budget = self._budget(c.max_seq_len)
        with torch.cuda.device(c.device):
            rc = _lib.lib().twl_decode_layer(ctypes.byref(a), stream_of(q))
        _lib.check(rc, "TwilightDecodeLayer")
        return self.out

    __call__ = forward
