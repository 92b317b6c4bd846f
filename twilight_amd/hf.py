"""Hugging Face Llama / Mistral integration of the Select-then-Prune decode path.

Mirrors ``enable_sparse_attention(model, sparse_config, enable_budget_info, enable_score_info)``
of twilight/pyimpl/attention.py:351-418 (config template :360-377, module patching :481-493) and
the budget statistics of twilight/pyimpl/state.py:158-234. Prefill (q_len > 1) runs the model's
own attention, as the reference runs flash attention there (attention.py:158-183); a decode step
(q_len == 1) of a patched layer appends the new token to a :class:`PagedKVCache` (K / V pages,
INT4 K shadow, Quest metadata) and calls :class:`TwilightDecodeLayer` instead of attending over the
whole context. The first two layers stay dense when ``skip_first_two_layers`` is set
(attention.py:199-201, config default :413).

Only the configuration the decode path implements is accepted: selector ``quest`` (chunk size 16),
weight estimator ``min_max_quant`` with 4 bits, weight pruner ``top_p``; anything else raises.
"""
from __future__ import annotations

import types
from typing import Dict, List, Optional, Tuple

import torch

from . import _lib
from .cache import PagedKVCache
from .kernel.attention import (group_attention_workspace_bytes, group_paged_decode_attention,
                               rope_qk_)
from .layer import TwilightDecodeLayer, parse_sparse_config

PAGE = _lib.PAGE


class HistoryBudgetInfo:
    """Per query (= one decode step through the model), per layer: survivors per head after
    pruning (the reference's "B1") and the selector's token budget ("B0"). Same accounting as
    twilight/pyimpl/state.py:158-234: a new query starts whenever the layer id does not follow the
    previous one, and averages skip layers 0 and 1."""

    def __init__(self) -> None:
        self.reset()

    def reset(self) -> None:
        self._budget_num: List[Dict[int, torch.Tensor]] = []
        self._B0: List[Dict[int, int]] = []
        self._last_layer_id = -999

    def update(self, layer_id: int, head_budgets: torch.Tensor) -> None:
        """``head_budgets``: survivors per (batch, head), any shape; stored flattened."""
        if layer_id != self._last_layer_id + 1:
            self._budget_num.append({})
            self._B0.append({})
        self._budget_num[-1][layer_id] = head_budgets.detach().flatten().clone()
        self._last_layer_id = layer_id

    def update_B0(self, layer_id: int, token_budget: int) -> None:
        if not self._B0:
            self._B0.append({})
        self._B0[-1][layer_id] = int(token_budget)

    def get_avg_budget_per_layer_single_query(self, query_index: int) -> List[float]:
        return [float(v.float().mean()) for v in self._budget_num[query_index].values()]

    def get_avg_budget_cur_query(self) -> List[float]:
        return self.get_avg_budget_per_layer_single_query(-1)

    def get_avg_budget_per_query(self) -> List[float]:
        out = []
        for q in self._budget_num:
            vals = [float(v.float().mean()) for lid, v in q.items() if lid > 1]
            out.append(sum(vals) / len(vals) if vals else float("nan"))
        return out

    def get_avg_budget_per_query_B0(self) -> List[float]:
        out = []
        for q in self._B0:
            vals = [b for lid, b in q.items() if lid > 1]
            out.append(sum(vals) / len(vals) if vals else float("nan"))
        return out

    def get_total_avg_budget(self) -> float:
        v = self.get_avg_budget_per_query()
        return sum(v) / len(v) if v else float("nan")

    def get_total_avg_budget_B0(self) -> float:
        v = self.get_avg_budget_per_query_B0()
        return sum(v) / len(v) if v else float("nan")

    def print_budget_info_single_query(self, query_index: int = -1) -> None:
        for lid, v in self._budget_num[query_index].items():
            print(f"Layer {lid}: {v.tolist()} Head Average: {float(v.float().mean()):.2f}")


class HistoryAccumulatedScoreInfo:
    """Per query and layer: the share of the TRUE attention mass (softmax of q·K/sqrt(d) over the
    whole context) that the kept tokens carry, per head, and its minimum over the heads. Same
    accounting as twilight/pyimpl/state.py:82-132 (queries split on the layer id, averages skip
    layers 0 and 1)."""

    def __init__(self) -> None:
        self.reset()

    def reset(self) -> None:
        self._score_sum: List[Dict[int, torch.Tensor]] = []
        self._min_sum: List[Dict[int, float]] = []
        self._last_layer_id = -999

    def update(self, layer_id: int, score_sum: torch.Tensor) -> None:
        """``score_sum``: kept attention mass per (batch, head), any shape; stored flattened."""
        if layer_id != self._last_layer_id + 1:
            self._score_sum.append({})
            self._min_sum.append({})
        flat = score_sum.detach().flatten().float().clone()
        self._score_sum[-1][layer_id] = flat
        self._min_sum[-1][layer_id] = float(flat.min())
        self._last_layer_id = layer_id

    def print_min_sum_single_query(self, query_index: int = -1) -> None:
        for lid, v in self._min_sum[query_index].items():
            print(f"Layer {lid}: {v:.2f}")

    def print_score_sum_single_query(self, query_index: int = -1) -> None:
        for lid, v in self._score_sum[query_index].items():
            print(f"Layer {lid}: {v}")

    def get_avg_score_per_query(self) -> List[float]:
        out = []
        for q in self._min_sum:
            vals = [v for lid, v in q.items() if lid > 1]
            out.append(sum(vals) / len(vals) if vals else float("nan"))
        return out

    def get_total_avg_score(self) -> float:
        v = self.get_avg_score_per_query()
        return sum(v) / len(v) if v else float("nan")


def kept_attention_mass(cache: PagedKVCache, q: torch.Tensor, idx: torch.Tensor,
                        count: torch.Tensor, sm_scale: float) -> torch.Tensor:
    """Diagnostic, not part of the decode path: for every (request, q head) the sum over the kept
    tokens ``idx[b, h, :count[b, h]]`` of softmax(q·K·sm_scale) taken over the request's WHOLE
    context, [B, H] fp32. It reads all of K with plain tensor operations on the GPU, which is what
    the decode path exists to avoid; the reference's statistic (state.py:96-110) costs the same
    there, since its dense-masked attention has the full weights at hand."""
    B, H, _ = q.shape
    Hkv = cache.num_kv_heads
    ptr = cache.kv_page_indptr.tolist()
    last = cache.kv_last_page_len.tolist()
    out = torch.zeros((B, H), dtype=torch.float32, device=q.device)
    for b in range(B):
        pages = cache.kv_page_indices[ptr[b]:ptr[b + 1]].long()
        n = (len(pages) - 1) * PAGE + last[b]
        k = cache.k_cache[pages].reshape(-1, Hkv, _lib.HEAD_DIM)[:n].float()      # [n, Hkv, D]
        k = k.repeat_interleave(H // Hkv, dim=1)                                  # [n, H, D]
        w = torch.softmax(torch.einsum("hd,nhd->hn", q[b].float(), k) * sm_scale, dim=-1)
        keep = torch.arange(idx.shape[-1], device=q.device)[None, :] < count[b][:, None]
        kept = torch.gather(w, 1, idx[b].long().clamp_(0, n - 1)) * keep
        out[b] = kept.sum(-1)
    return out


class _LayerState:
    """What a patched attention module carries between calls."""

    def __init__(self, cfg: dict, reserve_tokens: int, budget_info: Optional[HistoryBudgetInfo],
                 keep_hf_cache: bool, score_info: Optional[HistoryAccumulatedScoreInfo] = None,
                 dense: bool = False):
        self.cfg, self.reserve_tokens, self.budget_info = cfg, reserve_tokens, budget_info
        self.keep_hf_cache, self.score_info = keep_hf_cache, score_info
        self.dense = dense        # a layer the configuration leaves dense, served from paged K / V
        self.recorded = False     # the decode step is recorded / replayed by GraphedDecodeStep
        self.workspace: Optional[torch.Tensor] = None
        self.max_tokens = 0
        self.cache: Optional[PagedKVCache] = None
        self.layer: Optional[TwilightDecodeLayer] = None
        self.free: List[int] = []
        self.seq_len = 0          # tokens of the current sequence seen by this layer

    def reset(self) -> None:
        self.cache, self.layer, self.free, self.seq_len = None, None, [], 0
        self.workspace = None


def fill_from_prefill(st: _LayerState, k: torch.Tensor, v: torch.Tensor, num_q_heads: int) -> None:
    """Page the prefill K / V [B, Hkv, N, 128] of a layer and size everything for
    ``reserve_tokens`` more tokens per request. The first decode step of a patched module calls
    this on what the model's cache holds; a caller that has the K / V of a context from elsewhere
    may call it on ``module._twilight_state`` itself and decode from there."""
    B, _, N, _ = k.shape
    npg = (N + PAGE - 1) // PAGE
    spare_per_req = (st.reserve_tokens + PAGE - 1) // PAGE + 1
    # plane-layout metadata next to the records: the one-launch selector reads half the bytes from
    # it (with GQA it is used at the batch sizes where that launch runs, the records otherwise)
    planes = npg + spare_per_req
    st.cache = PagedKVCache.from_dense(k, v, k.device, spare_pages=B * spare_per_req,
                                       plane_pages=None if st.dense else planes)
    st.free = list(range(B * npg, B * (npg + spare_per_req)))
    st.seq_len = N
    if st.dense:
        st.max_tokens = (npg + spare_per_req) * PAGE
        st.workspace = torch.empty(group_attention_workspace_bytes(
            B, num_q_heads, k.shape[1], st.max_tokens, False), dtype=torch.uint8, device=k.device)
        return
    st.layer = TwilightDecodeLayer(st.cache, num_q_heads, reserve_pages=npg + spare_per_req, **st.cfg)


_mask_checked = None   # weak reference to the mask the last check passed (one check per step)


def _check_mask_hides_nothing(mask) -> None:
    """Raise for a decode-step attention mask that hides a position. Every layer of a step gets
    the same tensor, so the (synchronising) look at its values happens once per step."""
    global _mask_checked
    if _mask_checked is not None and _mask_checked() is mask:
        return
    hides = (~mask).any() if mask.dtype == torch.bool else (mask < 0).any()
    if bool(hides):
        raise RuntimeError("the Select-then-Prune decode step cannot honour an attention_mask "
                           "that hides positions (padded batches are not supported)")
    import weakref
    _mask_checked = weakref.ref(mask)


def _twilight_attention_forward(self, hidden_states, position_embeddings=None, attention_mask=None,
                                past_key_values=None, **kwargs):
    """Replacement of ``LlamaAttention.forward``: the module's own forward for prefill, the
    Select-then-Prune layer for decode (twilight/pyimpl/attention.py:59-306 split the same way)."""
    st: _LayerState = self._twilight_state
    q_len = hidden_states.shape[1]
    # a single token with nothing cached yet is a (one-token) prefill, not a decode step
    first_token = (past_key_values is not None and st.cache is None and st.seq_len == 0
                   and past_key_values.get_seq_length(self.layer_idx) == 0)
    if q_len > 1 or past_key_values is None or first_token:
        if past_key_values is None or past_key_values.get_seq_length(self.layer_idx) == 0:
            st.reset()                                    # a new sequence starts
        out = self._twilight_orig_forward(hidden_states, position_embeddings=position_embeddings,
                                          attention_mask=attention_mask,
                                          past_key_values=past_key_values, **kwargs)
        st.seq_len += q_len
        st.cache = st.layer = None                        # paged lazily at the next decode step
        return out
    if attention_mask is not None and not st.recorded:
        # The paged path attends to every cached position of every request, as the reference's
        # decode branch does (it asserts the mask away, twilight/pyimpl/attention.py:186): a mask
        # that hides positions (a left-padded batch) cannot be honoured, so it is refused rather
        # than ignored. Masks that hide nothing pass.
        _check_mask_hides_nothing(attention_mask)
    if st.cache is None:
        # first decode step after a prefill (possibly a prefill that ran before patching): page
        # the K / V the model's own cache holds for this layer
        lay = past_key_values.layers[self.layer_idx] if len(past_key_values.layers) > self.layer_idx else None
        keys = getattr(lay, "keys", None)
        if keys is None or not keys.is_cuda or keys.shape[-2] == 0:
            raise RuntimeError("decode step without prefilled K / V of this layer on a GPU (the "
                               "path has no CPU implementation and needs use_cache=True)")
        n = st.seq_len if st.seq_len > 0 else past_key_values.get_seq_length(self.layer_idx)
        fill_from_prefill(st, keys[:, :, :n], lay.values[:, :, :n], self.config.num_attention_heads)
    B = hidden_states.shape[0]
    # one token per request: the projections are already [B, heads, 128]; the rotary embedding
    # is one launch, in place, with the roundings of the model's own chain of tensor operations
    q = self.q_proj(hidden_states).view(B, -1, self.head_dim)
    k = self.k_proj(hidden_states).view(B, -1, self.head_dim)
    v = self.v_proj(hidden_states).view(B, -1, self.head_dim)
    cos, sin = position_embeddings
    cos, sin = cos[:, 0].expand(B, -1).contiguous(), sin[:, 0].expand(B, -1).contiguous()
    if cos.dtype != q.dtype:
        cos, sin = cos.to(q.dtype), sin.to(q.dtype)
    rope_qk_(q, k, cos, sin)
    q, k, v = q.unsqueeze(2), k.unsqueeze(2), v.unsqueeze(2)      # [B, heads, 1, 128] views
    if st.keep_hf_cache:
        past_key_values.update(k, v, self.layer_idx)  # keeps the model's own cache consistent
    if st.recorded:   # GraphedDecodeStep has done the host half for this step
        st.cache.append_device(k[:, :, 0], v[:, :, 0])
    else:
        st.cache.append(k[:, :, 0], v[:, :, 0], st.free)
        st.seq_len += 1
    if st.dense:
        c = st.cache
        out = group_paged_decode_attention(
            q[:, :, 0].contiguous(), c.k_cache, c.v_cache, c.kv_page_indices, c.kv_page_indptr,
            c.kv_last_page_len, max_tokens=st.max_tokens, sm_scale=getattr(self, "scaling", None),
            workspace=st.workspace)
        return self.o_proj(out.reshape(B, 1, -1)), None
    out = st.layer(q[:, :, 0].contiguous())           # [B, H, 128]
    if st.budget_info is not None and not st.recorded:
        st.budget_info.update(self.layer_idx, st.layer.count)
        st.budget_info.update_B0(self.layer_idx, min(st.layer._budget(st.seq_len), st.seq_len))
    if st.score_info is not None and not st.recorded:
        st.score_info.update(self.layer_idx, kept_attention_mass(
            st.cache, q[:, :, 0], st.layer.idx, st.layer.count, st.layer.sm_scale))
    attn_output = self.o_proj(out.reshape(B, 1, -1))
    return attn_output, None


def enable_sparse_attention(model, sparse_config: Dict, enable_budget_info: bool = False,
                            enable_score_info: bool = False, reserve_tokens: int = 4096,
                            high: str = "max", keep_hf_cache: bool = True,
                            dense_layers: str = "model",
                            group_select: bool = False) -> Tuple[Optional[HistoryBudgetInfo],
                                       Optional[HistoryAccumulatedScoreInfo]]:
    """Patch every Llama / Mistral attention module of ``model`` (twilight/pyimpl/attention.py:
    351-418, 481-493). ``sparse_config`` is the reference's JSON template
    (benchmark/configs/config_quest_twi.json). ``reserve_tokens``: decode tokens per request the
    paged caches are sized for. ``keep_hf_cache=False`` stops patched layers from also appending
    decode tokens to the model's own cache (a whole-context copy per step with ``DynamicCache``);
    it needs ``skip_first_two_layers`` (layer 0 keeps the sequence length the model asks its cache
    for) and a sequence that is only prefilled once. Returns ``(budget_info, score_info)`` as the
    reference does (attention.py:404-418). ``dense_layers``: how the layers the configuration
    leaves dense (``skip_first_two_layers``) decode — "model": through the model's own attention
    and cache, as in the reference; "paged": from paged K / V through the group attention kernel
    (K / V read once per kv head). With "paged" and ``keep_hf_cache=False`` nothing updates the
    model's cache at decode time, so the caller passes ``position_ids`` to the model itself. ``enable_score_info`` adds a dense pass over all of K
    to every patched layer's decode step (:func:`kept_attention_mass`): a diagnostic, not for
    timing runs. ``group_select``: with q heads that share kv heads (GQA), one Quest candidate list
    per kv head (a page scores the largest of its group's q-head scores) instead of the
    reference's list per q head (attention.py:124-126 repeats K per q head); top-p and attention
    stay per q head. Fewer bytes per layer; not the reference's selection."""
    for part in ("compressor",):
        t = sparse_config.get(part, {}).get("type", "none")
        if str(t).lower() not in ("none", ""):
            raise RuntimeError(f"{part} type {t!r} is not supported")
    cfg = parse_sparse_config(sparse_config)
    cfg["high"] = high
    cfg["group_select"] = bool(group_select)
    skip = 2 if sparse_config.get("skip_first_two_layers", True) else 0
    if dense_layers not in ("model", "paged"):
        raise RuntimeError(f"dense_layers must be 'model' or 'paged', got {dense_layers!r}")
    if not keep_hf_cache and skip == 0:
        raise RuntimeError("keep_hf_cache=False needs skip_first_two_layers")
    budget_info = HistoryBudgetInfo() if enable_budget_info else None
    score_info = HistoryAccumulatedScoreInfo() if enable_score_info else None
    patched = 0
    for name, module in model.named_modules():
        if not all(hasattr(module, a) for a in ("q_proj", "k_proj", "v_proj", "o_proj", "layer_idx")):
            continue
        if getattr(module, "head_dim", None) != _lib.HEAD_DIM:
            raise RuntimeError(f"{name}: head_dim must be {_lib.HEAD_DIM}")
        if hasattr(module, "_twilight_state"):
            raise RuntimeError("enable_sparse_attention was already called on this model")
        dense = module.layer_idx < skip
        if dense and dense_layers == "model":
            continue
        module._twilight_state = _LayerState(dict(cfg), reserve_tokens,
                                             None if dense else budget_info, keep_hf_cache,
                                             None if dense else score_info, dense=dense)
        module._twilight_orig_forward = module.forward
        module.forward = types.MethodType(_twilight_attention_forward, module)
        patched += 1
    if patched == 0:
        raise RuntimeError("no attention module was patched")
    return budget_info, score_info


class GraphedDecodeStep:
    """Decode steps of a patched model replayed from ONE recorded HIP graph.

    The model's eager decode step issues about a thousand small launches; at the speeds of this
    path the host cannot keep up with the GPU. Here the step is recorded once
    (``torch.cuda.graph``: the model's own kernels and the library's launches alike, all on the
    capture stream) and replayed; per step the host only advances the page tables
    (:meth:`PagedKVCache.advance_host`), writes the token ids and positions into fixed buffers and
    launches the graph. Page tables have fixed addresses (:meth:`PagedKVCache.reserve_page_table`),
    so the recording stays valid while the requests grow, up to ``reserve_tokens`` more tokens.

    Needs ``enable_sparse_attention(..., dense_layers="paged", keep_hf_cache=False)`` (nothing may
    touch the model's own cache inside the recording) and that every patched layer holds its paged
    K / V: run the first decode step after a prefill eagerly, or call :func:`fill_from_prefill`.
    Budget statistics are updated after every replay; the accumulated-score diagnostic is not
    available."""

    def __init__(self, model):
        self.model = model
        self.states: List[Tuple[int, _LayerState]] = []
        for _, module in model.named_modules():
            if all(hasattr(module, a) for a in ("q_proj", "k_proj", "v_proj", "o_proj", "layer_idx")):
                st = getattr(module, "_twilight_state", None)
                if st is None:
                    raise RuntimeError("GraphedDecodeStep needs dense_layers='paged': attention "
                                       f"layer {module.layer_idx} is not patched")
                if st.keep_hf_cache:
                    raise RuntimeError("GraphedDecodeStep needs keep_hf_cache=False")
                if st.score_info is not None:
                    raise RuntimeError("GraphedDecodeStep cannot record the score diagnostic")
                if not st.dense and st.cfg.get("sparsity_rate", -1) != -1:
                    # the budget is a launch argument: a recorded step would keep the first one
                    raise RuntimeError("GraphedDecodeStep cannot record a selector with "
                                       "sparsity_rate (its token budget changes every step)")
                self.states.append((module.layer_idx, st))
        if not self.states:
            raise RuntimeError("no patched attention module")
        self.states.sort(key=lambda t: t[0])
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.ids = self.pos = self.logits = self.past = None
        self._warm = False

    def _prepare(self, input_ids: torch.Tensor) -> None:
        from transformers import DynamicCache
        for lid, st in self.states:
            if st.cache is None:
                raise RuntimeError(f"layer {lid} has no paged K / V yet: run the first decode step "
                                   "after a prefill eagerly")
            cap = (st.max_tokens // PAGE) if st.dense else st.layer.reserve_pages
            st.cache.reserve_page_table(max(cap, st.cache.max_pages_per_req))
        self.ids = input_ids.clone()
        self.pos = torch.zeros_like(self.ids)
        self.past = DynamicCache(config=self.model.config)   # stays empty: nothing updates it

    def __call__(self, input_ids: torch.Tensor) -> torch.Tensor:
        """``input_ids`` [B, 1] -> logits [B, 1, vocab] (from the second call on the same buffer
        every call; the first call runs the step eagerly, the second records it)."""
        if self.ids is None:
            self._prepare(input_ids)
        seq = self.states[0][1].seq_len
        if any(st.seq_len != seq for _, st in self.states):
            raise RuntimeError("the patched layers disagree on the sequence length")
        for _, st in self.states:
            st.cache.advance_host(st.free)
            st.seq_len += 1
            st.recorded = True
        try:
            self.ids.copy_(input_ids)
            self.pos.fill_(seq)
            if not self._warm:
                # the first step runs eagerly, with the same shapes and buffers: libraries that
                # set themselves up on first use (GEMM workspaces) must not do so while recording
                with torch.no_grad():
                    self.logits = self.model(self.ids, past_key_values=self.past, use_cache=True,
                                             position_ids=self.pos).logits
                self._warm = True
            else:
                if self.graph is None:
                    graph = torch.cuda.CUDAGraph()
                    with torch.no_grad(), torch.cuda.graph(graph):
                        out = self.model(self.ids, past_key_values=self.past, use_cache=True,
                                         position_ids=self.pos)
                    self.graph, self.logits = graph, out.logits
                # recording does not execute: the step itself is the replay, the first time too
                self.graph.replay()
        finally:
            for _, st in self.states:
                st.recorded = False
        for lid, st in self.states:
            if st.budget_info is not None and not st.dense:
                st.budget_info.update(lid, st.layer.count)
                st.budget_info.update_B0(lid, min(st.layer._budget(st.seq_len), st.seq_len))
        return self.logits


def disable_sparse_attention(model) -> None:
    """Undo :func:`enable_sparse_attention` (the reference's ``reset_sparse_config``,
    attention.py:496-499, only clears its global flag)."""
    for _, module in model.named_modules():
        if hasattr(module, "_twilight_state"):
            module.forward = module._twilight_orig_forward
            del module._twilight_state, module._twilight_orig_forward
