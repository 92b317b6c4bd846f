"""TEST INFRASTRUCTURE ONLY — torch-CPU / numpy restatement of ``twilight/pyimpl`` decode math.

Every function cites the reference lines it follows. Functions whose names end in ``_records``
or ``_paged`` describe the storage formats of this build (INT4 shadow records, Quest metadata
records, FlashInfer-style page tables); the reference has no counterpart for them and they are
checked by round trips against the dense functions.

How each function is pinned (tests/test_oracle_*.py):
  min_max_quant_ref      known-answer vector of twilight/pyimpl/quantize.py:30-48 worked by hand
                         (min -3.56, max 4.32, 15 codes), min/max reproduce, |err| <= scale/2
  quest_selector_dense   brute force per chunk on N=40 (padding branch) + equality with the
                         min/max metadata form
  estimator_scores       reduces to a float64 matmul (library routine)
  top_p_unnormalized     softmax is torch's; the bisection is oracle.native.top_p_mask_f32
                         (pinned against the textbook nucleus set and brute force)
  masked_attention       reduces to softmax + matmul over gathered survivors (checked both ways),
                         also with given logits (use_estimated_weights_in_attn); a K the 4-bit
                         grid holds exactly makes both attention modes of decode_layer_dense meet
  sparsity_rate          closed forms of the budget rule: rate 1 keeps all, rate 0 one chunk
  quest_selector_group_dense
                         group 1 is quest_selector_dense; identical queries inside a group give
                         the per-head selection; brute force over the group maxima on 25 chunks
  get_label_tensor_ref, bgemv_int8_ref
                         the reference's own torch checks (channel.py:82-110, bgemv_int8.py:78-93),
                         i.e. a gather and a matmul
  qk_int8_lse_ref        closed form: float64 base-2 logsumexp of the dequantised product plus
                         the zero-padded tail of the last key block
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

from . import native

PAGE = 16
HEAD_DIM = 128
QGROUP = 32
INT4_RECORD_BYTES = 1280
META_RECORD_BYTES = 512


# --------------------------------------------------------------------------------------------
# a-2  INT4 estimator quantiser
# --------------------------------------------------------------------------------------------
def min_max_quant_ref(kv: torch.Tensor, qbit: int, group: Optional[int] = None) -> torch.Tensor:
    """twilight/pyimpl/quantize.py:4-13: asymmetric min/max fake-quant over the last dim.

    ``group`` (not in the reference) applies the same function to ``kv.view(..., D/group, group)``.
    """
    shape = kv.shape
    if group is not None:
        kv = kv.reshape(*shape[:-1], shape[-1] // group, group)
    max_val = kv.amax(dim=-1, keepdim=True)                       # quantize.py:5
    min_val = kv.amin(dim=-1, keepdim=True)                       # quantize.py:6
    max_int = 2 ** qbit - 1                                       # quantize.py:8
    scales = (max_val - min_val).clamp(min=1e-9) / max_int        # quantize.py:10
    zeros = -min_val                                              # quantize.py:11
    out = torch.clamp(torch.round((kv + zeros) / scales), 0, max_int) * scales - zeros  # :13
    return out.reshape(shape)


def int4_quant_storage(k: torch.Tensor):
    """Storage form of the quantiser: group 32, fp16 scale / zero (oracle.native.int4_quant).

    ``k`` [..., 128] -> codes uint8 [...,128], scale fp16 [...,4], zero fp16 [...,4], dequant fp32.
    """
    kn = k.detach().to(torch.float32).contiguous().numpy()
    codes, scale, zero = native.int4_quant(kn, QGROUP)
    deq = native.int4_dequant(codes, scale, zero, QGROUP)
    return codes, scale, zero, deq


def pack_int4_records(codes: np.ndarray, scale: np.ndarray, zero: np.ndarray) -> np.ndarray:
    """codes [P, Hkv, 16, 128] uint8, scale/zero [P, Hkv, 16, 4] fp16 -> uint8 [P, Hkv, 1280].

    Record = 16 tokens x 64 nibble bytes (low nibble = even element), then 64 (scale, zero) fp16
    pairs indexed token*4 + group.
    """
    P, H, T, D = codes.shape
    assert T == PAGE and D == HEAD_DIM
    rec = np.zeros((P, H, INT4_RECORD_BYTES), dtype=np.uint8)
    lo = codes[..., 0::2].astype(np.uint8)
    hi = codes[..., 1::2].astype(np.uint8)
    rec[..., :1024] = (lo | (hi << 4)).reshape(P, H, 1024)
    sz = np.stack([scale.astype(np.float16), zero.astype(np.float16)], axis=-1)  # [P,H,16,4,2]
    rec[..., 1024:] = np.ascontiguousarray(sz).view(np.uint8).reshape(P, H, 256)
    return rec


def unpack_int4_records(rec: np.ndarray):
    """Inverse of :func:`pack_int4_records`."""
    P, H, _ = rec.shape
    b = rec[..., :1024].reshape(P, H, PAGE, 64)
    codes = np.zeros((P, H, PAGE, HEAD_DIM), dtype=np.uint8)
    codes[..., 0::2] = b & 0xF
    codes[..., 1::2] = b >> 4
    sz = np.ascontiguousarray(rec[..., 1024:]).view(np.float16).reshape(P, H, PAGE, 4, 2)
    return codes, sz[..., 0].copy(), sz[..., 1].copy()


# --------------------------------------------------------------------------------------------
# a-1  Quest selector
# --------------------------------------------------------------------------------------------
def quest_chunk_budget(token_budget: int, chunk_size: int, n_chunks: int) -> int:
    """twilight/pyimpl/quest.py:93-98."""
    chunk_budget = max(1, token_budget // chunk_size)
    if token_budget % chunk_size != 0:
        chunk_budget += 1
    return min(chunk_budget, n_chunks)


def quest_chunk_scores_dense(q: torch.Tensor, k: torch.Tensor, chunk_size: int) -> torch.Tensor:
    """twilight/pyimpl/quest.py:36-84: q [B,H,1,D], k [B,H,N,D] -> estimate [B,H,1,chunks]."""
    sign = (q > 0) + (~(q > 0)) * -1                               # quest.py:37
    positive_query = q * sign                                      # quest.py:38
    max_key = k * sign                                             # quest.py:39
    seq_length = max_key.shape[-2]
    padding_length = chunk_size - (seq_length % chunk_size)        # quest.py:48
    if padding_length < chunk_size:                                # quest.py:49-65
        pad = torch.ones((max_key.shape[0], max_key.shape[1], padding_length, max_key.shape[3]))
        pad = pad * torch.tensor(torch.finfo(max_key.dtype).min)
        max_key = torch.cat([max_key, pad], dim=-2)
    chunk_max_key = max_key.reshape(max_key.shape[0], max_key.shape[1],
                                    max_key.shape[2] // chunk_size, chunk_size,
                                    max_key.shape[3]).amax(dim=-2)  # quest.py:68-74
    if chunk_max_key.dtype == torch.float32:                       # quest.py:76-77
        positive_query = positive_query.float()
    return torch.matmul(positive_query, chunk_max_key.transpose(2, 3))  # quest.py:81-84


def quest_selector_dense(q: torch.Tensor, k: torch.Tensor, chunk_size: int, token_budget: int):
    """twilight/pyimpl/quest.py:17-122 -> (token mask [B,H,1,N] bool, chunk ids [B,H,1,kc]).

    ``torch.topk`` leaves the order among equal scores unspecified; this restatement breaks ties
    toward the lower chunk number (stable descending sort).
    """
    B, H, _, _ = q.shape
    N = k.shape[-2]
    est = quest_chunk_scores_dense(q, k, chunk_size)
    n_chunks = est.shape[-1]
    kc = quest_chunk_budget(token_budget, chunk_size, n_chunks)
    order = torch.sort(est.double(), dim=-1, descending=True, stable=True).indices
    topk = order[..., :kc]                                         # quest.py:99
    tok = topk.unsqueeze(-1) * chunk_size + torch.arange(chunk_size)  # quest.py:104-108
    tok = tok.reshape(B, H, 1, -1)
    padded = n_chunks * chunk_size
    mask = torch.zeros((B, H, 1, padded), dtype=torch.bool)        # quest.py:111-118
    mask.scatter_(-1, tok, True)
    return mask[..., :N], topk                                     # quest.py:121-122


def quest_selector_group_dense(q: torch.Tensor, k: torch.Tensor, chunk_size: int,
                               token_budget: int, group: int):
    """Selection per kv head (an option of this build, not in the reference, which selects per q
    head): the chunk scores of quest.py:36-84 per q head, the largest of each group of ``group``
    consecutive q heads per chunk, then the top-k of quest.py:93-122 on those, the same for every
    q head of the group. Returns (token mask [B,H,1,N] bool, group scores [B,H,1,chunks])."""
    B, H, _, _ = q.shape
    N = k.shape[-2]
    est = quest_chunk_scores_dense(q, k, chunk_size)
    n_chunks = est.shape[-1]
    gmax = est.reshape(B, H // group, group, 1, n_chunks).amax(dim=2, keepdim=True)
    gmax = gmax.expand(B, H // group, group, 1, n_chunks).reshape(B, H, 1, n_chunks)
    kc = quest_chunk_budget(token_budget, chunk_size, n_chunks)
    order = torch.sort(gmax.double(), dim=-1, descending=True, stable=True).indices
    tok = order[..., :kc].unsqueeze(-1) * chunk_size + torch.arange(chunk_size)
    mask = torch.zeros((B, H, 1, n_chunks * chunk_size), dtype=torch.bool)
    mask.scatter_(-1, tok.reshape(B, H, 1, -1), True)
    return mask[..., :N], gmax


def quest_page_meta(k_pages: torch.Tensor, valid_len: Optional[torch.Tensor] = None):
    """Per-page channel-wise min / max over the valid tokens: k_pages [P,16,Hkv,D] -> [P,Hkv,2,D].

    Equivalent production form of quest.py:68-74: amax over a chunk of ``K*sign`` is ``max K`` where
    sign is +1 and ``-min K`` where it is -1.
    """
    P = k_pages.shape[0]
    kf = k_pages.float()
    if valid_len is None:
        valid_len = torch.full((P,), PAGE, dtype=torch.int64)
    t = torch.arange(PAGE).view(1, PAGE, 1, 1)
    valid = t < valid_len.view(P, 1, 1, 1)
    mn = torch.where(valid, kf, torch.tensor(float("inf"))).amin(dim=1)
    mx = torch.where(valid, kf, torch.tensor(float("-inf"))).amax(dim=1)
    return torch.stack([mn, mx], dim=2)  # [P, Hkv, 2, D]


def pack_meta_records(meta: torch.Tensor) -> np.ndarray:
    """meta [P,Hkv,2,D] (fp16-representable) -> uint8 [P,Hkv,512]: 32 chunks of (min4, max4) fp16."""
    P, H, _, D = meta.shape
    m = meta.to(torch.float16).numpy()
    mn = m[:, :, 0].reshape(P, H, D // 4, 4)
    mx = m[:, :, 1].reshape(P, H, D // 4, 4)
    rec = np.concatenate([mn, mx], axis=-1)  # [P,H,32,8]
    return np.ascontiguousarray(rec).view(np.uint8).reshape(P, H, META_RECORD_BYTES)


def quest_page_scores_meta(q: torch.Tensor, meta: torch.Tensor) -> torch.Tensor:
    """score = sum_d max(q_d*max_d, q_d*min_d): q [D] fp32, meta [pages,2,D] -> [pages] (fp64 sum)."""
    qd = q.double()
    md = meta.double()
    return torch.maximum(qd * md[:, 0], qd * md[:, 1]).sum(-1)


# --------------------------------------------------------------------------------------------
# a-3 / a-4 / a-5  estimator, softmax, top-p
# --------------------------------------------------------------------------------------------
def estimator_scores(q: torch.Tensor, k_deq: torch.Tensor, sm_scale: Optional[float] = None):
    """twilight/pyimpl/attention.py:252-254: q [...,1,D] @ Kq [...,N,D]^T / sqrt(D), in fp32."""
    D = q.shape[-1]
    s = 1.0 / math.sqrt(D) if sm_scale is None else sm_scale
    return torch.matmul(q.float(), k_deq.float().transpose(-1, -2)) * s


def top_p_unnormalized(weights: torch.Tensor, threshold, high_mode: int = native.HIGH_FIRST):
    """twilight/pyimpl/top_p.py:10-15: softmax(fp32) over the last dim, then the mask kernel.

    ``weights`` [B,H,1,N] -> (bool mask [B,H,1,N], probs fp32, low [B*H], iters [B*H]).
    """
    probs = torch.nn.functional.softmax(weights, dim=-1, dtype=torch.float32)   # top_p.py:11-13
    B, H, Q, N = probs.shape
    assert Q == 1  # csrc/src/sampling.cu:51-60 ignores dim 2
    p = threshold.numpy() if isinstance(threshold, torch.Tensor) else threshold
    mask, low, iters = native.top_p_mask_f32(probs.reshape(B * H, N).numpy(), p, high_mode)
    return torch.from_numpy(mask.astype(bool)).reshape(B, H, 1, N), probs, low, iters


# --------------------------------------------------------------------------------------------
# a-7  attention over the surviving tokens, dense-masked form
# --------------------------------------------------------------------------------------------
def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor,
                     prob_dtype: torch.dtype = torch.float32,
                     logits: Optional[torch.Tensor] = None) -> torch.Tensor:
    """twilight/pyimpl/attention.py:188-190,299-306 with every tensor held in fp32 on the CPU.

    ``prob_dtype`` is the reference's ``query_states.dtype`` to which the probabilities are cast
    (attention.py:302-304) before the V product. ``logits`` [B,H,1,N], when given, take the place
    of q.K/sqrt(D) (attention.py:295-296, use_estimated_weights_in_attn). Returns fp32 [B,H,1,D].
    """
    D = q.shape[-1]
    if logits is not None:
        w = logits.float().clone()                                            # attention.py:295-296
    else:
        w = torch.matmul(q.float(), k.float().transpose(2, 3)) / math.sqrt(D)  # attention.py:188-190
    w = w.masked_fill(~mask, torch.finfo(torch.float32).min)                  # attention.py:299
    pr = torch.nn.functional.softmax(w, dim=-1, dtype=torch.float32)          # attention.py:302
    pr = pr.to(prob_dtype).float()                                            # attention.py:302-304
    return torch.matmul(pr, v.float())                                        # attention.py:306


# --------------------------------------------------------------------------------------------
# whole decode layer, dense-masked (what pyimpl computes for q_len == 1)
# --------------------------------------------------------------------------------------------
def decode_layer_dense(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, top_p: float,
                       token_budget: Optional[int] = None, chunk_size: int = PAGE,
                       high_mode: int = native.HIGH_MAX, quant: str = "storage",
                       prob_dtype: torch.dtype = torch.float32, k_deq: Optional[torch.Tensor] = None,
                       mask0: Optional[torch.Tensor] = None, sparsity_rate: float = -1,
                       use_estimated_weights: bool = False):
    """twilight/pyimpl/attention.py:188-306 for one decode step.

    q [B,H,1,D], k/v [B,H,N,D] (K already repeated per q head, attention.py:124-126).
    ``quant``: "storage" = group 32 + fp16 scale/zero (this build's estimator), "ref128" = the
    reference's whole-head_dim group in fp32 (quantize.py:4-13 as called at attention.py:247-251).
    ``k_deq`` may carry a pre-dequantised K (variant B of the CPU baseline: quantise on append).
    ``mask0`` bool [B,H,1,N] replaces the selector's result (tests use it to follow the later
    stages on a selection that differs from the oracle's only by pages tied at the k-th score).
    ``sparsity_rate`` != -1 replaces the budget by int(N * rate) (quest.py:45-46);
    ``use_estimated_weights`` makes the attention use the estimator's logits (attention.py:295-296).
    Returns dict(scores, mask0, probs, pruned, mask, out, low, iters).
    """
    B, H, _, D = q.shape
    N = k.shape[-2]
    if sparsity_rate != -1:
        token_budget = int(N * sparsity_rate)                                 # quest.py:45-46
    if mask0 is not None:
        assert mask0.shape == (B, H, 1, N) and mask0.dtype == torch.bool
    elif token_budget is None:
        mask0 = torch.ones((B, H, 1, N), dtype=torch.bool)                    # attention.py:198-199
    else:
        mask0, _ = quest_selector_dense(q.float(), k.float(), chunk_size, token_budget)
    if k_deq is None:
        if quant == "storage":
            k_deq = torch.from_numpy(int4_quant_storage(k)[3])
        else:
            k_deq = min_max_quant_ref(k.float(), 4)                           # attention.py:247-251
    est = estimator_scores(q, k_deq)                                          # attention.py:252-254
    est = est.masked_fill(~mask0, torch.finfo(torch.float32).min)             # attention.py:255
    pruned, probs, low, iters = top_p_unnormalized(est, top_p, high_mode)     # attention.py:274-278
    mask = mask0 & pruned                                                     # attention.py:280-281
    out = masked_attention(q, k, v, mask, prob_dtype,                         # attention.py:295-306
                           logits=est if use_estimated_weights else None)
    return dict(scores=est, mask0=mask0, probs=probs, pruned=pruned, mask=mask, out=out,
                low=low, iters=iters)


# --------------------------------------------------------------------------------------------
# paging helpers (format of this build)
# --------------------------------------------------------------------------------------------
def dense_to_paged(x: torch.Tensor, perm: Optional[torch.Tensor] = None):
    """x [B,Hkv,N,D] -> pages [B*ceil(N/16), 16, Hkv, D] (zero padded), CSR page table.

    ``perm`` (a permutation of the page ids) shuffles the physical order. Returns
    ``(pages, kv_page_indices int32, kv_page_indptr int32 [B+1], kv_last_page_len int32 [B])``.
    """
    B, H, N, D = x.shape
    npg = (N + PAGE - 1) // PAGE
    pad = npg * PAGE - N
    xp = torch.nn.functional.pad(x, (0, 0, 0, pad)) if pad else x
    pages = xp.reshape(B, H, npg, PAGE, D).permute(0, 2, 3, 1, 4).reshape(B * npg, PAGE, H, D)
    total = B * npg
    if perm is None:
        perm = torch.arange(total)
    phys = torch.empty_like(pages)
    phys[perm] = pages  # logical page l of the flat order lives at physical perm[l]
    indices = perm.to(torch.int32).clone()
    indptr = (torch.arange(B + 1) * npg).to(torch.int32)
    last = torch.full((B,), N - (npg - 1) * PAGE, dtype=torch.int32)
    return phys.contiguous(), indices, indptr, last


def mask_to_lists(mask: torch.Tensor) -> Tuple[np.ndarray, np.ndarray]:
    """bool [B,H,1,N] -> (idx int32 [B*H, N] ascending, padded with -1; count int32 [B*H])."""
    B, H, _, N = mask.shape
    m = mask.reshape(B * H, N).numpy()
    count = m.sum(-1).astype(np.int32)
    idx = np.full((B * H, N), -1, dtype=np.int32)
    for r in range(B * H):
        nz = np.nonzero(m[r])[0]
        idx[r, :nz.size] = nz
    return idx, count


# --------------------------------------------------------------------------------------------
# Double-Sparse label ops (the reference's own torch references)
# --------------------------------------------------------------------------------------------
def get_label_tensor_ref(x: torch.Tensor, channel: torch.Tensor, r: int) -> torch.Tensor:
    """The indexing twilight/kernel/triton/channel.py:98-101 checks against: X[i, j, channel[j]]."""
    L, H, _ = x.shape
    out = torch.empty((L, H, r), dtype=x.dtype)
    for h in range(H):
        out[:, h] = x[:, h, channel[h, :r]]
    return out


def bgemv_int8_ref(q_label: torch.Tensor, k_label: torch.Tensor, k_scales: torch.Tensor):
    """torch_bgemv_int8, twilight/kernel/triton/bgemv_int8.py:78-93, evaluated in fp32."""
    B, H, r = q_label.shape
    n_ctx = k_label.shape[0] // B
    k = k_label.float() * k_scales.float()[:, :, None]                       # bgemv_int8.py:83
    q = q_label.float().view(B, H, 1, r)                                      # :86
    k = k.view(B, n_ctx, H, r).transpose(1, 2).transpose(2, 3)                # :87
    return torch.matmul(q, k).squeeze(-2)                                     # :89


def qk_int8_lse_ref(q: torch.Tensor, k: torch.Tensor, q_scale: torch.Tensor, k_scale: torch.Tensor):
    """The `lse` output of qk_int8_per_block, twilight/kernel/triton/qk_int8_per_block.py:22-109,
    block by block in the kernel's own order and arithmetic (fp32; exp2 / log2).

    ``q`` int8 [b,h_qo,qo_len,d], ``k`` int8 [b,h_kv,kv_len,d] (HND), ``q_scale`` fp32
    [b,h_qo,ceil(qo_len/128)], ``k_scale`` fp32 [b,h_kv,ceil(kv_len/64)]. Keys past kv_len in the
    last 64-block are zero rows (masked load, :36-37) and take part with score 0.
    Returns fp32 [b,h_qo,qo_len].
    """
    b, h_qo, qo_len, d = q.shape
    _, h_kv, kv_len, _ = k.shape
    group = h_qo // h_kv
    BM, BN = 128, 64                                                           # :112-113
    nb = (kv_len + BN - 1) // BN
    kp = torch.zeros((b, h_kv, nb * BN, d), dtype=torch.int64)
    kp[:, :, :kv_len] = k.long()
    kp = kp.repeat_interleave(group, dim=1)                                    # :74,80 (off_h // groups)
    ks = k_scale.float().reshape(b, h_kv, nb).repeat_interleave(group, dim=1)
    qs = q_scale.float().reshape(b, h_qo, -1)
    rows = torch.arange(qo_len)
    qsr = qs[:, :, rows // BM]                                                 # [b,h,qo_len]
    m_i = torch.full((b, h_qo, qo_len), float("-inf"))                         # :79
    l_i = torch.ones((b, h_qo, qo_len))                                        # :80
    ql = q.long()
    for j in range(nb):                                                        # :33
        dot = torch.matmul(ql, kp[:, :, j * BN:(j + 1) * BN].transpose(2, 3))  # exact in int64
        qk = dot.float() * qsr[..., None] * ks[:, :, j, None, None]            # :39
        m_ij = torch.maximum(m_i, qk.max(-1).values)                           # :40
        p = torch.exp2(qk - m_ij[..., None])                                   # :41-42
        l_i = l_i * torch.exp2(m_i - m_ij) + p.sum(-1)                         # :45-46
        m_i = m_ij                                                             # :48
    return torch.log2(l_i) + m_i                                               # :107-108
