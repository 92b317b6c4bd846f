"""Double-Sparse label ops with the names and signatures of twilight/kernel/triton/__init__.py:3-4."""
from __future__ import annotations

import torch

from .. import _lib
from ._check import check_cuda, check_dim, check_dtype, check_same_device, ptr, stream_of


def get_label_tensor(X: torch.Tensor, channel: torch.Tensor, Out: torch.Tensor,
                     HEAVY_CHANNEL_NUM: int) -> None:
    """``Out[l,h,c] = X[l,h,channel[h,c]]`` for c < HEAVY_CHANNEL_NUM
    (twilight/kernel/triton/channel.py:56-79). ``X`` [L,H,D] and ``Out`` [L,H,r] of one 2- or
    4-byte dtype, any strides; ``channel`` int64 [H, >= r]."""
    for name, t in (("X", X), ("channel", channel), ("Out", Out)):
        check_cuda(t, name)
    check_dim(3, X, "X"); check_dim(3, Out, "Out"); check_dim(2, channel, "channel")
    check_dtype(channel, torch.int64, "channel")
    if X.dtype != Out.dtype or X.element_size() not in (2, 4):
        raise RuntimeError("X and Out must share a 2- or 4-byte dtype")
    L, H, _ = X.shape
    r = int(HEAVY_CHANNEL_NUM)
    if tuple(Out.shape) != (L, H, r) or channel.size(0) != H or channel.size(1) < r or r <= 0:
        raise RuntimeError("shapes must be X [L,H,D], channel [H,>=r], Out [L,H,r]")
    check_same_device(X, ("channel", channel), ("Out", Out))
    if L == 0:
        return
    with torch.cuda.device(X.device):
        rc = _lib.lib().twl_get_label_tensor(ptr(X), ptr(channel), ptr(Out), X.element_size(), L, H,
                                             r, *X.stride(), *channel.stride(), *Out.stride(),
                                             stream_of(X))
    _lib.check(rc, "GetLabelTensor")


def bgemv_int8(Q_Label: torch.Tensor, K_Label: torch.Tensor, K_Scales: torch.Tensor,
               Out: torch.Tensor) -> torch.Tensor:
    """``Out[b,h,n] = (sum_c Q_Label[b,h,c] * K_Label[b*N+n,h,c]) * K_Scales[b*N+n,h]``
    (twilight/kernel/triton/bgemv_int8.py:53-75). ``Q_Label`` fp16 [B,H,r], ``K_Label`` int8
    [B*N,H,r], ``K_Scales`` fp16 [B*N,H], ``Out`` fp16 [B,H,N]; products are accumulated in fp32."""
    for name, t in (("Q_Label", Q_Label), ("K_Label", K_Label), ("K_Scales", K_Scales), ("Out", Out)):
        check_cuda(t, name)
    check_dim(3, Q_Label, "Q_Label"); check_dim(3, K_Label, "K_Label")
    check_dim(2, K_Scales, "K_Scales"); check_dim(3, Out, "Out")
    check_dtype(Q_Label, torch.float16, "Q_Label"); check_dtype(K_Label, torch.int8, "K_Label")
    check_dtype(K_Scales, torch.float16, "K_Scales"); check_dtype(Out, torch.float16, "Out")
    B, H, r = Q_Label.shape
    if B == 0 or K_Label.size(0) % B != 0:
        raise RuntimeError("K_Label must be [B*N_CTX, H, r]")
    N = K_Label.size(0) // B
    if K_Label.size(1) != H or K_Label.size(2) != r or tuple(K_Scales.shape) != (B * N, H) \
            or tuple(Out.shape) != (B, H, N):
        raise RuntimeError("shapes must be Q [B,H,r], K [B*N,H,r], scales [B*N,H], Out [B,H,N]")
    check_same_device(Q_Label, ("K_Label", K_Label), ("K_Scales", K_Scales), ("Out", Out))
    if N == 0:
        return Out
    with torch.cuda.device(Q_Label.device):
        rc = _lib.lib().twl_bgemv_int8(ptr(Q_Label), ptr(K_Label), ptr(K_Scales), ptr(Out), B, H, r,
                                       N, *Q_Label.stride(), *K_Label.stride(), *K_Scales.stride(),
                                       *Out.stride(), stream_of(Q_Label))
    _lib.check(rc, "BgemvInt8")
    return Out


def qk_int8_per_block(q: torch.Tensor, k: torch.Tensor, q_scale: torch.Tensor, k_scale: torch.Tensor,
                      tensor_layout: str = "HND", output_dtype: torch.dtype = torch.float16,
                      return_lse: bool = False):
    """Same call as twilight/kernel/triton/qk_int8_per_block.py:111-143: ``q`` / ``k`` int8
    [b,h,n,d] ("HND") or [b,n,h,d] ("NHD") quantised per 128 query rows / 64 key rows with fp32
    ``q_scale`` [b,h_qo,ceil(qo_len/128)] and ``k_scale`` [b,h_kv,ceil(kv_len/64)]. Returns
    ``(o, lse)``: ``o`` is the reference's first output, all zeros of ``q``'s shape (it never
    accumulates V, :30-49,101-102); ``lse`` fp32 [b,h_qo,qo_len] is the base-2 log-sum-exp of the
    scaled scores, or an empty CPU tensor when ``return_lse`` is False (:127-130)."""
    for name, t in (("q", q), ("k", k), ("q_scale", q_scale), ("k_scale", k_scale)):
        check_cuda(t, name)
    check_dim(4, q, "q"); check_dim(4, k, "k")
    check_dtype(q, torch.int8, "q"); check_dtype(k, torch.int8, "k")
    if tensor_layout == "HND":
        b, h_qo, qo_len, d = q.shape
        _, h_kv, kv_len, _ = k.shape
        sq, sk = (q.stride(0), q.stride(1), q.stride(2)), (k.stride(0), k.stride(1), k.stride(2))
    elif tensor_layout == "NHD":
        b, qo_len, h_qo, d = q.shape
        _, kv_len, h_kv, _ = k.shape
        sq, sk = (q.stride(0), q.stride(2), q.stride(1)), (k.stride(0), k.stride(2), k.stride(1))
    else:
        raise ValueError(f"tensor_layout {tensor_layout} not supported")
    if k.size(0) != b or k.size(3) != d or q.stride(3) != 1 or k.stride(3) != 1:
        raise RuntimeError("q and k must share batch and head_dim, with contiguous head_dim")
    if d not in (64, 128) or h_kv == 0 or h_qo % h_kv != 0:
        raise RuntimeError("head_dim must be 64 or 128 and h_qo a multiple of h_kv")
    o = torch.zeros(q.shape, dtype=output_dtype, device=q.device)
    if not return_lse:
        return o, torch.empty([0], dtype=torch.float32, device="cpu")
    mb, nb = (qo_len + 127) // 128, (kv_len + 63) // 64
    qs = q_scale.to(torch.float32).contiguous()
    ks = k_scale.to(torch.float32).contiguous()
    if qs.numel() != b * h_qo * mb or ks.numel() != b * h_kv * nb:
        raise RuntimeError("q_scale must have b*h_qo*ceil(qo_len/128) and k_scale "
                           "b*h_kv*ceil(kv_len/64) elements")
    check_same_device(q, ("k", k), ("q_scale", q_scale), ("k_scale", k_scale))
    with torch.cuda.device(q.device):
        lse = torch.empty([b, h_qo, qo_len], dtype=torch.float32, device=q.device)
        if qo_len and kv_len:
            rc = _lib.lib().twl_qk_int8_lse(ptr(q), ptr(k), ptr(qs), ptr(ks), ptr(lse), b, h_qo,
                                            h_kv, qo_len, kv_len, d, *sq, *sk, stream_of(q))
            _lib.check(rc, "QkInt8PerBlock")
    return o, lse
