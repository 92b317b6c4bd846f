"""Seeded synthetic inputs of the shapes the benchmarks and parity tests use.

Everything is drawn from a CPU ``torch.Generator`` (identical on every machine) unless the
function name ends in ``_device`` — those fill multi-GB tensors directly on the GPU for the
benchmark, where only shapes and statistics matter.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from . import _lib

PAGE, HEAD_DIM = _lib.PAGE, _lib.HEAD_DIM


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def heavy_hitter_qkv(B: int, H: int, N: int, n_heavy: int = 16, mass: float = 0.60, seed: int = 0,
                     dtype: torch.dtype = torch.float32) -> Tuple[torch.Tensor, ...]:
    """q [B,H,1,D], K, V [B,H,N,D] ~ N(0,1); ``n_heavy`` random tokens per head get
    ``K += alpha * q`` with alpha solved per head (bisection) so that they carry ``mass`` of the
    exact softmax. Values are rounded to ``dtype`` first, then returned as fp32."""
    D = HEAD_DIM
    g = _gen(seed)
    q = torch.randn((B, H, 1, D), generator=g).to(dtype).float()
    k = torch.randn((B, H, N, D), generator=g).to(dtype).float()
    v = torch.randn((B, H, N, D), generator=g).to(dtype).float()
    gp = _gen(seed + 1)
    for b in range(B):
        for h in range(H):
            pos = torch.randperm(N, generator=gp)[:n_heavy]
            qv = q[b, h, 0]
            base = (k[b, h] @ qv) / math.sqrt(D)
            qq = float(qv @ qv) / math.sqrt(D)
            lo, hi = 0.0, 4.0
            for _ in range(40):
                a = 0.5 * (lo + hi)
                logits = base.clone()
                logits[pos] += a * qq
                pr = torch.softmax(logits.double(), dim=-1)
                if float(pr[pos].sum()) < mass:
                    lo = a
                else:
                    hi = a
            k[b, h, pos] = (k[b, h, pos] + 0.5 * (lo + hi) * qv).to(dtype).float()
    return q, k, v


def topp_scores(B: int, H: int, M: int, seed: int = 0, L0: float = 12.0, zipf_s: float = 1.2,
                max_spikes: int = 512, first_is_max: bool = False) -> torch.Tensor:
    """fp32 [B,H,M] logits: N(0,1) background plus, per row, 1..max_spikes spikes at random
    positions with logit ``L0 - zipf_s * ln(rank)`` (a Zipf(s) probability profile).
    ``first_is_max`` places the largest spike at position 0 (the attention-sink case)."""
    g = _gen(seed)
    x = torch.randn((B, H, M), generator=g)
    gp, gs = _gen(seed + 1), _gen(seed + 2)
    for b in range(B):
        for h in range(H):
            ns = int(torch.randint(1, min(max_spikes, M) + 1, (1,), generator=gs))
            pos = torch.randperm(M, generator=gp)[:ns]
            if first_is_max:
                pos = pos[pos != 0]
                pos = torch.cat([torch.zeros(1, dtype=pos.dtype), pos])[:ns]
            ranks = torch.arange(1, pos.numel() + 1, dtype=torch.float32)
            x[b, h, pos] = L0 - zipf_s * torch.log(ranks)
    return x


def int4_records_random(n_pages: int, n_kv_heads: int, seed: int = 0, device="cpu") -> torch.Tensor:
    """uint8 [n_pages, n_kv_heads, 1280] records: uniform nibbles, scale ~ U(0.01, 0.1) as fp16,
    zero = fp16(-8 * scale) (centres the dequantised values)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    rec = torch.empty((n_pages, n_kv_heads, _lib.INT4_RECORD_BYTES), dtype=torch.uint8, device=dev)
    rec[..., :1024] = torch.randint(0, 256, (n_pages, n_kv_heads, 1024), dtype=torch.uint8,
                                    device=dev, generator=g)
    scale = (torch.rand((n_pages, n_kv_heads, 64), device=dev, generator=g) * 0.09 + 0.01).half()
    zero = (-8.0 * scale.float()).half()
    sz = torch.stack([scale, zero], dim=-1).contiguous()  # [P,H,64,2] fp16
    rec[..., 1024:] = sz.view(torch.uint8).reshape(n_pages, n_kv_heads, 256)
    return rec


def identity_page_table(B: int, pages_per_req: int, last_len: int = PAGE, device="cpu",
                        shuffle_seed: Optional[int] = None):
    """CSR page table of B equal-length requests; physical ids are the identity or a seeded
    permutation. Returns (kv_page_indices, kv_page_indptr, kv_last_page_len) int32."""
    total = B * pages_per_req
    if shuffle_seed is None:
        ids = torch.arange(total, dtype=torch.int32)
    else:
        ids = torch.randperm(total, generator=_gen(shuffle_seed)).to(torch.int32)
    indptr = (torch.arange(B + 1) * pages_per_req).to(torch.int32)
    last = torch.full((B,), last_len, dtype=torch.int32)
    return ids.to(device), indptr.to(device), last.to(device)


def layer_inputs_device(B: int, H: int, Hkv: int, N: int, dtype: torch.dtype, device,
                        seed: int = 0, heavy_pages: int = 8, alpha: float = 0.9,
                        shuffle_pages: bool = True):
    """Decode-layer inputs built on the GPU: q [B,H,128], paged K, V [B*N/16, 16, Hkv, 128]
    ~ N(0,1) in ``dtype``; per (batch, q head) ``heavy_pages`` random pages get ``K += alpha*q`` on
    3 of their tokens (planted heavy hitters). Returns (q, k_pages, v_pages, page table tuple)."""
    assert N % PAGE == 0
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    npg = N // PAGE
    total = B * npg
    q = torch.randn((B, H, HEAD_DIM), device=dev, generator=g).to(dtype)
    k = torch.empty((total, PAGE, Hkv, HEAD_DIM), dtype=dtype, device=dev)
    v = torch.empty_like(k)
    step = max(1, total // 16)
    for s in range(0, total, step):  # chunked so the fp32 temporaries stay small
        e = min(total, s + step)
        k[s:e] = torch.randn((e - s, PAGE, Hkv, HEAD_DIM), device=dev, generator=g).to(dtype)
        v[s:e] = torch.randn((e - s, PAGE, Hkv, HEAD_DIM), device=dev, generator=g).to(dtype)
    ids, indptr, last = identity_page_table(B, npg, PAGE, "cpu", seed + 7 if shuffle_pages else None)
    ids_d = ids.to(dev).long()
    group = H // Hkv
    gp = _gen(seed + 1)
    for b in range(B):
        for h in range(H):
            lp = torch.randperm(npg, generator=gp)[:heavy_pages]
            phys = ids_d[b * npg + lp.to(dev)]
            slots = torch.randint(0, PAGE, (heavy_pages, 3), generator=gp).to(dev)
            kvh = h // group
            for j in range(3):
                cur = k[phys, slots[:, j], kvh].float()
                k[phys, slots[:, j], kvh] = (cur + alpha * q[b, h].float()).to(dtype)
    return q, k, v, (ids.to(dev), indptr.to(dev), last.to(dev))
