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
                        shuffle_pages: bool = True,
                        survivors: Optional[Tuple[int, int]] = None, top_p: float = 0.95,
                        budget: int = 8192):
    """Decode-layer inputs built on the GPU: q [B,H,128], paged K, V [B*N/16, 16, Hkv, 128]
    ~ N(0,1) in ``dtype``; per (batch, q head) ``heavy_pages`` random pages get ``K += a*q`` on
    3 of their tokens (planted heavy hitters). Returns (q, k_pages, v_pages, page table tuple).

    ``survivors=None`` ("peaked" workload): ``a = alpha`` for every row and the 3 token slots of a
    page are drawn with replacement, so most rows hold a token planted twice that takes nearly
    all of the softmax mass (a top-p of 0.95 keeps 2 tokens at the median, thousands in the few
    rows without such a token).

    ``survivors=(lo, hi)`` ("calibrated" workload): the slots are distinct and ``a`` is solved per
    row, by bisection on the row's own logits, so that a nucleus of mass ``top_p`` over the row's
    ``budget`` Quest candidates (whole pages by the min/max upper bound, the planted pages among
    them) holds a target number of tokens drawn log-uniformly from [lo, hi]."""
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
    if survivors is not None:
        _plant_calibrated(q, k, ids_d, B, H, Hkv, npg, heavy_pages, gp, survivors, top_p, budget)
        return q, k, v, (ids.to(dev), indptr.to(dev), last.to(dev))
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


def nucleus_size(logits: torch.Tensor, top_p: float) -> torch.Tensor:
    """Size of the smallest set of entries of each row of ``logits`` [R, M] whose softmax mass
    reaches ``top_p`` (sort descending, cumulative sum)."""
    pr = torch.softmax(logits.double(), dim=-1)
    cs = torch.cumsum(torch.sort(pr, dim=-1, descending=True).values, dim=-1)
    return (cs < top_p).sum(-1) + 1


def _plant_calibrated(q, k, ids_d, B, H, Hkv, npg, heavy_pages, gp, survivors, top_p, budget):
    """Plants 3 distinct tokens in each of ``heavy_pages`` pages per (batch, q head) with
    ``K += a*q``, ``a`` solved per row for a target nucleus size (see layer_inputs_device)."""
    dev, dtype, D = q.device, q.dtype, HEAD_DIM
    group = H // Hkv
    kpages = min(npg, max(1, budget // PAGE) + (1 if budget % PAGE else 0))
    lo_t, hi_t = survivors
    hrow = torch.arange(H, device=dev)
    kvh_of = hrow // group
    for b in range(B):
        phys_b = ids_d[b * npg:(b + 1) * npg]
        kk = k[phys_b].float()                                       # [npg, 16, Hkv, D]
        qf = q[b].float()                                            # [H, D]
        logits = torch.einsum("pthd,hgd->hgpt", kk, qf.view(Hkv, group, D)).reshape(H, npg, PAGE)
        logits /= math.sqrt(D)
        pmax = kk.amax(1).permute(1, 0, 2)[kvh_of]                   # [H, npg, D]
        pmin = kk.amin(1).permute(1, 0, 2)[kvh_of]
        bound = torch.maximum(qf[:, None, :] * pmax, qf[:, None, :] * pmin).sum(-1)   # [H, npg]
        del kk, pmax, pmin
        lps, sls, tgt = [], [], []
        for _ in range(H):
            lps.append(torch.randperm(npg, generator=gp)[:heavy_pages])
            sls.append(torch.stack([torch.randperm(PAGE, generator=gp)[:3]
                                    for _ in range(heavy_pages)]))
            u = float(torch.rand((), generator=gp))
            tgt.append(math.exp(math.log(lo_t) + u * (math.log(hi_t) - math.log(lo_t))))
        lp = torch.stack(lps).to(dev)                                # [H, heavy_pages]
        sl = torch.stack(sls).to(dev)                                # [H, heavy_pages, 3]
        target = torch.tensor(tgt, device=dev)
        heavy = torch.zeros((H, npg, PAGE), dtype=torch.bool, device=dev)
        hi_ = hrow[:, None, None].expand_as(sl)
        heavy[hi_, lp[:, :, None].expand_as(sl), sl] = True
        bound.scatter_(1, lp, float("inf"))                          # planted pages are selected
        sel = torch.topk(bound, kpages, dim=1).indices               # [H, kpages]
        take = sel[:, :, None].expand(-1, -1, PAGE)
        cand = torch.gather(logits, 1, take).reshape(H, -1)
        hm = torch.gather(heavy, 1, take).reshape(H, -1).float()
        qq = (qf * qf).sum(-1) / math.sqrt(D)
        a_lo = torch.zeros(H, device=dev)
        a_hi = torch.full((H,), 4.0, device=dev)
        for _ in range(28):
            a = 0.5 * (a_lo + a_hi)
            n = nucleus_size(cand + (a * qq)[:, None] * hm, top_p)
            more = n.float() > target                                # too many kept: plant harder
            a_lo = torch.where(more, a, a_lo)
            a_hi = torch.where(more, a_hi, a)
        a = 0.5 * (a_lo + a_hi)
        pg = phys_b[lp][:, :, None].expand_as(sl)                    # [H, heavy_pages, 3] physical
        hh = kvh_of[:, None, None].expand_as(sl)
        cur = k[pg, sl, hh].float()                                  # [H, heavy_pages, 3, D]
        k[pg, sl, hh] = (cur + a[:, None, None, None] * qf[:, None, None, :]).to(dtype)
