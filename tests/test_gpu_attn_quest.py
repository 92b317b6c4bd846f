"""GPU parity of the Quest selector and the sparse paged decode attention against the oracle's
restatement of twilight/pyimpl/quest.py:17-122 and twilight/pyimpl/attention.py:188-190,299-306."""
import math

import numpy as np
import pytest
import torch

from oracle import pyimpl_port as P
from twilight_amd import synth
from twilight_amd.cache import PagedKVCache
import twilight_amd.kernel as K

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt,N,budget,H,Hkv", [
    (torch.float16, 1000, 256, 4, 2), (torch.float16, 4096, 1000, 4, 4),
    (torch.bfloat16, 777, 64, 8, 2), (torch.float16, 40, 4096, 4, 2),
    (torch.float16, 600, 100, 8, 1), (torch.bfloat16, 333, 48, 6, 2)])
def test_quest_select_vs_dense_reference(dev, dt, N, budget, H, Hkv):
    B = 2
    g = torch.Generator().manual_seed(N)
    q = torch.randn((B, H, 1, 128), generator=g).to(dt)
    k = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    v = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(B * npg, generator=g))
    sel, cnt, scores = K.quest_select(q[:, :, 0].contiguous().to(dev), cache.meta,
                                      cache.kv_page_indices, cache.kv_page_indptr, budget, npg)
    krep = k.float().repeat_interleave(H // Hkv, dim=1)                    # attention.py:124-126
    est = P.quest_chunk_scores_dense(q.float(), krep, 16)[:, :, 0]         # [B,H,chunks]
    got_scores = scores.cpu()
    assert torch.allclose(got_scores, est, rtol=1e-4, atol=1e-3)
    kc = P.quest_chunk_budget(budget, 16, npg)
    assert cnt.cpu().unique().tolist() == [kc] and sel.shape[-1] == kc
    s = sel.cpu().long()
    for b in range(B):
        for h in range(H):
            mine = s[b, h]
            assert torch.all(mine[1:] > mine[:-1])                         # ascending, distinct
            # the selection is exactly the top-k of the scores the kernel itself produced
            # (ties to the lower page), and it agrees with the fp32 reference scores except
            # for pages within rounding of the k-th score
            order = torch.sort(got_scores[b, h].double(), descending=True, stable=True).indices[:kc]
            assert set(order.tolist()) == set(mine.tolist())
            ref = set(torch.sort(est[b, h].double(), descending=True, stable=True).indices[:kc].tolist())
            kth = torch.sort(est[b, h], descending=True).values[kc - 1]
            for pg in ref.symmetric_difference(set(mine.tolist())):
                assert abs(float(est[b, h, pg]) - float(kth)) <= 1e-3 * max(1.0, abs(float(kth)))


def test_quest_ties_go_to_the_lower_page(dev):
    # identical pages -> identical scores: the first k pages are selected
    k = torch.ones((1, 1, 160, 128), dtype=torch.float16)
    cache = PagedKVCache.from_dense(k, k, dev)
    q = torch.ones((1, 1, 128), dtype=torch.float16, device=dev)
    sel, cnt, _ = K.quest_select(q, cache.meta, cache.kv_page_indices, cache.kv_page_indptr, 48, 10)
    assert sel.cpu().reshape(-1).tolist() == [0, 1, 2] and int(cnt) == 3


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_sparse_attention_vs_masked_reference(dev, dt):
    B, H, Hkv, N = 2, 8, 2, 1500
    g = torch.Generator().manual_seed(4)
    q = torch.randn((B, H, 1, 128), generator=g).to(dt)
    k = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    v = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    mask = torch.rand((B, H, 1, N), generator=g) < 0.08
    mask[0, 0] = False; mask[0, 0, 0, 5] = True           # a single survivor
    mask[0, 1] = False                                    # no survivor -> zeros
    mask[0, 2] = True                                     # everything survives
    mask[1, 7, 0, N - 1] = True                           # last token of a partial page
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(B * npg, generator=g))
    idx, count = P.mask_to_lists(mask)
    idx_t = torch.from_numpy(np.maximum(idx, 0)).reshape(B, H, N).to(dev)
    cnt_t = torch.from_numpy(count).reshape(B, H).to(dev)
    out, lse = K.sparse_paged_decode_attention(q[:, :, 0].contiguous().to(dev), cache.k_cache,
                                               cache.v_cache, idx_t, cnt_t, cache.kv_page_indices,
                                               cache.kv_page_indptr, return_lse=True)
    krep = k.float().repeat_interleave(H // Hkv, dim=1)
    vrep = v.float().repeat_interleave(H // Hkv, dim=1)
    ref = P.masked_attention(q.float(), krep, vrep, mask, prob_dtype=dt)[:, :, 0]
    got = out.cpu().float()
    assert torch.all(got[0, 1] == 0)
    rows = torch.ones(B, H, dtype=torch.bool); rows[0, 1] = False
    # output is rounded to the q dtype: half an ulp of fp16 (2^-11) / bf16 (2^-8) relative
    tol = 1e-3 if dt == torch.float16 else 8e-3
    assert torch.allclose(got[rows], ref[rows], rtol=tol, atol=tol)
    w = torch.matmul(q.float(), krep.transpose(2, 3)) / math.sqrt(128)
    ref_lse = torch.logsumexp(w.masked_fill(~mask, float("-inf")), dim=-1)[:, :, 0]
    assert torch.allclose(lse.cpu()[rows], ref_lse[rows], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_weighted_attention_vs_closed_form(dev, dt):
    """Given weights in place of q.K logits (attention.py:295-296): out = sum w V / sum w over
    the listed tokens, for rows of one survivor, a few, exactly 128, and thousands (split rows)."""
    B, H, Hkv, N = 2, 8, 2, 3000
    g = torch.Generator().manual_seed(14)
    k = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    v = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(B * npg, generator=g))
    counts = [1, 0, 7, 128, 129, 1000, N, 300, 64, 2, 2999, 257, 5, 90, 511, 12]
    idx = torch.zeros((B, H, N), dtype=torch.int32)
    w = torch.rand((B, H, N), generator=g) ** 4 + 1e-6
    for r, n in enumerate(counts):
        idx[r // H, r % H, :n] = torch.sort(torch.randperm(N, generator=g)[:n]).values.int()
    cnt = torch.tensor(counts, dtype=torch.int32).reshape(B, H)
    out, lse = K.weighted_paged_decode_attention(w.to(dev), cache.v_cache, idx.to(dev), cnt.to(dev),
                                                 cache.kv_page_indices, cache.kv_page_indptr,
                                                 return_lse=True)
    got = out.cpu().double()
    vrep = v.double().repeat_interleave(H // Hkv, dim=1)
    tol = 1e-3 if dt == torch.float16 else 8e-3
    for r, n in enumerate(counts):
        b, h = r // H, r % H
        if n == 0:
            assert torch.all(got[b, h] == 0)
            continue
        ww = w[b, h, :n].double()
        pr = ww / ww.sum()
        if n <= 128:
            pr = pr.float().to(dt).double()                                # attention.py:302-304
        ref = pr @ vrep[b, h, idx[b, h, :n].long()]
        assert torch.allclose(got[b, h], ref, rtol=tol, atol=tol), (r, n)
        assert abs(float(lse[b, h]) - math.log(float(ww.sum()))) < 1e-4
    # the same lists a second time on the same workspace words
    out2 = K.weighted_paged_decode_attention(w.to(dev), cache.v_cache, idx.to(dev), cnt.to(dev),
                                             cache.kv_page_indices, cache.kv_page_indptr)
    assert torch.allclose(out2.float(), out.float(), rtol=tol, atol=tol)


def test_sparse_attention_hnd_layout_view(dev):
    # the same kernel over an HND-stored cache ([pages, Hkv, 16, 128] viewed as [pages,16,Hkv,128])
    g = torch.Generator().manual_seed(6)
    B, H, N = 1, 2, 320
    q = torch.randn((B, H, 128), generator=g).half().to(dev)
    k = torch.randn((B, H, N, 128), generator=g).half()
    v = torch.randn((B, H, N, 128), generator=g).half()
    cache = PagedKVCache.from_dense(k, v, dev)
    k_hnd = cache.k_cache.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    v_hnd = cache.v_cache.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    idx = torch.arange(0, N, 3, dtype=torch.int32).repeat(B, H, 1).to(dev)
    cnt = torch.full((B, H), idx.shape[-1], dtype=torch.int32, device=dev)
    a = K.sparse_paged_decode_attention(q, cache.k_cache, cache.v_cache, idx, cnt,
                                        cache.kv_page_indices, cache.kv_page_indptr)
    b = K.sparse_paged_decode_attention(q, k_hnd, v_hnd, idx, cnt, cache.kv_page_indices,
                                        cache.kv_page_indptr)
    assert torch.equal(a, b)


def test_sparse_attention_split_rows_share_a_workspace(dev):
    # rows of 1..3000 survivors (1 to 24 chunks of 128), two calls in a row on one workspace:
    # the ticket counters must come back to zero and both results must match the reference
    B, H, N = 1, 8, 3000
    g = torch.Generator().manual_seed(8)
    q = torch.randn((B, H, 1, 128), generator=g).half()
    k = torch.randn((B, H, N, 128), generator=g).half()
    v = torch.randn((B, H, N, 128), generator=g).half()
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(188, generator=g))
    ws = torch.zeros(K.attention_workspace_bytes(B * H, N), dtype=torch.uint8, device=dev)
    for trial, lens in enumerate(([1, 127, 128, 129, 256, 257, 1000, 3000], [3000, 5, 640, 128, 2, 1999, 384, 129])):
        mask = torch.zeros((B, H, 1, N), dtype=torch.bool)
        for h, n in enumerate(lens):
            mask[0, h, 0, torch.randperm(N, generator=g)[:n]] = True
        idx, count = P.mask_to_lists(mask)
        out = K.sparse_paged_decode_attention(
            q[:, :, 0].contiguous().to(dev), cache.k_cache, cache.v_cache,
            torch.from_numpy(np.maximum(idx, 0)).reshape(B, H, N).to(dev),
            torch.from_numpy(count).reshape(B, H).to(dev), cache.kv_page_indices,
            cache.kv_page_indptr, workspace=ws)
        ref = P.masked_attention(q.float(), k.float(), v.float(), mask, prob_dtype=torch.float16)[:, :, 0]
        assert torch.allclose(out.cpu().float(), ref, rtol=1e-3, atol=1e-3), trial
        assert int(ws[:B * H * 8].view(torch.int64).abs().sum()) == 0
    # ticket words that are not zero when the call starts (a call that never finished, memory that
    # was never cleared) carry another call's 48-bit tag or none: they count as zero. Small
    # counts, words shaped like (small tag << 16) | count, all ones, and arbitrary bits.
    ws[:B * H * 8].view(torch.int64).copy_(torch.tensor(
        [2, 0x00070003, 0x7FFF0001, 1, -1, (0x1234 << 16) | 0x17, 0x0123456789ABCDEF, 3 << 32]))
    out = K.sparse_paged_decode_attention(
        q[:, :, 0].contiguous().to(dev), cache.k_cache, cache.v_cache,
        torch.from_numpy(np.maximum(idx, 0)).reshape(B, H, N).to(dev),
        torch.from_numpy(count).reshape(B, H).to(dev), cache.kv_page_indices,
        cache.kv_page_indptr, workspace=ws)
    assert torch.allclose(out.cpu().float(), ref, rtol=1e-3, atol=1e-3)
    split = torch.from_numpy(count).reshape(-1) > 512     # rows that used their ticket for sure
    assert int(ws[:B * H * 8].view(torch.int64)[split].abs().sum()) == 0


def test_attention_folds_positions_outside_the_request(dev):
    # a list entry beyond the request's pages must not be read past the page table: it is folded
    # onto the request's last page (the kernel must finish and give finite numbers)
    g = torch.Generator().manual_seed(21)
    B, H, N = 1, 2, 100
    q = torch.randn((B, H, 128), generator=g).half().to(dev)
    k = torch.randn((B, H, N, 128), generator=g).half()
    cache = PagedKVCache.from_dense(k, k, dev)
    idx = torch.tensor([[[0, 5, 1 << 20, -7], [3, 99, 100000, 0]]], dtype=torch.int32, device=dev)
    cnt = torch.tensor([[4, 3]], dtype=torch.int32, device=dev)
    out = K.sparse_paged_decode_attention(q, cache.k_cache, cache.v_cache, idx, cnt,
                                          cache.kv_page_indices, cache.kv_page_indptr)
    assert torch.isfinite(out).all()
    gi = torch.tensor([[[0, 1 << 22], [5, -3]]], dtype=torch.int32, device=dev)
    gc = torch.tensor([[2, 2]], dtype=torch.int32, device=dev)
    out2 = K.group_paged_decode_attention(q, cache.k_cache, cache.v_cache, cache.kv_page_indices,
                                          cache.kv_page_indptr, group_idx=gi, group_count=gc)
    assert torch.isfinite(out2).all()
