"""GPU parity of the group attention (one token list per kv head, shared by its q heads) and of
the list union against the oracle's masked attention (twilight/pyimpl/attention.py:188-190,
299-306 with K / V repeated per q head as at attention.py:124-126)."""
import math

import numpy as np
import pytest
import torch

from oracle import pyimpl_port as P
from twilight_amd.cache import PagedKVCache
import twilight_amd.kernel as K

pytestmark = pytest.mark.gpu


def _ragged(cache, lens):
    """Cut the requests of a uniformly paged cache down to ``lens`` tokens."""
    ptr = cache.kv_page_indptr.tolist()
    ind = cache.kv_page_indices.cpu()
    per, last = [], []
    for b, n in enumerate(lens):
        npg = (n + 15) // 16
        per.append(ind[ptr[b]:ptr[b] + npg])
        last.append(n - (npg - 1) * 16 if n else 0)
    indptr = torch.tensor([0] + np.cumsum([len(x) for x in per]).tolist(), dtype=torch.int32)
    cache.set_page_table(torch.cat(per) if per else ind[:0], indptr,
                         torch.tensor(last, dtype=torch.int32))


def _tol(dt):
    # the output is rounded to the q dtype: half an ulp of fp16 (2^-11) / bf16 (2^-8) relative
    return 1e-3 if dt == torch.float16 else 8e-3


@pytest.mark.parametrize("dt,H,Hkv,lens", [
    (torch.float16, 8, 2, [1500, 17, 640]),        # G = 4, two heads per workgroup
    (torch.bfloat16, 8, 8, [333, 1]),              # G = 1, eight heads per workgroup
    (torch.float16, 16, 2, [100, 2049]),           # G = 8
    (torch.bfloat16, 6, 3, [700, 64, 65]),         # G = 2, a head count that is not a power of 2
    (torch.float16, 32, 32, [130, 47]),            # MHA: sixteen heads per workgroup, two blocks
    (torch.bfloat16, 32, 8, [5000])])              # Llama-3 grouping, 79 chunks of 64
def test_dense_decode_vs_reference(dev, dt, H, Hkv, lens):
    B, N = len(lens), max(lens)
    g = torch.Generator().manual_seed(N + H)
    q = torch.randn((B, H, 1, 128), generator=g).to(dt)
    k = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    v = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(B * npg, generator=g))
    _ragged(cache, lens)
    out, lse = K.group_paged_decode_attention(
        q[:, :, 0].contiguous().to(dev), cache.k_cache, cache.v_cache, cache.kv_page_indices,
        cache.kv_page_indptr, cache.kv_last_page_len, max_tokens=N, return_lse=True)
    mask = torch.zeros((B, H, 1, N), dtype=torch.bool)
    for b, n in enumerate(lens):
        mask[b, :, :, :n] = True
    krep = k.float().repeat_interleave(H // Hkv, dim=1)
    vrep = v.float().repeat_interleave(H // Hkv, dim=1)
    ref = P.masked_attention(q.float(), krep, vrep, mask)[:, :, 0]
    assert torch.allclose(out.cpu().float(), ref, rtol=_tol(dt), atol=_tol(dt))
    w = torch.matmul(q.float(), krep.transpose(2, 3)) / math.sqrt(128)
    ref_lse = torch.logsumexp(w.masked_fill(~mask, float("-inf")), dim=-1)[:, :, 0]
    assert torch.allclose(lse.cpu(), ref_lse, rtol=1e-5, atol=1e-5)


def test_dense_decode_empty_request_and_spiky_rows(dev):
    # a request without pages gives zeros and lse = -inf; logits of very different magnitude
    # (one token far above the rest, placed last so every running maximum is replaced) survive
    # the rescaling
    B, H, Hkv, N = 2, 4, 1, 300
    g = torch.Generator().manual_seed(3)
    q = torch.randn((B, H, 1, 128), generator=g).half()
    k = torch.randn((B, Hkv, N, 128), generator=g).half()
    v = torch.randn((B, Hkv, N, 128), generator=g).half()
    k[0, 0, N - 1] = (q[0, 0, 0].float() * 4).half()
    cache = PagedKVCache.from_dense(k, v, dev)
    _ragged(cache, [N, 0])
    out, lse = K.group_paged_decode_attention(
        q[:, :, 0].contiguous().to(dev), cache.k_cache, cache.v_cache, cache.kv_page_indices,
        cache.kv_page_indptr, cache.kv_last_page_len, max_tokens=N, return_lse=True)
    assert torch.all(out[1] == 0) and torch.all(torch.isinf(lse[1])) and torch.all(lse[1] < 0)
    mask = torch.ones((1, H, 1, N), dtype=torch.bool)
    ref = P.masked_attention(q[:1].float(), k[:1].float().repeat_interleave(H, 1),
                             v[:1].float().repeat_interleave(H, 1), mask)[:, :, 0]
    assert torch.allclose(out[:1].cpu().float(), ref, rtol=1e-3, atol=1e-3)
    assert torch.allclose(out[0, 0].cpu().float(), v[0, 0, N - 1].float(), atol=2e-3)  # one-hot row


@pytest.mark.parametrize("dt,H,Hkv", [(torch.float16, 8, 2), (torch.bfloat16, 4, 4),
                                      (torch.float16, 16, 2)])
def test_union_lists_and_group_attention_vs_reference(dev, dt, H, Hkv):
    B, N, G = 2, 1100, H // Hkv
    g = torch.Generator().manual_seed(H)
    q = torch.randn((B, H, 1, 128), generator=g).to(dt)
    k = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    v = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    mask = torch.rand((B, H, 1, N), generator=g) < 0.1
    mask[0, :G] = False                                   # an empty group
    mask[1, 0] = True                                     # one head keeps everything
    mask[1, G:2 * G] = False; mask[1, G, 0, N - 1] = True  # a group of one token, the last one
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(B * npg, generator=g))
    idx, count = P.mask_to_lists(mask)
    idx_t = torch.from_numpy(np.maximum(idx, 0)).reshape(B, H, N).to(dev)
    cnt_t = torch.from_numpy(count).reshape(B, H).to(dev)
    gidx, gcnt = K.group_union_lists(idx_t, cnt_t, Hkv, N)
    union = mask.reshape(B, Hkv, G, 1, N).any(2)          # [B,Hkv,1,N]
    uidx, ucount = P.mask_to_lists(union)
    assert np.array_equal(gcnt.cpu().numpy().reshape(-1), ucount)
    got_idx = gidx.cpu().numpy().reshape(B * Hkv, -1)
    for r in range(B * Hkv):
        assert np.array_equal(got_idx[r, :ucount[r]], uidx[r, :ucount[r]])
    out, lse = K.group_paged_decode_attention(
        q[:, :, 0].contiguous().to(dev), cache.k_cache, cache.v_cache, cache.kv_page_indices,
        cache.kv_page_indptr, group_idx=gidx, group_count=gcnt, return_lse=True)
    umask = union.repeat_interleave(G, dim=1)
    krep = k.float().repeat_interleave(G, dim=1)
    vrep = v.float().repeat_interleave(G, dim=1)
    ref = P.masked_attention(q.float(), krep, vrep, umask)[:, :, 0]
    got = out.cpu().float()
    assert torch.all(got[0, :G] == 0)
    rows = torch.ones(B, H, dtype=torch.bool); rows[0, :G] = False
    assert torch.allclose(got[rows], ref[rows], rtol=_tol(dt), atol=_tol(dt))
    w = torch.matmul(q.float(), krep.transpose(2, 3)) / math.sqrt(128)
    ref_lse = torch.logsumexp(w.masked_fill(~umask, float("-inf")), dim=-1)[:, :, 0]
    assert torch.allclose(lse.cpu()[rows], ref_lse[rows], rtol=1e-5, atol=1e-5)
    # a stride shorter than the union cuts it to its first positions
    cut_idx, cut_cnt = K.group_union_lists(idx_t, cnt_t, Hkv, N, group_stride=40)
    assert np.array_equal(cut_cnt.cpu().numpy().reshape(-1), np.minimum(ucount, 40))
    r = B * Hkv - 1
    assert np.array_equal(cut_idx.cpu().numpy().reshape(B * Hkv, -1)[r, :min(ucount[r], 40)],
                          uidx[r, :min(ucount[r], 40)])


def test_dense_decode_full_size_equals_the_per_head_kernel(dev):
    # Llama-3 shape at full context: the group kernel over every token against the per-head
    # kernel over full lists (an independent code path), and linearity in V
    B, H, Hkv, N = 2, 32, 8, 32768
    g = torch.Generator(device=dev).manual_seed(5)
    q = torch.randn((B, H, 128), generator=g, device=dev, dtype=torch.bfloat16)
    k = torch.randn((B, Hkv, N, 128), generator=g, device=dev, dtype=torch.bfloat16)
    v = torch.randn((B, Hkv, N, 128), generator=g, device=dev, dtype=torch.bfloat16)
    cache = PagedKVCache.from_dense(k, v, dev)
    out, lse = K.group_paged_decode_attention(q, cache.k_cache, cache.v_cache, cache.kv_page_indices,
                                              cache.kv_page_indptr, cache.kv_last_page_len,
                                              max_tokens=N, return_lse=True)
    idx = torch.arange(N, dtype=torch.int32, device=dev).expand(B, H, N).contiguous()
    cnt = torch.full((B, H), N, dtype=torch.int32, device=dev)
    ref, ref_lse = K.sparse_paged_decode_attention(q, cache.k_cache, cache.v_cache, idx, cnt,
                                                   cache.kv_page_indices, cache.kv_page_indptr,
                                                   return_lse=True)
    assert torch.allclose(lse, ref_lse, rtol=1e-5, atol=1e-5)
    # outputs are means of 32768 N(0,1) values (|out| ~ 1e-2): compare on that scale
    assert float((out.float() - ref.float()).abs().max()) < 2e-4
    dense = torch.nn.functional.scaled_dot_product_attention(
        q[:, :, None].float(), k.float().repeat_interleave(4, 1), v.float().repeat_interleave(4, 1))
    assert float((out.float() - dense[:, :, 0]).abs().max()) < 2e-4


def test_group_attention_rejects_bad_arguments(dev):
    k = torch.zeros((1, 2, 32, 128), dtype=torch.float16)
    cache = PagedKVCache.from_dense(k, k, dev)
    q = torch.zeros((1, 6, 128), dtype=torch.float16, device=dev)       # 6 / 2 = 3 heads per group
    with pytest.raises(RuntimeError):
        K.group_paged_decode_attention(q, cache.k_cache, cache.v_cache, cache.kv_page_indices,
                                       cache.kv_page_indptr, cache.kv_last_page_len, max_tokens=32)
    q = torch.zeros((1, 4, 128), dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError):                                    # dense form without lengths
        K.group_paged_decode_attention(q, cache.k_cache, cache.v_cache, cache.kv_page_indices,
                                       cache.kv_page_indptr)
    with pytest.raises(RuntimeError):                                    # list without counts
        K.group_paged_decode_attention(q, cache.k_cache, cache.v_cache, cache.kv_page_indices,
                                       cache.kv_page_indptr,
                                       group_idx=torch.zeros((1, 2, 8), dtype=torch.int32, device=dev))
    idx = torch.zeros((1, 4, 8), dtype=torch.int32, device=dev)
    cnt = torch.zeros((1, 4), dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):                                    # bitmap limit
        K.group_union_lists(idx, cnt, 2, 1 << 20)


@pytest.mark.parametrize("seed", range(8))
def test_group_attention_random_shapes(dev, seed):
    # random batch, grouping, dtype and request lengths around the chunk and page boundaries,
    # dense form and list form (random per-group subsets) against the masked reference
    rng = np.random.default_rng(100 + seed)
    dt = [torch.float16, torch.bfloat16][seed % 2]
    G = int(rng.choice([1, 2, 4, 8]))
    Hkv = int(rng.choice([1, 2, 3, 4, 8]))
    H = G * Hkv
    B = int(rng.integers(1, 5))
    edges = [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 513, 1000, 2047]
    lens = [int(rng.choice(edges)) for _ in range(B)]
    N = max(lens)
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, 1, 128), generator=g).to(dt)
    k = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    v = torch.randn((B, Hkv, N, 128), generator=g).to(dt)
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(B * npg, generator=g))
    _ragged(cache, lens)
    qd = q[:, :, 0].contiguous().to(dev)
    krep, vrep = k.float().repeat_interleave(G, dim=1), v.float().repeat_interleave(G, dim=1)
    dense_mask = torch.zeros((B, H, 1, N), dtype=torch.bool)
    for b, n in enumerate(lens):
        dense_mask[b, :, :, :n] = True
    out = K.group_paged_decode_attention(qd, cache.k_cache, cache.v_cache, cache.kv_page_indices,
                                         cache.kv_page_indptr, cache.kv_last_page_len, max_tokens=N)
    ref = P.masked_attention(q.float(), krep, vrep, dense_mask)[:, :, 0]
    assert torch.allclose(out.cpu().float(), ref, rtol=_tol(dt), atol=_tol(dt)), (lens, H, Hkv)
    # list form: a random subset of each request's tokens per kv head (some empty)
    gmask = (torch.rand((B, Hkv, 1, N), generator=g) < float(rng.uniform(0.05, 0.9))) & dense_mask[:, ::G]
    gmask[0, 0] = False
    gidx, gcount = P.mask_to_lists(gmask)
    out2 = K.group_paged_decode_attention(
        qd, cache.k_cache, cache.v_cache, cache.kv_page_indices, cache.kv_page_indptr,
        group_idx=torch.from_numpy(np.maximum(gidx, 0)).reshape(B, Hkv, N).to(dev),
        group_count=torch.from_numpy(gcount).reshape(B, Hkv).to(dev))
    umask = gmask.repeat_interleave(G, dim=1)
    ref2 = P.masked_attention(q.float(), krep, vrep, umask)[:, :, 0]
    rows = umask.any(-1)[:, :, 0]
    got2 = out2.cpu().float()
    assert torch.all(got2[~rows] == 0)
    assert torch.allclose(got2[rows], ref2[rows], rtol=_tol(dt), atol=_tol(dt)), (lens, H, Hkv)
