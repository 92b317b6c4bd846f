"""GPU parity of the one-launch estimator + pruner (INT4 score GEMV, softmax, top-p, compaction)
against the oracle's restatement of twilight/pyimpl/attention.py:252-255 and
twilight/pyimpl/top_p.py:10-15 (csrc/include/sampling.cuh:156-231), and against the two-launch
sequence of the same library."""
import math

import numpy as np
import pytest
import torch

from oracle import native
from oracle import pyimpl_port as P
from twilight_amd import synth
import twilight_amd.kernel as K
from _checks import assert_scores_close, assert_top_p_parity

pytestmark = pytest.mark.gpu


def _peaky_q(B, H, rec, ids, indptr, seed):
    """q aligned with a few random tokens of each request so that the softmax has heavy hitters."""
    g = torch.Generator().manual_seed(seed)
    codes, scale, zero = P.unpack_int4_records(rec.numpy())
    deq = torch.from_numpy(native.int4_dequant(codes, scale, zero))       # [P,Hkv,16,128]
    Hkv = deq.shape[1]
    q = torch.randn((B, H, 128), generator=g) * 0.5
    for b in range(B):
        npg = int(indptr[b + 1] - indptr[b])
        for h in range(H):
            for _ in range(int(torch.randint(1, 6, (1,), generator=g))):
                pg = int(ids[int(indptr[b]) + int(torch.randint(0, npg, (1,), generator=g))])
                tok = int(torch.randint(0, 16, (1,), generator=g))
                q[b, h] += deq[pg, h // (H // Hkv), tok] * float(torch.rand(1, generator=g) * 12 + 4)
    return q, deq


def _case(dev, B, H, Hkv, npg, S, last_len, p, high, qdt, seed, ragged=True, per_row_p=False):
    rec = synth.int4_records_random(B * npg, Hkv, seed=seed)
    ids, indptr, last = synth.identity_page_table(B, npg, last_len=last_len, shuffle_seed=seed + 1)
    q, deq = _peaky_q(B, H, rec, ids, indptr, seed + 2)
    q = q.to(qdt)
    g = torch.Generator().manual_seed(seed + 3)
    sel = torch.stack([torch.sort(torch.randperm(npg, generator=g)[:S]).values
                       for _ in range(B * H)]).reshape(B, H, S).to(torch.int32)
    if ragged:
        cnt_in = torch.randint(1, S + 1, (B, H), generator=g).to(torch.int32)
        cnt_in[0, 0] = S
        cnt_in[-1, -1] = 1
        if B * H > 2:
            cnt_in[0, 1] = 0                                           # a row without candidates
    else:
        cnt_in = torch.full((B, H), S, dtype=torch.int32)
    rows = B * H
    top_p = (torch.rand(rows, generator=g) * 0.5 + 0.45) if per_row_p else p
    d = lambda t: t.to(dev)
    args = (d(q), d(rec), d(ids), d(indptr), d(last))
    idx, count, cand, scores, low = K.sparse_gemv_int4_top_p(
        *args, d(sel), d(cnt_in), d(top_p) if per_row_p else top_p, high=high,
        sm_scale=1 / math.sqrt(128), return_scores=True, return_low=True)
    M = S * 16
    assert torch.equal(cand.cpu(), cnt_in * 16)
    sc = scores.cpu().numpy().reshape(rows, M)
    ix = idx.cpu().numpy().reshape(rows, M)
    cn = count.cpu().numpy().reshape(rows)
    # 1. scores: oracle GEMV over the dequantised records (1e-3 relative), -inf past last_len
    want = np.full((rows, M), -np.inf)
    qf = q.float()
    for b in range(B):
        for h in range(H):
            r = b * H + h
            n = int(cnt_in[b, h])
            phys = ids[indptr[b] + sel[b, h, :n].long()].long()
            w = (deq[phys, h // (H // Hkv)].reshape(-1, 128).double() @ qf[b, h].double()) / math.sqrt(128)
            w = w.numpy()
            tok = (sel[b, h, :n, None].long() * 16 + torch.arange(16)[None]).reshape(-1).numpy()
            w[tok >= (npg - 1) * 16 + last_len] = -np.inf
            want[r, :n * 16] = w
    assert_scores_close(sc, want)
    # 2. the pruned lists against the oracle run on the GPU's own scores
    x = torch.from_numpy(sc).masked_fill(torch.from_numpy(np.isinf(sc)), torch.finfo(torch.float32).min)
    hm = native.HIGH_MAX if high == "max" else native.HIGH_FIRST
    if high == "first":
        # The reference's bound is the probability of TOKEN 0 of the context on a full-length row
        # (csrc/include/sampling.cuh:156-159 after attention.py:255,274-278): when logical page 0
        # is not the list's first page the oracle sees an extra leading entry of probability 0
        # (dropped again below), otherwise the candidate row as it is.
        lead = torch.full((rows, 1), torch.finfo(torch.float32).min)
        no0 = (sel.reshape(rows, S)[:, 0] != 0) | (cnt_in.reshape(rows) == 0)
        xs = [torch.cat([lead[r], x[r]]) if no0[r] else torch.cat([x[r], lead[r]]) for r in range(rows)]
        x = torch.stack(xs)
    p_np = top_p.numpy().astype(np.float32) if per_row_p else p
    live = np.nonzero(cnt_in.reshape(-1).numpy() > 0)[0]
    Mx = x.shape[1]
    om, oprobs, ol, _ = P.top_p_unnormalized(x.reshape(rows, 1, 1, Mx)[live], p_np[live] if per_row_p else p_np, hm)
    pn = oprobs.reshape(len(live), Mx).numpy()
    _, _, _, og = native.top_p_mask_f32(pn, p_np[live] if per_row_p else p_np, hm, return_margin=True)
    om = om.reshape(len(live), Mx)
    if high == "first":
        # back to candidate positions (the padding entry has probability 0 and is never kept)
        keep = [slice(1, Mx) if no0[r] else slice(0, M) for r in live]
        assert not any(bool(om[i, 0]) for i, r in enumerate(live) if no0[r])
        pn = np.stack([pn[i, k] for i, k in enumerate(keep)])
        om = torch.stack([om[i, k] for i, k in enumerate(keep)])
    selr = sel.reshape(rows, S).numpy()
    gm = np.zeros((rows, M), dtype=bool)
    for r in range(rows):
        toks = ix[r, :cn[r]]
        assert np.all(np.diff(toks) > 0)
        pos = np.searchsorted(selr[r], toks // 16) * 16 + toks % 16
        assert np.array_equal(selr[r][pos // 16] * 16 + pos % 16, toks)
        gm[r, pos] = True
    for r in range(rows):
        if r not in live:
            assert cn[r] == 0
    n_exact = assert_top_p_parity(pn, p_np[live] if per_row_p else p_np, gm[live],
                                  om.reshape(len(live), M).numpy(), ol, og, margin_tol=5e-6)
    assert n_exact >= 0.9 * len(live)
    # 3. the two-launch sequence of the same library: same scores bit for bit, same lists
    s2, c2 = K.sparse_gemv_int4(*args, sel_pages=d(sel), sel_count=d(cnt_in))
    assert torch.equal(c2.cpu(), cand.cpu())
    s2n = s2.cpu().numpy().reshape(rows, M)
    for r in range(rows):
        n = int(cnt_in.reshape(-1)[r]) * 16
        assert np.array_equal(s2n[r, :n].view(np.uint32), sc[r, :n].view(np.uint32))
    i2, n2, l2 = K.softmax_top_p(s2, d(top_p) if per_row_p else top_p, lens=c2, sel_pages=d(sel),
                                 high=high, return_low=True)
    n2 = n2.cpu().numpy().reshape(rows)
    i2 = i2.cpu().numpy().reshape(rows, M)
    margin = np.full(rows, np.inf, dtype=np.float32)
    margin[live] = og
    same = [bool(n2[r] == cn[r] and np.array_equal(i2[r, :n2[r]], ix[r, :cn[r]])) for r in range(rows)]
    assert sum(same) >= 0.9 * rows
    for r in range(rows):
        assert same[r] or margin[r] < 5e-6, r


@pytest.mark.parametrize("S", [5, 16, 29, 64, 100, 256, 400, 1000, 2048])
def test_every_kernel_shape(dev, S):
    # one case per instantiated (threads, values per thread) shape; full lists, MHA, fp16
    B, H = (2, 4) if S <= 400 else (1, 4)
    npg = max(S + 3, int(S * 1.3))
    _case(dev, B, H, H, npg, S, 16, 0.9, "max", torch.float16, seed=S, ragged=False)


@pytest.mark.parametrize("S,Hkv,qdt,high,last_len,per_row_p", [
    (70, 8, torch.float16, "max", 16, False),
    (70, 2, torch.bfloat16, "max", 7, False),      # GQA 4:1, bf16 q, partial last page
    (130, 8, torch.float16, "first", 16, False),   # the reference's initial upper bound
    (300, 1, torch.float16, "max", 1, True),       # MQA, per-row p (top_p_arr)
    (513, 4, torch.bfloat16, "first", 3, True),
])
def test_ragged_lists(dev, S, Hkv, qdt, high, last_len, per_row_p):
    _case(dev, 2, 8, Hkv, S + 40, S, last_len, 0.85, high, qdt, seed=7 * S, per_row_p=per_row_p)


def test_errors(dev):
    rec = synth.int4_records_random(8, 2, seed=0).to(dev)
    ids, indptr, last = [t.to(dev) for t in synth.identity_page_table(1, 8)]
    q = torch.randn((1, 4, 128), device=dev).half()
    sel = torch.arange(4, dtype=torch.int32, device=dev).repeat(1, 4, 1).contiguous()
    cnt = torch.full((1, 4), 4, dtype=torch.int32, device=dev)
    K.sparse_gemv_int4_top_p(q, rec, ids, indptr, last, sel, cnt, 0.9)
    with pytest.raises(RuntimeError):
        K.sparse_gemv_int4_top_p(q, rec, ids, indptr, last, sel, cnt, 1.5)
    with pytest.raises(RuntimeError):
        K.sparse_gemv_int4_top_p(q.float(), rec, ids, indptr, last, sel, cnt, 0.9)
    with pytest.raises(RuntimeError):
        K.sparse_gemv_int4_top_p(q, rec, ids, indptr, last, sel.long(), cnt, 0.9)
    with pytest.raises(RuntimeError):
        K.sparse_gemv_int4_top_p(q, rec, ids, indptr, last, sel, cnt, 0.9, max_pages=4096)
    with pytest.raises(RuntimeError):
        K.sparse_gemv_int4_top_p(q[:, :3], rec, ids, indptr, last, sel, cnt, 0.9)


@pytest.mark.parametrize("N,lens,budget,H,Hkv,dt", [
    (1600, None, 320, 4, 4, torch.float16),          # 100 pages, keep 20
    (1000, None, 100, 4, 2, torch.bfloat16),         # GQA, bf16, budget not a multiple of 16, partial page
    (11200, None, 16384, 2, 2, torch.float16),       # budget beyond the context: every page (700)
    (40000, None, 4096, 2, 1, torch.float16),        # 2500 pages per request (> 2048)
    (8192 + 40, None, 8192, 2, 2, torch.float16),    # 512 selected pages: the benchmark's list length
])
def test_one_launch_row_kernel_equals_three_launches(dev, N, lens, budget, H, Hkv, dt):
    """twl_select_estimate_prune against twl_quest_select + twl_gemv_top_p on a real paged cache:
    page scores and page lists bit for bit, candidate scores bit for bit, survivor lists equal
    (a row whose bisection meets |S - p| within rounding may differ: other reduction shape)."""
    from twilight_amd.cache import PagedKVCache
    B, p = 2, 0.9
    g = torch.Generator().manual_seed(N)
    q = torch.randn((B, H, 128), generator=g)
    k = torch.randn((B, Hkv, N, 128), generator=g)
    group = H // Hkv
    for b in range(B):                               # a few heavy hitters per head
        for h in range(H):
            pos = torch.randint(0, N, (6,), generator=g)
            k[b, h // group, pos] += q[b, h] * (0.3 + torch.rand(6, 1, generator=g))
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k.to(dt), k.to(dt), dev,
                                    page_perm=torch.randperm(B * npg, generator=g))
    qd = q.to(dt).to(dev)
    tab = (cache.kv_page_indices, cache.kv_page_indptr, cache.kv_last_page_len)
    selA, selcA, psA = K.quest_select(qd, cache.meta, tab[0], tab[1], budget, npg)
    kk = selA.shape[-1]
    idxA, cntA, candA, scA = K.sparse_gemv_int4_top_p(qd, cache.k_int4, *tab, selA, selcA, p,
                                                     max_pages=kk, return_scores=True)
    selB, selcB, idxB, cntB, candB, psB, scB = K.quest_gemv_int4_top_p(
        qd, cache.meta, cache.k_int4, *tab, budget, npg, p, return_scores=True)
    assert torch.equal(psA.view(torch.int32), psB.view(torch.int32))
    assert torch.equal(selcA, selcB) and torch.equal(selA, selB) and torch.equal(candA, candB)
    assert int(selcA.min()) == min(kk, npg)
    n = int(selcA[0, 0]) * 16
    assert torch.equal(scA[..., :n].view(torch.int32), scB[..., :n].view(torch.int32))
    cA, cB, iA, iB = cntA.cpu(), cntB.cpu(), idxA.cpu(), idxB.cpu()
    differ = 0
    for b in range(B):
        for h in range(H):
            same = int(cA[b, h]) == int(cB[b, h]) and torch.equal(iA[b, h, :cA[b, h]], iB[b, h, :cB[b, h]])
            differ += 0 if same else 1
            toks = iB[b, h, :cB[b, h]].long()
            assert torch.all(toks[1:] > toks[:-1]) and int(toks.max()) < N
    assert differ <= 1


@pytest.mark.parametrize("N,budget,H,Hkv,dt", [
    (1600, 320, 4, 4, torch.float16),
    (1000, 100, 4, 4, torch.bfloat16),       # partial last page, budget not a multiple of 16
    (11200, 16384, 2, 2, torch.float16),     # every page
    (40000, 4096, 2, 2, torch.float16),      # 2500 pages per request (four scoring passes)
    (32768, 8192, 2, 2, torch.float16),      # the benchmark's row shape
    (32768 + 32, 8192, 2, 2, torch.float16),   # 2050 pages: the 2 beyond 2048 come from records
    (32768 + 250, 8192, 4, 2, torch.bfloat16), # 2064 pages, the last one partial, GQA
    (34816, 8192, 2, 2, torch.float16),      # 2176 pages: a tail of 128 pages from records
    (34832, 8192, 2, 2, torch.float16),      # 2177 pages: a second plane pass, last page from its record
    (65536 + 48, 8192, 2, 2, torch.float16), # 4099 pages: three pages beyond two plane passes
    (1600, 320, 16, 4, torch.float16),       # GQA 4:1, 32 rows: a group's rows share an XCD
    (1000, 100, 4, 2, torch.bfloat16),       # GQA 2:1, 8 rows: rows in launch order
    (1600, 320, 8, 1, torch.float16),        # eight q heads on one kv head
    (34832, 8192, 8, 2, torch.bfloat16),     # GQA 4:1 with a second plane pass and a record tail
])
def test_row_kernel_with_plane_metadata(dev, N, budget, H, Hkv, dt):
    """The plane layout (minima / maxima of all pages of a request contiguous per channel) against
    the record layout: planes hold exactly the records' numbers; page scores agree to summation
    order; the page lists are equal except pages whose score ties the k-th within rounding; rows
    with equal lists give identical candidate scores and survivors."""
    from twilight_amd.cache import PagedKVCache
    B, p = 2, 0.9
    g = torch.Generator().manual_seed(N + 1)
    q = torch.randn((B, H, 128), generator=g)
    k = torch.randn((B, Hkv, N, 128), generator=g)
    for b in range(B):
        for h in range(H):
            pos = torch.randint(0, N, (6,), generator=g)
            k[b, h // (H // Hkv), pos] += q[b, h] * (0.3 + torch.rand(6, 1, generator=g))
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(k.to(dt), k.to(dt), dev,
                                    page_perm=torch.randperm(B * npg, generator=g), plane_pages=npg + 9)
    # planes == transposed records, bit for bit
    cap = cache.meta_planes.shape[-1]
    assert cap % 8 == 0 and cap >= npg
    rec = cache.meta.view(torch.int16).reshape(-1, Hkv, 32, 2, 4)            # [page, h, chunk, min|max, 4]
    phys = cache.kv_page_indices.long().reshape(B, npg)
    want = rec[phys].permute(0, 2, 3, 5, 4, 1).reshape(B, Hkv, 128, 2, npg)  # [b, h, d, min|max, page]
    assert torch.equal(cache.meta_planes.view(torch.int16)[..., :npg], want)
    qd = q.to(dt).to(dev)
    tab = (cache.kv_page_indices, cache.kv_page_indptr, cache.kv_last_page_len)
    A = K.quest_gemv_int4_top_p(qd, cache.meta, cache.k_int4, *tab, budget, npg, p, return_scores=True)
    Bv = K.quest_gemv_int4_top_p(qd, cache.meta, cache.k_int4, *tab, budget, npg, p, return_scores=True,
                                 meta_planes=cache.meta_planes)
    # the stand-alone plane scoring kernel does the same arithmetic as the row kernel's first phase
    from twilight_amd import _lib
    ps2 = torch.zeros((B, H, npg), dtype=torch.float32, device=dev)
    rc = _lib.lib().twl_quest_page_scores_planes(
        qd.data_ptr(), 0 if dt == torch.float16 else 1, cache.meta_planes.data_ptr(), cap, 0, 0,
        cache.meta.data_ptr(), cache.kv_page_indices.data_ptr(), cache.kv_page_indptr.data_ptr(), B, H, Hkv, npg, ps2.data_ptr(), npg,
        torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.equal(ps2.view(torch.int32), Bv[5].view(torch.int32))
    selA, selcA, idxA, cntA, candA, psA, scA = [t.cpu() for t in A]
    selB, selcB, idxB, cntB, candB, psB, scB = [t.cpu() for t in Bv]
    assert torch.allclose(psA, psB, rtol=1e-5, atol=1e-4)
    assert torch.equal(selcA, selcB) and torch.equal(candA, candB)
    kk = int(selcA[0, 0])
    same_rows = 0
    for b in range(B):
        for h in range(H):
            a_set, b_set = set(selA[b, h, :kk].tolist()), set(selB[b, h, :kk].tolist())
            assert torch.all(selB[b, h, 1:kk] > selB[b, h, :kk - 1])
            kth = torch.sort(psA[b, h, :npg], descending=True).values[kk - 1]
            for pg in a_set ^ b_set:       # only pages tied with the k-th score may differ
                assert abs(float(psA[b, h, pg]) - float(kth)) <= 1e-4 * max(1.0, abs(float(kth)))
            if a_set == b_set:
                same_rows += 1
                n = kk * 16
                assert torch.equal(scA[b, h, :n].view(torch.int32), scB[b, h, :n].view(torch.int32))
                assert int(cntA[b, h]) == int(cntB[b, h])
                assert torch.equal(idxA[b, h, :cntA[b, h]], idxB[b, h, :cntB[b, h]])
    assert same_rows >= B * H - 1


@pytest.mark.parametrize("planes", [False, True])
def test_row_kernel_ragged_batch(dev, planes):
    """Requests of different lengths in one batch (one with a partial last page, one of a single
    page, one shorter than the budget): the one-launch kernel against quest_select + gemv_top_p."""
    from twilight_amd.cache import PagedKVCache
    H, N, p, budget = 4, 2000, 0.9, 480
    lens = [2000, 597, 16, 333]                       # tokens per request
    B = len(lens)
    g = torch.Generator().manual_seed(12)
    q = torch.randn((B, H, 128), generator=g)
    k = torch.randn((B, H, N, 128), generator=g)
    for b in range(B):
        for h in range(H):
            pos = torch.randint(0, lens[b], (4,), generator=g)
            k[b, h, pos] += q[b, h] * 0.5
    npg = N // 16
    full = PagedKVCache.from_dense(k.half(), k.half(), dev,
                                   page_perm=torch.randperm(B * npg, generator=g))
    phys = full.kv_page_indices.cpu().reshape(B, npg)
    pages = [(n + 15) // 16 for n in lens]
    ids = torch.cat([phys[b, :pages[b]] for b in range(B)])
    indptr = torch.tensor([0] + list(np.cumsum(pages)), dtype=torch.int32)
    last = torch.tensor([n - (pg - 1) * 16 for n, pg in zip(lens, pages)], dtype=torch.int32)
    full.set_page_table(ids, indptr, last)
    # last pages now hold fewer valid tokens: refresh their records
    last_pages = torch.stack([phys[b, pages[b] - 1] for b in range(B)]).to(torch.int32).to(dev)
    full.rebuild_shadow(last_pages, last.to(dev))
    if planes:
        full.enable_planes()
    qd = q.half().to(dev)
    tab = (full.kv_page_indices, full.kv_page_indptr, full.kv_last_page_len)
    mp = max(pages)
    selA, selcA, psA = K.quest_select(qd, full.meta, tab[0], tab[1], budget, mp)
    kk = selA.shape[-1]
    idxA, cntA, candA = K.sparse_gemv_int4_top_p(qd, full.k_int4, *tab, selA, selcA, p, max_pages=kk)
    selB, selcB, idxB, cntB, candB = K.quest_gemv_int4_top_p(
        qd, full.meta, full.k_int4, *tab, budget, mp, p, meta_planes=full.meta_planes)
    assert torch.equal(selcA, selcB) and torch.equal(candA, candB)
    want_k = [min(kk, pg) for pg in pages]
    assert selcB.cpu()[:, 0].tolist() == want_k
    # candidates of the last page stop at the request's length
    assert candB.cpu()[:, 0].tolist() == [16 * w for w in want_k]
    differ = 0
    for b in range(B):
        for h in range(H):
            n = want_k[b]
            if not torch.equal(selA[b, h, :n], selB[b, h, :n]):
                differ += 1
                continue
            ca, cb = int(cntA[b, h]), int(cntB[b, h])
            same = ca == cb and torch.equal(idxA[b, h, :ca], idxB[b, h, :cb])
            differ += 0 if same else 1
            assert int(idxB[b, h, :cb].max()) < lens[b]        # nothing past the request's end
    assert differ <= 1
