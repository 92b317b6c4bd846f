"""GPU parity of the INT4 path: shadow build (quantiser), unpack, and the score GEMV, against the
oracle's restatement of twilight/pyimpl/quantize.py:4-13 and twilight/pyimpl/attention.py:252-255."""
import math

import numpy as np
import pytest
import torch

from oracle import native
from oracle import pyimpl_port as P
from twilight_amd import synth
from twilight_amd.cache import PagedKVCache
import twilight_amd.kernel as K
from _checks import assert_scores_close

pytestmark = pytest.mark.gpu


def _oracle_records(k_pages):
    """k_pages [P,16,Hkv,128] (fp16-representable fp32) -> records + dequantised fp32 [P,Hkv,16,128]."""
    kk = k_pages.permute(0, 2, 1, 3).contiguous()          # [P,Hkv,16,128]
    codes, scale, zero, deq = P.int4_quant_storage(kk)
    return P.pack_int4_records(codes, scale, zero), deq


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_shadow_build_bit_exact(dev, dt):
    g = torch.Generator().manual_seed(0)
    k = (torch.randn((37, 16, 3, 128), generator=g) * torch.rand((37, 1, 3, 1), generator=g) * 3).to(dt)
    k[5, :, 1, 32:64] = 0.25                                  # a constant group
    k[6, 3, 2, :] = 0                                         # an all-zero token
    rec_o, deq_o = _oracle_records(k.float())
    kd = k.to(dev)
    k_int4 = torch.zeros((37, 3, 1280), dtype=torch.uint8, device=dev)
    meta = torch.zeros((37, 3, 512), dtype=torch.uint8, device=dev)
    K.kv_shadow_build(kd, k_int4, meta)
    assert np.array_equal(k_int4.cpu().numpy(), rec_o)       # nibbles, scale, zero: bit-exact
    deq = K.dequant_int4(k_int4).cpu().numpy()
    assert np.array_equal(deq.view(np.uint32), deq_o.view(np.uint32))   # dequantised: bit-exact
    # Quest metadata = channel-wise min / max of the page, in the cache dtype
    m = P.quest_page_meta(k.float())
    if dt == torch.float16:
        assert np.array_equal(meta.cpu().numpy(), P.pack_meta_records(m))
    else:
        got = meta.cpu().view(torch.bfloat16).reshape(37, 3, 32, 2, 4).float()
        assert torch.equal(got[:, :, :, 0].reshape(37, 3, 128), m[:, :, 0])
        assert torch.equal(got[:, :, :, 1].reshape(37, 3, 128), m[:, :, 1])


def test_shadow_partial_pages_and_page_ids(dev):
    g = torch.Generator().manual_seed(1)
    k = torch.randn((10, 16, 2, 128), generator=g).half()
    kd = k.to(dev)
    k_int4 = torch.full((10, 2, 1280), 0xAB, dtype=torch.uint8, device=dev)
    meta = torch.full((10, 2, 512), 0xCD, dtype=torch.uint8, device=dev)
    ids = torch.tensor([7, 2, 9], dtype=torch.int32, device=dev)
    valid = torch.tensor([16, 5, 1], dtype=torch.int32, device=dev)
    K.kv_shadow_build(kd, k_int4, meta, ids, valid)
    rec_o, _ = _oracle_records(k.float())
    got = k_int4.cpu().numpy()
    untouched = [i for i in range(10) if i not in (7, 2, 9)]
    assert np.all(got[untouched] == 0xAB) and np.all(meta.cpu().numpy()[untouched] == 0xCD)
    assert np.array_equal(got[7], rec_o[7])
    for page, v in ((2, 5), (9, 1)):
        c, s, z = P.unpack_int4_records(got[page:page + 1])
        co, so, zo = P.unpack_int4_records(rec_o[page:page + 1])
        assert np.array_equal(c[0, :, :v], co[0, :, :v]) and np.array_equal(s[0, :, :v], so[0, :, :v])
        assert np.all(c[0, :, v:] == 0) and np.all(s[0, :, v:] == 0) and np.all(z[0, :, v:] == 0)
    vl = torch.full((10,), 16, dtype=torch.int64); vl[2] = 5; vl[9] = 1
    m = P.pack_meta_records(P.quest_page_meta(k.float(), vl))
    assert np.array_equal(meta.cpu().numpy()[[7, 2, 9]], m[[7, 2, 9]])


def _gemv_oracle(q, deq_rows, sm_scale):
    """q [D] fp32, deq_rows [n,D] fp32 -> fp64 scores."""
    return (deq_rows.astype(np.float64) @ q.double().numpy()) * sm_scale


@pytest.mark.parametrize("qdt", [torch.float16, torch.bfloat16])
def test_gemv_full_context_shuffled_pages(dev, qdt):
    # every page of each request (sel_pages = None), shuffled physical pages, partial last page
    B, H, Hkv, npg = 3, 4, 2, 21
    rec = synth.int4_records_random(B * npg, Hkv, seed=3)
    ids, indptr, last = synth.identity_page_table(B, npg, last_len=9, shuffle_seed=4)
    g = torch.Generator().manual_seed(5)
    q = torch.randn((B, H, 128), generator=g).to(qdt)
    out, cnt = K.sparse_gemv_int4(q.to(dev), rec.to(dev), ids.to(dev), indptr.to(dev), last.to(dev),
                                  max_pages=npg)
    assert cnt.cpu().unique().tolist() == [npg * 16]
    codes, scale, zero = P.unpack_int4_records(rec.numpy())
    deq = native.int4_dequant(codes, scale, zero)            # [P,Hkv,16,128]
    got = out.cpu().numpy()
    qh = q.float()                                            # the true q, bf16 included
    for b in range(B):
        phys = ids[indptr[b]:indptr[b + 1]].long().numpy()
        for h in range(H):
            want = _gemv_oracle(qh[b, h], deq[phys, h // 2].reshape(-1, 128), 1 / math.sqrt(128))
            want[(npg - 1) * 16 + 9:] = -np.inf
            assert_scores_close(got[b, h], want)


def test_gemv_bf16_query_range(dev):
    # a bf16 query is converted to fp16 for the dot products: exact from 2^-17 to 65504, tiny
    # values rounded to multiples of 2^-24, larger ones saturated (finite scores, never NaN)
    npg = 5
    rec = synth.int4_records_random(npg, 1, seed=31)
    ids, indptr, last = synth.identity_page_table(1, npg, last_len=16)
    codes, scale, zero = P.unpack_int4_records(rec.numpy())
    deq = native.int4_dequant(codes, scale, zero)[:, 0].reshape(-1, 128)
    g = torch.Generator().manual_seed(32)
    base = torch.randn((1, 1, 128), generator=g)
    for mag, exact in ((1.0, True), (300.0, True), (2.0 ** -15, True), (2.0 ** -21, False), (3e5, False)):
        q = (base * mag).to(torch.bfloat16)
        out, _ = K.sparse_gemv_int4(q.to(dev), rec.to(dev), ids.to(dev), indptr.to(dev), last.to(dev),
                                    max_pages=npg)
        got = out.cpu().numpy()[0, 0]
        assert np.isfinite(got).all(), mag
        # what the kernel is documented to compute: q rounded to fp16 with saturation
        qk = q.float().clamp(-65504.0, 65504.0).to(torch.float16).float()[0, 0]
        assert_scores_close(got, _gemv_oracle(qk, deq, 1 / math.sqrt(128)))
        if exact and mag >= 1.0:   # inside the exact range the true bf16 q gives the same scores
            assert torch.equal(qk, q.float()[0, 0])
            assert_scores_close(got, _gemv_oracle(q.float()[0, 0], deq, 1 / math.sqrt(128)))


def test_gemv_selected_pages_and_ragged_counts(dev):
    B, H, npg, S = 2, 8, 150, 70
    rec = synth.int4_records_random(B * npg, H, seed=6)
    ids, indptr, last = synth.identity_page_table(B, npg, last_len=16, shuffle_seed=7)
    g = torch.Generator().manual_seed(8)
    q = torch.randn((B, H, 128), generator=g).half()
    sel = torch.stack([torch.sort(torch.randperm(npg, generator=g)[:S]).values
                       for _ in range(B * H)]).reshape(B, H, S).to(torch.int32)
    cnt_in = torch.randint(1, S + 1, (B, H), generator=g).to(torch.int32)
    cnt_in[0, 0] = S; cnt_in[1, 3] = 1; cnt_in[1, 4] = 16; cnt_in[1, 5] = 17; cnt_in[1, 6] = 64; cnt_in[1, 7] = 65
    out = torch.full((B, H, S * 16), 123.0, device=dev)
    out, cnt = K.sparse_gemv_int4(q.to(dev), rec.to(dev), ids.to(dev), indptr.to(dev), last.to(dev),
                                  sel_pages=sel.to(dev), sel_count=cnt_in.to(dev), out=out)
    assert torch.equal(cnt.cpu(), cnt_in * 16)
    codes, scale, zero = P.unpack_int4_records(rec.numpy())
    deq = native.int4_dequant(codes, scale, zero)
    got = out.cpu().numpy()
    for b in range(B):
        for h in range(H):
            n = int(cnt_in[b, h])
            phys = ids[indptr[b] + sel[b, h, :n].long()].long().numpy()
            want = _gemv_oracle(q[b, h].float(), deq[phys, h].reshape(-1, 128), 1 / math.sqrt(128))
            assert_scores_close(got[b, h, :n * 16], want)
            assert np.all(got[b, h, n * 16:] == 123.0)      # nothing written past the row's pages


@pytest.mark.parametrize("H,Hkv,qdt", [(8, 2, torch.float16), (8, 4, torch.bfloat16), (8, 1, torch.float16)])
def test_gemv_group_lists_against_oracle_and_per_head_gemv(dev, H, Hkv, qdt):
    """One page list per kv head, records fetched once per group and multiplied with the group's
    queries on the matrix cores: every q head's scores against the fp64 product over the
    dequantised records (1e-3 relative, as for the per-head GEMV) and against the per-head GEMV
    over the same list (exact products, fp32 sums in another order: a few ulps of the terms);
    ragged counts, partial last page, slots past a row's count untouched."""
    B, npg, S = 3, 90, 70
    G = H // Hkv
    rec = synth.int4_records_random(B * npg, Hkv, seed=16)
    ids, indptr, last = synth.identity_page_table(B, npg, last_len=5, shuffle_seed=17)
    g = torch.Generator().manual_seed(18)
    q = torch.randn((B, H, 128), generator=g).to(qdt)
    lists = torch.stack([torch.sort(torch.randperm(npg, generator=g)[:S]).values
                         for _ in range(B * Hkv)]).reshape(B, Hkv, S).to(torch.int32)
    first = torch.cat([torch.randperm(npg - 1, generator=g)[:S - 1], torch.tensor([npg - 1])])
    lists[0, 0] = torch.sort(first).values.to(torch.int32)       # the partial last page is a candidate
    cnt_kv = torch.randint(1, S + 1, (B, Hkv), generator=g).to(torch.int32)
    cnt_kv[0, 0] = S; cnt_kv[1, 0] = 1; cnt_kv[2, 0] = 33
    sel = lists.repeat_interleave(G, dim=1).contiguous()
    cnt = cnt_kv.repeat_interleave(G, dim=1).contiguous()
    # the group kernel only looks at the first q head's list: the other rows may hold anything
    junk = sel.clone()
    junk.reshape(B, Hkv, G, S)[:, :, 1:] = 0
    args = (q.to(dev), rec.to(dev), ids.to(dev), indptr.to(dev), last.to(dev))
    want, wc = K.sparse_gemv_int4(*args, sel_pages=sel.to(dev), sel_count=cnt.to(dev),
                                  out=torch.full((B, H, S * 16), 7.0, device=dev))
    got, gc = K.sparse_gemv_int4(*args, sel_pages=junk.to(dev), sel_count=cnt.to(dev),
                                 out=torch.full((B, H, S * 16), 7.0, device=dev), group_lists=True)
    assert torch.equal(gc, wc)
    want, got = want.cpu().numpy(), got.cpu().numpy()
    assert np.isneginf(want).any()                                # the partial page was exercised
    assert np.array_equal(np.isneginf(got), np.isneginf(want))
    assert np.array_equal(got == 7.0, want == 7.0)                # nothing written past a row's count
    codes, scale, zero = P.unpack_int4_records(rec.numpy())
    deq = native.int4_dequant(codes, scale, zero)                 # [pages, Hkv, 16, 128]
    # the kernel takes a bf16 query as its nearest fp16 value
    qf = q.float() if qdt == torch.float16 else q.float().half().float()
    sm = 1.0 / math.sqrt(128)
    for b in range(B):
        for h in range(H):
            n = int(cnt[b, h])
            phys = ids[indptr[b] + sel[b, h, :n].long()].long()
            ref = _gemv_oracle(qf[b, h], deq[phys, h // G].reshape(-1, 128), sm)
            live = np.isfinite(want[b, h, :n * 16])
            assert_scores_close(got[b, h, :n * 16][live][None], ref[live][None])
            # against the per-head kernel: both add exact products in fp32
            rms = float(np.sqrt((ref[live] ** 2).mean()))
            assert np.abs(got[b, h, :n * 16][live] - want[b, h, :n * 16][live]).max() <= 2e-5 * max(rms, 1.0)


def test_gemv_constant_case_of_the_reference_bench(dev):
    # benchmark/efficiency/bench_gemv.py:390-422: q = 1, nibbles 3, scale 1, zero 0 -> 3*128 = 384
    npg = 8
    codes = np.full((npg, 1, 16, 128), 3, np.uint8)
    rec = torch.from_numpy(P.pack_int4_records(codes, np.ones((npg, 1, 16, 4), np.float16),
                                               np.zeros((npg, 1, 16, 4), np.float16)))
    ids, indptr, last = synth.identity_page_table(1, npg)
    q = torch.ones((1, 1, 128), dtype=torch.float16)
    out, _ = K.sparse_gemv_int4(q.to(dev), rec.to(dev), ids.to(dev), indptr.to(dev), last.to(dev),
                                max_pages=npg, sm_scale=1.0)
    assert torch.all(out == 384.0)


def test_gemv_matches_quantised_k_of_a_real_cache(dev):
    # end to end with the shadow builder: scores == q . dequant(quant(K)) / sqrt(D)
    q, k, v = synth.heavy_hitter_qkv(1, 4, 1000, n_heavy=4, seed=2, dtype=torch.float16)
    cache = PagedKVCache.from_dense(k.half(), v.half(), dev, page_perm=torch.randperm(63))
    out, _ = K.sparse_gemv_int4(q[:, :, 0].half().to(dev), cache.k_int4, cache.kv_page_indices,
                                cache.kv_page_indptr, cache.kv_last_page_len, max_pages=63)
    _, _, _, deq = P.int4_quant_storage(k)
    want = P.estimator_scores(q, torch.from_numpy(deq))[0, :, 0].double().numpy()
    got = out.cpu().numpy()[0]
    assert_scores_close(got[:, :1000], want)
    assert np.all(np.isneginf(got[:, 1000:]))


@pytest.mark.parametrize("H", [4, 6, 32])   # 6: a head count that does not divide the workgroup
def test_ftka_shaped_entry(dev, H):
    # call shape of benchmark/efficiency/bench_gemv.py:445-454: NHD uint8 cache, per-token scale/zero
    B, page_size, pages = 2, 4, 30
    g = torch.Generator().manual_seed(10)
    k_u8 = torch.randint(0, 256, (pages, page_size, H, 64), dtype=torch.uint8, generator=g)
    scales = (torch.rand((pages, page_size, H), generator=g) * 0.1 + 0.01).half()
    zeros = (torch.randn((pages, page_size, H), generator=g) * 0.2).half()
    q = torch.randn((B, H, 128), generator=g).half()
    per_req = [11, 15]
    perm = torch.randperm(pages, generator=g)
    idx = perm[:sum(per_req)].to(torch.int32)
    indptr = torch.tensor([0, 11, 26], dtype=torch.int32)
    last = torch.tensor([4, 2], dtype=torch.int32)
    N = 15 * page_size
    o = torch.full((B, H, N), 7.0, dtype=torch.float16, device=dev)
    K.batched_sparse_gemv_int4_k(q.to(dev), o, k_u8.to(dev), scales.to(dev), zeros.to(dev),
                                 idx.to(dev), indptr.to(dev), last.to(dev))
    lo = (k_u8 & 0xF).float(); hi = (k_u8 >> 4).float()
    kk = torch.stack([lo, hi], dim=-1).reshape(pages, page_size, H, 128)
    deq = kk * scales.float()[..., None] + zeros.float()[..., None]       # bench_gemv.py:181
    got = o.cpu().float()
    for b in range(B):
        n_tok = (per_req[b] - 1) * page_size + int(last[b])
        phys = idx[indptr[b]:indptr[b + 1]].long()
        kb = deq[phys].reshape(-1, H, 128)[:n_tok]
        want = torch.einsum("hd,nhd->hn", q[b].double(), kb.double())
        assert torch.allclose(got[b, :, :n_tok].double(), want, rtol=2e-3, atol=2e-2)   # fp16 output
        assert torch.all(got[b, :, n_tok:] == 7.0)


@pytest.mark.parametrize("paged", [False, True])
def test_gemv_full_size_cfg2_sampled_and_linear(dev, paged):
    # the stand-alone GEMV benchmark shape: B=8, H=32, 32768 candidates per head. The oracle checks a sample of
    # (row, page) pairs; linearity in q checks every output: f(q1) + f(q2) == f(q1 + q2) when q1, q2
    # have disjoint supports (exact up to fp32 accumulation order).
    B, H, npg = 8, 32, 2048
    rec = synth.int4_records_random(B * npg, H, seed=0, device=dev)
    ids, indptr, last = synth.identity_page_table(B, npg, device=dev, shuffle_seed=1 if paged else None)
    g = torch.Generator().manual_seed(2)
    q = torch.randn((B, H, 128), generator=g).half()
    out, _ = K.sparse_gemv_int4(q.to(dev), rec, ids, indptr, last, max_pages=npg)
    got = out.cpu().numpy()
    rng = np.random.default_rng(3)
    ids_c = ids.cpu().numpy()
    for _ in range(64):
        b, h, lp = int(rng.integers(B)), int(rng.integers(H)), int(rng.integers(npg))
        phys = int(ids_c[b * npg + lp])
        c, s, z = P.unpack_int4_records(rec[phys:phys + 1, h:h + 1].cpu().numpy())
        deq = native.int4_dequant(c, s, z)[0, 0]
        want = _gemv_oracle(q[b, h].float(), deq, 1 / math.sqrt(128))
        np.testing.assert_allclose(got[b, h, lp * 16:(lp + 1) * 16], want, rtol=1e-3, atol=3e-4)
    q1 = q.clone(); q1[..., 64:] = 0
    q2 = q.clone(); q2[..., :64] = 0
    o1, _ = K.sparse_gemv_int4(q1.to(dev), rec, ids, indptr, last, max_pages=npg)
    o2, _ = K.sparse_gemv_int4(q2.to(dev), rec, ids, indptr, last, max_pages=npg)
    err = (o1 + o2 - out).abs().max().item()
    assert err < 2e-5, err


@pytest.mark.parametrize("H", [4, 6, 32])
def test_ftka_shaped_fp16_int8_and_single_entries(dev, H):
    # call shapes of benchmark/efficiency/bench_gemv.py:33 (single), :135-144 (int8), :234-241 (fp16);
    # the references there are plain matmuls (:36-42, :181, :259-296)
    B, page_size, pages = 2, 2, 40
    g = torch.Generator().manual_seed(12)
    q = torch.randn((B, H, 128), generator=g).half()
    k16 = torch.randn((pages, page_size, H, 128), generator=g).half()
    k_i8 = torch.randint(-128, 128, (pages, page_size, H, 128), generator=g, dtype=torch.int16)
    k_u8 = (k_i8 + 128).to(torch.uint8)                                    # bench_gemv.py:93
    scales = (torch.rand((pages, page_size, H), generator=g) * 0.02 + 0.001).half()
    zeros = (torch.randn((pages, page_size, H), generator=g) * 0.1).half()
    per_req = [13, 20]
    idx = torch.randperm(pages, generator=g)[:sum(per_req)].to(torch.int32)
    indptr = torch.tensor([0, 13, 33], dtype=torch.int32)
    last = torch.tensor([1, 2], dtype=torch.int32)
    N = 20 * page_size
    d = lambda t: t.to(dev)
    o16 = torch.full((B, H, 1, N), 9.0, dtype=torch.float16, device=dev)
    K.batched_sparse_gemv(d(q), o16, d(k16), d(idx), d(indptr), d(last))
    o8 = torch.full((B, H, N), 9.0, dtype=torch.float16, device=dev)
    K.batched_sparse_gemv_int8_k(d(q), o8, d(k_u8), d(scales), d(zeros), d(idx), d(indptr), d(last))
    deq8 = k_i8.float() * scales.float()[..., None] + zeros.float()[..., None]
    for b in range(B):
        n_tok = (per_req[b] - 1) * page_size + int(last[b])
        phys = idx[indptr[b]:indptr[b + 1]].long()
        w16 = torch.einsum("hd,nhd->hn", q[b].double(), k16[phys].reshape(-1, H, 128)[:n_tok].double())
        assert torch.allclose(o16.cpu()[b, :, 0, :n_tok].double(), w16, rtol=2e-3, atol=2e-2)
        w8 = torch.einsum("hd,nhd->hn", q[b].double(), deq8[phys].reshape(-1, H, 128)[:n_tok].double())
        assert torch.allclose(o8.cpu()[b, :, :n_tok].double(), w8, rtol=2e-3, atol=2e-2)
        assert torch.all(o16.cpu()[b, :, 0, n_tok:] == 9.0) and torch.all(o8.cpu()[b, :, n_tok:] == 9.0)
    # constant case of bench_gemv.py:80-112: int8 value 3, scale 1, zero 0, q = 1 -> 384
    ones_q = torch.ones((1, 2, 128), dtype=torch.float16, device=dev)
    k3 = torch.full((8, 1, 2, 128), 131, dtype=torch.uint8, device=dev)
    o3 = torch.zeros((1, 2, 8), dtype=torch.float16, device=dev)
    K.batched_sparse_gemv_int8_k(ones_q, o3, k3, torch.ones((8, 1, 2), dtype=torch.float16, device=dev),
                                 torch.zeros((8, 1, 2), dtype=torch.float16, device=dev),
                                 torch.arange(8, dtype=torch.int32, device=dev),
                                 torch.tensor([0, 8], dtype=torch.int32, device=dev),
                                 torch.ones(1, dtype=torch.int32, device=dev))
    assert torch.all(o3 == 384.0)
    # single request (bench_gemv.py:23-42)
    qs = torch.randn((H, 128), generator=g).half()
    ks = torch.randn((77, H, 128), generator=g).half()
    os_ = torch.empty((H, 77), dtype=torch.float16, device=dev)
    K.single_sparse_gemv(d(qs), os_, d(ks))
    ref = torch.matmul(qs.double().unsqueeze(1), ks.double().transpose(0, 1).transpose(1, 2)).squeeze(1)
    assert torch.allclose(os_.cpu().double(), ref, rtol=1e-2, atol=2e-2)      # tolerances of :41-42
