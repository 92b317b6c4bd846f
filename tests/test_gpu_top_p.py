"""GPU parity of the top-p pruner (through the C-ABI) against the oracle's restatement of
csrc/include/sampling.cuh:156-231 and twilight/pyimpl/top_p.py:10-15."""
import os

import numpy as np
import pytest
import torch

from oracle import native
from oracle import pyimpl_port as P
from twilight_amd import synth
import twilight_amd.kernel as K
from _checks import assert_top_p_parity

pytestmark = pytest.mark.gpu


def _softmax(x):
    return torch.softmax(x, dim=-1, dtype=torch.float32)


@pytest.mark.parametrize("p", [0.85, 0.95])
@pytest.mark.parametrize("first_is_max", [True, False])
def test_mask_dropin_cfg3(dev, p, first_is_max):
    # the pruner-alone benchmark shape: [8, 32, 8192] Zipf-spiked rows
    x = synth.topp_scores(8, 32, 8192, seed=0, first_is_max=first_is_max)
    probs = _softmax(x).reshape(8, 32, 1, 8192)
    pn = probs.reshape(256, 8192).numpy()
    for high, mode in (("first", native.HIGH_FIRST), ("max", native.HIGH_MAX)):
        om, ol, oi, og = native.top_p_mask_f32(pn, p, mode, return_margin=True)
        idx, count, mask, low, iters = K.top_p_select(probs.to(dev), p, high=high,
                                                      return_mask=True, return_stats=True)
        gm = mask.cpu().numpy().reshape(256, 8192)
        assert mask.dtype == torch.bool and mask.shape == probs.shape
        n_exact = assert_top_p_parity(pn, p, gm, om, ol, og, gpu_low=low.cpu().numpy())
        assert n_exact >= 250
        ok = og >= 2e-6
        assert np.array_equal(iters.cpu().numpy()[ok], oi[ok])
        # index list == positions of the mask, ascending
        cn = count.cpu().numpy().reshape(256)
        ix = idx.cpu().numpy().reshape(256, 8192)
        assert np.array_equal(cn, gm.sum(-1))
        for r in range(256):
            assert np.array_equal(ix[r, :cn[r]], np.nonzero(gm[r])[0])
        # the reference entry point itself
        m2 = K.top_p_fp32_return_mask(probs.to(dev), p, high=high)
        assert torch.equal(m2, mask)


@pytest.mark.parametrize("d", [1, 3, 17, 1000, 1024, 1025, 4097, 9000, 20000, 32768])
def test_ragged_lengths(dev, d):
    g = torch.Generator().manual_seed(d)
    x = torch.randn((3, 2, d), generator=g) * 3
    probs = _softmax(x).reshape(3, 2, 1, d)
    pn = probs.reshape(6, d).numpy()
    om, ol, oi, og = native.top_p_mask_f32(pn, 0.9, native.HIGH_MAX, return_margin=True)
    idx, count, mask = K.top_p_select(probs.to(dev), 0.9, high="max", return_mask=True)
    gm = mask.cpu().numpy().reshape(6, d)
    assert_top_p_parity(pn, 0.9, gm, om, ol, og)
    assert np.array_equal(count.cpu().numpy().reshape(6), gm.sum(-1))


@pytest.mark.parametrize("d", [2048, 8192, 32768])
def test_rows_that_exercise_the_heavy_element_phase(dev, d):
    """Rows built around the bisection's first phase (one wavefront iterating over the elements
    above max/256, the other elements entering through their maximum and the smallest positive
    element): termination inside the phase, a list that is exactly full, one element too many
    (whole-row fallback), no light elements, no heavy elements but the maximum, a first element
    far below the maximum in `first` mode. Masks, `low` and iteration counts against the oracle."""
    g = torch.Generator().manual_seed(d)
    rows = []
    tail = torch.rand(d, generator=g) * 1e-6 + 1e-7

    def norm(v):
        return (v / v.sum()).float()
    a = tail.clone(); a[5] = 2.0                                   # one dominant element
    rows.append(norm(a))
    b = tail.clone(); b[:12] = 0.5 ** torch.arange(1, 13)          # geometric heavy hitters
    rows.append(norm(b))
    c = tail.clone() * 1e-3; c[torch.randperm(d, generator=g)[:256]] = 1.0   # list exactly full
    rows.append(norm(c))
    e = tail.clone() * 1e-3; e[torch.randperm(d, generator=g)[:257]] = 1.0   # one too many
    rows.append(norm(e))
    f = torch.zeros(d); f[torch.randperm(d, generator=g)[:40]] = torch.rand(40, generator=g) + 0.5
    rows.append(norm(f))                                           # only heavy elements and zeros
    h = torch.full((d,), 1.0); h[9] = 300.0                        # the maximum alone is heavy
    rows.append(norm(h))
    u = torch.rand(d, generator=g) + 0.5                           # flat: everything is heavy
    rows.append(norm(u))
    w = tail.clone(); w[0] = 1e-4; w[100:110] = 1.0                # `first` far below the maximum
    rows.append(norm(w))
    probs = torch.stack(rows).reshape(1, len(rows), 1, d).contiguous()
    pn = probs.reshape(len(rows), d).numpy()
    for p in (0.3, 0.9, 0.999):
        for high, mode in (("max", native.HIGH_MAX), ("first", native.HIGH_FIRST)):
            om, ol, oi, og = native.top_p_mask_f32(pn, p, mode, return_margin=True)
            idx, count, mask, low, iters = K.top_p_select(probs.to(dev), p, high=high,
                                                          return_mask=True, return_stats=True)
            gm = mask.cpu().numpy().reshape(len(rows), d)
            assert_top_p_parity(pn, p, gm, om, ol, og, gpu_low=low.cpu().numpy().reshape(-1))
            ok = og >= 2e-6
            assert np.array_equal(iters.cpu().numpy().reshape(-1)[ok], oi[ok]), (p, high)
            assert np.array_equal(count.cpu().numpy().reshape(-1), gm.sum(-1))


@pytest.mark.parametrize("seed", range(int(os.environ.get("TWL_RANDOM_SHAPES", "12"))))
def test_random_rows(dev, seed):
    """Row length, sharpness, number and weight of spikes, zeros, p and the `high` mode drawn at
    random: masks, `low` and iteration counts against the oracle."""
    rng = np.random.default_rng(500 + seed)
    d = int(rng.choice([int(rng.integers(1, 300)), int(rng.integers(300, 5000)),
                        int(rng.integers(5000, 32769))]))
    rows = int(rng.integers(1, 9))
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((rows, d), generator=g) * float(rng.choice([0.3, 1.0, 3.0, 8.0]))
    for r in range(rows):
        n_spike = int(rng.integers(0, min(d, 40) + 1))
        if n_spike:
            pos = torch.randperm(d, generator=g)[:n_spike]
            x[r, pos] += float(rng.choice([2.0, 6.0, 12.0])) * torch.rand(n_spike, generator=g)
        if rng.random() < 0.3:                     # masked candidates: probability exactly 0
            x[r, torch.rand(d, generator=g) < 0.4] = float("-inf")
            x[r, int(rng.integers(0, d))] = 0.0    # at least one live element
    probs = _softmax(x).reshape(1, rows, 1, d).contiguous()
    pn = probs.reshape(rows, d).numpy()
    p = float(rng.choice([0.1, 0.5, 0.85, 0.9, 0.95, 0.99, 1.0]))
    high, mode = (("max", native.HIGH_MAX) if rng.random() < 0.6 else ("first", native.HIGH_FIRST))
    om, ol, oi, og = native.top_p_mask_f32(pn, p, mode, return_margin=True)
    idx, count, mask, low, iters = K.top_p_select(probs.to(dev), p, high=high, return_mask=True,
                                                  return_stats=True)
    gm = mask.cpu().numpy().reshape(rows, d)
    assert_top_p_parity(pn, p, gm, om, ol, og, gpu_low=low.cpu().numpy().reshape(-1))
    ok = og >= 2e-6
    assert np.array_equal(iters.cpu().numpy().reshape(-1)[ok], oi[ok])
    assert np.array_equal(count.cpu().numpy().reshape(-1), gm.sum(-1))
    # the fused softmax + top-p entry on the raw scores of the same rows (top_p.py:10-15)
    idx2, count2, probs2 = K.softmax_top_p(x.reshape(1, rows, d).contiguous().to(dev), p, high=high,
                                           return_probs=True)
    # fp32 normalisers of up to 32768 terms, summed in different orders: a common factor per row
    np.testing.assert_allclose(probs2.cpu().numpy().reshape(rows, d), pn, rtol=1e-5, atol=1e-12)
    gm2 = np.zeros((rows, d), dtype=bool)
    c2 = count2.cpu().numpy().reshape(-1)
    i2 = idx2.cpu().numpy().reshape(rows, d)
    for r in range(rows):
        assert np.all(np.diff(i2[r, :c2[r]]) > 0)
        gm2[r, i2[r, :c2[r]]] = True
    assert_top_p_parity(pn, p, gm2, om, ol, og, margin_tol=5e-6)


def test_per_row_p_and_degenerate_rows(dev):
    d = 2048
    g = torch.Generator().manual_seed(1)
    probs = _softmax(torch.randn((2, 4, d), generator=g) * 4)
    probs[0, 0] = 0; probs[0, 0, 77] = 1.0            # one-hot
    probs[0, 1] = 1.0 / d                              # uniform: everything ties, all kept
    probs[0, 2] = 0                                    # all zero: nothing kept
    probs = probs.reshape(2, 4, 1, d).contiguous()
    ps = torch.tensor([0.95, 0.5, 0.9, 0.3, 0.6, 0.85, 0.99, 1.0])
    pn = probs.reshape(8, d).numpy()
    om, ol, oi, og = native.top_p_mask_f32(pn, ps.numpy(), native.HIGH_MAX, return_margin=True)
    mask = K.top_p_fp32_return_mask(probs.to(dev), ps.to(dev), high="max")
    gm = mask.cpu().numpy().reshape(8, d)
    assert gm[0].sum() == 1 and gm[0, 77] and gm[1].sum() == d and gm[2].sum() == 0
    assert_top_p_parity(pn[3:], ps.numpy()[3:], gm[3:], om[3:], ol[3:], og[3:])


def test_sink_quirk_first_mode(dev):
    # probs[...,0] == 0 under high="first": the reference prunes nothing (mask = probs > 0)
    g = torch.Generator().manual_seed(2)
    probs = _softmax(torch.randn((1, 4, 1, 512), generator=g) * 3)
    probs[..., 0] = 0
    m = K.top_p_fp32_return_mask(probs.to(dev), 0.5, high="first")
    assert torch.equal(m.cpu(), probs > 0)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_16bit_entry(dev, dt):
    # the reference's DType = half / nv_bfloat16 instantiation (csrc/src/sampling.cu:22-43): every
    # operation in the 16-bit type, sums in cub::BlockReduce's order. Oracle and kernel follow the
    # same order, so masks, final pivots and iteration counts must be identical on EVERY row: there
    # is no margin in this comparison. Shapes cover VEC = gcd(8, d) in {8, 4, 2, 1}, one to four
    # chunks of 1024 * VEC elements, both upper bounds, scalar and per-row p.
    code = 0 if dt == torch.float16 else 1
    g = torch.Generator().manual_seed(3)
    for d, rows, scale in ((3000, 16, 4.0), (8192, 32, 5.0), (4100, 8, 4.0), (1002, 8, 3.0),
                           (999, 8, 3.0), (32768, 8, 6.0), (20000, 4, 5.0), (24, 4, 1.0), (5, 4, 1.0)):
        probs = _softmax(torch.randn((1, rows, 1, d), generator=g) * scale).to(dt)
        bits = probs.view(torch.int16).numpy().view(np.uint16).reshape(rows, d)
        for high, mode in (("max", native.HIGH_MAX), ("first", native.HIGH_FIRST)):
            for p in (0.9, 0.85 + 0.1 * torch.rand(rows, generator=g)):
                pn = p.numpy().astype(np.float32) if torch.is_tensor(p) else p
                om, ol, oi = native.top_p_mask_cub(bits, code, pn, mode)
                pd = p.to(dev) if torch.is_tensor(p) else p
                idx, count, mask, low, iters = K.top_p_select(probs.to(dev), pd, high=high,
                                                              return_mask=True, return_stats=True)
                gm = mask.cpu().numpy().reshape(rows, d)
                assert np.array_equal(gm, om.astype(bool)), (d, high)
                assert np.array_equal(low.cpu().numpy(), ol) and np.array_equal(iters.cpu().numpy(), oi)
                cn = count.cpu().numpy().reshape(-1)
                ix = idx.cpu().numpy().reshape(rows, d)
                for r in range(rows):
                    assert np.array_equal(ix[r, :cn[r]], np.nonzero(gm[r])[0])
        assert torch.equal(K.top_p_fp16_return_mask(probs.to(dev), 0.9), 
                           torch.from_numpy(native.top_p_mask_cub(bits, code, 0.9, native.HIGH_FIRST)[0]
                                            .astype(bool)).reshape(1, rows, 1, d).to(dev))


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_16bit_entry_cfg3_shape(dev, dt):
    # the pruner workload (8 x 32 rows of 8192, Zipf spikes over a normal background) in 16 bits
    code = 0 if dt == torch.float16 else 1
    x = synth.topp_scores(8, 32, 8192, seed=13, first_is_max=True)
    probs = _softmax(x).reshape(8, 32, 1, 8192).to(dt)
    bits = probs.view(torch.int16).numpy().view(np.uint16).reshape(256, 8192)
    for p in (0.85, 0.95):
        for high, mode in (("first", native.HIGH_FIRST), ("max", native.HIGH_MAX)):
            om, ol, oi = native.top_p_mask_cub(bits, code, p, mode)
            idx, count, mask, low, iters = K.top_p_select(probs.to(dev), p, high=high,
                                                          return_mask=True, return_stats=True)
            assert np.array_equal(mask.cpu().numpy().reshape(256, 8192), om.astype(bool))
            assert np.array_equal(low.cpu().numpy(), ol) and np.array_equal(iters.cpu().numpy(), oi)
            assert oi.mean() > 5     # the rows really iterate


def test_fp32_exact_entry(dev):
    # the reference's DType = float instantiation (csrc/src/sampling.cu:45-63) with the sums in
    # cub::BlockReduce's order (VEC = gcd(4, d) in {4, 2, 1}, one to eight chunks of 1024 * VEC):
    # masks, final pivots and iteration counts identical on EVERY row, no margin; both upper
    # bounds, scalar and per-row p, mask-only and list outputs.
    g = torch.Generator().manual_seed(4)
    for d, rows, scale in ((3000, 16, 4.0), (8192, 32, 5.0), (4100, 8, 4.0), (1002, 8, 3.0),
                           (999, 8, 3.0), (32768, 8, 6.0), (20000, 4, 5.0), (24, 4, 1.0), (5, 4, 1.0),
                           (1, 3, 1.0), (17, 4, 2.0), (1025, 4, 3.0), (4097, 4, 4.0), (9000, 4, 4.0)):
        probs = _softmax(torch.randn((1, rows, 1, d), generator=g) * scale)
        pn32 = probs.numpy().reshape(rows, d)
        for high, mode in (("max", native.HIGH_MAX), ("first", native.HIGH_FIRST)):
            for p in (0.9, 0.85 + 0.1 * torch.rand(rows, generator=g)):
                pn = p.numpy().astype(np.float32) if torch.is_tensor(p) else p
                om, ol, oi = native.top_p_mask_cub(pn32, native.DT_F32, pn, mode)
                pd = p.to(dev) if torch.is_tensor(p) else p
                idx, count, mask, low, iters = K.top_p_select(probs.to(dev), pd, high=high,
                                                              return_mask=True, return_stats=True,
                                                              exact=True)
                gm = mask.cpu().numpy().reshape(rows, d)
                assert np.array_equal(gm, om.astype(bool)), (d, high)
                assert np.array_equal(low.cpu().numpy(), ol) and np.array_equal(iters.cpu().numpy(), oi)
                cn = count.cpu().numpy().reshape(-1)
                ix = idx.cpu().numpy().reshape(rows, d)
                for r in range(rows):
                    assert np.array_equal(ix[r, :cn[r]], np.nonzero(gm[r])[0])
        assert torch.equal(K.top_p_fp32_return_mask(probs.to(dev), 0.9, exact=True),
                           torch.from_numpy(native.top_p_mask_cub(pn32, native.DT_F32, 0.9, native.HIGH_FIRST)[0]
                                            .astype(bool)).reshape(1, rows, 1, d).to(dev))


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16, torch.float32])
def test_exact_entries_on_ties_zeros_and_degenerate_rows(dev, dt):
    # rows the random tests do not produce, for the three kernels that follow the reference's
    # arithmetic: values from a tiny set (ties everywhere, so the min{x > low} / max{x <= high}
    # searches return repeated values and the bracket closes on them), rows that are mostly zero,
    # one-hot, flat and all-zero rows, a zero in front (the `first` bound is then 0: the loop runs
    # once and keeps every positive entry). Masks, pivots and iteration counts equal the oracle's.
    g = torch.Generator().manual_seed(11)
    code = {torch.float16: 0, torch.bfloat16: 1, torch.float32: native.DT_F32}[dt]
    for d in (8192, 4100, 999, 64, 7):
        rows = []
        levels = torch.tensor([0.0, 1.0, 2.0, 3.0, 8.0, 64.0])
        for zeros in (0.0, 0.5, 0.97):
            r = levels[torch.randint(1, 6, (d,), generator=g)]
            r[torch.rand(d, generator=g) < zeros] = 0.0
            rows.append(r)
        one_hot = torch.zeros(d); one_hot[d // 3] = 1.0
        first_zero = levels[torch.randint(1, 6, (d,), generator=g)].clone(); first_zero[0] = 0.0
        rows += [one_hot, torch.ones(d), torch.zeros(d), first_zero]
        x = torch.stack(rows)
        probs = (x / x.sum(-1, keepdim=True).clamp(min=1.0)).to(dt)   # rounded to the type once
        n = probs.shape[0]
        vals = (probs.numpy() if dt == torch.float32
                else probs.view(torch.int16).numpy().view(np.uint16)).reshape(n, d)
        for high, mode in (("max", native.HIGH_MAX), ("first", native.HIGH_FIRST)):
            for p in (0.5, 0.9, 1.0):
                om, ol, oi = native.top_p_mask_cub(vals, code, p, mode)
                idx, count, mask, low, iters = K.top_p_select(
                    probs.reshape(1, n, 1, d).to(dev), p, high=high, return_mask=True,
                    return_stats=True, exact=True)
                gm = mask.cpu().numpy().reshape(n, d)
                assert np.array_equal(gm, om.astype(bool)), (d, high, p)
                assert np.array_equal(low.cpu().numpy().reshape(-1), ol), (d, high, p)
                assert np.array_equal(iters.cpu().numpy().reshape(-1), oi), (d, high, p)
                cn = count.cpu().numpy().reshape(-1)
                assert np.array_equal(cn, gm.sum(-1))
        # the zero in front under the reference's bound: one iteration, every positive entry kept
        om, _, oi = native.top_p_mask_cub(vals[-1:], code, 0.9, native.HIGH_FIRST)
        assert int(oi[0]) == 1 and np.array_equal(om[0].astype(bool), vals[-1] != 0)


@pytest.mark.parametrize("first_is_max", [True, False])
def test_fp32_exact_entry_cfg3(dev, first_is_max):
    # the pruner workload (8 x 32 rows of 8192 probabilities, Zipf spikes over a normal
    # background), both p, both upper bounds: equal to the float oracle on every row
    x = synth.topp_scores(8, 32, 8192, seed=13, first_is_max=first_is_max)
    probs = _softmax(x).reshape(8, 32, 1, 8192)
    pn32 = probs.numpy().reshape(256, 8192)
    for p in (0.85, 0.95):
        for high, mode in (("first", native.HIGH_FIRST), ("max", native.HIGH_MAX)):
            om, ol, oi = native.top_p_mask_cub(pn32, native.DT_F32, p, mode)
            idx, count, mask, low, iters = K.top_p_select(probs.to(dev), p, high=high,
                                                          return_mask=True, return_stats=True,
                                                          exact=True)
            assert np.array_equal(mask.cpu().numpy().reshape(256, 8192), om.astype(bool))
            assert np.array_equal(low.cpu().numpy(), ol) and np.array_equal(iters.cpu().numpy(), oi)
            assert oi.mean() > 5 or not first_is_max
            # the default kernel (its own order of additions) keeps the same set wherever no
            # decision of the search came within rounding of p
            fast = K.top_p_fp32_return_mask(probs.to(dev), p, high=high).cpu().numpy().reshape(256, 8192)
            assert (fast == om.astype(bool)).all(-1).sum() >= 250


def test_fused_softmax_top_p_lists(dev):
    # twilight/pyimpl/top_p.py:10-15 on candidate scores with -inf slots, ragged lens, page mapping
    B, H, S = 2, 4, 40
    M = S * 16
    x = synth.topp_scores(B, H, M, seed=5, max_spikes=40)
    lens = torch.tensor([[640, 600, 16, 333], [1, 640, 500, 48]], dtype=torch.int32)
    x[0, 0, 5:9] = float("-inf")
    g = torch.Generator().manual_seed(9)
    sel = torch.stack([torch.sort(torch.randperm(200, generator=g)[:S]).values
                       for _ in range(B * H)]).reshape(B, H, S).to(torch.int32)
    xm = x.clone()
    for b in range(B):
        for h in range(H):
            xm[b, h, lens[b, h]:] = float("-inf")
    ref_in = xm.masked_fill(torch.isinf(xm), torch.finfo(torch.float32).min).reshape(B, H, 1, M)
    om, oprobs, ol, _ = P.top_p_unnormalized(ref_in, 0.9, native.HIGH_MAX)
    pn = oprobs.reshape(B * H, M).numpy()
    _, _, _, og = native.top_p_mask_f32(pn, 0.9, native.HIGH_MAX, return_margin=True)
    idx, count, probs, low = K.softmax_top_p(x.to(dev), 0.9, lens=lens.to(dev), sel_pages=sel.to(dev),
                                             high="max", return_probs=True, return_low=True)
    gp = probs.cpu().numpy().reshape(B * H, M)
    for r in range(B * H):
        n = int(lens.reshape(-1)[r])
        np.testing.assert_allclose(gp[r, :n], pn[r, :n], rtol=2e-6, atol=1e-12)
    cn = count.cpu().numpy().reshape(-1)
    ix = idx.cpu().numpy().reshape(B * H, M)
    gm = np.zeros((B * H, M), dtype=bool)
    selr = sel.reshape(B * H, S).numpy()
    for r in range(B * H):
        toks = ix[r, :cn[r]]
        assert np.all(np.diff(toks) > 0)
        # invert the page mapping: token -> candidate position
        pos = np.searchsorted(selr[r], toks // 16) * 16 + toks % 16
        assert np.array_equal(selr[r][pos // 16] * 16 + pos % 16, toks)
        gm[r, pos] = True
    assert_top_p_parity(pn, 0.9, gm, om.reshape(B * H, M).numpy(), ol, og, margin_tol=5e-6)


def test_repeatable(dev):
    x = synth.topp_scores(2, 8, 8192, seed=11).to(dev)
    a = K.softmax_top_p(x, 0.95, return_low=True)
    b = K.softmax_top_p(x, 0.95, return_low=True)
    assert torch.equal(a[1], b[1]) and torch.equal(a[2], b[2])
    ca = a[1].reshape(-1).cpu()
    ia, ib = a[0].reshape(16, -1).cpu(), b[0].reshape(16, -1).cpu()
    for r in range(16):
        assert torch.equal(ia[r, :ca[r]], ib[r, :ca[r]])


def test_errors(dev):
    p = torch.rand(2, 3, 1, 64, device=dev)
    with pytest.raises(RuntimeError):
        K.top_p_fp32_return_mask(p[..., ::2], 0.9)           # not contiguous
    with pytest.raises(RuntimeError):
        K.top_p_fp32_return_mask(p.reshape(6, 64), 0.9)       # not 4-D
    with pytest.raises(RuntimeError):
        K.top_p_fp32_return_mask(p.half(), 0.9)               # wrong dtype for the fp32 entry
    with pytest.raises(RuntimeError):
        K.top_p_fp32_return_mask(p, float("nan"))
    with pytest.raises(RuntimeError):
        K.softmax_top_p(p[:, :, 0].contiguous(), 1.5)         # not one of the reference's ops: 0 < p <= 1
    with pytest.raises(RuntimeError):
        K.top_p_fp32_return_mask(p, torch.rand(5, device=dev))


@pytest.mark.parametrize("exact", [False, True])
def test_reference_takes_any_p_and_any_qo_len(dev, exact):
    """What csrc/src/sampling.cu:22-63 does with arguments it does not check, reproduced by the
    drop-in ops: a scalar p outside (0, 1] (p >= 1: no sum reaches it, low stays 0, every positive
    probability is kept; p <= 0: every sum reaches it) and qo_len != 1 (dim 2 is ignored: the
    first batch * heads rows of the buffer are processed, the rest of the mask stays False)."""
    g = torch.Generator().manual_seed(12)
    probs = _softmax(torch.randn((2, 3, 1, 700), generator=g) * 3.0)
    probs[0, 1, 0, 5:9] = 0.0
    pn = probs.numpy().reshape(6, 700)
    for p in (1.5, 1.0, 0.0, -0.25):
        for high, mode in (("first", native.HIGH_FIRST), ("max", native.HIGH_MAX)):
            om, ol, oi = native.top_p_mask_f32(pn, p, mode)
            idx, count, mask, low, iters = K.top_p_select(probs.to(dev), p, high=high, return_mask=True,
                                                          return_stats=True, exact=exact)
            assert np.array_equal(mask.cpu().numpy().reshape(6, 700), om.astype(bool)), (p, high)
            if not exact:
                assert np.array_equal(low.cpu().numpy(), ol) and np.array_equal(iters.cpu().numpy(), oi)
            if p > 1:
                assert np.array_equal(om.astype(bool), pn > 0)
        for dt, code in ((torch.float16, 0), (torch.bfloat16, 1)):
            bits = probs.to(dt).view(torch.int16).numpy().view(np.uint16).reshape(6, 700)
            om16 = native.top_p_mask_cub(bits, code, p, native.HIGH_FIRST)[0]
            got = K.top_p_fp16_return_mask(probs.to(dt).to(dev), p).cpu().numpy().reshape(6, 700)
            assert np.array_equal(got, om16.astype(bool)), (p, dt)
    # qo_len = 3: rows 0..5 of the flattened [18, 700] buffer are the kernel's six rows
    wide = _softmax(torch.randn((2, 3, 3, 700), generator=g) * 3.0)
    om = native.top_p_mask_f32(wide.numpy().reshape(18, 700)[:6], 0.9, native.HIGH_FIRST)[0]
    got = K.top_p_fp32_return_mask(wide.to(dev), 0.9, exact=exact).cpu().numpy().reshape(18, 700)
    assert np.array_equal(got[:6], om.astype(bool)) and not got[6:].any()
    with pytest.raises(RuntimeError):
        K.top_p_select(wide.to(dev), 0.9)                     # the list form is decode-only
