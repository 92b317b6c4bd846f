"""The known-answer vectors of tests/golden/known_answers.json (written by
tests/golden/make_fixtures.py from the closed forms the reference states, without running the
reference or the oracle) against the oracle on the CPU and against the HIP path through the C ABI."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import native
from oracle import pyimpl_port as P

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")) as f:
    KA = json.load(f)


def test_fixture_file_is_what_the_generator_writes():
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        "make_fixtures", os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_fixtures.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    assert m.int4_quant() == KA["int4_quant"] and m.top_p_figure() == KA["top_p_figure"]
    assert m.top_p_trace() == KA["top_p_trace"] and m.gemv_constant() == KA["gemv_constant"]
    assert m.top_p_dyadic() == KA["top_p_dyadic"]
    assert m.top_p_cub_order() == KA["top_p_cub_order"]


def test_oracle_quantiser_on_the_reference_vector():
    k = KA["int4_quant"]
    out = P.min_max_quant_ref(torch.tensor(k["x"]), 4)                      # quantize.py:4-13
    np.testing.assert_allclose(out.numpy(), np.array(k["dequant"], np.float32), rtol=0, atol=3e-6)
    codes, scale, zero = native.int4_quant(np.array(k["x"], np.float32)[None], group=15)
    assert codes[0].tolist() == k["codes"]
    assert scale[0, 0] == np.float16(k["scale"]) and zero[0, 0] == np.float16(k["min"])


def test_oracle_top_p_on_the_figure_and_the_hand_trace():
    fig = KA["top_p_figure"]
    w = np.array([fig["weights"]], np.float32)
    for mode in (native.HIGH_FIRST, native.HIGH_MAX):
        mask, _, _ = native.top_p_mask_f32(w, fig["p"], mode)
        assert np.nonzero(mask[0])[0].tolist() == fig["keep"]
    tr = KA["top_p_trace"]
    mask, low, iters = native.top_p_mask_f32(np.array([tr["probs"]], np.float32), tr["p"], native.HIGH_FIRST)
    assert mask[0].tolist() == tr["mask"] and iters[0] == tr["iterations"] and low[0] == np.float32(tr["low"])


def test_oracle_top_p_on_the_dyadic_rows_in_every_width():
    # exact in fp32, fp16 and bf16: the one known answer for the 16-bit restatement
    dy = KA["top_p_dyadic"]
    for r in dy["rows"]:
        pr = np.array([r["probs"]], np.float32)
        for mode in (native.HIGH_FIRST, native.HIGH_MAX):
            mask, low, iters = native.top_p_mask_f32(pr, dy["p"], mode)
            assert mask[0].tolist() == r["mask"] and low[0] == np.float32(r["low"])
            assert iters[0] == r["iterations"]
            bits16 = pr.astype(np.float16).view(np.uint16)
            bitsbf = (pr.view(np.uint32) >> 16).astype(np.uint16)          # exact: dyadic values
            for bits, code in ((bits16, 0), (bitsbf, 1)):
                m16, low16, it16 = native.top_p_mask_cub(bits, code, dy["p"], mode)
                assert m16[0].tolist() == r["mask"] and float(low16[0]) == r["low"]
                assert it16[0] == r["iterations"]


def _cub_row(r):
    """(bits uint16 [1, d], dtype code, high mode) of one ``top_p_cub_order`` fixture row."""
    code = {"f16": 0, "bf16": 1, "f32": 2}[r["dtype"]]
    bits = np.zeros((1, r["d"]), np.uint32 if code == 2 else np.uint16)
    for i, b in r["nonzero"]:
        bits[0, i] = b
    if code == 2:
        bits = bits.view(np.float32)          # the float oracle takes the values themselves
    return bits, code, (native.HIGH_FIRST if r["high"] == "first" else native.HIGH_MAX)


def _low_bits(low: float, code: int) -> int:
    if code == 0:
        return int(np.float32(low).astype(np.float16).view(np.uint16))
    if code == 2:
        return int(np.float32(low).view(np.uint32))
    return int(np.float32(low).view(np.uint32) >> 16)


def test_oracle_top_p_in_16_bit_arithmetic_and_cub_order():
    # rows followed in exact rational arithmetic with explicit rounding; each one comes out
    # differently under at least one plausible mistake (see make_fixtures.top_p_cub_order)
    rows = KA["top_p_cub_order"]["rows"]
    seen = set()
    for r in rows:
        bits, code, mode = _cub_row(r)
        mask, low, iters = native.top_p_mask_cub(bits, code, r["p"], mode)
        assert np.nonzero(mask[0])[0].tolist() == r["kept"], (r["dtype"], r["d"])
        assert _low_bits(low[0], code) == r["low_bits"] and iters[0] == r["iterations"]
        seen |= {(r["dtype"], a) for a in r["differs_under"]}
    for fmt in ("f16", "bf16", "f32"):
        for alt in ("exact_sums", "flat_sum", "thread_tree", "warp_tree", "chunks_merged",
                    "exact_mid", "exact_eps"):
            # (no float lies between 1e-5 and its float rounding: that mistake cannot show there)
            assert (fmt, alt) in seen or (fmt, alt) == ("f32", "exact_eps")


def test_oracle_estimator_on_the_constant_inputs():
    c = KA["gemv_constant"]
    deq = native.int4_dequant(np.full((1, c["head_dim"]), c["nibble"], np.uint8),
                              np.full((1, 4), c["scale"], np.float16), np.full((1, 4), c["zero"], np.float16))
    q = torch.full((1, 1, 1, c["head_dim"]), c["q"])
    assert float(P.estimator_scores(q, torch.from_numpy(deq)[None, None], sm_scale=1.0)) == c["raw_score"]


@pytest.mark.gpu
def test_hip_top_p_on_the_figure_and_the_hand_trace(dev):
    import twilight_amd.kernel as K
    fig = KA["top_p_figure"]
    w = torch.tensor(fig["weights"], dtype=torch.float32, device=dev).reshape(1, 1, 1, -1)
    mask = K.top_p_fp32_return_mask(w, fig["p"])
    assert torch.nonzero(mask[0, 0, 0]).flatten().tolist() == fig["keep"]
    idx, count = K.top_p_select(w, fig["p"])
    assert idx[0, 0, :int(count[0, 0])].tolist() == fig["keep"]
    tr = KA["top_p_trace"]                                  # token 0 is the maximum: both bounds agree
    pr = torch.tensor(tr["probs"], dtype=torch.float32, device=dev).reshape(1, 1, 1, -1)
    assert K.top_p_fp32_return_mask(pr, tr["p"])[0, 0, 0].int().tolist() == tr["mask"]


@pytest.mark.gpu
def test_hip_top_p_on_the_dyadic_rows_in_every_width(dev):
    import twilight_amd.kernel as K
    dy = KA["top_p_dyadic"]
    pr = torch.tensor([r["probs"] for r in dy["rows"]], dtype=torch.float32, device=dev)
    pr = pr.reshape(1, len(dy["rows"]), 1, -1)
    want = torch.tensor([r["mask"] for r in dy["rows"]], dtype=torch.bool)
    for high in ("first", "max"):
        assert torch.equal(K.top_p_fp32_return_mask(pr, dy["p"], high=high)[0, :, 0].cpu(), want)
        idx, count, low, iters = K.top_p_select(pr, dy["p"], high=high, return_stats=True)
        assert low.flatten().tolist() == [r["low"] for r in dy["rows"]]
        assert iters.flatten().tolist() == [r["iterations"] for r in dy["rows"]]
        for dt in (torch.float16, torch.bfloat16):
            m16 = K.top_p_fp16_return_mask(pr.to(dt), dy["p"], high=high)
            assert torch.equal(m16[0, :, 0].cpu(), want)


@pytest.mark.gpu
def test_hip_top_p_in_16_bit_arithmetic_and_cub_order(dev):
    import twilight_amd.kernel as K
    for r in KA["top_p_cub_order"]["rows"]:
        bits, code, _ = _cub_row(r)
        if code == 2:
            t = torch.from_numpy(bits)
        else:
            t = torch.from_numpy(bits.view(np.int16)).view(torch.float16 if code == 0 else torch.bfloat16)
        t = t.reshape(1, 1, 1, -1).to(dev)
        idx, count, mask, low, iters = K.top_p_select(t, r["p"], high=r["high"], return_mask=True,
                                                      return_stats=True, exact=True)
        kept = torch.nonzero(mask[0, 0, 0]).flatten().tolist()
        assert kept == r["kept"], (r["dtype"], r["d"], r["differs_under"])
        assert idx[0, 0, :int(count[0, 0])].tolist() == r["kept"]
        assert _low_bits(float(low[0]), code) == r["low_bits"] and int(iters[0]) == r["iterations"]
        if code == 2:
            assert torch.equal(K.top_p_fp32_return_mask(t, r["p"], high=r["high"], exact=True), mask)
        else:
            assert torch.equal(K.top_p_fp16_return_mask(t, r["p"], high=r["high"]), mask)


@pytest.mark.gpu
def test_hip_quantiser_on_the_reference_vector(dev):
    import twilight_amd.kernel as K
    k = KA["int4_quant"]
    # one page, one kv head; token 0's first quantisation group holds the vector twice and its
    # first two values once more (same minimum and maximum), everything else is zero
    x = torch.tensor(k["x"] + k["x"] + k["x"][:2], dtype=torch.float16)
    page = torch.zeros((1, 16, 1, 128), dtype=torch.float16)
    page[0, 0, 0, :32] = x
    page = page.to(dev)
    rec = torch.zeros((1, 1, 1280), dtype=torch.uint8, device=dev)
    K.kv_shadow_build(page, rec, None)
    nib = rec[0, 0, :16].cpu().numpy()                      # token 0, elements 0..31
    codes = np.stack([nib & 15, nib >> 4], axis=-1).reshape(-1)
    assert codes[:15].tolist() == k["codes"] and codes[15:30].tolist() == k["codes"]
    sz = rec[0, 0, 1024:1028].cpu().numpy().view(np.float16)
    assert sz[0] == np.float16(k["scale"]) and sz[1] == np.float16(k["min"])
    deq = K.dequant_int4(rec)[0, 0, 0, :15].cpu().numpy()
    # storage form: fp16 scale and zero, one fp32 rounding of code * scale + zero
    want = np.array(k["codes"], np.float32) * np.float32(sz[0]) + np.float32(sz[1])
    assert np.array_equal(deq, want)
    np.testing.assert_allclose(deq, np.array(k["dequant"], np.float32), atol=0.5 * 2 ** -9 * 16)


@pytest.mark.gpu
def test_hip_estimator_on_the_constant_inputs(dev):
    import twilight_amd.kernel as K
    from twilight_amd import synth
    c = KA["gemv_constant"]
    H, pages = 2, 3
    rec = np.zeros((pages, H, 1280), np.uint8)
    rec[:, :, :1024] = c["nibble"] | (c["nibble"] << 4)
    sz = np.tile(np.array([c["scale"], c["zero"]], np.float16), 64)
    rec[:, :, 1024:] = sz.view(np.uint8)
    ids, indptr, last = synth.identity_page_table(1, pages, 16, dev)
    q = torch.full((1, H, 128), c["q"], dtype=torch.float16, device=dev)
    scores, cnt = K.sparse_gemv_int4(q, torch.from_numpy(rec).to(dev), ids, indptr, last,
                                     max_pages=pages, sm_scale=1.0)
    assert int(cnt.min()) == pages * 16
    assert torch.all(scores[:, :, :pages * 16] == c["raw_score"])
