"""Pins the oracle's INT4 quantiser (twilight/pyimpl/quantize.py:4-13) without running the
reference: a hand-worked known-answer vector, invariants, and the fp16 helpers against numpy."""
import numpy as np
import torch

from oracle import native
from oracle import pyimpl_port as P

# input fixture of twilight/pyimpl/quantize.py:30-48; expected values worked by hand:
# min -3.56, max 4.32, scale = 7.88/15 = 0.5253333, code = round((x + 3.56)/scale)
KAT_X = [0.31, 0.42, -0.57, 0.23, -1.79, -2.18, 1.90, 4.32, -3.56, 0.78, 0.69, 1.45, 2.84,
         -2.09, -1.26]
KAT_CODES = [7, 8, 6, 7, 3, 3, 10, 15, 0, 8, 8, 10, 12, 3, 4]


def test_quant_ref_known_answer():
    x = torch.tensor(KAT_X)
    out = P.min_max_quant_ref(x, 4)
    scale = np.float32(7.88) / np.float32(15)
    expect = np.array(KAT_CODES, dtype=np.float32) * scale - np.float32(3.56)
    np.testing.assert_allclose(out.numpy(), expect, rtol=0, atol=2e-6)
    # spot values from the arithmetic done by hand
    assert abs(float(out[0]) - 0.117333) < 1e-5
    assert abs(float(out[7]) - 4.32) < 1e-5 and abs(float(out[8]) + 3.56) < 1e-6


def test_quant_ref_invariants():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((64, 128), generator=g)
    for group in (None, 32):
        y = P.min_max_quant_ref(x, 4, group)
        xv = x.reshape(64, -1, 128 if group is None else group)
        yv = y.reshape(xv.shape)
        scale = (xv.amax(-1) - xv.amin(-1)) / 15
        assert torch.all((xv - yv).abs() <= scale[..., None] / 2 + 1e-6)
        # the group minimum and maximum are reproduced
        assert torch.allclose(yv.amin(-1), xv.amin(-1), atol=1e-6)
        assert torch.allclose(yv.amax(-1), xv.amax(-1), atol=2e-6)
    # a constant row survives unchanged (scale clamps to 1e-9/15)
    c = torch.full((1, 128), 0.75)
    assert torch.equal(P.min_max_quant_ref(c, 4), c)


def test_storage_quant_known_answer_codes():
    x = np.array(KAT_X, dtype=np.float32)[None, :]
    codes, scale, zero = native.int4_quant(x, group=15)
    assert codes[0].tolist() == KAT_CODES
    assert scale[0, 0] == np.float16(7.88 / 15) and zero[0, 0] == np.float16(-3.56)
    deq = native.int4_dequant(codes, scale, zero, group=15)
    expect = np.array(KAT_CODES, np.float32) * np.float32(scale[0, 0]) + np.float32(zero[0, 0])
    assert np.array_equal(deq[0], expect)


def test_storage_quant_matches_reference_formula_up_to_fp16_rounding():
    g = torch.Generator().manual_seed(1)
    k = torch.randn((8, 16, 128), generator=g).half().float()
    codes, scale, zero, deq = P.int4_quant_storage(k)
    assert codes.max() <= 15 and codes.dtype == np.uint8
    ref = P.min_max_quant_ref(k, 4, 32).numpy()
    s = scale.astype(np.float32).repeat(32, axis=-1)
    kg = k.numpy().reshape(8, 16, 4, 32)
    mn = kg.min(-1, keepdims=True)
    ref_codes = np.rint((kg - mn) / ((kg.max(-1, keepdims=True) - mn) / 15)).reshape(8, 16, 128)
    # same function apart from the fp16 rounding of scale (rel 2^-11) and zero (rel 2^-11):
    # codes agree except where (k-min)/scale sits next to a .5 boundary, and then by one step
    diff = np.abs(codes.astype(np.int32) - ref_codes.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.02
    same = diff == 0
    tol = 16 * s * 2.0 ** -11 + np.abs(mn).repeat(32, -1).reshape(8, 16, 128) * 2.0 ** -11 + 1e-6
    assert np.all(np.abs(deq - ref)[same] <= tol[same])
    err = np.abs(deq - k.numpy())
    assert np.all(err <= s * 0.5 + 2e-3)
    # dequantised values are exactly code*scale+zero in fp32
    z = zero.astype(np.float32).repeat(32, axis=-1)
    assert np.array_equal(deq, codes.astype(np.float32) * s + z)


def test_storage_quant_degenerate_groups():
    k = np.zeros((3, 128), dtype=np.float32)
    k[1] = 0.5                      # constant group: scale floors at 2^-14, codes 0
    k[2, :32] = np.linspace(-1, 1, 32)
    codes, scale, zero = native.int4_quant(k, 32)
    assert np.all(codes[0] == 0) and np.all(codes[1] == 0)
    assert np.all(scale[1] == np.float16(2.0 ** -14)) and np.all(zero[1] == np.float16(0.5))
    deq = native.int4_dequant(codes, scale, zero, 32)
    assert np.array_equal(deq[1], k[1]) and np.array_equal(deq[0], k[0])
    assert codes[2, 0] == 0 and codes[2, 31] == 15


def test_fp16_helpers_match_numpy():
    L = native.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(2000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 2000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0001, 2.0 ** -14, 6.1e-5, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11],
                 dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.twl_oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    allh = np.arange(0, 0x7C00, 7, dtype=np.uint16)
    back = np.array([L.twl_oracle_f16_to_f32(int(h)) for h in allh], dtype=np.float32)
    assert np.array_equal(back, allh.view(np.float16).astype(np.float32))
    bf = torch.tensor(vals[:2000]).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    gotb = np.array([L.twl_oracle_f32_to_bf16(float(v)) for v in vals[:2000]], dtype=np.uint16)
    assert np.array_equal(gotb, bf)


def test_record_pack_roundtrip_and_nibble_order():
    rng = np.random.default_rng(3)
    codes = rng.integers(0, 16, (3, 2, 16, 128), dtype=np.uint8)
    scale = rng.uniform(0.01, 0.1, (3, 2, 16, 4)).astype(np.float16)
    zero = rng.uniform(-1, 0, (3, 2, 16, 4)).astype(np.float16)
    rec = P.pack_int4_records(codes, scale, zero)
    assert rec.shape == (3, 2, 1280)
    c2, s2, z2 = P.unpack_int4_records(rec)
    assert np.array_equal(c2, codes) and np.array_equal(s2, scale) and np.array_equal(z2, zero)
    # every value in every nibble slot of a 32-bit word: element j sits in bits [4(j%8), +4) of word j//8
    for slot in range(8):
        for val in range(16):
            c = np.zeros((1, 1, 16, 128), dtype=np.uint8)
            c[0, 0, 5, 40 + slot] = val
            r = P.pack_int4_records(c, np.zeros((1, 1, 16, 4), np.float16), np.zeros((1, 1, 16, 4), np.float16))
            words = r[0, 0, :1024].view("<u4")
            assert words[5 * 16 + 5] == (val << (4 * slot))
            assert words.astype(np.uint64).sum() == (val << (4 * slot))
    # (scale, zero) pair of token t, group g at byte 1024 + 4*(4t+g)
    sz = rec[1, 1, 1024:].view(np.float16).reshape(16, 4, 2)
    assert sz[7, 2, 0] == scale[1, 1, 7, 2] and sz[7, 2, 1] == zero[1, 1, 7, 2]
