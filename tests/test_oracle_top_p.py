"""Pins the oracle's top-p bisection (csrc/include/sampling.cuh:156-231) with things the
mathematics fixes: a hand-traced run, the textbook nucleus set, brute force over subsets,
degenerate rows, and the documented behaviour of the `high = probs[0]` initialisation."""
import itertools

import numpy as np
import pytest
import torch

from oracle import native
from oracle import pyimpl_port as P


def softmax_rows(x):
    return torch.softmax(torch.from_numpy(x), dim=-1, dtype=torch.float32).numpy()


def test_hand_traced_run():
    # probs [0.5,0.3,0.2], p=0.7, high=probs[0]=0.5. By hand:
    #  it1 mid=.25   S=.8>=p  -> low=.25          a=min{x>0}=.2   b=max{x<=.5}=.5   b-a=.3
    #  it2 mid=.375  S=.5<p   -> high=min(.375,b=.5)=.375   a=min{x>.25}=.3  b-a=.2
    #  it3 mid=.3125 S=.5<p   -> b=max{x<=.375}=.3 high=.3  a=.3  b-a=0 -> stop
    probs = np.array([[0.5, 0.3, 0.2]], dtype=np.float32)
    mask, low, iters = native.top_p_mask_f32(probs, 0.7, native.HIGH_FIRST)
    assert mask.tolist() == [[1, 1, 0]] and iters[0] == 3 and low[0] == np.float32(0.25)


def test_worked_example_of_the_paper_figure():
    # figures/arch.png: W = [0.5, 0.03, ., 0.02, 0.15, ., 0.04, 0.25] keeps {0.5, 0.15, 0.25};
    # their mass is exactly 0.9, so p = 0.89 keeps the test away from fp rounding of the sum.
    w = np.array([[0.5, 0.03, 0.005, 0.02, 0.15, 0.005, 0.04, 0.25]], dtype=np.float32)
    for mode in (native.HIGH_FIRST, native.HIGH_MAX):
        mask, _, _ = native.top_p_mask_f32(w, 0.89, mode)
        assert mask.tolist() == [[1, 0, 0, 0, 1, 0, 0, 1]]


def test_nucleus_is_minimal_by_brute_force():
    rng = np.random.default_rng(0)
    for trial in range(40):
        d = int(rng.integers(2, 13))
        x = softmax_rows(rng.standard_normal((1, d)).astype(np.float32) * 2)[0]
        p = float(rng.uniform(0.3, 0.98))
        mask, pivot, mass = native.nucleus(x, p)
        k = int(mask.sum())
        assert mass >= p
        # no smaller subset reaches p; the kept set is the k largest values
        best = d
        for r in range(1, d + 1):
            if any(sum(float(x[i]) for i in c) >= p for c in itertools.combinations(range(d), r)):
                best = r
                break
        assert k == best
        assert set(np.argsort(-x, kind="stable")[:k]) == set(np.nonzero(mask)[0])
        assert pivot == x[mask.astype(bool)].min()


@pytest.mark.parametrize("p", [0.5, 0.85, 0.95])
def test_bisection_vs_nucleus(p):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((64, 2048)).astype(np.float32)
    x[:, :8] += rng.uniform(4, 9, (64, 8)).astype(np.float32)   # a few heavy tokens
    probs = softmax_rows(x)
    mask, low, iters = native.top_p_mask_f32(probs, p, native.HIGH_MAX)
    assert iters.max() <= 24
    for r in range(probs.shape[0]):
        star, pivot, mass = native.nucleus(probs[r], p)
        kept = mask[r].astype(bool)
        assert probs[r][kept].astype(np.float64).sum() >= p - 1e-6       # kept mass >= p
        if abs(mass - float(probs[r][star.astype(bool)].min()) - p) < 2e-6 or abs(mass - p) < 2e-6:
            continue  # the fp32 value of a partial sum decides: not pinned by the mathematics
        assert np.all(kept >= star.astype(bool))                           # superset of S*
        extra = kept & ~star.astype(bool)
        assert np.all(probs[r][extra] > pivot - 1e-5) and np.all(probs[r][extra] < pivot)
        assert low[r] < pivot


def test_first_vs_max_and_sink_quirk():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((16, 512)).astype(np.float32)
    x[:, 0] = 8.0                       # token 0 is the row maximum: both initialisations agree
    probs = softmax_rows(x)
    m0, l0, i0 = native.top_p_mask_f32(probs, 0.9, native.HIGH_FIRST)
    m1, l1, i1 = native.top_p_mask_f32(probs, 0.9, native.HIGH_MAX)
    assert np.array_equal(m0, m1) and np.array_equal(l0, l1) and np.array_equal(i0, i1)
    # probs[0] == 0 (sink not among the candidates): the loop exits at once, nothing is pruned
    probs2 = probs.copy()
    probs2[:, 0] = 0.0
    m2, l2, i2 = native.top_p_mask_f32(probs2, 0.9, native.HIGH_FIRST)
    assert np.array_equal(m2, (probs2 > 0).astype(np.uint8)) and np.all(i2 == 1) and np.all(l2 == 0)
    # token 0 small but non-zero: a superset of the max-initialised answer, mass still >= p
    probs3 = softmax_rows(rng.standard_normal((16, 512)).astype(np.float32) * 3)
    m3, _, _ = native.top_p_mask_f32(probs3, 0.9, native.HIGH_FIRST)
    m4, _, _ = native.top_p_mask_f32(probs3, 0.9, native.HIGH_MAX)
    assert np.all(m3 >= m4)
    assert np.all((probs3 * m3).sum(-1) >= 0.9 - 1e-6)


def test_degenerate_rows():
    d = 256
    onehot = np.zeros((1, d), np.float32); onehot[0, 17] = 1.0
    m, _, _ = native.top_p_mask_f32(onehot, 0.95, native.HIGH_MAX)
    assert m.sum() == 1 and m[0, 17] == 1
    uni = np.full((1, d), 1.0 / d, np.float32)      # every element ties with the pivot: all kept
    m, _, _ = native.top_p_mask_f32(uni, 0.5, native.HIGH_MAX)
    assert m.sum() == d
    rng = np.random.default_rng(4)
    pr = softmax_rows(rng.standard_normal((4, d)).astype(np.float32))
    m, low, _ = native.top_p_mask_f32(pr, 1.0, native.HIGH_MAX)   # p = 1: everything kept
    assert np.array_equal(m, (pr > low[:, None]).astype(np.uint8))
    assert np.all((pr * m).sum(-1) >= 1.0 - 1e-5)
    z = np.zeros((2, d), np.float32)                 # an all-zero row keeps nothing
    m, _, it = native.top_p_mask_f32(z, 0.9, native.HIGH_MAX)
    assert m.sum() == 0 and np.all(it == 1)


def test_per_row_p_array():
    rng = np.random.default_rng(5)
    pr = softmax_rows(rng.standard_normal((6, 300)).astype(np.float32) * 2)
    ps = np.array([0.5, 0.6, 0.7, 0.8, 0.9, 0.99], dtype=np.float32)
    m, _, _ = native.top_p_mask_f32(pr, ps, native.HIGH_MAX)
    for r in range(6):
        mr, _, _ = native.top_p_mask_f32(pr[r:r + 1], float(ps[r]), native.HIGH_MAX)
        assert np.array_equal(m[r], mr[0])


def test_top_p_unnormalized_wrapper_shapes_and_mask_of_masked_entries():
    # twilight/pyimpl/top_p.py:10-15 + attention.py:255: entries at finfo.min get probability 0
    g = torch.Generator().manual_seed(0)
    w = torch.randn((2, 3, 1, 200), generator=g) * 3
    w[..., 100:] = torch.finfo(torch.float32).min
    mask, probs, low, iters = P.top_p_unnormalized(w, 0.9, native.HIGH_MAX)
    assert mask.shape == w.shape and mask.dtype == torch.bool
    assert not mask[..., 100:].any() and torch.all(probs[..., 100:] == 0)
    assert torch.all((probs * mask).sum(-1) >= 0.9 - 1e-6)


def test_16_bit_addition_against_numpy_and_bf16_by_bit_trick():
    # one addition of the element type, the building block of the CUB-order restatement: fp16
    # against numpy's float16 arithmetic, bf16 against fp32 addition + round-to-nearest-even of
    # the upper half (24 >= 2 * 8 + 2 bits: the double rounding is innocuous)
    rng = np.random.default_rng(5)
    a = (rng.random(3000) * 2.0 ** rng.integers(-26, 1, 3000)).astype(np.float16)
    b = (rng.random(3000) * 2.0 ** rng.integers(-26, 1, 3000)).astype(np.float16)
    for x, y in zip(a, b):
        assert native.dt_add(float(x), float(y), native.DT_F16) == float(np.float16(x + y))
    def bf(v):
        u = np.float32(v).view(np.uint32)
        return float(np.uint32(((int(u) + 0x7FFF + ((int(u) >> 16) & 1)) >> 16) << 16).view(np.float32))
    for x, y in zip(a[:1500], b[:1500]):
        xb, yb = bf(float(x)), bf(float(y))
        assert native.dt_add(xb, yb, native.DT_BF16) == bf(np.float32(xb) + np.float32(yb))
    # fp16 specials: the tolerance, a subnormal tie, overflow
    assert native.dt_round(1e-5, native.DT_F16) == 168 * 2.0 ** -24
    assert native.dt_round(1e-5, native.DT_BF16) == 168 * 2.0 ** -24
    assert native.dt_round(1.5 * 2.0 ** -24, native.DT_F16) == 2.0 ** -23
    assert native.dt_round(2.5 * 2.0 ** -24, native.DT_F16) == 2.0 ** -23
    assert native.dt_round(65520.0, native.DT_F16) == float("inf")


def test_cub_order_in_fp32_agrees_with_the_fp64_sum_form_where_the_margin_allows():
    # the float instantiation (csrc/src/sampling.cu:45-63) in CUB's order against the same
    # bisection with sums accumulated in fp64: wherever no decision came close to a rounding flip
    # both must give the same mask, pivot and iteration count
    rng = np.random.default_rng(9)
    pr = softmax_rows(rng.standard_normal((24, 5000)).astype(np.float32) * 4)
    for mode in (native.HIGH_FIRST, native.HIGH_MAX):
        m0, low0, it0, margin = native.top_p_mask_f32(pr, 0.9, mode, return_margin=True)
        m1, low1, it1 = native.top_p_mask_cub(pr, native.DT_F32, 0.9, mode)
        clear = margin > 2e-6
        assert clear.sum() >= 20
        assert np.array_equal(m0[clear], m1[clear]) and np.array_equal(low0[clear], low1[clear])
        assert np.array_equal(it0[clear], it1[clear])


def test_16_bit_rows_stay_in_the_value_set():
    rng = np.random.default_rng(6)
    pr = softmax_rows(rng.standard_normal((8, 400)).astype(np.float32) * 3).astype(np.float16)
    m, low, _ = native.top_p_mask_cub(pr.view(np.uint16), native.DT_F16, 0.9, native.HIGH_MAX)
    assert np.all(low.astype(np.float16).astype(np.float32) == low)   # pivots are fp16 values
    assert np.array_equal(m, (pr.astype(np.float32) > low[:, None]).astype(np.uint8))
    assert np.all((pr.astype(np.float64) * m).sum(-1) >= 0.9 - 5e-3)
