"""Shared assertions of the GPU parity tests (tolerances as stated in each docstring)."""
import numpy as np


def assert_top_p_parity(probs, p, gpu_mask, ora_mask, ora_low, ora_margin, gpu_low=None,
                        margin_tol=2e-6, band=1e-5):
    """The pruned set must equal the oracle's except for tokens whose probability lies within
    ``band`` (1e-5, the kernel's own stopping tolerance) of the threshold, and the kept mass must
    be >= p. Rows where some bisection decision had |S - p| < ``margin_tol`` are decided by fp32
    summation order: for them only the structural properties are required."""
    probs = np.asarray(probs, dtype=np.float32)
    gpu_mask = np.asarray(gpu_mask).astype(bool)
    ora_mask = np.asarray(ora_mask).astype(bool)
    rows = probs.shape[0]
    p_arr = np.broadcast_to(np.asarray(p, dtype=np.float64), (rows,))
    n_exact = 0
    for r in range(rows):
        kept = gpu_mask[r]
        mass = probs[r][kept].astype(np.float64).sum()
        assert mass >= p_arr[r] - 2e-6, f"row {r}: kept mass {mass} < p {p_arr[r]}"
        if kept.any() and (~kept).any():
            # a threshold set: nothing dropped is larger than something kept (beyond rounding)
            assert probs[r][~kept].max() <= probs[r][kept].min() * (1 + 1e-5) + 1e-12, f"row {r}"
        if np.array_equal(kept, ora_mask[r]):
            n_exact += 1
            if gpu_low is not None and ora_margin[r] >= margin_tol:
                assert gpu_low[r] == ora_low[r], f"row {r}: low {gpu_low[r]} vs {ora_low[r]}"
            continue
        diff = kept != ora_mask[r]
        if ora_margin[r] < margin_tol:
            continue
        thr = ora_low[r]
        assert np.all(np.abs(probs[r][diff] - thr) <= band), \
            f"row {r}: {diff.sum()} tokens differ outside the {band} band around {thr}"
    return n_exact


def assert_scores_close(got, want, rtol=1e-3, atol_frac=1e-4):
    """Scores agree within 1e-3 relative; entries much smaller than the row's typical score (where
    a relative bound is meaningless under cancellation) get an absolute bound of ``atol_frac``
    times the row RMS."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    finite = np.isfinite(want)
    assert np.array_equal(finite, np.isfinite(got))
    assert np.array_equal(got[~finite], want[~finite])
    w = np.where(finite, want, 0.0)
    rms = np.sqrt((w ** 2).sum(-1, keepdims=True) / np.maximum(finite.sum(-1, keepdims=True), 1))
    err = np.abs(np.where(finite, got, 0.0) - w)
    bound = rtol * np.abs(w) + atol_frac * rms + 1e-30
    bad = err > bound
    assert not bad.any(), f"{bad.sum()} scores off; worst err {err.max()} (bound {bound[bad].min()})"
