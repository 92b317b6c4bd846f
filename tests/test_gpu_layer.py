"""End-to-end GPU parity of the decode layer (select -> INT4 estimate -> top-p -> attention)
against the oracle's dense-masked restatement of twilight/pyimpl/attention.py:188-306."""
import os

import numpy as np
import pytest
import torch

from oracle import native
from oracle import pyimpl_port as P
from twilight_amd import synth
from twilight_amd.cache import PagedKVCache
from twilight_amd.layer import TwilightDecodeLayer
from _checks import assert_scores_close, assert_top_p_parity

pytestmark = pytest.mark.gpu


def _lists_to_mask(idx, count, N):
    rows = idx.shape[0]
    m = np.zeros((rows, N), dtype=bool)
    for r in range(rows):
        m[r, idx[r, :count[r]]] = True
    return m


def _pages_to_mask(sel, selc, npg):
    """Page lists [rows, k] with counts -> bool token mask [rows, npg * 16]."""
    m = np.zeros((sel.shape[0], npg * 16), dtype=bool)
    for r in range(sel.shape[0]):
        for pg in sel[r, :selc[r]]:
            m[r, pg * 16:(pg + 1) * 16] = True
    return m


def _assert_selection_ties(page_scores, gpu_pages, ora_mask0, npg):
    """A page on one side of the selection only must score within 1e-3 * max(1, |k-th|) of the
    oracle's k-th page score (the two top-k sets differ by ties at the boundary only)."""
    padded = np.zeros(npg * 16, dtype=bool)
    padded[:ora_mask0.size] = ora_mask0.reshape(-1)
    ora_pages = set(np.nonzero(padded.reshape(npg, 16).any(-1))[0].tolist())
    mine = set(int(x) for x in gpu_pages)
    assert len(mine) == len(ora_pages)
    kth = float(torch.sort(page_scores, descending=True).values[len(ora_pages) - 1])
    for pg in ora_pages.symmetric_difference(mine):
        assert abs(float(page_scores[pg]) - kth) <= 1e-3 * max(1.0, abs(kth)), (pg, float(page_scores[pg]), kth)


def _run_case(dev, B, H, Hkv, N, budget, p, dt, seed, shuffle=True, n_heavy=16, fused=True,
              planes=False, rate=-1, use_est=False, group_select=False, high="max", sink=None):
    q, k, v = synth.heavy_hitter_qkv(B, H, N, n_heavy=n_heavy, mass=0.6, seed=seed, dtype=dt)
    group = H // Hkv
    if sink is not None:
        # an attention sink: token 0 of every kv head leans towards its group's first query
        k[:, :, 0] = (k[:, :, 0] + sink * q[:, ::group, 0].repeat_interleave(group, dim=1)).to(dt).float()
    HM = native.HIGH_FIRST if high == "first" else native.HIGH_MAX
    kk, vv = k[:, ::group].contiguous(), v[:, ::group].contiguous()        # one K/V per kv head
    npg = (N + 15) // 16
    perm = torch.randperm(B * npg, generator=torch.Generator().manual_seed(seed)) if shuffle else None
    cache = PagedKVCache.from_dense(kk.to(dt), vv.to(dt), dev, page_perm=perm,
                                    plane_pages=npg if planes else None)
    layer = TwilightDecodeLayer(cache, H, token_budget=budget, top_p=p, high=high,
                                fused_estimator=fused, keep_scores=True, sparsity_rate=rate,
                                use_estimated_weights=use_est, group_select=group_select)
    if rate != -1:
        budget = int(N * rate)                                              # quest.py:45-46
    out = layer(q[:, :, 0].to(dt).to(dev)).cpu().float()
    krep = kk.repeat_interleave(group, dim=1)                               # attention.py:124-126
    vrep = vv.repeat_interleave(group, dim=1)
    ref = P.decode_layer_dense(q, krep, vrep, top_p=p, token_budget=budget if budget < N else None,
                               high_mode=HM, quant="storage", prob_dtype=dt,
                               sparsity_rate=rate, use_estimated_weights=use_est)
    est_pg = None
    if group_select:
        # one candidate list per kv head: the oracle's group selection replaces the per-head one
        gmask, gsc = P.quest_selector_group_dense(q.float(), krep.float(), 16, budget, group)
        est_pg = gsc[:, :, 0].reshape(B * H, -1)
        ref = P.decode_layer_dense(q, krep, vrep, top_p=p, token_budget=budget, high_mode=HM,
                                   quant="storage", prob_dtype=dt, use_estimated_weights=use_est,
                                   mask0=gmask)
    rows = B * H
    # 1. selector: the oracle's pages, except pages whose score ties the k-th within rounding
    #    (checked on the oracle's own page scores); the later stages are then followed on the
    #    GPU's own selection, for every row
    sel = layer.sel_pages.cpu().numpy().reshape(rows, -1)
    selc = layer.sel_count.cpu().numpy().reshape(rows)
    mask0 = ref["mask0"].reshape(rows, N).numpy()
    gmask0 = _pages_to_mask(sel, selc, npg)[:, :N]
    differ = np.nonzero((gmask0 != mask0).any(-1))[0]
    if group_select:
        assert (sel.reshape(B, Hkv, group, -1) == sel.reshape(B, Hkv, group, -1)[:, :, :1]).all()
    if differ.size:
        if est_pg is None:
            est_pg = P.quest_chunk_scores_dense(q.float(), krep.float(), 16)[:, :, 0].reshape(rows, -1)
        for r in differ:
            _assert_selection_ties(est_pg[r], sel[r, :selc[r]], mask0[r], npg)
        ref = P.decode_layer_dense(q, krep, vrep, top_p=p, token_budget=budget, high_mode=HM,
                                   quant="storage", prob_dtype=dt, use_estimated_weights=use_est,
                                   mask0=torch.from_numpy(gmask0).reshape(B, H, 1, N))
    # 2. estimator scores on the selected candidates (1e-3 relative)
    scores = layer.scores.cpu().numpy().reshape(rows, -1)
    est = ref["scores"].reshape(rows, N).double().numpy()
    cand_tok = (sel[:, :, None] * 16 + np.arange(16)[None, None, :]).reshape(rows, -1)
    for r in range(rows):
        n = selc[r] * 16
        tok = cand_tok[r, :n]
        inside = tok < N
        assert_scores_close(scores[r, :n][inside][None], est[r, tok[inside]][None])
        assert np.all(np.isneginf(scores[r, :n][~inside]))
    # 3. pruned index lists (identical except within 1e-5 of the threshold; kept mass >= p)
    idx = layer.idx.cpu().numpy().reshape(rows, -1)
    cnt = layer.count.cpu().numpy().reshape(rows)
    gm = _lists_to_mask(idx, cnt, N)
    probs = ref["probs"].reshape(rows, N).numpy()
    _, _, _, margin = native.top_p_mask_f32(probs, p, HM, return_margin=True)
    assert_top_p_parity(probs, p, gm, ref["mask"].reshape(rows, N).numpy(), ref["low"], margin,
                        margin_tol=5e-6)
    # 4. attention: exact over the GPU's own survivors, and end to end against the oracle
    tol = 1e-3 if dt == torch.float16 else 8e-3
    if use_est:
        # the estimator's probability of every survivor, in list order beside idx
        sp = layer.surv_probs.cpu().numpy().reshape(rows, -1)
        for r in range(rows):
            np.testing.assert_allclose(sp[r, :cnt[r]], probs[r, idx[r, :cnt[r]]], rtol=1e-4, atol=1e-9)
    own = P.masked_attention(q, krep, vrep, torch.from_numpy(gm).reshape(B, H, 1, N), prob_dtype=dt,
                             logits=ref["scores"] if use_est else None)
    assert torch.allclose(out, own[:, :, 0], rtol=tol, atol=tol)
    e2e = (out.reshape(rows, 128) - ref["out"].reshape(rows, 128)).abs().max().item()
    assert e2e < 5 * tol, e2e
    return layer, ref


@pytest.mark.parametrize("fused", [True, False])
def test_cfg1_full_context(dev, fused):
    # the reference's CPU-runnable case: B=1, 32 heads MHA, D=128, N=4096, 16 heavy hitters with ~60 % of the mass,
    # all tokens are candidates, p = 0.95
    layer, ref = _run_case(dev, 1, 32, 32, 4096, 4096, 0.95, torch.float16, seed=0, fused=fused)
    cnt = layer.count.cpu().float()
    assert 16 <= cnt.min() and cnt.mean() < 4096 * 0.8


@pytest.mark.parametrize("B,H,Hkv,N,budget,p,dt", [
    (2, 8, 8, 2048, 512, 0.95, torch.float16),     # Longchat-7B shape in the small (MHA)
    (2, 8, 2, 2048, 512, 0.90, torch.bfloat16),    # Llama-3-8B shape in the small (GQA 4:1, bf16)
    (3, 4, 4, 1000, 250, 0.85, torch.float16),     # ragged: partial last page, budget not /16
    (1, 4, 1, 100, 8192, 0.95, torch.float16),     # budget larger than the context
])
@pytest.mark.parametrize("fused", [True, False])
def test_small_layer_configs(dev, B, H, Hkv, N, budget, p, dt, fused):
    _run_case(dev, B, H, Hkv, N, budget, p, dt, seed=B * 100 + H, n_heavy=8, fused=fused)


@pytest.mark.parametrize("B,H,Hkv,N,budget,dt,fused,planes", [
    (2, 8, 8, 2048, 512, torch.float16, True, False),     # estimator + pruner in one launch
    (2, 8, 8, 2048, 512, torch.float16, False, False),    # every stage its own launch
    (8, 32, 32, 1024, 256, torch.float16, True, True),    # the one-launch row kernel
    (2, 8, 2, 2048, 512, torch.bfloat16, True, False),    # GQA
])
@pytest.mark.parametrize("sink", [None, 0.6, 1.5])
def test_layer_high_first_is_the_reference_bound(dev, B, H, Hkv, N, budget, dt, fused, planes, sink):
    """high="first": the bisection starts from the probability of TOKEN 0 of the context, as
    csrc/include/sampling.cuh:156-159 does on the full-length row that attention.py:274-278 hands
    it. Without a sink page 0 is rarely among the selected pages: token 0 then has probability 0,
    the loop ends at once and every candidate with a positive probability is kept. With a sink
    token 0 is a candidate; a moderate one (0.6, about as heavy as the planted tokens) is often
    not the row maximum, so the result is a superset of the minimal set; a strong one (1.5) is
    the maximum. With q heads sharing kv heads the sink leans towards the group's first query."""
    layer, ref = _run_case(dev, B, H, Hkv, N, budget, 0.9, dt, seed=11 * B + H, n_heavy=8, fused=fused,
                           planes=planes, high="first", sink=sink)
    rows = B * H
    sel = layer.sel_pages.cpu().numpy().reshape(rows, -1)
    cnt = layer.count.cpu().numpy().reshape(rows)
    cand = layer.cand_count.cpu().numpy().reshape(rows)
    no_page0 = sel[:, 0] != 0
    if sink is None:
        assert no_page0.any()
        # nothing is pruned in those rows (probabilities that underflow to 0 aside)
        probs = ref["probs"].reshape(rows, N).numpy()
        assert np.array_equal(cnt[no_page0], (probs[no_page0] > 0).sum(-1))
        assert (cnt[no_page0] >= 0.9 * np.minimum(cand[no_page0], N)).all()
    else:
        lead = (np.arange(rows) % H) % (H // Hkv) == 0      # the rows the sink was planted for
        with0 = lead & ~no_page0
        assert with0.sum() >= 0.5 * lead.sum()      # the sink page is selected in most rows
        assert (cnt[with0] < cand[with0]).all()     # and there the search prunes


@pytest.mark.parametrize("B,H,Hkv,N,budget", [
    (2, 8, 8, 2048, 512),    # 16 rows: separate launches, page scores from the plane layout
    (8, 32, 32, 1024, 256),  # 256 rows: the one-launch row kernel reading the plane layout
    (8, 32, 8, 1024, 256),   # the same with 4 q heads per kv head (a group's rows share an XCD)
    (2, 8, 2, 2048, 512),    # GQA, 16 rows: separate launches, records (planes present, unused)
])
def test_layer_with_plane_metadata(dev, B, H, Hkv, N, budget):
    _run_case(dev, B, H, Hkv, N, budget, 0.95, torch.float16, seed=B + N, n_heavy=8, planes=True)


@pytest.mark.parametrize("B,H,Hkv,planes", [
    (20, 32, 32, True),    # 640 rows, planes: the row kernel beyond two rows per compute unit
    (20, 32, 32, False),   # 640 rows, records: scores, top-k and fused estimator as three launches
    (6, 32, 8, True),      # 192 rows, 4 q heads per kv head, planes: row kernel, groups per XCD
    (5, 28, 4, True),      # 140 rows, 7 q heads per kv head: rows stay in launch order
    (4, 32, 8, True),      # 128 rows with GQA: every stage its own launch
    (3, 32, 32, True),     # 96 rows: every stage its own launch, short GEMV wavefronts
])
def test_layer_dispatch_regimes(dev, B, H, Hkv, planes):
    """One case per branch of the layer's choice of launches (by rows per compute unit, GQA and
    metadata layout): every branch gives the oracle's result."""
    _run_case(dev, B, H, Hkv, 512, 128, 0.9, torch.float16, seed=B * H + Hkv, n_heavy=4,
              planes=planes)


@pytest.mark.parametrize("B,H,Hkv,N,budget,dt,fused,planes", [
    (1, 32, 32, 4096, 4096, torch.float16, True, False),   # every token a candidate, few rows
    (8, 32, 32, 1024, 256, torch.float16, True, True),     # the one-launch row kernel
    (20, 32, 32, 512, 128, torch.bfloat16, True, False),   # estimator + pruner in one launch
    (2, 8, 2, 2048, 512, torch.bfloat16, False, False),    # every stage its own launch, GQA
    (3, 4, 4, 1000, 250, torch.float16, True, False),      # ragged, budget not a page multiple
])
def test_layer_attention_on_estimated_weights(dev, B, H, Hkv, N, budget, dt, fused, planes):
    """use_estimated_weights_in_attn (attention.py:295-296): the survivors' estimator
    probabilities are emitted beside the index lists and weigh V; K is not read again."""
    _run_case(dev, B, H, Hkv, N, budget, 0.95, dt, seed=7 * B + H, n_heavy=8, fused=fused,
              planes=planes, use_est=True)


def test_layer_estimated_weights_long_rows(dev):
    """Rows of more than 128 survivors (flat attention: no heavy tokens, p close to 1) take the
    split path of the weighted attention and its merge."""
    layer, _ = _run_case(dev, 2, 8, 8, 4096, 2048, 0.99, torch.float16, seed=5, n_heavy=0,
                         use_est=True)
    assert int(layer.count.max()) > 256


@pytest.mark.parametrize("B,H,Hkv,N,budget,dt", [
    (2, 8, 2, 2048, 512, torch.bfloat16),     # Llama-3 grouping in the small
    (8, 32, 8, 1024, 256, torch.float16),     # 256 rows
    (3, 8, 4, 1000, 250, torch.float16),      # two q heads per kv head, ragged
    (1, 8, 1, 600, 100, torch.bfloat16),      # eight q heads on one kv head
    (2, 4, 4, 512, 128, torch.float16),       # no grouping: the option changes nothing
])
def test_layer_group_select(dev, B, H, Hkv, N, budget, dt):
    """group_select: one Quest selection per kv head (largest q-head score per page), records read
    once per kv head; every later stage per q head as before."""
    _run_case(dev, B, H, Hkv, N, budget, 0.9, dt, seed=3 * B + H + Hkv, n_heavy=6, group_select=True)


@pytest.mark.parametrize("N,rate,planes", [(2048, 0.25, False), (1000, 0.13, True), (300, 0.0, False),
                                           (777, 1.0, False)])
def test_layer_sparsity_rate(dev, N, rate, planes):
    """selector.sparsity_rate (quest.py:45-46): the budget follows the context length."""
    layer, ref = _run_case(dev, 2, 8, 8, N, 99999, 0.9, torch.float16, seed=N, n_heavy=4, planes=planes,
                           rate=rate)
    kc = P.quest_chunk_budget(int(N * rate), 16, (N + 15) // 16)
    assert (layer.sel_count.cpu().numpy() == kc).all()


def test_sparsity_rate_follows_appends(dev):
    """The budget is recomputed from the host-side length every step."""
    B, H, N = 2, 4, 160
    q, k, v = synth.heavy_hitter_qkv(B, H, N, n_heavy=2, mass=0.5, seed=3, dtype=torch.float16)
    k, v = k.half(), v.half()
    cache = PagedKVCache.from_dense(k, v, dev, spare_pages=8)
    layer = TwilightDecodeLayer(cache, H, top_p=0.9, sparsity_rate=0.5, reserve_pages=20)
    qd = q[:, :, 0].half().to(dev)
    layer(qd)
    assert (layer.sel_count.cpu().numpy() == 5).all()                 # int(160 * 0.5) = 80 tokens
    free = list(range(cache.num_pages - 8, cache.num_pages))
    for _ in range(33):                                               # 193 tokens: budget 96
        cache.append(k[:, :, 0].to(dev), v[:, :, 0].to(dev), free)
    layer(qd)
    assert (layer.sel_count.cpu().numpy() == P.quest_chunk_budget(96, 16, 13)).all()


@pytest.mark.parametrize("seed", range(int(os.environ.get("TWL_RANDOM_SHAPES", "12"))))
def test_layer_random_shapes(dev, seed):
    """Shapes drawn at random (batch, head counts and grouping, context with a partial last page,
    budget, p, dtype, metadata layout, fused / split launches): every draw against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    Hkv = int(rng.choice([1, 2, 3, 4, 8]))
    H = Hkv * int(rng.choice([1, 1, 2, 4, 7]))
    B = int(rng.integers(1, 9))
    N = int(rng.integers(20, 1500)) if seed % 3 else int(rng.integers(1500, 9000))
    budget = int(rng.choice([16, 40, 128, 300, 512, 4096]))
    p = float(rng.choice([0.5, 0.85, 0.9, 0.95, 0.99]))
    dt = torch.float16 if rng.random() < 0.6 else torch.bfloat16
    _run_case(dev, B, H, Hkv, N, budget, p, dt, seed=seed, n_heavy=int(rng.integers(1, 12)),
              fused=bool(rng.random() < 0.7), planes=bool(rng.random() < 0.5))


def test_layer_at_128k_context(dev):
    # 8192 pages per request: the widest selector shapes (8 pages per thread in the radix select,
    # four scoring passes over the plane layout), 512 selected pages, against the dense oracle
    _run_case(dev, 1, 4, 4, 131072, 8192, 0.95, torch.float16, seed=77, n_heavy=12, planes=True)
    from twilight_amd.cache import PagedKVCache as C
    g = torch.Generator().manual_seed(78)
    k = torch.randn((1, 2, 131072, 128), generator=g).half()
    cache = C.from_dense(k, k, dev, plane_pages=8192)
    q = torch.randn((1, 2, 128), generator=g).half().to(dev)
    tab = (cache.kv_page_indices, cache.kv_page_indptr, cache.kv_last_page_len)
    import twilight_amd.kernel as K
    a = K.quest_gemv_int4_top_p(q, cache.meta, cache.k_int4, *tab, 8192, 8192, 0.9, return_scores=True,
                                meta_planes=cache.meta_planes)
    sel, selc, ps = K.quest_select(q, cache.meta, *tab[:2], 8192, 8192)
    assert torch.allclose(a[5], ps, rtol=1e-5, atol=1e-4)                  # page scores: planes vs records
    same = [set(a[0][0, h].tolist()) == set(sel[0, h].tolist()) for h in range(2)]
    assert all(same) or int(selc.min()) == 512


def test_decode_append_keeps_shadow_fresh(dev):
    # append tokens one at a time (crossing a page boundary) and compare with a cache built at once
    g = torch.Generator().manual_seed(0)
    B, Hkv, N0, steps = 2, 2, 60, 9
    k = torch.randn((B, Hkv, N0 + steps, 128), generator=g).half()
    v = torch.randn((B, Hkv, N0 + steps, 128), generator=g).half()
    cache = PagedKVCache.from_dense(k[:, :, :N0].contiguous(), v[:, :, :N0].contiguous(), dev,
                                    spare_pages=4)
    free = [8, 9, 10, 11]
    for s in range(steps):
        cache.append(k[:, :, N0 + s], v[:, :, N0 + s], free)
    full = PagedKVCache.from_dense(k, v, dev)
    q = torch.randn((B, 4, 128), generator=g).half().to(dev)
    a = TwilightDecodeLayer(cache, 4, token_budget=32, top_p=0.9)
    b = TwilightDecodeLayer(full, 4, token_budget=32, top_p=0.9)
    oa, ob = a(q).clone(), b(q).clone()
    assert torch.equal(a.sel_pages, b.sel_pages) and torch.equal(a.count, b.count)
    assert torch.equal(oa, ob)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_append_kernel_records_equal_bulk_build(dev, dt):
    # token-by-token append (one launch per step) must leave K, V, INT4 records and Quest metadata
    # bit-identical to paging the final tensors at once; ragged: 3 requests of different phase
    g = torch.Generator().manual_seed(5)
    B, Hkv, N0, steps = 3, 5, 47, 40                     # crosses two page boundaries
    k = (torch.randn((B, Hkv, N0 + steps, 128), generator=g) * 2).to(dt)
    v = torch.randn((B, Hkv, N0 + steps, 128), generator=g).to(dt)
    cache = PagedKVCache.from_dense(k[:, :, :N0].contiguous(), v[:, :, :N0].contiguous(), dev,
                                    spare_pages=12, plane_pages=8)
    free = list(range(9, 21))
    for s in range(steps):
        # a strided view (the layout a projection + transpose hands over)
        cache.append(k[:, :, N0 + s].to(dev), v[:, :, N0 + s].to(dev), free)
    full = PagedKVCache.from_dense(k, v, dev, plane_pages=8)
    assert torch.equal(cache.kv_last_page_len.cpu(), full.kv_last_page_len.cpu())
    # plane-layout metadata too, for every COMPLETE page: the last page of a request is scored from
    # its record, and its plane entries are written when its 16th token arrives
    done = (N0 + steps) // 16
    assert torch.equal(cache.meta_planes.view(torch.int16)[..., :done],
                       full.meta_planes.view(torch.int16)[..., :done])
    ia, ib = cache.kv_page_indices.long(), full.kv_page_indices.long()
    assert ia.numel() == ib.numel()
    for name in ("k_cache", "v_cache", "k_int4", "meta"):
        assert torch.equal(getattr(cache, name)[ia], getattr(full, name)[ib]), name


@pytest.mark.parametrize("B,H,Hkv,dt,p,planes,survivors", [
    (16, 32, 32, torch.float16, 0.95, False, None),       # Longchat-7B shape (32 MHA heads, fp16), records
    (16, 32, 32, torch.float16, 0.95, True, (100, 400)),  # through the plane-layout metadata, on the
                                                          # benchmark's calibrated heavy hitters
    (8, 32, 8, torch.bfloat16, 0.90, True, None),         # Llama-3-8B shape (32 q / 8 kv heads, bf16)
    (8, 32, 8, torch.bfloat16, 0.90, True, (100, 400)),
])
def test_full_size_layer_sampled_rows_and_properties(dev, B, H, Hkv, dt, p, planes, survivors):
    # The two model shapes of the headline benchmark at their full size: ctx 32768, paged KV (shuffled pages), Quest
    # budget 8192, on both planted workloads of the benchmark. The oracle (dense, CPU) checks 32
    # (batch, head) rows end to end: the longest, the shortest and 30 drawn at random;
    # size-independent properties check every row.
    N, budget = 32768, 8192
    npg = N // 16
    q, k, v, (ids, indptr, last) = synth.layer_inputs_device(B, H, Hkv, N, dt, dev, seed=3,
                                                             survivors=survivors, top_p=p,
                                                             budget=budget)
    cache = PagedKVCache(B * npg, Hkv, dt, dev)
    cache.k_cache, cache.v_cache = k, v
    cache.set_page_table(ids, indptr, last)
    cache.rebuild_shadow()
    if planes:
        cache.enable_planes()
    layer = TwilightDecodeLayer(cache, H, token_budget=budget, top_p=p, high="max",
                                keep_scores=True)
    out = layer(q).clone()
    torch.cuda.synchronize()
    rows = B * H
    cnt = layer.count.reshape(rows).cpu().numpy()
    selc = layer.sel_count.reshape(rows).cpu().numpy()
    assert np.all(selc == 512) and np.all(cnt >= 1) and np.all(cnt <= 8192)
    assert torch.isfinite(out.float()).all()
    # every row: survivors ascending, inside the selected pages, and they carry >= p of the
    # softmax of the row's own candidate scores
    sel = layer.sel_pages.reshape(rows, -1)
    idx = layer.idx.reshape(rows, -1)
    scores = layer.scores.reshape(rows, -1)
    probs = torch.softmax(scores, dim=-1)
    pos = torch.arange(idx.shape[1], device=dev)[None, :]
    valid = pos < layer.count.reshape(rows, 1)
    tok = torch.where(valid, idx, torch.full_like(idx, -1))
    assert bool(((tok[:, 1:] > tok[:, :-1]) | ~valid[:, 1:]).all())
    page_of = (idx // 16).long()
    slot = torch.searchsorted(sel.long().contiguous(), page_of.clamp(min=0).contiguous())
    slot = slot.clamp(max=sel.shape[1] - 1)
    assert bool(((torch.gather(sel.long(), 1, slot) == page_of) | ~valid).all())
    cand = slot * 16 + (idx % 16).long()
    kept = torch.where(valid, torch.gather(probs, 1, cand.clamp(0, probs.shape[1] - 1)), torch.zeros_like(probs[:, :1]).expand_as(cand))
    assert float(kept.sum(-1).min()) >= p - 1e-5
    # sampled rows against the dense oracle
    ids_c = ids.cpu().long()
    rng = np.random.default_rng(0)
    picks = [int(np.argmax(cnt)), int(np.argmin(cnt))]
    while len(picks) < 32:
        r = int(rng.integers(0, rows))
        if r not in picks:
            picks.append(r)
    if survivors is not None:
        # the generator's target: a nucleus of 100-400 tokens per row
        assert survivors[0] * 0.8 <= np.median(cnt) <= survivors[1] * 1.2, np.median(cnt)
    tol = 1e-3 if dt == torch.float16 else 8e-3
    for r in picks:
        b, h = divmod(r, H)
        kvh = h // (H // Hkv)
        phys = ids_c[b * npg:(b + 1) * npg].to(dev)
        kd = k[phys, :, kvh].reshape(N, 128).float().cpu()[None, None]
        vd = v[phys, :, kvh].reshape(N, 128).float().cpu()[None, None]
        qd = q[b, h].float().cpu()[None, None, None]
        ref = P.decode_layer_dense(qd, kd, vd, top_p=p, token_budget=budget,
                                   high_mode=native.HIGH_MAX, quant="storage",
                                   prob_dtype=dt)
        m0 = np.zeros(N, dtype=bool)
        for pg in sel[r, :selc[r]].cpu().numpy():
            m0[pg * 16:(pg + 1) * 16] = True
        if not np.array_equal(m0, ref["mask0"].reshape(N).numpy()):
            # pages tied with the 512th score within rounding: checked as ties, then the later
            # stages are followed on the GPU's own selection
            est_pg = P.quest_chunk_scores_dense(qd, kd, 16)[0, 0, 0]
            _assert_selection_ties(est_pg, sel[r, :selc[r]].cpu().numpy(),
                                   ref["mask0"].reshape(N).numpy(), npg)
            ref = P.decode_layer_dense(qd, kd, vd, top_p=p, token_budget=budget,
                                       high_mode=native.HIGH_MAX, quant="storage", prob_dtype=dt,
                                       mask0=torch.from_numpy(m0).reshape(1, 1, 1, N))
        gm = np.zeros((1, N), dtype=bool)
        gm[0, idx[r, :cnt[r]].cpu().numpy()] = True
        pr = ref["probs"].reshape(1, N).numpy()
        _, _, _, margin = native.top_p_mask_f32(pr, p, native.HIGH_MAX, return_margin=True)
        assert_top_p_parity(pr, p, gm, ref["mask"].reshape(1, N).numpy(), ref["low"], margin,
                            margin_tol=5e-6)
        own = P.masked_attention(qd, kd, vd, torch.from_numpy(gm).reshape(1, 1, 1, N),
                                 prob_dtype=dt if cnt[r] <= 128 else torch.float32)
        assert torch.allclose(out[b, h].float().cpu(), own[0, 0, 0], rtol=tol, atol=tol), r
        e2e = (out[b, h].float().cpu() - ref["out"][0, 0, 0]).abs().max().item()
        assert e2e < 5 * tol, (r, e2e)


def test_full_size_options_every_row(dev):
    """The optional forms of the layer at the Llama-3 shape's full size (B=8, 32 q / 8 kv heads,
    bf16, ctx 32768, budget 8192), every row, through properties that need no dense oracle:
    use_estimated_weights (same lists, the survivors' estimator probabilities, out = sum w V /
    sum w against a torch gather) and group_select (one list per kv head = the top pages of the
    group's largest page scores; kept mass >= p on its own scores)."""
    B, H, Hkv, N, budget, p, dt = 8, 32, 8, 32768, 8192, 0.9, torch.bfloat16
    G, npg, rows = H // Hkv, N // 16, B * H
    q, k, v, (ids, indptr, last) = synth.layer_inputs_device(B, H, Hkv, N, dt, dev, seed=4)
    cache = PagedKVCache(B * npg, Hkv, dt, dev)
    cache.k_cache, cache.v_cache = k, v
    cache.set_page_table(ids, indptr, last)
    cache.rebuild_shadow()
    cache.enable_planes()
    base = TwilightDecodeLayer(cache, H, token_budget=budget, top_p=p, keep_scores=True)
    base(q)
    est = TwilightDecodeLayer(cache, H, token_budget=budget, top_p=p, use_estimated_weights=True)
    out = est(q).float()
    assert torch.equal(est.count, base.count) and torch.isfinite(out).all()
    cnt = base.count.reshape(rows)
    pos = torch.arange(base.idx.shape[-1], device=dev)[None, :]
    valid = pos < cnt[:, None]
    assert torch.equal(torch.where(valid, est.idx.reshape(rows, -1), 0),
                       torch.where(valid, base.idx.reshape(rows, -1), 0))
    # the emitted weights are the softmax of the candidate scores at the survivors' slots
    sel = base.sel_pages.reshape(rows, -1).long().contiguous()
    idx = base.idx.reshape(rows, -1).long()
    slot = torch.searchsorted(sel, (idx // 16).clamp(min=0).contiguous()).clamp(max=sel.shape[1] - 1)
    cand = slot * 16 + idx % 16
    probs = torch.softmax(base.scores.reshape(rows, -1), dim=-1)
    want_w = torch.gather(probs, 1, cand.clamp(0, probs.shape[1] - 1))
    got_w = est.surv_probs.reshape(rows, -1)
    assert torch.allclose(torch.where(valid, got_w, 0), torch.where(valid, want_w, 0), rtol=1e-4, atol=1e-10)
    # out = sum w V / sum w, for every row of at most 1024 survivors (all but a handful)
    cap = 1024
    short = (cnt <= cap).nonzero().squeeze(-1)
    assert short.numel() >= rows * 0.9
    r_b, r_kv = short // H, (short % H) // G
    tok = idx[short, :cap].clamp(min=0)
    phys = ids.long()[(r_b * npg)[:, None] + tok // 16]                       # physical page
    vv = v[phys, tok % 16, r_kv[:, None]].float()                             # [rows', cap, 128]
    w = torch.where(valid[short, :cap], got_w[short, :cap], 0.0)
    wn = w / w.sum(-1, keepdim=True)
    wn = torch.where((cnt[short] <= 128)[:, None], wn.to(dt).float(), wn)     # attention.py:302-304
    ref = torch.einsum("rc,rcd->rd", wn, vv)
    assert torch.allclose(out.reshape(rows, 128)[short], ref, rtol=8e-3, atol=8e-3)
    del vv, est

    grp = TwilightDecodeLayer(cache, H, token_budget=budget, top_p=p, group_select=True)
    gout = grp(q)
    assert torch.isfinite(gout.float()).all() and bool((grp.sel_count == 512).all())
    gs = grp.sel_pages.reshape(B, Hkv, G, -1)
    assert bool((gs == gs[:, :, :1]).all())
    # the group's list = the 512 pages with the largest group score; the row kernel of `base`
    # scores the same pages from the plane layout (another summation order): pages at the
    # boundary may differ within rounding
    gmax = base.page_scores.reshape(B, Hkv, G, -1)[..., :npg].amax(dim=2)     # [B, Hkv, npg]
    kth = torch.sort(gmax, dim=-1, descending=True).values[..., 511]
    chosen = torch.zeros_like(gmax, dtype=torch.bool)
    chosen.scatter_(-1, gs[:, :, 0].long(), True)
    tolr = 1e-3 * kth.abs().clamp(min=1.0)[..., None]
    assert bool((gmax[chosen].reshape(B, Hkv, 512) >= (kth[..., None] - tolr)).all())
    assert bool((torch.where(chosen, torch.full_like(gmax, -1e30), gmax) <= kth[..., None] + tolr).all())
    # kept mass on the group layer's own scores
    gcnt = grp.count.reshape(rows)
    gvalid = pos < gcnt[:, None]
    gsel = grp.sel_pages.reshape(rows, -1).long().contiguous()
    gidx = grp.idx.reshape(rows, -1).long()
    gslot = torch.searchsorted(gsel, (gidx // 16).clamp(min=0).contiguous()).clamp(max=gsel.shape[1] - 1)
    assert bool(((torch.gather(gsel, 1, gslot) == gidx // 16) | ~gvalid).all())
    gprobs = torch.softmax(grp.scores.reshape(rows, -1), dim=-1)
    gkept = torch.where(gvalid, torch.gather(gprobs, 1, (gslot * 16 + gidx % 16).clamp(0, gprobs.shape[1] - 1)), 0.0)
    assert float(gkept.sum(-1).min()) >= p - 1e-5


@pytest.mark.parametrize("H,Hkv", [(8, 8), (8, 2)])
def test_layer_step_replays_from_a_hip_graph(dev, H, Hkv):
    # a serving loop captures the decode step: every replay, with eager work and synchronisations
    # between replays and new q / K contents each time, must equal the eager result (the library
    # enqueues kernels only: no allocation, no memset, no host synchronisation)
    B, N = 32, 1024                  # MHA: 256 rows -> the one-launch row kernel; GQA: three launches
    g = torch.Generator().manual_seed(H + Hkv)
    k = torch.randn((B, Hkv, N, 128), generator=g).half()
    v = torch.randn((B, Hkv, N, 128), generator=g).half()
    cache = PagedKVCache.from_dense(k, v, dev, spare_pages=B)
    layer = TwilightDecodeLayer(cache, H, token_budget=256, top_p=0.9, reserve_pages=N // 16 + 1)
    q = torch.randn((B, H, 128), generator=g).half().to(dev)
    layer(q)                          # warm-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        layer(q)
    torch.cuda.synchronize()
    for step in range(4):
        q.copy_(torch.randn((B, H, 128), generator=g).half())      # same buffer, new contents
        if step == 2:                 # the cache contents change under the graph too
            cache.k_cache.mul_(-0.5)
            cache.rebuild_shadow()
        eager = layer(q).clone()
        cnt_e, idx_e = layer.count.clone(), layer.idx.clone()
        torch.cuda.synchronize()
        layer.out.zero_(); layer.count.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(layer.out, eager), step
        assert torch.equal(layer.count, cnt_e)
        mx = int(cnt_e.max())
        assert torch.equal(layer.idx[..., :mx] * (torch.arange(mx, device=dev) < cnt_e[..., None]),
                           idx_e[..., :mx] * (torch.arange(mx, device=dev) < cnt_e[..., None]))


def test_plane_slot_table(dev):
    """Plane-layout metadata addressed through a slot table: requests sit in any slots of a larger
    buffer, a request leaves the batch and the others keep their planes, appends go to the right
    slot. Everything is compared bit for bit with slot = batch position on the same data."""
    from twilight_amd import kernel as K
    g = torch.Generator().manual_seed(21)
    B, H, N, budget, p = 3, 4, 700, 160, 0.9
    npg = (N + 15) // 16
    q = torch.randn((B, H, 128), generator=g).half()
    k = torch.randn((B, H, N + 20, 128), generator=g).half()
    v = torch.randn((B, H, N + 20, 128), generator=g).half()

    def fresh(**kw):
        return PagedKVCache.from_dense(k[:, :, :N].contiguous(), v[:, :, :N].contiguous(), dev,
                                       page_perm=torch.randperm(B * npg, generator=torch.Generator().manual_seed(3)),
                                       spare_pages=2 * B, **kw)

    plain = fresh(plane_pages=npg + 8)
    slotted = fresh()
    slots = torch.tensor([4, 0, 2], dtype=torch.int32)
    slotted.enable_planes(npg + 8, num_slots=5, slots=slots)
    assert slotted.meta_planes.shape[0] == 5
    pl = slotted.meta_planes.view(torch.int16)
    assert torch.equal(pl[slots.long()], plain.meta_planes.view(torch.int16))
    assert not pl[1].any() and not pl[3].any()                   # slots of nobody stay untouched
    qd = q.to(dev)

    def run(c, qq):
        out = list(K.quest_gemv_int4_top_p(qq, c.meta, c.k_int4, c.kv_page_indices, c.kv_page_indptr,
                                           c.kv_last_page_len, budget, c.max_pages_per_req, p,
                                           return_scores=True, meta_planes=c.meta_planes,
                                           plane_slots=c.plane_slots))
        idx, count = out[2], out[3]          # entries past a row's count are not written
        live = torch.arange(idx.shape[-1], device=idx.device)[None, None, :] < count[..., None]
        out[2] = torch.where(live, idx, torch.full_like(idx, -1))
        return out
    want, got = run(plain, qd), run(slotted, qd)
    for a, b in zip(want, got):
        assert torch.equal(a, b)
    # the whole layer, and the separate-launch scoring kernel (12 rows: the split path)
    la = TwilightDecodeLayer(plain, H, token_budget=budget, top_p=p)
    lb = TwilightDecodeLayer(slotted, H, token_budget=budget, top_p=p)
    assert torch.equal(la(qd), lb(qd)) and torch.equal(la.count, lb.count)
    # decode appends across a page boundary land in the request's own slot
    free_a, free_b = list(range(B * npg, B * npg + 2 * B)), list(range(B * npg, B * npg + 2 * B))
    for s in range(20):
        plain.append(k[:, :, N + s].to(dev), v[:, :, N + s].to(dev), free_a)
        slotted.append(k[:, :, N + s].to(dev), v[:, :, N + s].to(dev), free_b)
    pl = slotted.meta_planes.view(torch.int16)
    assert torch.equal(pl[slots.long()], plain.meta_planes.view(torch.int16))
    assert not pl[1].any() and not pl[3].any()
    # request 1 leaves: requests 0 and 2 move to positions 0 and 1, their planes stay in place
    per = [plain._per_req[b] for b in (0, 2)]
    ids = torch.tensor(per[0] + per[1], dtype=torch.int32)
    indptr = torch.tensor([0, len(per[0]), len(per[0]) + len(per[1])], dtype=torch.int32)
    last = torch.tensor([plain._last[0], plain._last[2]], dtype=torch.int32)
    before = slotted.meta_planes.clone()
    slotted.set_page_table(ids, indptr, last)
    slotted.set_plane_slots(torch.tensor([4, 2], dtype=torch.int32))
    assert torch.equal(before, slotted.meta_planes)              # nothing was rebuilt
    got2 = run(slotted, qd[[0, 2]].contiguous())
    want2 = run(plain, qd)
    for a, b in zip(want2, got2):
        assert torch.equal(a[[0, 2]], b)
    with pytest.raises(RuntimeError):
        slotted.set_plane_slots(torch.tensor([4, 4], dtype=torch.int32))   # one slot, two requests
    with pytest.raises(RuntimeError):
        slotted.set_plane_slots(torch.tensor([4, 5], dtype=torch.int32))   # outside the buffer


@pytest.mark.parametrize("B,H,Hkv,N,budget,dt,planes", [
    (2, 8, 2, 1200, 512, torch.float16, False),          # three launches, G = 4
    (4, 32, 8, 2048, 1024, torch.bfloat16, True),        # Llama-3 grouping, one-launch kernel
    (1, 4, 4, 700, 256, torch.float16, False)])          # G = 1: the union is the head's own list
def test_layer_group_union_attention(dev, B, H, Hkv, N, budget, dt, planes):
    # group_union: the q heads of a kv head attend over the union of their survivor lists. The
    # per-head lists are the pruner's (unchanged); the union and the attention over it are checked
    # against the oracle's masked attention with the OR of the group's masks
    p, G = 0.9, H // Hkv
    q, k, v = synth.heavy_hitter_qkv(B, H, N, n_heavy=12, mass=0.6, seed=N, dtype=dt)
    kk, vv = k[:, ::G].contiguous(), v[:, ::G].contiguous()
    npg = (N + 15) // 16
    cache = PagedKVCache.from_dense(kk.to(dt), vv.to(dt), dev,
                                    page_perm=torch.randperm(B * npg, generator=torch.Generator().manual_seed(1)),
                                    plane_pages=npg if planes else None)
    qd = q[:, :, 0].to(dt).to(dev)
    plain = TwilightDecodeLayer(cache, H, token_budget=budget, top_p=p)
    out_plain = plain(qd).clone()
    layer = TwilightDecodeLayer(cache, H, token_budget=budget, top_p=p, group_union=True)
    out = layer(qd).cpu().float()
    rows = B * H
    assert torch.equal(layer.count, plain.count)
    idx = layer.idx.cpu().numpy().reshape(rows, -1)
    cnt = layer.count.cpu().numpy().reshape(rows)
    own = _lists_to_mask(idx, cnt, N)                                        # [rows, N]
    union = own.reshape(B, Hkv, G, N).any(2)                                 # [B, Hkv, N]
    gidx = layer.group_idx.cpu().numpy().reshape(B * Hkv, -1)
    gcnt = layer.group_count.cpu().numpy().reshape(B * Hkv)
    assert np.array_equal(_lists_to_mask(gidx, gcnt, N), union.reshape(B * Hkv, N))
    assert np.array_equal(gcnt, union.reshape(B * Hkv, N).sum(-1))
    for r in range(B * Hkv):
        assert np.all(np.diff(gidx[r, :gcnt[r]]) > 0)                        # ascending, distinct
    umask = torch.from_numpy(np.repeat(union, G, axis=1)).reshape(B, H, 1, N)
    krep, vrep = kk.repeat_interleave(G, dim=1), vv.repeat_interleave(G, dim=1)
    ref = P.masked_attention(q, krep, vrep, umask)[:, :, 0]
    tol = 1e-3 if dt == torch.float16 else 8e-3
    assert torch.allclose(out, ref, rtol=tol, atol=tol)
    if G == 1:
        assert torch.allclose(out, out_plain.cpu().float(), rtol=tol, atol=tol)
