"""Pins the oracle's Quest selector (twilight/pyimpl/quest.py:17-122), estimator GEMV and masked
attention (twilight/pyimpl/attention.py:188-306) against brute force / library routines."""
import math

import numpy as np
import torch

from oracle import native
from oracle import pyimpl_port as P


def test_quest_dense_vs_brute_force_with_padding():
    g = torch.Generator().manual_seed(0)
    B, H, N, D, C = 1, 2, 40, 128, 16        # 40 = 2.5 chunks: exercises quest.py:48-65
    q = torch.randn((B, H, 1, D), generator=g)
    k = torch.randn((B, H, N, D), generator=g)
    est = P.quest_chunk_scores_dense(q, k, C)
    assert est.shape == (B, H, 1, 3)
    for h in range(H):
        for c in range(3):
            toks = range(c * C, min(N, (c + 1) * C))
            s = 0.0
            for d in range(D):
                qd = float(q[0, h, 0, d])
                s += max(qd * float(k[0, h, t, d]) for t in toks)
            assert abs(s - float(est[0, h, 0, c])) < 1e-3
    mask, topk = P.quest_selector_dense(q, k, C, token_budget=20)   # 20 -> 1 + 1 chunks
    assert topk.shape[-1] == 2
    for h in range(H):
        best = torch.argsort(est[0, h, 0], descending=True)[:2].tolist()
        want = torch.zeros(N, dtype=torch.bool)
        for c in best:
            want[c * C:min(N, (c + 1) * C)] = True
        assert torch.equal(mask[0, h, 0], want)


def test_quest_budget_rule():
    # quest.py:93-98
    assert P.quest_chunk_budget(8192, 16, 2048) == 512
    assert P.quest_chunk_budget(8200, 16, 2048) == 513
    assert P.quest_chunk_budget(5, 16, 2048) == 2      # max(1, 0) + 1 for the remainder
    assert P.quest_chunk_budget(16, 16, 2048) == 1
    assert P.quest_chunk_budget(8192, 16, 100) == 100


def test_quest_meta_form_equals_dense_form():
    g = torch.Generator().manual_seed(1)
    B, Hkv, N, D = 2, 2, 72, 128                 # last page holds 8 valid tokens
    q = torch.randn((B, Hkv, 1, D), generator=g).half().float()
    q[0, 0, 0, 5] = 0.0                            # quest.py:37: sign(0) = -1, contributes 0
    k = torch.randn((B, Hkv, N, D), generator=g).half().float()
    dense = P.quest_chunk_scores_dense(q, k, 16)
    pages, ids, indptr, last = P.dense_to_paged(k, torch.randperm(B * 5, generator=g))
    valid = torch.full((B * 5,), 16, dtype=torch.int64)
    for b in range(B):
        valid[ids[indptr[b + 1] - 1].long()] = int(last[b])
    meta = P.quest_page_meta(pages, valid)
    rec = P.pack_meta_records(meta)
    assert rec.shape == (B * 5, Hkv, 512)
    # record layout: chunk c = fp16 min[4c..4c+3] then max[4c..4c+3]
    r = rec[3, 1].view(np.float16).reshape(32, 2, 4)
    assert np.array_equal(r[:, 0].reshape(-1), meta[3, 1, 0].numpy().astype(np.float16))
    assert np.array_equal(r[:, 1].reshape(-1), meta[3, 1, 1].numpy().astype(np.float16))
    for b in range(B):
        for h in range(Hkv):
            phys = ids[indptr[b]:indptr[b + 1]].long()
            s = P.quest_page_scores_meta(q[b, h, 0], meta[phys, h])
            assert torch.allclose(s.float(), dense[b, h, 0], rtol=1e-5, atol=1e-4)


def test_group_selection_reduces_to_the_per_head_selection():
    g = torch.Generator().manual_seed(11)
    B, H, N = 2, 8, 400
    q = torch.randn((B, H, 1, 128), generator=g)
    k = torch.randn((B, H, N, 128), generator=g)
    per_head, _ = P.quest_selector_dense(q, k, 16, 96)
    m1, _ = P.quest_selector_group_dense(q, k, 16, 96, 1)
    assert torch.equal(m1, per_head)
    # identical queries (and keys) inside a group: the group's choice is every head's own choice
    q4 = q[:, ::4].repeat_interleave(4, dim=1)
    k4 = k[:, ::4].repeat_interleave(4, dim=1)
    m4, _ = P.quest_selector_group_dense(q4, k4, 16, 96, 4)
    assert torch.equal(m4, P.quest_selector_dense(q4, k4, 16, 96)[0])
    # different queries over shared keys: one mask per group, of the budget's size; brute force:
    # no chunk outside it has a larger group score than a chunk inside it
    kk = k[:, ::4].repeat_interleave(4, dim=1)
    mg, _ = P.quest_selector_group_dense(q, kk, 16, 96, 4)
    assert mg.sum(-1).unique().tolist() == [96]
    mgr = mg.reshape(B, 2, 4, N)
    assert (mgr == mgr[:, :, :1]).all()
    sc = P.quest_chunk_scores_dense(q, kk, 16)[:, :, 0]                       # [B, H, 25]
    for b in range(B):
        for kv in range(2):
            gsc = [max(float(sc[b, 4 * kv + j, c]) for j in range(4)) for c in range(25)]
            chosen = [c for c in range(25) if mg[b, 4 * kv, 0, c * 16]]
            assert len(chosen) == 6
            assert min(gsc[c] for c in chosen) >= max(gsc[c] for c in range(25) if c not in chosen)


def test_estimator_scores_is_a_matmul():
    g = torch.Generator().manual_seed(2)
    q = torch.randn((1, 4, 1, 128), generator=g).half().float()
    k = torch.randn((1, 4, 96, 128), generator=g).half().float()
    _, _, _, deq = P.int4_quant_storage(k)
    s = P.estimator_scores(q, torch.from_numpy(deq))
    ref = np.einsum("bhqd,bhnd->bhqn", q.double().numpy(), deq.astype(np.float64)) / math.sqrt(128)
    np.testing.assert_allclose(s.numpy(), ref, rtol=1e-5, atol=1e-5)
    # the constant-input case of benchmark/efficiency/bench_gemv.py:390-422: q = 1, nibble 3,
    # scale 1, zero 0 -> every raw score is 3 * 128
    ones = torch.ones((1, 1, 1, 128))
    deq3 = native.int4_dequant(np.full((1, 128), 3, np.uint8), np.ones((1, 4), np.float16),
                               np.zeros((1, 4), np.float16))
    assert float(P.estimator_scores(ones, torch.from_numpy(deq3)[None, None], sm_scale=1.0)) == 384.0


def test_masked_attention_equals_gathered_softmax():
    g = torch.Generator().manual_seed(3)
    B, H, N, D = 2, 3, 200, 128
    q = torch.randn((B, H, 1, D), generator=g).half().float()
    k = torch.randn((B, H, N, D), generator=g).half().float()
    v = torch.randn((B, H, N, D), generator=g).half().float()
    mask = torch.rand((B, H, 1, N), generator=g) < 0.1
    mask[..., 0] = True
    for dt in (torch.float32, torch.float16):
        out = P.masked_attention(q, k, v, mask, dt)
        for b in range(B):
            for h in range(H):
                sel = mask[b, h, 0].nonzero().squeeze(-1)
                logit = (k[b, h, sel].double() @ q[b, h, 0].double()) / math.sqrt(D)
                pr = torch.softmax(logit, -1)
                if dt == torch.float16:
                    pr = pr.float().half().double()
                ref = pr @ v[b, h, sel].double()
                assert torch.allclose(out[b, h, 0].double(), ref, rtol=1e-4, atol=1e-5)
    idx, count = P.mask_to_lists(mask)
    assert count.sum() == int(mask.sum()) and idx[0, 0] == 0


def test_masked_attention_on_given_logits():
    """attention.py:295-296: given logits replace q.K. Pinned by the gathered closed form with
    logits unrelated to q.K, and by logits equal to q.K reproducing the default path."""
    g = torch.Generator().manual_seed(5)
    B, H, N, D = 1, 2, 96, 128
    q = torch.randn((B, H, 1, D), generator=g)
    k = torch.randn((B, H, N, D), generator=g)
    v = torch.randn((B, H, N, D), generator=g)
    logits = torch.randn((B, H, 1, N), generator=g) * 3
    mask = torch.rand((B, H, 1, N), generator=g) < 0.3
    mask[..., 5] = True
    out = P.masked_attention(q, k, v, mask, logits=logits)
    for h in range(H):
        sel = mask[0, h, 0].nonzero().squeeze(-1)
        pr = torch.softmax(logits[0, h, 0, sel].double(), -1)
        assert torch.allclose(out[0, h, 0].double(), pr @ v[0, h, sel].double(), rtol=1e-5, atol=1e-6)
    same = P.masked_attention(q, k, v, mask, logits=torch.matmul(q, k.transpose(2, 3)) / math.sqrt(D))
    assert torch.allclose(same, P.masked_attention(q, k, v, mask), rtol=1e-5, atol=1e-6)
    assert not torch.allclose(out, same, atol=1e-2)      # the given logits are really used


def test_decode_layer_dense_knobs():
    """sparsity_rate (quest.py:45-46) and use_estimated_weights_in_attn (attention.py:295-296)."""
    from twilight_amd import synth
    q, k, v = synth.heavy_hitter_qkv(1, 2, 512, n_heavy=8, mass=0.6, seed=1)
    # rate 1 keeps everything, rate 0 keeps the one chunk the budget rule never goes below
    assert P.decode_layer_dense(q, k, v, top_p=0.9, sparsity_rate=1.0)["mask0"].all()
    assert P.decode_layer_dense(q, k, v, top_p=0.9, sparsity_rate=0.0)["mask0"].sum(-1).unique().tolist() == [16]
    assert P.decode_layer_dense(q, k, v, top_p=0.9, sparsity_rate=0.26)["mask0"].sum(-1).unique().tolist() == [144]
    # a K that the 4-bit grid holds exactly: the estimator's logits are the exact ones and the two
    # attention modes meet
    g = torch.Generator().manual_seed(2)
    codes = torch.randint(0, 16, (1, 2, 512, 128), generator=g).float()
    codes[..., 0::32] = 0
    codes[..., 1::32] = 15                     # every group of 32 spans the full range
    kq = codes * 0.125 - 1.0                   # scale 1/8, zero -1: fp16-exact
    a = P.decode_layer_dense(q, kq, v, top_p=0.9, token_budget=256)
    b = P.decode_layer_dense(q, kq, v, top_p=0.9, token_budget=256, use_estimated_weights=True)
    assert torch.equal(a["mask"], b["mask"])
    assert torch.allclose(a["out"], b["out"], rtol=1e-4, atol=1e-5)
    # with an inexact K the estimated weights change the result
    c = P.decode_layer_dense(q, k, v, top_p=0.9, token_budget=256, use_estimated_weights=True)
    d = P.decode_layer_dense(q, k, v, top_p=0.9, token_budget=256)
    assert not torch.allclose(c["out"], d["out"], atol=1e-4)


def test_decode_layer_dense_consistency():
    from twilight_amd import synth
    q, k, v = synth.heavy_hitter_qkv(1, 2, 512, n_heavy=8, mass=0.6, seed=0)
    r = P.decode_layer_dense(q, k, v, top_p=0.95, token_budget=256)
    assert r["mask0"].sum(-1).unique().tolist() == [256]
    assert torch.all(r["mask"] <= r["mask0"])
    kept = (r["probs"] * r["mask"]).sum(-1)
    assert torch.all(kept >= 0.95 - 1e-6)
    # heavy hitters carry ~0.6 of the exact softmax by construction
    w = torch.softmax((q @ k.transpose(2, 3)) / math.sqrt(128), -1)
    top8 = w.topk(8, dim=-1).values.sum(-1)
    assert torch.all((top8 > 0.55) & (top8 < 0.66))


def test_qk_int8_lse_oracle_is_a_base2_logsumexp():
    # closed form: lse = log2( sum_n 2^s[m][n] + (#padded keys) * 2^0 ), evaluated in float64 from
    # the dequantised product; pins scale indexing (q block 128, k block 64, GQA head mapping) and
    # the zero-padded tail of the last key block
    g = torch.Generator().manual_seed(0)
    b, h_qo, h_kv, qo_len, kv_len, d = 2, 4, 2, 150, 100, 64
    q = torch.randint(-127, 128, (b, h_qo, qo_len, d), generator=g, dtype=torch.int8)
    k = torch.randint(-127, 128, (b, h_kv, kv_len, d), generator=g, dtype=torch.int8)
    qs = torch.rand((b, h_qo, 2), generator=g) * 2e-3 + 1e-3
    ks = torch.rand((b, h_kv, 2), generator=g) * 2e-3 + 1e-3
    got = P.qk_int8_lse_ref(q, k, qs, ks).double()
    krep = k.double().repeat_interleave(2, dim=1)
    s = torch.matmul(q.double(), krep.transpose(2, 3))
    s = s * qs.double()[:, :, torch.arange(qo_len) // 128][..., None]
    s = s * ks.double().repeat_interleave(2, dim=1)[:, :, torch.arange(kv_len) // 64][:, :, None, :]
    want = torch.log2(torch.exp2(s).sum(-1) + (128 - kv_len))
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-5)
    # no padding when kv_len is a multiple of 64: a plain logsumexp (in base 2)
    got2 = P.qk_int8_lse_ref(q, k[:, :, :64], qs, ks[:, :, :1]).double()
    want2 = torch.logsumexp(s[..., :64] * math.log(2.0), dim=-1) / math.log(2.0)
    assert torch.allclose(got2, want2, rtol=1e-5, atol=1e-5)
