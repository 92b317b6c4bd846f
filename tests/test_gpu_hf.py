"""GPU test of the Hugging Face integration: a random-initialised Llama decodes through the
patched attention modules (twilight/pyimpl/attention.py:351-418, 481-493 is what is mirrored)."""
import json

import pytest
import torch

from twilight_amd import hf
from test_hf_host import CFG, _tiny_llama

pytestmark = pytest.mark.gpu


def _decode(model, ids, steps):
    """Greedy decode; returns the logits of every decode step [steps, B, vocab] and the tokens."""
    logits, toks = [], []
    with torch.no_grad():
        out = model(ids, use_cache=True)
        past = out.past_key_values
        nxt = out.logits[:, -1].argmax(-1, keepdim=True)
        for _ in range(steps):
            out = model(nxt, past_key_values=past, use_cache=True)
            past = out.past_key_values
            logits.append(out.logits[:, -1].float())
            toks.append(nxt)
            nxt = out.logits[:, -1].argmax(-1, keepdim=True)
    return torch.stack(logits), torch.cat(toks, dim=1)


def _forced_decode(model, ids, forced):
    """Decode feeding the given tokens (so two models see identical inputs at every step)."""
    logits = []
    with torch.no_grad():
        out = model(ids, use_cache=True)
        past = out.past_key_values
        for s in range(forced.shape[1]):
            out = model(forced[:, s:s + 1], past_key_values=past, use_cache=True)
            past = out.past_key_values
            logits.append(out.logits[:, -1].float())
    return torch.stack(logits)


@pytest.mark.parametrize("kv_heads", [4, 2])
def test_decode_with_p_one_equals_dense_decode(dev, kv_heads):
    # p = 1 and a budget beyond the context keep every token with non-zero estimated probability:
    # the patched model must reproduce dense decoding up to fp16 rounding of the attention output
    model = _tiny_llama(layers=4, heads=4, kv_heads=kv_heads, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (2, 200), generator=torch.Generator().manual_seed(2)).to(dev)
    ref_logits, toks = _decode(model, ids, 12)           # crosses a page boundary at step 8
    cfg = json.loads(json.dumps(CFG))
    cfg["selector"]["token_budget"] = 4096
    cfg["weight_pruner"]["threshold"] = 1.0
    info, _ = hf.enable_sparse_attention(model, cfg, enable_budget_info=True, reserve_tokens=64)
    got = _forced_decode(model, ids, toks)
    assert torch.isfinite(got).all()
    assert torch.allclose(got, ref_logits, rtol=2e-2, atol=2e-2), (got - ref_logits).abs().max()
    # budget statistics: one query per decode step, layers 2 and 3 report, everything is kept
    assert len(info._budget_num) == 12 and sorted(info._budget_num[0]) == [2, 3]
    first = info._budget_num[0][2].cpu()
    assert first.numel() == 2 * 4 and int(first.min()) >= 195 and int(first.max()) <= 201
    hf.disable_sparse_attention(model)
    again = _forced_decode(model, ids, toks)
    assert torch.allclose(again, ref_logits, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("kv_heads", [2, 1])
def test_group_select_through_the_model_patch(dev, kv_heads):
    """enable_sparse_attention(group_select=True): one Quest list per kv head. With everything
    kept it is dense decoding; with a real budget the q heads of a kv head share their page list
    and the step still prunes."""
    model = _tiny_llama(layers=4, heads=4, kv_heads=kv_heads, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (2, 200), generator=torch.Generator().manual_seed(6)).to(dev)
    ref_logits, toks = _decode(model, ids, 6)
    cfg = json.loads(json.dumps(CFG))
    cfg["selector"]["token_budget"] = 4096
    cfg["weight_pruner"]["threshold"] = 1.0
    hf.enable_sparse_attention(model, cfg, reserve_tokens=64, group_select=True)
    got = _forced_decode(model, ids, toks)
    assert torch.allclose(got, ref_logits, rtol=2e-2, atol=2e-2), (got - ref_logits).abs().max()
    hf.disable_sparse_attention(model)
    cfg["selector"]["token_budget"] = 64
    cfg["weight_pruner"]["threshold"] = 0.9
    info, _ = hf.enable_sparse_attention(model, cfg, enable_budget_info=True, reserve_tokens=64,
                                         group_select=True)
    got = _forced_decode(model, ids, toks)
    assert torch.isfinite(got).all()
    lay = model.model.layers[2].self_attn._twilight_state.layer
    assert lay.group_select
    sel = lay.sel_pages.reshape(2, kv_heads, 4 // kv_heads, -1)
    assert bool((sel == sel[:, :, :1]).all()) and int(lay.sel_count.max()) == 4
    assert 0 < info.get_total_avg_budget() <= 64
    hf.disable_sparse_attention(model)


def test_decode_with_estimated_weights_and_sparsity_rate(dev):
    """use_estimated_weights_in_attn and selector.sparsity_rate through the model patch: with
    everything kept the estimator's weights move the logits only by the 4-bit error, and the
    reported selector budget follows the context length."""
    model = _tiny_llama(layers=4, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (2, 200), generator=torch.Generator().manual_seed(5)).to(dev)
    ref_logits, toks = _decode(model, ids, 4)
    cfg = json.loads(json.dumps(CFG))
    cfg["selector"] = {"type": "quest", "sparsity_rate": 0.5, "chunk_size": 16}
    cfg["weight_pruner"]["threshold"] = 1.0
    cfg["use_estimated_weights_in_attn"] = True
    info, _ = hf.enable_sparse_attention(model, cfg, enable_budget_info=True, reserve_tokens=32)
    got = _forced_decode(model, ids, toks)
    assert torch.isfinite(got).all()
    cos = torch.nn.functional.cosine_similarity(got.flatten(1), ref_logits.flatten(1), dim=1)
    assert float(cos.min()) > 0.8
    assert info.get_avg_budget_per_query_B0() == [float(int((201 + s) * 0.5)) for s in range(4)]
    hf.disable_sparse_attention(model)
    # a recorded step would freeze the first budget: refused
    hf.enable_sparse_attention(model, cfg, reserve_tokens=32, dense_layers="paged", keep_hf_cache=False)
    with pytest.raises(RuntimeError, match="sparsity_rate"):
        hf.GraphedDecodeStep(model)
    hf.disable_sparse_attention(model)


def test_decode_prunes_and_reports_budgets(dev):
    model = _tiny_llama(layers=4, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (3, 333), generator=torch.Generator().manual_seed(3)).to(dev)
    ref_logits, toks = _decode(model, ids, 6)
    info, _ = hf.enable_sparse_attention(model, CFG, enable_budget_info=True, reserve_tokens=32)
    got = _forced_decode(model, ids, toks)                # budget 64 tokens, p = 0.9
    assert torch.isfinite(got).all()
    per_query = info.get_avg_budget_per_query()
    assert len(per_query) == 6 and all(1 <= b <= 64 for b in per_query)
    assert info.get_total_avg_budget_B0() == 64.0
    # a random-initialised model attends diffusely, so pruning to <= 64 of 333 tokens moves the
    # logits, but not arbitrarily: the same tokens stay likely
    cos = torch.nn.functional.cosine_similarity(got.flatten(1), ref_logits.flatten(1), dim=1)
    assert float(cos.min()) > 0.5
    # a second prompt through the same patched model starts from a fresh paged cache
    ids2 = ids[:, :100].contiguous()
    got2 = _forced_decode(model, ids2, toks[:, :3])
    assert torch.isfinite(got2).all()
    assert model.model.layers[2].self_attn._twilight_state.seq_len == 103


def test_patch_after_prefill_and_without_hf_cache_updates(dev):
    # (a) patching a model whose prompt was prefilled before: the first decode step pages the K / V
    # found in the model's cache; (b) keep_hf_cache=False gives the same logits (patched layers
    # never read the model's cache at decode) while their DynamicCache layers stop growing
    model = _tiny_llama(layers=4, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (2, 90), generator=torch.Generator().manual_seed(4)).to(dev)
    nxt = torch.randint(0, 97, (2, 5), generator=torch.Generator().manual_seed(5)).to(dev)

    def run(patch_before, keep):
        with torch.no_grad():
            if patch_before:
                hf.enable_sparse_attention(model, CFG, keep_hf_cache=keep)
            out = model(ids, use_cache=True)
            past = out.past_key_values
            if not patch_before:
                hf.enable_sparse_attention(model, CFG, keep_hf_cache=keep)
            logits = []
            for s in range(nxt.shape[1]):
                out = model(nxt[:, s:s + 1], past_key_values=past, use_cache=True)
                past = out.past_key_values
                logits.append(out.logits[:, -1].float())
        lens = [past.get_seq_length(i) for i in range(4)]
        hf.disable_sparse_attention(model)
        return torch.stack(logits), lens

    a, la = run(True, True)
    b, lb = run(False, True)
    c, lc = run(True, False)
    assert torch.equal(a, b) and torch.equal(a, c)
    assert la == [95, 95, 95, 95] and lb == la and lc == [95, 95, 90, 90]


def test_score_info_reports_kept_attention_mass(dev):
    # p = 1 with a budget beyond the context keeps every token whose estimated probability is not
    # zero: the kept share of the true attention mass is 1 up to the tokens the estimate flushed;
    # at p = 0.9 with 64 of 300 tokens it lies strictly between 0 and 1 and equals a direct
    # evaluation from the layer's own lists
    model = _tiny_llama(layers=4, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (2, 300), generator=torch.Generator().manual_seed(6)).to(dev)
    nxt = torch.randint(0, 97, (2, 3), generator=torch.Generator().manual_seed(7)).to(dev)
    cfg = json.loads(json.dumps(CFG))
    cfg["selector"]["token_budget"] = 4096
    cfg["weight_pruner"]["threshold"] = 1.0
    _, score = hf.enable_sparse_attention(model, cfg, enable_score_info=True)
    _forced_decode(model, ids, nxt)
    assert len(score._score_sum) == 3 and sorted(score._score_sum[0]) == [2, 3]
    for q in score._score_sum:
        for v in q.values():
            assert v.shape == (8,) and float(v.min()) > 0.999 and float(v.max()) < 1.0001
    assert score.get_total_avg_score() > 0.999
    hf.disable_sparse_attention(model)

    _, score = hf.enable_sparse_attention(model, CFG, enable_score_info=True)
    _forced_decode(model, ids, nxt)
    v = score._score_sum[-1][3].cpu()
    assert float(v.min()) > 0.2 and float(v.max()) < 0.9999
    # the function itself, on layer 3's cache: every token kept gives 1 ...
    st = model.model.layers[3].self_attn._twilight_state
    c, lay = st.cache, st.layer
    B, H = lay.count.shape
    n = st.seq_len
    ptr = c.kv_page_indptr.tolist()
    full = torch.arange(n, dtype=torch.int32, device=dev).expand(B, H, n).contiguous()
    cnt_full = torch.full((B, H), n, dtype=torch.int32, device=dev)
    q = torch.randn(B, H, 128, generator=torch.Generator().manual_seed(8)).to(dev, torch.float16)
    ones = hf.kept_attention_mass(c, q, full, cnt_full, lay.sm_scale)
    assert torch.allclose(ones, torch.ones_like(ones), atol=1e-5)
    # ... and a hand-made list its closed form: mass of tokens {0, n-1} = (e^{s0} + e^{s_last}) / sum e^{s}
    two = torch.zeros((B, H, 4), dtype=torch.int32, device=dev)
    two[:, :, 1] = n - 1
    got = hf.kept_attention_mass(c, q, two, torch.full((B, H), 2, dtype=torch.int32, device=dev),
                                 lay.sm_scale).cpu()
    for b in range(B):
        pages = c.kv_page_indices[ptr[b]:ptr[b + 1]].long()
        k = c.k_cache[pages].reshape(-1, c.num_kv_heads, 128)[:n].double().cpu()
        for h in range(H):
            s = (k[:, h // (H // c.num_kv_heads)] @ q[b, h].double().cpu()) * lay.sm_scale
            want = float((s[0].exp() + s[-1].exp()) / s.exp().sum())
            assert abs(float(got[b, h]) - want) < 1e-4
    hf.disable_sparse_attention(model)


def test_paged_dense_layers_reproduce_dense_decode(dev):
    # dense_layers="paged": layers 0-1 decode from paged K / V through the group attention kernel;
    # with p = 1 and a budget beyond the context the whole model must reproduce dense decoding.
    # With keep_hf_cache=False nothing updates the model's cache, so positions are passed in.
    model = _tiny_llama(layers=4, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (2, 150), generator=torch.Generator().manual_seed(9)).to(dev)
    ref_logits, toks = _decode(model, ids, 20)            # crosses a page boundary
    cfg = json.loads(json.dumps(CFG))
    cfg["selector"]["token_budget"] = 4096
    cfg["weight_pruner"]["threshold"] = 1.0
    for keep in (True, False):
        hf.enable_sparse_attention(model, cfg, reserve_tokens=64, dense_layers="paged",
                                   keep_hf_cache=keep)
        states = [l.self_attn._twilight_state for l in model.model.layers]
        assert [s.dense for s in states] == [True, True, False, False]
        logits = []
        with torch.no_grad():
            out = model(ids, use_cache=True)
            past = out.past_key_values
            for s in range(toks.shape[1]):
                pos = torch.full((2, 1), 150 + s, device=dev)
                out = model(toks[:, s:s + 1], past_key_values=past, use_cache=True, position_ids=pos)
                past = out.past_key_values
                logits.append(out.logits[:, -1].float())
        got = torch.stack(logits)
        assert torch.allclose(got, ref_logits, rtol=2e-2, atol=2e-2), (keep, (got - ref_logits).abs().max())
        assert past.get_seq_length(0) == (170 if keep else 150)
        hf.disable_sparse_attention(model)
    with pytest.raises(RuntimeError):
        hf.enable_sparse_attention(model, cfg, dense_layers="flash")


def test_graphed_decode_step_equals_eager_decode(dev):
    # the whole decode step recorded once into a HIP graph and replayed: same logits as the eager
    # patched model at every step, across page boundaries (tokens 160 and 176) and with the
    # budget statistics still collected
    model = _tiny_llama(layers=4, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    ids = torch.randint(0, 97, (2, 150), generator=torch.Generator().manual_seed(11)).to(dev)
    toks = torch.randint(0, 97, (2, 30), generator=torch.Generator().manual_seed(12)).to(dev)

    def eager():
        hf.enable_sparse_attention(model, CFG, reserve_tokens=64, dense_layers="paged",
                                   keep_hf_cache=False)
        logits = []
        with torch.no_grad():
            past = model(ids, use_cache=True).past_key_values
            for s in range(toks.shape[1]):
                pos = torch.full((2, 1), 150 + s, device=dev)
                out = model(toks[:, s:s + 1], past_key_values=past, use_cache=True, position_ids=pos)
                logits.append(out.logits[:, -1].float().clone())
        hf.disable_sparse_attention(model)
        return torch.stack(logits)

    want = eager()
    info, _ = hf.enable_sparse_attention(model, CFG, reserve_tokens=64, dense_layers="paged",
                                         keep_hf_cache=False, enable_budget_info=True)
    got = []
    with torch.no_grad():
        past = model(ids, use_cache=True).past_key_values
        pos = torch.full((2, 1), 150, device=dev)     # first decode step eagerly: pages the prefill
        out = model(toks[:, :1], past_key_values=past, use_cache=True, position_ids=pos)
        got.append(out.logits[:, -1].float().clone())
        step = hf.GraphedDecodeStep(model)
        for s in range(1, toks.shape[1]):
            got.append(step(toks[:, s:s + 1])[:, -1].float().clone())
            torch.cuda.synchronize()                  # eager work and syncs between the replays
    got = torch.stack(got)
    assert torch.equal(got, want), (got - want).abs().max()
    st = model.model.layers[3].self_attn._twilight_state
    assert st.seq_len == 180 and st.cache._seq_lens == [180, 180]
    assert st.cache.kv_last_page_len.cpu().tolist() == [4, 4]
    assert len(info._budget_num) == 30 and sorted(info._budget_num[-1]) == [2, 3]
    hf.disable_sparse_attention(model)
    # the recording needs paged dense layers and an untouched model cache
    hf.enable_sparse_attention(model, CFG)
    with pytest.raises(RuntimeError):
        hf.GraphedDecodeStep(model)
    hf.disable_sparse_attention(model)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_fused_rotary_embedding_equals_the_tensor_form(dev, dt):
    # one launch, in place, bit-identical to apply_rotary_pos_emb on tensors of the same dtype
    # (twilight/pyimpl/attention.py:118-123 calls that function)
    import twilight_amd.kernel as K
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    B, H, Hkv = 3, 8, 2
    g = torch.Generator().manual_seed(13)
    q = (torch.randn((B, H, 1, 128), generator=g) * 3).to(dt).to(dev)
    k = (torch.randn((B, Hkv, 1, 128), generator=g) * 3).to(dt).to(dev)
    pos = torch.tensor([[5.0], [1234.0], [32767.0]])
    inv = 1.0 / (500000.0 ** (torch.arange(0, 128, 2).float() / 128))
    ang = torch.cat([pos * inv, pos * inv], dim=-1)                       # [B, 128]
    cos, sin = ang.cos().to(dt).to(dev), ang.sin().to(dt).to(dev)
    want_q, want_k = apply_rotary_pos_emb(q, k, cos[:, None], sin[:, None])
    q3, k3 = q[:, :, 0].contiguous(), k[:, :, 0].contiguous()
    K.rope_qk_(q3, k3, cos, sin)
    assert torch.equal(q3, want_q[:, :, 0]) and torch.equal(k3, want_k[:, :, 0])
    with pytest.raises(RuntimeError):
        K.rope_qk_(q3, k3, cos.float(), sin.float())


def test_decode_refuses_a_mask_that_hides_positions_and_takes_a_single_first_token(dev):
    # the reference asserts the decode-step mask away (twilight/pyimpl/attention.py:186); here a
    # mask that hides nothing passes, one that hides a position (a left-padded batch) raises, and
    # a single token with nothing cached is a one-token prefill through the model's own forward
    model = _tiny_llama(layers=3, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    hf.enable_sparse_attention(model, json.loads(json.dumps(CFG)), reserve_tokens=32)
    ids = torch.randint(0, 97, (2, 40), generator=torch.Generator().manual_seed(5)).to(dev)
    with torch.no_grad():
        out = model(ids, use_cache=True)
        past = out.past_key_values
        nxt = out.logits[:, -1].argmax(-1, keepdim=True)
        full = torch.ones((2, 41), dtype=torch.long, device=dev)
        ok = model(nxt, past_key_values=past, use_cache=True, attention_mask=full)
        assert torch.isfinite(ok.logits).all()
        padded = full.clone()
        padded = torch.cat([padded, torch.ones((2, 1), dtype=torch.long, device=dev)], dim=1)
        padded[1, :3] = 0
        with pytest.raises(RuntimeError, match="attention_mask"):
            model(nxt, past_key_values=ok.past_key_values, use_cache=True, attention_mask=padded)
    hf.disable_sparse_attention(model)
    # one token, empty cache: prefill path, then ordinary decode steps
    model2 = _tiny_llama(layers=3, heads=4, kv_heads=2, dtype=torch.float16).to(dev)
    from transformers import DynamicCache
    with torch.no_grad():
        ref = model2(ids[:, :1], past_key_values=DynamicCache(config=model2.config), use_cache=True)
        hf.enable_sparse_attention(model2, json.loads(json.dumps(CFG)), reserve_tokens=32)
        got = model2(ids[:, :1], past_key_values=DynamicCache(config=model2.config), use_cache=True)
        assert torch.allclose(got.logits.float(), ref.logits.float(), rtol=1e-3, atol=1e-3)
        step = model2(ids[:, 1:2], past_key_values=got.past_key_values, use_cache=True)
        assert torch.isfinite(step.logits).all()


def test_full_size_model_keeping_everything_equals_dense_decode(dev):
    """The whole model at the benchmark's shape (Llama-3-8B: 32 layers, 32 q heads on 8 kv heads,
    head_dim 128, bf16, random weights) over a 32704-token context: with p = 1 and a budget that
    holds every page the patched model (paged caches filled from given K / V, layers 0-1 through the
    dense paged attention, layers 2-31 through select -> estimate -> prune -> attention over all
    32704 + step tokens, RoPE, append) must reproduce the model's own dense decode. Size-dependent
    parts are exercised here: 2044-page tables, 32736-candidate rows, split attention rows of 256
    chunks, appends that cross a page boundary."""
    from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM
    B, N, nl, steps = 1, 32704, 32, 3
    cfg = LlamaConfig(vocab_size=128256, hidden_size=4096, intermediate_size=14336,
                      num_hidden_layers=nl, num_attention_heads=32, num_key_value_heads=8,
                      head_dim=128, max_position_embeddings=N + 4096, rope_theta=500000.0,
                      attn_implementation="sdpa")
    torch.manual_seed(0)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            model = LlamaForCausalLM(cfg).eval()
    finally:
        torch.set_default_dtype(old)

    def kv(layer):
        g = torch.Generator(device=dev).manual_seed(1000 + layer)
        k = torch.randn((B, 8, N, 128), generator=g, device=dev, dtype=torch.bfloat16)
        v = torch.randn((B, 8, N, 128), generator=g, device=dev, dtype=torch.bfloat16)
        return k, v

    ids = torch.randint(0, cfg.vocab_size, (steps, B, 1), generator=torch.Generator().manual_seed(7)).to(dev)

    def run(cache, m=None):
        out = []
        with torch.no_grad():
            for s in range(steps):
                o = (m or model)(ids[s], past_key_values=cache, use_cache=True,
                                 position_ids=torch.full((B, 1), N + s, device=dev))
                out.append(o.logits[:, -1].float())
        return torch.stack(out)

    # the yardstick: the same weights and K / V in fp32 (eager attention), against which both
    # bf16 runs are measured; then the model's own bf16 dense decode
    import copy
    model32 = copy.deepcopy(model).float()
    model32.config._attn_implementation = "eager"
    cache = DynamicCache(config=cfg)
    for i in range(nl):
        k, v = kv(i)
        cache.update(k.float(), v.float(), i)
    exact = run(cache, model32)
    del cache, model32
    torch.cuda.empty_cache()
    cache = DynamicCache(config=cfg)
    for i in range(nl):
        cache.update(*kv(i), i)
    ref = run(cache)
    del cache
    torch.cuda.empty_cache()
    sparse_cfg = json.loads(json.dumps(CFG))
    sparse_cfg["selector"]["token_budget"] = 32768
    sparse_cfg["weight_pruner"]["threshold"] = 1.0
    info, _ = hf.enable_sparse_attention(model, sparse_cfg, enable_budget_info=True, reserve_tokens=16,
                                         keep_hf_cache=False, dense_layers="paged")
    for i in range(nl):
        hf.fill_from_prefill(model.model.layers[i].self_attn._twilight_state, *kv(i), cfg.num_attention_heads)
    got = run(DynamicCache(config=cfg))
    hf.disable_sparse_attention(model)
    assert torch.isfinite(got).all()
    # every token is kept in every pruned layer
    first = info._budget_num[0]
    assert sorted(first) == list(range(2, nl))
    assert all(int(first[l].min()) >= N for l in first)
    # both bf16 runs against the fp32 one: the patched model may not be further from it than the
    # model's own bf16 decode is (plus a fifth), and the two agree with each other
    err_got = (got - exact).abs().max().item()
    err_ref = (ref - exact).abs().max().item()
    rms_got = (got - exact).pow(2).mean().sqrt().item()
    rms_ref = (ref - exact).pow(2).mean().sqrt().item()
    scale = exact.abs().max().item()
    cosf = torch.nn.functional.cosine_similarity
    cos_got = float(cosf(got.flatten(1), exact.flatten(1), dim=1).min())
    cos_ref = float(cosf(ref.flatten(1), exact.flatten(1), dim=1).min())
    rms_between = (got - ref).pow(2).mean().sqrt().item()
    print(f"full-size model vs fp32: patched max {err_got:.4f} rms {rms_got:.5f} cosine {cos_got:.6f}; "
          f"bf16 dense max {err_ref:.4f} rms {rms_ref:.5f} cosine {cos_ref:.6f}; max |logit| "
          f"{scale:.3f}; patched vs bf16 dense rms {rms_between:.5f}")
    # (measured: rms 0.0556 against 0.0543, cosine 0.99899 against 0.99904 at max |logit| 5.7:
    # the distance to fp32 is the bf16 arithmetic of the model around the attention)
    assert rms_got <= 1.2 * rms_ref and err_got <= 1.5 * err_ref
    assert cos_got >= cos_ref - 5e-4 and cos_got > 0.995
    assert rms_between <= 2.0 * rms_ref
