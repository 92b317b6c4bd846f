"""Host logic of the Hugging Face integration (no GPU): config validation, module patching,
prefill pass-through and the budget statistics of twilight/pyimpl/state.py:158-234."""
import json
import os

import pytest
import torch

from twilight_amd import hf

CFG = {
    "compressor": {"type": "none"},
    "selector": {"type": "quest", "token_budget": 64, "chunk_size": 16},
    "weight_estimator": {"type": "min_max_quant", "quant_bit": 4},
    "weight_pruner": {"type": "top_p", "threshold": 0.9},
    "skip_first_two_layers": True,
    "use_estimated_weights_in_attn": False,
}


def _tiny_llama(layers=4, heads=2, kv_heads=1, dtype=torch.float32):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=97, hidden_size=heads * 128, intermediate_size=256,
                      num_hidden_layers=layers, num_attention_heads=heads,
                      num_key_value_heads=kv_heads, head_dim=128, max_position_embeddings=2048,
                      attn_implementation="sdpa")
    return LlamaForCausalLM(cfg).to(dtype).eval()


def test_budget_info_accounting():
    info = hf.HistoryBudgetInfo()
    for q in range(2):                                  # two decode steps through a 4-layer model
        for lid in range(2, 4):                         # layers 0, 1 are dense and never report
            info.update(lid, torch.tensor([[10 * (q + 1), 30 * (q + 1)]]))
            info.update_B0(lid, 64)
    assert len(info._budget_num) == 2                   # layer id jumped back -> a new query
    assert info.get_avg_budget_per_query() == [20.0, 40.0]
    assert info.get_total_avg_budget() == 30.0
    assert info.get_total_avg_budget_B0() == 64.0
    assert info.get_avg_budget_cur_query() == [40.0, 40.0]
    info.reset()
    assert info._budget_num == []


def test_config_validation():
    m = _tiny_llama()
    for key, bad in (("selector", {"type": "ds"}), ("weight_estimator", {"type": "none"}),
                     ("weight_pruner", {"type": "top_k"}), ("compressor", {"type": "snap_kv"})):
        cfg = json.loads(json.dumps(CFG))
        cfg[key] = bad
        with pytest.raises(RuntimeError):
            hf.enable_sparse_attention(m, cfg)
    cfg = json.loads(json.dumps(CFG))
    cfg["selector"]["chunk_size"] = 32
    with pytest.raises(RuntimeError):
        hf.enable_sparse_attention(m, cfg)


def test_score_info_accounting():
    # queries split where the layer id does not follow the previous one; averages are over the
    # per-layer MINIMUM over heads and skip layers 0 and 1 (twilight/pyimpl/state.py:96-132)
    m = _tiny_llama()
    info, score = hf.enable_sparse_attention(m, CFG, enable_budget_info=True, enable_score_info=True)
    assert isinstance(score, hf.HistoryAccumulatedScoreInfo)
    assert m.model.layers[3].self_attn._twilight_state.score_info is score
    for query in range(2):
        for lid in range(4):
            score.update(lid, torch.tensor([[0.9 + 0.01 * lid, 0.95], [0.99, 0.97 - 0.1 * query]]))
    assert len(score._min_sum) == 2 and sorted(score._min_sum[0]) == [0, 1, 2, 3]
    assert score._score_sum[0][2].shape == (4,)
    per_query = score.get_avg_score_per_query()
    assert per_query[0] == pytest.approx((0.92 + 0.93) / 2, abs=1e-6)
    assert per_query[1] == pytest.approx(0.87, abs=1e-6)
    assert score.get_total_avg_score() == pytest.approx((0.925 + 0.87) / 2, abs=1e-6)


def test_reference_config_file_shape_is_accepted():
    # the literal contents of benchmark/configs/config_quest_twi.json
    cfg = {"compressor": {"type": "none"},
           "selector": {"type": "quest", "token_budget": 8192, "chunk_size": 16},
           "weight_estimator": {"type": "min_max_quant", "quant_bit": 4},
           "weight_pruner": {"type": "top_p", "threshold": 0.85},
           "skip_first_two_layers": True, "use_estimated_weights_in_attn": False}
    m = _tiny_llama()
    info, score = hf.enable_sparse_attention(m, cfg, enable_budget_info=True)
    assert isinstance(info, hf.HistoryBudgetInfo) and score is None
    st = m.model.layers[2].self_attn._twilight_state
    assert st.cfg["token_budget"] == 8192 and st.cfg["top_p"] == 0.85


def test_patching_and_prefill_passthrough_on_cpu():
    m = _tiny_llama()
    ids = torch.randint(0, 97, (2, 40), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        ref = m(ids, use_cache=True).logits
    hf.enable_sparse_attention(m, CFG)
    patched = [hasattr(l.self_attn, "_twilight_state") for l in m.model.layers]
    assert patched == [False, False, True, True]        # skip_first_two_layers
    with pytest.raises(RuntimeError):
        hf.enable_sparse_attention(m, CFG)              # twice
    with torch.no_grad():
        out = m(ids, use_cache=True)
        assert torch.equal(out.logits, ref)             # prefill runs the model's own attention
        with pytest.raises(RuntimeError):               # decode needs the GPU path
            m(ids[:, :1], past_key_values=out.past_key_values, use_cache=True)
    hf.disable_sparse_attention(m)
    assert not any(hasattr(l.self_attn, "_twilight_state") for l in m.model.layers)
    with torch.no_grad():
        assert torch.equal(m(ids, use_cache=True).logits, ref)
