#!/usr/bin/env python3
"""Benchmark of the Select-then-Prune decode layer on one MI355X.

A step is one pass of the hot path (Quest page selection -> INT4-K score GEMV -> softmax + top-p
prune -> sparse paged attention) over one batch of synthetic decode queries, enqueued by a single
``twl_decode_layer`` call with every input already resident in HBM.

Workload (``config.workload``): the Longchat-7B-shaped layer of the reference's headline figure at
the batch the target is quoted on — 32 MHA heads, head_dim 128, fp16 paged KV (page 16), batch 8,
context 32768, Quest budget 8192, top-p 0.95. q, K, V ~ N(0,1) with planted heavy-hitter pages whose
strength is solved per row so that the pruner keeps 100-400 tokens per row (``--planted
calibrated``, the default; ``--planted peaked`` is one fixed strength, under which most rows keep
1-2 tokens and a few keep thousands).

Prints ONE JSON line. ``value`` is microseconds per layer (lower is better). ``roofline`` is for
the step's dominant kernel (the one-launch selector + estimator + pruner); ``kernels`` lists every
kernel of the layer with its algorithmic bytes, time and fraction of the 8 TB/s peak, and
``gemv_cfg2`` the stand-alone INT4 GEMV at 8 x 32 x 32768 candidates. ``b8_peaked`` is the same
layer on the other planted workload, ``cfg4_b16`` / ``cfg4_b32`` / ``cfg4_b64`` the same layer at
the other batch sizes of the reference's latency figure and ``cfg5_layer`` the Llama-3 shape (32 q
heads on 8 kv heads, bf16, p 0.9, with the dense paged decode and the one-list-per-kv-head option
beside it), all measured the same way with fewer steps; ``cfg5_model`` is the whole 32-layer model
at that shape (random weights, tokens/s, 8 decode steps replayed from one HIP graph, against the
model's own dense decode).
``cpu_baseline`` is the CPU oracle (a port of the reference's torch path) timed on this host on
one of the 8 batch elements and scaled by 8, plus the reference's own CPU case (B=1, context 4096)
with warm-ups, repeats, median and per-stage times.

Other workloads (``--workload``), each printing one JSON line of its own: ``llama3`` (the same
layer with 32 q heads on 8 kv heads, bf16, p 0.9, plus dense-decode comparisons), ``topp`` (the
pruner alone), ``ftka`` (the NHD GEMV call shapes and the Double-Sparse label ops),
``llama3-model`` (whole-model decode of a random-initialised Llama-3-8B shape, tokens/s, dense
against the patched model).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch of quest_score_kernel at the default workload, measured with
# `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` (131404.9 KiB x 2.000 + 2048.0 KiB x 1.000, the
# factors being what the same counters read for a 1 GiB device copy; the summary of those runs is
# kept under profiles/). bench.py cannot read counters itself, so the figure is reported only for
# the exact configuration it was measured on.
QUEST_SCORE_TRAFFIC_BYTES_DEFAULT = int((131404.9 * 2.000 + 2048.0 * 1.000) * 1024)
# The same for select_estimate_prune_kernel (FETCH_SIZE KiB x 2.000 + WRITE_SIZE KiB x 1.000).
ROW_KERNEL_TRAFFIC_BYTES_RECORDS = int((213640.2 * 2.000 + 596.1 * 1.000) * 1024)  # --no-planes
ROW_KERNEL_TRAFFIC_BYTES_DEFAULT = int((148074.2 * 2.000 + 775.4 * 1.000) * 1024)  # plane layout, calibrated
ROW_KERNEL_TRAFFIC_BYTES_PEAKED = int((148094.6 * 2.000 + 596.1 * 1.000) * 1024)   # plane layout, peaked


def _time_calls(fn, iters: int, warmup: int) -> float:
    """Average microseconds per call of ``fn`` (which enqueues on the current stream), measured
    with events on that stream around ``iters`` back-to-back calls."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1000.0 / iters


def _median_time(fn, warmups: int, repeats: int):
    """(median seconds, last result) of ``fn`` after ``warmups`` untimed calls."""
    for _ in range(warmups):
        out = fn()
    ts = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        out = fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], out


def cpu_baseline_cfg1(warmups: int = 3, repeats: int = 20):
    """The CPU restatement of the reference's decode math on its own CPU-runnable case: B=1, 32 MHA
    heads, head_dim 128, context 4096, fp32, 16 heavy hitters per head with ~60 % of the softmax
    mass, every token a candidate, p = 0.95. time.perf_counter, warm-ups, repeats, median; stages
    timed one by one and two totals: (A) K re-quantised inside the step as
    twilight/pyimpl/attention.py:247-251 does, (B) K quantised beforehand."""
    from oracle import native, pyimpl_port as P
    from twilight_amd import synth
    q, k, v = synth.heavy_hitter_qkv(1, 32, 4096, n_heavy=16, mass=0.6, seed=0)
    mask0 = torch.ones((1, 32, 1, 4096), dtype=torch.bool)
    t_quant, quant = _median_time(lambda: torch.from_numpy(P.int4_quant_storage(k)[3]), warmups, repeats)
    t_gemv, est = _median_time(lambda: P.estimator_scores(q, quant), warmups, repeats)
    t_topp, pruned = _median_time(lambda: P.top_p_unnormalized(est, 0.95, native.HIGH_MAX), warmups, repeats)
    mask = mask0 & pruned[0]
    t_attn, _ = _median_time(lambda: P.masked_attention(q, k, v, mask, torch.float32), warmups, repeats)
    t_a, ra = _median_time(lambda: P.decode_layer_dense(q, k, v, top_p=0.95, token_budget=None,
                                                       high_mode=native.HIGH_MAX, quant="storage"),
                           warmups, repeats)
    t_b, _ = _median_time(lambda: P.decode_layer_dense(q, k, v, top_p=0.95, token_budget=None,
                                                      high_mode=native.HIGH_MAX, k_deq=quant),
                          warmups, repeats)
    us = lambda t: round(t * 1e6, 1)
    return {"workload": "B=1, 32 MHA heads, head_dim 128, context 4096, fp32, 16 heavy hitters per "
                        "head (~60 % of the mass), all tokens candidates, p 0.95, INT4 group 32",
            "warmups": warmups, "repeats": repeats, "statistic": "median",
            "us_A_requantise_every_step": us(t_a), "us_B_k_prequantised": us(t_b),
            "stages_us": {"quantise": us(t_quant), "gemv": us(t_gemv), "softmax_top_p": us(t_topp),
                          "attention": us(t_attn)},
            "survivors_mean": float(ra["mask"].sum(-1).float().mean())}


def cpu_baseline(N: int, H: int, budget: int, top_p: float, batch_scale: int, dev, seed: int = 0,
                 warmups: int = 1, repeats: int = 3, survivors=None):
    """Times the CPU oracle (torch fp32 + the C quantiser and top-p restatement) on one batch
    element drawn by the generator the GPU workload uses (same planted heavy hitters), un-paged to
    dense K / V: one warm-up, the median of three runs, scaled by the batch size. The reference's
    own CPU case (B=1, context 4096) is timed as well, with its per-stage split."""
    from oracle import native, pyimpl_port as P
    from twilight_amd import synth
    torch.set_num_threads(os.cpu_count() or 1)
    threads = torch.get_num_threads()
    qd, kd, vd, (ids, _, _) = synth.layer_inputs_device(1, H, H, N, torch.float16, dev, seed=seed,
                                                        survivors=survivors, top_p=top_p,
                                                        budget=budget)
    order = ids.long()
    q = qd.float().cpu().reshape(1, H, 1, 128)
    k = kd[order].reshape(N, H, 128).permute(1, 0, 2).float().cpu().reshape(1, H, N, 128).contiguous()
    v = vd[order].reshape(N, H, 128).permute(1, 0, 2).float().cpu().reshape(1, H, N, 128).contiguous()
    del qd, kd, vd
    # (A) as the reference does it: K is re-quantised inside every decode step
    ta, ra = _median_time(lambda: P.decode_layer_dense(
        q, k, v, top_p=top_p, token_budget=budget, high_mode=native.HIGH_MAX, quant="storage",
        prob_dtype=torch.float16), warmups, repeats)
    # (B) K quantised once on append, as the GPU path does
    k_deq = torch.from_numpy(P.int4_quant_storage(k)[3])
    tb, _ = _median_time(lambda: P.decode_layer_dense(
        q, k, v, top_p=top_p, token_budget=budget, high_mode=native.HIGH_MAX, k_deq=k_deq,
        prob_dtype=torch.float16), warmups, repeats)
    del k, v, k_deq
    return {
        "value": ta * 1e6 * batch_scale, "unit": "us/layer", "cores": threads, "kind": "port",
        "value_k_prequantised": tb * 1e6 * batch_scale,
        "sample": (f"1 of {batch_scale} batch elements (32 heads x {N} tokens, budget {budget}, "
                   f"p {top_p}; same generator as the GPU workload) through "
                   f"oracle.pyimpl_port.decode_layer_dense, {warmups} warm-up, median of {repeats} "
                   f"runs, time x {batch_scale}; `value` re-quantises K every step like "
                   "twilight/pyimpl/attention.py:247-251 (variant A), `value_k_prequantised` does "
                   f"not (variant B); torch uses {threads} threads "
                   f"(os.cpu_count() = {os.cpu_count()}), the C quantiser / top-p one"),
        "survivors_mean": float(ra["mask"].sum(-1).float().mean()),
        "survivors_median": float(ra["mask"].sum(-1).float().median()),
        "cfg1": cpu_baseline_cfg1(),
    }


def bench_topp(args, L, dev) -> int:
    """The pruner alone: fp32 scores [8, 32, 8192], N(0,1) background + a Zipf(1.2) spike set of
    1..512 tokens per row at random positions; softmax + top-p + compaction in one launch
    (twl_softmax_top_p_f32), p in {0.85, 0.95}. Four score tensors are visited round-robin."""
    from twilight_amd import synth
    B, H, M = 8, 32, 8192
    rows = B * H
    xs = [synth.topp_scores(B, H, M, seed=100 * i, max_spikes=512).to(dev) for i in range(4)]
    idx = torch.empty((B, H, M), dtype=torch.int32, device=dev)
    cnt = torch.empty((B, H), dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    res = {}
    for p in (0.85, 0.95):
        state = {"i": 0}

        def call():
            x = xs[state["i"] % 4]
            state["i"] += 1
            L.twl_softmax_top_p_f32(x.data_ptr(), M, 0, rows, M, 0, p, 1, 0, 0, idx.data_ptr(), M,
                                    cnt.data_ptr(), 0, 0, stream)
        us = _time_calls(call, args.steps, args.warmup)
        surv = []
        for x in xs:
            L.twl_softmax_top_p_f32(x.data_ptr(), M, 0, rows, M, 0, p, 1, 0, 0, idx.data_ptr(), M,
                                    cnt.data_ptr(), 0, 0, stream)
            torch.cuda.synchronize()
            surv.append(cnt.float().cpu())
        sv = torch.cat([t.flatten() for t in surv])
        nbytes = rows * M * 4 + int(sv.mean() * rows) * 4 + rows * 4
        res[str(p)] = {"us": round(us, 2), "survivors_median": float(sv.median()),
                       "survivors_mean": round(float(sv.mean()), 1), "survivors_max": int(sv.max()),
                       "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1)}
    # the drop-in mask ops on normalised probabilities (top_p_fp32_return_mask /
    # top_p_fp16_return_mask, high = probs[..., 0] as the reference has it, token 0 the maximum)
    xs1 = [synth.topp_scores(B, H, M, seed=100 * i + 7, max_spikes=512, first_is_max=True).to(dev)
           for i in range(4)]
    masks = {}
    mask = torch.empty((rows, M), dtype=torch.uint8, device=dev)
    for name, dt in (("fp32", torch.float32), ("fp32_exact", torch.float32), ("fp16", torch.float16),
                     ("bf16", torch.bfloat16)):
        ps = [torch.softmax(x, -1).to(dt).contiguous() for x in xs1]
        state = {"i": 0}

        def call_mask():
            pr = ps[state["i"] % 4]
            state["i"] += 1
            if name == "fp32_exact":
                L.twl_top_p_f32_exact(pr.data_ptr(), mask.data_ptr(), 0, 0, 0, 0.95, rows, M, M, 0, 0, 0, stream)
            elif dt == torch.float32:
                L.twl_top_p_f32(pr.data_ptr(), mask.data_ptr(), 0, 0, 0, 0.95, rows, M, M, 0, 0, 0, stream)
            else:
                L.twl_top_p_f16(pr.data_ptr(), 0 if dt == torch.float16 else 1, mask.data_ptr(), 0, 0, 0,
                                0.95, rows, M, M, 0, 0, 0, stream)
        masks[name] = round(_time_calls(call_mask, args.steps, args.warmup), 2)
    line = {"metric": "us/top-p call (softmax + top-p + compaction)", "value": res["0.95"]["us"],
            "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(res["0.95"]["us"] / 1e3, 5), "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "top-p pruner alone, fp32 scores [8, 32, 8192], Zipf(1.2) spike "
                                   "sets of 1-512 tokens per row, high = row max"},
            "per_p": res,
            "mask_ops_us_p095": masks,
            "mask_ops_what": "twl_top_p_f32 / twl_top_p_f32_exact / twl_top_p_f16 on [8, 32, 8192] "
                             "probabilities writing the byte mask; fp32_exact and the 16-bit forms "
                             "run the reference's arithmetic in cub::BlockReduce's order (1024 "
                             "threads per row)"}
    print(json.dumps(line))
    return 0


def bench_ftka(args, dev) -> int:
    """The GEMV call shapes of benchmark/efficiency/bench_gemv.py (32 heads, head_dim 128, token
    pages, page lists shared by the heads of a request) and the Double-Sparse label ops, at batch
    8 and 32768 tokens per request. Unlike the reference's bench every request has pages of its own
    (its requests all point at the same 32768 pages, which a cache then serves 7 times out of 8)
    and two caches are visited in turn, so every call streams cold data."""
    import twilight_amd.kernel as K
    B, H, D, N = args.batch, 32, 128, args.context
    g = torch.Generator(device=dev); g.manual_seed(0)
    pages = B * N
    idx = torch.arange(pages, dtype=torch.int32, device=dev)
    indptr = (torch.arange(B + 1, dtype=torch.int32) * N).to(dev)
    last = torch.ones(B, dtype=torch.int32, device=dev)
    q = torch.randn((B, H, D), device=dev, generator=g, dtype=torch.float16)
    res = {}

    def timed(name, make, nbytes, note=None):
        fns = [make(i) for i in range(2)]
        state = {"i": 0}

        def call():
            fns[state["i"] & 1]()
            state["i"] += 1
        us = _time_calls(call, max(args.steps // 4, 20), 4)
        res[name] = {"us": round(us, 2), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                     "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        if note:
            res[name]["note"] = note

    # fp16 K (bench_gemv.py:191-247)
    k16 = [torch.randn((pages, 1, H, D), device=dev, generator=g, dtype=torch.float16) for _ in range(2)]
    o16 = torch.empty((B, H, 1, N), dtype=torch.float16, device=dev)
    timed("batched_sparse_gemv", lambda i: lambda: K.batched_sparse_gemv(q, o16, k16[i], idx, indptr, last),
          pages * H * D * 2 + B * H * N * 2 + pages * 4)
    del k16
    # int8 K + per-token scale / zero (bench_gemv.py:67-147)
    k8 = [torch.randint(0, 256, (pages, 1, H, D), device=dev, generator=g, dtype=torch.uint8) for _ in range(2)]
    sc = [torch.rand((pages, 1, H), device=dev, generator=g).half() * 0.02 + 0.001 for _ in range(2)]
    zr = [torch.randn((pages, 1, H), device=dev, generator=g).half() * 0.1 for _ in range(2)]
    o8 = torch.empty((B, H, N), dtype=torch.float16, device=dev)
    timed("batched_sparse_gemv_int8_k",
          lambda i: lambda: K.batched_sparse_gemv_int8_k(q, o8, k8[i], sc[i], zr[i], idx, indptr, last),
          pages * H * (D + 4) + B * H * N * 2 + pages * 4)
    del k8
    # int4 K, two nibbles per byte (bench_gemv.py:377-454)
    k4 = [torch.randint(0, 256, (pages, 1, H, D // 2), device=dev, generator=g, dtype=torch.uint8) for _ in range(2)]
    timed("batched_sparse_gemv_int4_k",
          lambda i: lambda: K.batched_sparse_gemv_int4_k(q, o8, k4[i], sc[i], zr[i], idx, indptr, last),
          pages * H * (D // 2 + 4) + B * H * N * 2 + pages * 4)
    del k4, sc, zr
    # one request, contiguous K (bench_gemv.py:13-53; its largest length is 16384)
    ks = [torch.randn((16384, H, D), device=dev, generator=g, dtype=torch.float16) for _ in range(2)]
    os_ = torch.empty((H, 16384), dtype=torch.float16, device=dev)
    timed("single_sparse_gemv", lambda i: lambda: K.single_sparse_gemv(q[0], os_, ks[i]),
          16384 * H * D * 2 + H * 16384 * 2, note="one request of 16384 tokens")
    del ks
    # Double-Sparse label ops (twilight/pyimpl/double_sparse.py:17): 16 heavy channels
    r = 16
    chan = torch.stack([torch.randperm(D, device=dev, generator=g)[:r] for _ in range(H)]).to(torch.int64)
    xk = [torch.randn((B * N, H, D), device=dev, generator=g, dtype=torch.float16) for _ in range(2)]
    lab = torch.empty((B * N, H, r), dtype=torch.float16, device=dev)
    timed("get_label_tensor", lambda i: lambda: K.get_label_tensor(xk[i], chan, lab, r),
          B * N * H * (D + r) * 2, note="16 of 128 channels at random positions touch every "
                                        "32-byte sector of a 256-byte row: the rows are counted whole")
    del xk
    ql = torch.randn((B, H, r), device=dev, generator=g, dtype=torch.float16)
    kl = [torch.randint(-128, 128, (B * N, H, r), device=dev, generator=g, dtype=torch.int8) for _ in range(2)]
    ksc = [torch.rand((B * N, H), device=dev, generator=g).half() for _ in range(2)]
    ob = torch.empty((B, H, N), dtype=torch.float16, device=dev)
    timed("bgemv_int8", lambda i: lambda: K.bgemv_int8(ql, kl[i], ksc[i], ob),
          B * N * H * (r + 2) + B * H * N * 2)
    del kl, ksc
    # per-block int8 QK^T log-sum-exp, prefill shape (qk_int8_per_block.py:111-143)
    bq, hq, nq = 1, 32, 4096
    qi = torch.randint(-128, 128, (bq, hq, nq, D), device=dev, generator=g, dtype=torch.int8)
    ki = torch.randint(-128, 128, (bq, hq, nq, D), device=dev, generator=g, dtype=torch.int8)
    qs = torch.rand((bq, hq, nq // 128), device=dev, generator=g) * 0.01
    kss = torch.rand((bq, hq, nq // 64), device=dev, generator=g) * 0.01
    us = _time_calls(lambda: K.qk_int8_per_block(qi, ki, qs, kss, return_lse=True), 20, 3)
    ops = 2.0 * bq * hq * nq * nq * D
    res["qk_int8_per_block"] = {"us": round(us, 2), "int8_TOPs": round(ops / us / 1e6, 1),
                                "frac_of_int8_mfma_peak": round(ops / us / 1e6 / 5000.0, 4),
                                "note": "1 x 32 heads x 4096 x 4096 x 128, includes allocating and "
                                        "zeroing the reference's first output"}
    line = {"metric": "us per call, ftka GEMV call shapes and Double-Sparse ops",
            "value": res["batched_sparse_gemv_int4_k"]["us"], "unit": "us", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(res["batched_sparse_gemv_int4_k"]["us"] / 1e3, 5),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic",
            "config": {"workload": f"ftka-shaped GEMVs and label ops, B={B}, 32 heads, head_dim 128, "
                                   f"{N} tokens per request, token pages; value = the INT4 GEMV"},
            "ops": res}
    print(json.dumps(line))
    return 0


def bench_llama3_model(args, dev, emit: bool = True):
    """Whole-model decode at the Llama-3-8B shape: every layer of a random-initialised model
    (GQA 32 / 8 heads, bf16), B requests with a synthetic context of N tokens already in the
    caches, decode steps timed end to end — once dense (torch SDPA over a static KV cache) and once
    with the Select-then-Prune path in layers 2.. (the first two layers stay dense, as the
    reference's configuration has them, twilight/pyimpl/attention.py:199-201). Everything outside
    the attention modules is the model's own eager PyTorch code in both runs."""
    from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM, StaticCache
    from twilight_amd import hf
    B, N, nl = args.batch, args.context, args.model_layers
    steps, warmup = min(args.steps, 32), min(args.warmup, 4)
    top_p = args.top_p
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
    # A random-initialised model attends almost uniformly, which no trained model does: scale the
    # query projection so that the softmax over the context is as peaked as the few hundred kept
    # tokens per head that the reference reports; the kept count is part of the output.
    with torch.no_grad():
        for lay in model.model.layers:
            lay.self_attn.q_proj.weight.mul_(args.q_gain)

    def kv(layer):
        g = torch.Generator(device=dev).manual_seed(1000 + layer)
        k = torch.randn((B, 8, N, 128), generator=g, device=dev, dtype=torch.bfloat16)
        v = torch.randn((B, 8, N, 128), generator=g, device=dev, dtype=torch.bfloat16)
        return k, v

    ids = torch.randint(0, cfg.vocab_size, (steps + warmup, B, 1),
                        generator=torch.Generator().manual_seed(7)).to(dev)

    def run(cache, positions=False):
        # positions: pass position_ids explicitly (needed when nothing updates the model's cache)
        def pos(s):
            return {"position_ids": torch.full((B, 1), N + s, device=dev)} if positions else {}
        with torch.no_grad():
            for s in range(warmup):
                model(ids[s], past_key_values=cache, use_cache=True, **pos(s))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for s in range(warmup, warmup + steps):
                out = model(ids[s], past_key_values=cache, use_cache=True, **pos(s))
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / steps, out.logits[:, -1].float()

    reserve = steps + warmup + 16

    def make_cache(kind, layers):
        # "static": preallocated K / V, attention over the whole buffer under a mask;
        # "dynamic": K / V grown by concatenation every step, attention without a mask
        c = (StaticCache(config=cfg, max_cache_len=N + reserve) if kind == "static"
             else DynamicCache(config=cfg))
        for i in layers:
            c.update(*kv(i), i)
        return c

    dense = {}
    if not args.no_dense:
        for kind in ("static", "dynamic"):
            cache = make_cache(kind, range(nl))
            t, _ = run(cache)
            dense[kind] = t * 1e3
            del cache
            torch.cuda.empty_cache()

    sparse_cfg = {"compressor": {"type": "none"},
                  "selector": {"type": "quest", "token_budget": args.budget, "chunk_size": 16},
                  "weight_estimator": {"type": "min_max_quant", "quant_bit": 4},
                  "weight_pruner": {"type": "top_p", "threshold": top_p},
                  "skip_first_two_layers": True, "use_estimated_weights_in_attn": False}
    def run_graphed():
        step = hf.GraphedDecodeStep(model)
        for s in range(warmup):              # the first call records the step
            step(ids[s])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s in range(warmup, warmup + steps):
            logits = step(ids[s])
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps, logits[:, -1].float()

    twi = {}
    modes = ("model", "paged", "paged+graph") if args.model_mode == "all" else (args.model_mode,)
    for mode in modes:
        # "model": the two dense layers run the model's own attention over a DynamicCache;
        # "paged": they run twl_group_attn over paged K / V and the model's cache stays empty;
        # "paged+graph": the same step recorded once into a HIP graph and replayed
        info, _ = hf.enable_sparse_attention(model, sparse_cfg, enable_budget_info=True,
                                             reserve_tokens=reserve + 16, keep_hf_cache=False,
                                             dense_layers="model" if mode == "model" else "paged")
        states = [getattr(model.model.layers[i].self_attn, "_twilight_state", None) for i in range(nl)]
        cache = make_cache("dynamic", [i for i in range(nl) if states[i] is None])
        for i in range(nl):
            if states[i] is not None:
                hf.fill_from_prefill(states[i], *kv(i), cfg.num_attention_heads)
        t, logits = run_graphed() if mode == "paged+graph" else run(cache, positions=True)
        twi[mode] = t * 1e3
        kept = info.get_total_avg_budget()
        if mode != modes[-1]:
            hf.disable_sparse_attention(model)
            del cache, states
            torch.cuda.empty_cache()
    best = min(twi, key=twi.get)
    twi_ms = twi[best]
    dense_best = min(dense, key=dense.get) if dense else None
    dense_ms = dense[dense_best] if dense else None
    # GPU time of the decode-layer calls alone, by events around them in one more step
    ev = []

    def timed(lay):
        def call(q):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            o = lay(q)
            e1.record()
            ev.append((e0, e1))
            return o
        return call

    for i in range(nl):
        st = getattr(model.model.layers[i].self_attn, "_twilight_state", None)
        if st is not None and not st.dense:
            st.layer = _Timed(st.layer, timed(st.layer))
    with torch.no_grad():
        model(ids[0], past_key_values=cache, use_cache=True,
              position_ids=torch.full((B, 1), N + steps + warmup, device=dev))
    torch.cuda.synchronize()
    layer_us = sum(a.elapsed_time(b) for a, b in ev) * 1e3 / max(len(ev), 1)
    hf.disable_sparse_attention(model)
    del cache, states
    torch.cuda.empty_cache()
    # one more run: the graph-replayed step with one Quest candidate list per kv head
    info, _ = hf.enable_sparse_attention(model, sparse_cfg, enable_budget_info=True,
                                         reserve_tokens=reserve + 16, keep_hf_cache=False,
                                         dense_layers="paged", group_select=True)
    for i in range(nl):
        hf.fill_from_prefill(model.model.layers[i].self_attn._twilight_state, *kv(i),
                             cfg.num_attention_heads)
    tg, lg = run_graphed()
    grp_run = {"what": "enable_sparse_attention(group_select=True): one Quest candidate list per "
                       "kv head instead of one per q head (not the reference's selection); the "
                       "step replayed from a HIP graph",
               "ms_per_step": round(tg * 1e3, 3), "tokens_per_s": round(B / tg, 1),
               "kept_tokens_per_head_mean": round(info.get_total_avg_budget(), 1),
               "finite_logits": bool(torch.isfinite(lg).all())}
    hf.disable_sparse_attention(model)
    line = {
        "metric": "tokens/s, whole-model decode with Twilight applied", "value": round(B / twi_ms * 1e3, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(twi_ms, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"random-init Llama-3-8B shape, {nl} layers, GQA 32/8, bf16, B={B}, "
                               f"context {N} (synthetic K/V), budget {args.budget}, p={top_p}, "
                               f"layers 0-1 dense, q_proj x{args.q_gain}"},
        "dense_layers_what": "how layers 0-1 decode: 'model' = the model's own attention (torch "
                             "SDPA) over a DynamicCache, 'paged' = twl_group_attn over paged K/V, "
                             "'paged+graph' = that step recorded into one HIP graph and replayed",
        "dense_layers": best,
        "ms_per_step_by_dense_layers": {k: round(v, 3) for k, v in twi.items()},
        "dense": None if dense_ms is None else {
            "ms_per_step": round(dense_ms, 3), "tokens_per_s": round(B / dense_ms * 1e3, 1),
            "model_cache": dense_best,
            "ms_per_step_by_model_cache": {k: round(v, 3) for k, v in dense.items()},
            "what": "same model and context, every layer through the model's own attention "
                    "(torch SDPA) over the transformers cache class named"},
        "speedup_vs_dense": None if dense_ms is None else round(dense_ms / twi_ms, 2),
        "kept_tokens_per_head_mean": round(kept, 1),
        "twilight_layer_us": round(layer_us, 1),
        "finite_logits": bool(torch.isfinite(logits).all()),
        "group_select": grp_run,
    }
    del model
    torch.cuda.empty_cache()
    if emit:
        print(json.dumps(line))
        return 0
    return line


class _Timed:
    """Stands in for a decode layer object: calls go through ``fn``, attributes to the layer."""

    def __init__(self, layer, fn):
        self._layer, self._fn = layer, fn

    def __call__(self, q):
        return self._fn(q)

    def __getattr__(self, name):
        return getattr(self._layer, name)


def _planted_name(survivors) -> str:
    return ("peaked (a fixed shift of 0.9 q, slots with replacement: most rows hold one "
            "dominant token)" if survivors is None else
            f"calibrated (shift solved per row for a top-p nucleus of {survivors[0]}-{survivors[1]} "
            "tokens over the row's candidates)")


def measure_shape(L, dev, B, H, Hkv, N, dt, budget, top_p, n_layers, steps, warmup,
                  dense: bool = False, survivors=None):
    """One more shape of the same layer, measured the way the headline figure is: ``n_layers``
    independent caches visited round-robin, wall time per ``twl_decode_layer`` step, and the two
    kernels of the step timed alone with events. Returns a dict for the JSON line."""
    from twilight_amd import synth
    from twilight_amd.cache import PagedKVCache
    from twilight_amd.layer import TwilightDecodeLayer
    D, npg = 128, N // 16
    qcode = 1 if dt == torch.bfloat16 else 0
    layers, qs = [], []
    for li in range(n_layers):
        q, k, v, (ids, indptr, last) = synth.layer_inputs_device(
            B, H, Hkv, N, dt, dev, seed=500 + 10 * li, survivors=survivors, top_p=top_p,
            budget=budget)
        cache = PagedKVCache(B * npg, Hkv, dt, dev)
        cache.k_cache, cache.v_cache = k, v
        cache.set_page_table(ids, indptr, last)
        cache.rebuild_shadow()
        cache.enable_planes()
        layers.append(TwilightDecodeLayer(cache, H, token_budget=budget, top_p=top_p, high="max"))
        qs.append(q)
    torch.cuda.synchronize()
    for i in range(warmup):
        layers[i % n_layers].forward(qs[i % n_layers])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        layers[i % n_layers].forward(qs[i % n_layers])
    torch.cuda.synchronize()
    wall_us = (time.perf_counter() - t0) * 1e6 / steps
    for i in range(n_layers):
        layers[i].forward(qs[i])
    torch.cuda.synchronize()
    cnts = torch.stack([l.count for l in layers]).float()
    n_bar = float(cnts.mean())
    rows, kp = B * H, layers[0].k_pages
    M = kp * 16
    stream = torch.cuda.current_stream().cuda_stream
    p = lambda t: 0 if t is None else t.data_ptr()
    sm = 1.0 / math.sqrt(D)
    state = {"i": 0}

    def rot(make):
        fns = [make(layers[i], layers[i].cache, qs[i]) for i in range(n_layers)]

        def call():
            fns[state["i"] % n_layers]()
            state["i"] += 1
        return call
    row_us = _time_calls(rot(lambda l, c, q: lambda: L.twl_select_estimate_prune(
        p(q), qcode, p(c.meta), p(c.k_int4), p(c.kv_page_indices), p(c.kv_page_indptr),
        p(c.kv_last_page_len), B, H, Hkv, budget, npg, sm, 0, top_p, 1, p(l.sel_pages), kp,
        p(l.sel_count), p(l.idx), M, p(l.count), 0, 0, 0, M, p(l.cand_count), p(c.meta_planes),
        c.meta_planes.size(4), 0, 0, stream)), max(steps, 40), 2 * n_layers)
    attn_us = _time_calls(rot(lambda l, c, q: lambda: L.twl_sparse_attn(
        p(q), p(l.out), qcode, p(c.k_cache), p(c.v_cache), *c.k_cache.stride()[:3], p(l.idx), M,
        p(l.count), p(c.kv_page_indices), p(c.kv_page_indptr), B, H, Hkv, sm, 0,
        p(l.attn_workspace), l.attn_workspace.numel(), stream)), max(steps, 40), 2 * n_layers)
    attn_bytes = int(rows * n_bar) * (2 * D * 2 + 4) + rows * D * 4
    lists = rows * npg * 4 + rows * kp * 8 + int(rows * n_bar) * 4 + rows * 12 + rows * D * 2
    # per q head, as the reference's code selects and prunes (attention.py:124-126): metadata once
    # per kv head (the record is shared by the group), INT4 records once per q-head row
    per_head = B * Hkv * npg * 512 + rows * M * 80 + lists + attn_bytes
    # one candidate list per kv head (INT4 records read once for the group's q heads, fp32
    # scores per q head): the lower count for GQA; equal to the above without GQA
    shared = B * Hkv * npg * 512 + B * Hkv * M * 80 + rows * M * 4 * (1 if H != Hkv else 0) \
        + lists + attn_bytes
    by_design = per_head - (B * Hkv * npg * 512 >> (H // Hkv))
    gb = lambda n: round(n / wall_us / 1e3 / HBM_PEAK_GBS, 4)
    out = {"workload": f"B={B}, {H} q / {Hkv} kv heads, {'bf16' if qcode else 'fp16'}, context {N}, "
                       f"budget {budget}, p {top_p}, {n_layers} caches rotated",
           "us_per_layer": round(wall_us, 2), "steps": steps,
           "select_estimate_prune_us": round(row_us, 2), "sparse_attn_us": round(attn_us, 2),
           "survivors_mean": round(n_bar, 1), "survivors_median": float(cnts.median()),
           "survivors_max": int(cnts.max()), "planted": _planted_name(survivors),
           "layer_bytes_per_q_head_lists": per_head, "frac_of_hbm_peak_per_q_head_lists": gb(per_head),
           "layer_bytes_read_by_design": by_design, "frac_of_hbm_peak_read_by_design": gb(by_design)}
    if H != Hkv:
        out["layer_bytes_shared_candidate_lists"] = shared
        out["frac_of_hbm_peak_shared_candidate_lists"] = gb(shared)
    if H != Hkv and H // Hkv in (2, 4, 8):
        # the option that realises the shared count: one Quest selection per kv head, metadata and
        # INT4 records read once per kv head, five launches (scores, top-k, group GEMV, pruner,
        # attention)
        glayers = [TwilightDecodeLayer(l.cache, H, token_budget=budget, top_p=top_p, high="max",
                                       group_select=True) for l in layers]
        for i in range(warmup):
            glayers[i % n_layers].forward(qs[i % n_layers])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            glayers[i % n_layers].forward(qs[i % n_layers])
        torch.cuda.synchronize()
        g_us = (time.perf_counter() - t0) * 1e6 / steps
        for i in range(n_layers):
            glayers[i].forward(qs[i])
        torch.cuda.synchronize()
        g_bar = float(torch.stack([l.count for l in glayers]).float().mean())
        gemv_us = _time_calls(rot(lambda l, c, q: lambda: L.twl_gemv_int4_group(
            p(q), qcode, p(l.scores), M, p(l.cand_count), p(c.k_int4), p(l.sel_pages),
            p(l.sel_count), kp, p(c.kv_page_indices), p(c.kv_page_indptr), p(c.kv_last_page_len),
            B, H, Hkv, kp, sm, stream)), max(steps, 40), 2 * n_layers)
        gemv_bytes = B * Hkv * M * 80 + rows * M * 4
        out["group_select"] = {
            "what": "TwilightDecodeLayer(group_select=True): one candidate list per kv head "
                    "(largest q-head page score), not the reference's per-q-head selection",
            "us_per_layer": round(g_us, 2), "survivors_mean": round(g_bar, 1),
            "frac_of_hbm_peak_shared_candidate_lists": round(shared / g_us / 1e3 / HBM_PEAK_GBS, 4),
            "gemv_int4_group_us": round(gemv_us, 2), "gemv_int4_group_bytes": gemv_bytes,
            "gemv_int4_group_frac_of_hbm_peak": round(gemv_bytes / gemv_us / 1e3 / HBM_PEAK_GBS, 4)}
        del glayers
    if dense:
        gws = torch.empty(int(L.twl_group_attn_workspace_bytes(B, H, Hkv, N, 0)), dtype=torch.uint8,
                          device=dev)
        outd = torch.empty_like(qs[0])
        us = _time_calls(rot(lambda l, c, q: lambda: L.twl_group_attn(
            p(q), p(outd), qcode, p(c.k_cache), p(c.v_cache), *c.k_cache.stride()[:3], 0, 0, 0, N,
            p(c.kv_page_indices), p(c.kv_page_indptr), p(c.kv_last_page_len), B, H, Hkv, sm, 0,
            p(gws), gws.numel(), stream)), 40, n_layers)
        nbytes = B * Hkv * N * 2 * D * 2
        out["dense_group_attn_us"] = round(us, 2)
        out["dense_group_attn_frac_of_hbm_peak"] = round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)
        out["speedup_vs_dense_decode"] = round(us / wall_us, 2)
    del layers, qs
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=32768)
    ap.add_argument("--budget", type=int, default=8192)
    ap.add_argument("--top-p", type=float, default=None,
                    help="pruning threshold (default 0.95; 0.9 for the Llama-3 workloads)")
    ap.add_argument("--workload", choices=["longchat", "llama3", "llama3-model", "topp", "ftka"],
                    default="longchat",
                    help="longchat: 32 MHA heads fp16 (the headline workload); llama3: GQA 32/8 "
                         "bf16, with a dense-decode baseline (the same attention kernel over "
                         "every token); topp: the pruner kernel alone on [8,32,8192] scores; "
                         "ftka: the NHD GEMV call shapes of the reference's bench_gemv.py and the "
                         "Double-Sparse label ops; llama3-model: whole-model decode of a "
                         "random-initialised Llama-3-8B shape, dense against Twilight, tokens/s")
    ap.add_argument("--model-layers", type=int, default=32, help="llama3-model: number of layers")
    ap.add_argument("--q-gain", type=float, default=3.0,
                    help="llama3-model: factor on the random q_proj weights (peakedness of attention)")
    ap.add_argument("--no-dense", action="store_true", help="llama3-model: skip the dense run")
    ap.add_argument("--model-mode", choices=["all", "model", "paged", "paged+graph"], default="all",
                    help="llama3-model: which of the patched runs to time (see dense_layers_what)")
    ap.add_argument("--layers", type=int, default=4,
                    help="independent layer caches visited round-robin (cold-cache steps)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 4 device copies of 1 GiB (a kernel of known traffic, used to "
                         "scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--split-estimator", action="store_true",
                    help="run the INT4 GEMV and the softmax + top-p as two launches instead of one")
    ap.add_argument("--no-planes", action="store_true",
                    help="keep the Quest metadata in the 512-byte record layout only")
    ap.add_argument("--group-union", action="store_true",
                    help="attention over the union of each kv head's survivor lists (GQA)")
    ap.add_argument("--group-select", action="store_true",
                    help="one Quest selection per kv head, INT4 records read once per group (GQA)")
    ap.add_argument("--planted", choices=["calibrated", "peaked"], default="calibrated",
                    help="planted heavy hitters: calibrated = K shift solved per row so that top-p "
                         "keeps 100-400 tokens; peaked = one fixed shift (median 2 kept tokens)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-shapes", action="store_true",
                    help="default workload: skip the B=16 and the Llama-3-shape sections")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel breakdown")
    args = ap.parse_args()
    if args.top_p is None:
        args.top_p = 0.9 if args.workload in ("llama3", "llama3-model") else 0.95
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (every (batch, head) "
              "row is independent); run with --gpus 1", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2

    from twilight_amd import _lib, build, synth
    from twilight_amd.cache import PagedKVCache
    from twilight_amd.layer import TwilightDecodeLayer
    if not os.path.exists(build.LIB_PATH):
        build.build_library()
    L = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "topp":
        return bench_topp(args, L, dev)
    if args.workload == "ftka":
        return bench_ftka(args, dev)
    if args.workload == "llama3-model":
        return bench_llama3_model(args, dev)
    llama = args.workload == "llama3"
    survivors = (100, 400) if args.planted == "calibrated" else None
    B, H, Hkv, N, D = args.batch, 32, (8 if llama else 32), args.context, 128
    npg = N // 16
    dt = torch.bfloat16 if llama else torch.float16
    qcode = 1 if llama else 0   # twl_dtype of q / K / V

    if args.calibrate_copy:
        src = torch.full((1 << 28,), 1.0, dtype=torch.float32, device=dev)   # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- inputs, resident in HBM before anything is timed ----------------------------------
    # `--layers` independent caches (different data, same shape) are visited round-robin, as the
    # layers of a model are during decode: no step finds its KV, INT4 shadow or Quest metadata
    # left in the 256 MB last-level cache by the previous step.
    layers, qs = [], []
    for li in range(args.layers):
        q, k, v, (ids, indptr, last) = synth.layer_inputs_device(
            B, H, Hkv, N, dt, dev, seed=10 * li, survivors=survivors, top_p=args.top_p,
            budget=args.budget)
        cache = PagedKVCache(B * npg, Hkv, dt, dev)
        cache.k_cache, cache.v_cache = k, v
        cache.set_page_table(ids, indptr, last)
        cache.rebuild_shadow()
        if not args.no_planes:
            cache.enable_planes()      # metadata also in plane layout: the row kernel reads half
        layers.append(TwilightDecodeLayer(cache, H, token_budget=args.budget, top_p=args.top_p,
                                          high="max", fused_estimator=not args.split_estimator,
                                          group_union=args.group_union,
                                          group_select=args.group_select))
        qs.append(q)
    torch.cuda.synchronize()
    nl = len(layers)

    # ---- the timed region: K steps of the whole layer --------------------------------------
    for i in range(args.warmup):
        layers[i % nl].forward(qs[i % nl])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        layers[i % nl].forward(qs[i % nl])
    torch.cuda.synchronize()
    wall_us = (time.perf_counter() - t0) * 1e6 / args.steps
    for i in range(nl):                      # leave every layer's buffers as a whole step does
        layers[i].forward(qs[i])
    torch.cuda.synchronize()
    # the same steps recorded once into a HIP graph (one step of each rotated layer) and replayed,
    # as a serving loop that records its decode step would run them (reported beside `value`)
    graph_us = None
    if args.steps >= nl:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(nl):
                layers[i].forward(qs[i])
        reps = max(args.steps // nl, 1)
        g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            g.replay()
        torch.cuda.synchronize()
        graph_us = (time.perf_counter() - t0) * 1e6 / (reps * nl)
    counts = torch.stack([l.count for l in layers]).float()
    n_bar = float(counts.mean())
    n_max = int(counts.max())
    kp = layers[0].k_pages
    M = kp * 16
    rows = B * H

    # ---- per-kernel times through the stand-alone entry points, same buffers, same rotation ----
    kernels = {}
    stream = torch.cuda.current_stream().cuda_stream
    p = lambda t: 0 if t is None else t.data_ptr()
    sm = 1.0 / math.sqrt(D)

    def rotating(make):
        fns = [make(layers[i], layers[i].cache, qs[i]) for i in range(nl)]
        state = {"i": 0}

        def call():
            fns[state["i"] % nl]()
            state["i"] += 1
        return call

    if not args.no_kernels:
        it, wu = max(args.steps, 50), 2 * nl
        calls = {
            "quest_score": (rotating(lambda l, c, q: lambda: L.twl_quest_page_scores(
                p(q), qcode, p(c.meta), p(c.kv_page_indices), p(c.kv_page_indptr), B, H, Hkv,
                npg, p(l.page_scores), npg, stream)),
                B * Hkv * npg * 512 + rows * npg * 4 + rows * D * 2),
            "quest_topk": (rotating(lambda l, c, q: lambda: L.twl_quest_topk_pages(
                p(l.page_scores), npg, p(c.kv_page_indptr), B, H, args.budget, npg,
                p(l.sel_pages), kp, p(l.sel_count), stream)), rows * (npg * 4 + kp * 4 + 4)),
            "gemv_int4": (rotating(lambda l, c, q: lambda: L.twl_gemv_int4(
                p(q), qcode, p(l.scores), M, p(l.cand_count), p(c.k_int4), p(l.sel_pages),
                p(l.sel_count), kp, p(c.kv_page_indices), p(c.kv_page_indptr),
                p(c.kv_last_page_len), B, H, Hkv, kp, sm, stream)),
                rows * M * (64 + 16 + 4) + rows * D * 2 + rows * kp * 8),
            "select_estimate_prune": (rotating(lambda l, c, q: lambda: L.twl_select_estimate_prune(
                p(q), qcode, p(c.meta), p(c.k_int4), p(c.kv_page_indices), p(c.kv_page_indptr),
                p(c.kv_last_page_len), B, H, Hkv, args.budget, npg, sm, 0, args.top_p, 1,
                p(l.sel_pages), kp, p(l.sel_count), p(l.idx), M, p(l.count), 0, 0, 0, M,
                p(l.cand_count), p(c.meta_planes),
                0 if c.meta_planes is None else c.meta_planes.size(4), 0, 0, stream)),
                B * Hkv * npg * 512 + rows * M * (64 + 16) + rows * D * 2 + rows * npg * 4
                + rows * kp * 8 + int(rows * n_bar) * 4 + rows * 12),
            "gemv_top_p": (rotating(lambda l, c, q: lambda: L.twl_gemv_top_p(
                p(q), qcode, p(c.k_int4), p(l.sel_pages), p(l.sel_count), kp,
                p(c.kv_page_indices), p(c.kv_page_indptr), p(c.kv_last_page_len), B, H, Hkv, kp,
                sm, 0, args.top_p, 1, p(l.idx), M, p(l.count), 0, M, p(l.cand_count), 0, stream)),
                rows * M * (64 + 16) + rows * D * 2 + rows * kp * 8 + int(rows * n_bar) * 4
                + rows * 8),
            "softmax_top_p": (rotating(lambda l, c, q: lambda: L.twl_softmax_top_p_f32(
                p(l.scores), M, p(l.cand_count), rows, M, 0, args.top_p, 1, p(l.sel_pages),
                kp, p(l.idx), M, p(l.count), 0, 0, stream)),
                rows * M * 4 + int(rows * n_bar) * 4 + rows * 4),
            "sparse_attn": (rotating(lambda l, c, q: lambda: L.twl_sparse_attn(
                p(q), p(l.out), qcode, p(c.k_cache), p(c.v_cache), *c.k_cache.stride()[:3],
                p(l.idx), M, p(l.count), p(c.kv_page_indices), p(c.kv_page_indptr),
                B, H, Hkv, sm, 0, p(l.attn_workspace), l.attn_workspace.numel(), stream)),
                int(rows * n_bar) * (2 * D * 2 + 4) + rows * D * 4),
        }
        if layers[0].cache.meta_planes is not None and H == Hkv:
            calls["quest_score_planes"] = (rotating(
                lambda l, c, q: lambda: L.twl_quest_page_scores_planes(
                    p(q), qcode, p(c.meta_planes), c.meta_planes.size(4), 0, 0, p(c.meta),
                    p(c.kv_page_indices), p(c.kv_page_indptr),
                    B, H, Hkv, npg, p(l.page_scores), npg, stream)),
                rows * npg * 256 + rows * npg * 4 + rows * D * 2)   # the sign-selected runs only
        for name, (fn, nbytes) in calls.items():
            us = _time_calls(fn, it, wu)
            kernels[name] = {"us": round(us, 2), "bytes": nbytes,
                             "GBps": round(nbytes / us / 1e3, 1),
                             "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        if layers[0].cache.meta_planes is not None:
            # `bytes` above is the algorithm's figure (512 B of min/max metadata per row and
            # page); with the plane layout the kernel reads only the sign-selected half of it
            for name in ("select_estimate_prune",):
                k = kernels.get(name)
                if k:
                    # a (channel, plane) run stays unread when every q head of the kv head's
                    # group has the same sign there: 2^-G of the metadata on average
                    k["bytes_read_by_design"] = k["bytes"] - (B * Hkv * npg * 512 >> (H // Hkv))
                    k["GBps_read_by_design"] = round(k["bytes_read_by_design"] / k["us"] / 1e3, 1)

    # the kernels one layer step launches (the choice twl_decode_layer makes)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    split = args.split_estimator or 2 * rows < cus or (H != Hkv and 2 * rows == cus)
    has_planes = layers[0].cache.meta_planes is not None
    row_kernel = (not split and (H == Hkv or has_planes) and npg <= 8192
                  and (has_planes or rows <= 2 * cus))
    score = ("quest_score_planes" if layers[0].cache.meta_planes is not None and H == Hkv
             else "quest_score")
    if split:
        used = (score, "quest_topk", "gemv_int4", "softmax_top_p", "sparse_attn")
    elif row_kernel:
        used = ("select_estimate_prune", "sparse_attn")
    else:
        used = (score, "quest_topk", "gemv_top_p", "sparse_attn")
    if not row_kernel and kp == npg:
        used = tuple(n for n in used if n != score)   # every page is kept: no scoring launch
    for name in kernels:
        kernels[name]["in_layer_step"] = name in used
    layer_bytes = sum(kernels[n]["bytes"] for n in used) if kernels else None
    # dominant kernel of the step: the one-launch selector + estimator + pruner when the step
    # uses it, else the metadata stream
    if "select_estimate_prune" in used:
        dom_name = "select_estimate_prune"
    elif score in used:
        dom_name = score
    else:                                    # no scoring launch: the INT4 stream dominates
        dom_name = "gemv_top_p" if "gemv_top_p" in used else "gemv_int4"
    dom = kernels.get(dom_name)
    roofline = None
    if dom:
        default_cfg = (B, N, args.budget, llama) == (8, 32768, 8192, False)
        traffic = None
        if default_cfg:
            if dom_name == "quest_score":
                traffic = QUEST_SCORE_TRAFFIC_BYTES_DEFAULT
            elif dom_name == "quest_score_planes":
                traffic = None  # not measured for this kernel
            elif layers[0].cache.meta_planes is not None:
                traffic = (ROW_KERNEL_TRAFFIC_BYTES_DEFAULT if survivors is not None
                           else ROW_KERNEL_TRAFFIC_BYTES_PEAKED)
            else:
                traffic = ROW_KERNEL_TRAFFIC_BYTES_RECORDS
        roofline = {"bound": "hbm",
                    "kernel": ("quest_score_kernel" if dom_name == "quest_score"
                               else dom_name + "_kernel"),
                    "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": dom["frac_of_hbm_peak"], "bytes_per_launch": dom["bytes"],
                    "us_per_launch": dom["us"], "traffic": traffic,
                    "frac_traffic": (None if traffic is None else
                                     round(traffic / dom["us"] / 1e3 / HBM_PEAK_GBS, 4)),
                    "traffic_source": (None if traffic is None else
                                       "HBM counters of an earlier rocprofv3 --pmc run of this "
                                       "command (FETCH_SIZE, WRITE_SIZE scaled by a 1 GiB copy; "
                                       "summary under profiles/), not read in this run")}
        if "bytes_read_by_design" in dom:
            roofline["note"] = ("achieved = algorithmic bytes / time; the kernel reads only the "
                                "min or max runs that the signs of its queries select (plane "
                                "layout: half the metadata with one q head per kv head), so "
                                "its HBM traffic is below the algorithmic bytes: "
                                f"{dom['bytes_read_by_design']} B by design = "
                                f"{dom['GBps_read_by_design']} GB/s of real traffic")

    # ---- stand-alone INT4 GEMV at 8 x 32 x 32768 candidates (all pages of every request) ----
    gemv_cfg2 = None
    if not args.no_kernels and B == 8 and N == 32768 and not llama:
        out2 = torch.empty((B, H, N), dtype=torch.float32, device=dev)
        cnt2 = torch.empty((B, H), dtype=torch.int32, device=dev)
        fn = rotating(lambda l, c, q: lambda: L.twl_gemv_int4(
            p(q), qcode, p(out2), N, p(cnt2), p(c.k_int4), 0, 0, 0, p(c.kv_page_indices),
            p(c.kv_page_indptr), p(c.kv_last_page_len), B, H, Hkv, npg, sm, stream))
        us = _time_calls(fn, 50, 2 * nl)
        nbytes = rows * N * 84 + rows * D * 2
        gemv_cfg2 = {"us": round(us, 2), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                     "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                     "workload": "INT4 GEMV alone, B=8 H=32 D=128, 32768 candidates per head, "
                                 "shuffled pages"}
        del out2

    # ---- dense-decode baseline on the same GPU: the same attention kernel over every token ----
    dense = None
    if llama and not args.no_kernels:
        full_idx = torch.arange(N, dtype=torch.int32, device=dev).repeat(B, H, 1).contiguous()
        full_cnt = torch.full((B, H), N, dtype=torch.int32, device=dev)
        ws = torch.zeros(int(L.twl_sparse_attn_workspace_bytes(rows, N)), dtype=torch.uint8, device=dev)
        outd = torch.empty_like(qs[0])
        fn = rotating(lambda l, c, q: lambda: L.twl_sparse_attn(
            p(q), p(outd), qcode, p(c.k_cache), p(c.v_cache), *c.k_cache.stride()[:3], p(full_idx), N,
            p(full_cnt), p(c.kv_page_indices), p(c.kv_page_indptr), B, H, Hkv, sm, 0, p(ws),
            ws.numel(), stream))
        us = _time_calls(fn, 20, nl)
        nbytes = B * Hkv * N * 2 * D * 2
        dense = {"us": round(us, 2), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                 "what": "twl_sparse_attn over all 32768 tokens of every row (the sparse kernel "
                         "used densely: K/V are fetched per q head, 4x the bytes counted here, "
                         "which count K/V once per kv head)"}
        del full_idx, ws
        # the group kernel: K / V of a token fetched once for the 4 q heads of its kv head
        gws = torch.empty(int(L.twl_group_attn_workspace_bytes(B, H, Hkv, N, 0)), dtype=torch.uint8,
                          device=dev)
        fn = rotating(lambda l, c, q: lambda: L.twl_group_attn(
            p(q), p(outd), qcode, p(c.k_cache), p(c.v_cache), *c.k_cache.stride()[:3], 0, 0, 0, N,
            p(c.kv_page_indices), p(c.kv_page_indptr), p(c.kv_last_page_len), B, H, Hkv, sm, 0,
            p(gws), gws.numel(), stream))
        us = _time_calls(fn, 40, nl)
        dense["group_attn_us"] = round(us, 2)
        dense["group_attn_GBps"] = round(nbytes / us / 1e3, 1)
        dense["group_attn_frac_of_hbm_peak"] = round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)
        dense["group_attn_what"] = ("twl_group_attn over every token (dense paged decode, K/V read "
                                    "once per kv head, two launches: partial results + merge), "
                                    "cold caches")
        del gws
        # torch's own dense decode attention over contiguous K/V of one layer (GQA-aware)
        try:
            c0 = layers[0].cache
            phys = c0.kv_page_indices.long().reshape(B, npg)
            kd = c0.k_cache[phys].reshape(B, N, Hkv, D).permute(0, 2, 1, 3).contiguous()
            vd = c0.v_cache[phys].reshape(B, N, Hkv, D).permute(0, 2, 1, 3).contiguous()
            q4 = qs[0].reshape(B, H, 1, D)
            sdpa = lambda: torch.nn.functional.scaled_dot_product_attention(
                q4, kd, vd, is_causal=False, enable_gqa=True)
            dense["torch_sdpa_us"] = round(_time_calls(sdpa, 20, 3), 2)
            dense["torch_sdpa_what"] = ("torch.nn.functional.scaled_dot_product_attention, q "
                                        "[B,32,1,128], contiguous bf16 K/V [B,8,32768,128], "
                                        "enable_gqa=True, same data every call (warm caches)")
            del kd, vd
        except Exception as e:  # a missing SDPA backend must not fail the benchmark
            dense["torch_sdpa_us"] = None
            dense["torch_sdpa_what"] = f"not available: {type(e).__name__}: {e}"

    # ---- the two other layer shapes of the headline figure, in the same line ------------------
    extra = {}
    if (not llama and not args.no_extra_shapes and not args.split_estimator and not args.no_planes
            and (B, N, args.budget) == (8, 32768, 8192)):
        es, ew = max(20, min(args.steps, 60)), max(4, min(args.warmup, 10))
        # the same layer on the other planted workload (the headline of earlier runs)
        other = None if survivors is not None else (100, 400)
        extra["b8_" + ("peaked" if other is None else "calibrated")] = measure_shape(
            L, dev, 8, 32, 32, N, torch.float16, args.budget, args.top_p, 4, es, ew, survivors=other)
        extra["cfg4_b16"] = measure_shape(L, dev, 16, 32, 32, N, torch.float16, args.budget,
                                          args.top_p, 2, es, ew, survivors=survivors)
        # the rest of the batch axis of the reference's latency figure (figures/kernels.png)
        free_b = torch.cuda.mem_get_info()[0]
        for bb, ncache in ((32, 2), (64, 1)):
            need = ncache * bb * N * 32 * 128 * 2 * 2 * 1.45   # K, V, INT4 shadow, metadata twice
            if need > free_b * 0.9:
                extra[f"cfg4_b{bb}"] = {"skipped": f"needs about {need / 2**30:.0f} GiB, "
                                                   f"{free_b / 2**30:.0f} GiB free"}
                continue
            extra[f"cfg4_b{bb}"] = measure_shape(L, dev, bb, 32, 32, N, torch.float16, args.budget,
                                                 args.top_p, ncache, 20, 4, survivors=survivors)
        extra["cfg5_layer"] = measure_shape(L, dev, 8, 32, 8, N, torch.bfloat16, args.budget, 0.9,
                                            4, es, ew, dense=True, survivors=survivors)
        # the whole model at that shape (32 layers, random weights), a few decode steps: tokens/s
        # of the patched model replayed from one HIP graph against the model's own dense decode
        margs = argparse.Namespace(**vars(args))
        margs.steps, margs.warmup, margs.top_p, margs.model_mode, margs.no_dense = 8, 2, 0.9, "paged+graph", False
        m = bench_llama3_model(margs, dev, emit=False)
        extra["cfg5_model"] = {k: m[k] for k in ("config", "value", "unit", "ms_per_step", "steps",
                                                 "dense", "speedup_vs_dense",
                                                 "kept_tokens_per_head_mean", "twilight_layer_us",
                                                 "finite_logits", "group_select")}

    cpu = None
    if not args.no_cpu_baseline and not llama:
        cpu = cpu_baseline(N, H, args.budget, args.top_p, B, dev, survivors=survivors)

    line = {
        "metric": "\u00b5s/decode-layer at 32k ctx (select+prune+attn); GEMV & attn HBM GB/s vs peak",
        "value": round(wall_us, 2), "unit": "us", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall_us / 1e3, 5), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if llama else "f16",
        "data": "synthetic",
        "config": {"workload": (f"Select-then-Prune decode layer, "
                                f"{'Llama-3-8B shape: GQA 32/8' if llama else 'Longchat-7B shape: 32 MHA'}"
                                f" heads, B={B}, head_dim 128, {'bf16' if llama else 'fp16'} paged KV "
                                f"(page 16), context {N}, Quest budget {args.budget}, INT4 K estimate "
                                f"(group 32), top-p {args.top_p}"),
                   "batch": B, "context": N, "budget": args.budget, "top_p": args.top_p,
                   "layers_rotated": nl, "planted": _planted_name(survivors),
                   "survivors_mean": round(n_bar, 1), "survivors_median": float(counts.median()),
                   "survivors_max": n_max,
                   **({"group_select": True} if args.group_select else {})},
        "us_per_step_graph_replay": None if graph_us is None else round(graph_us, 2),
        "layer_bytes": layer_bytes,
        "layer_frac_of_hbm_peak": (round(layer_bytes / wall_us / 1e3 / HBM_PEAK_GBS, 4)
                                   if layer_bytes else None),
        "roofline": roofline, "kernels": kernels, "gemv_cfg2": gemv_cfg2, "cpu_baseline": cpu,
    }
    if dense:
        line["dense_decode_baseline"] = dense
    line.update(extra)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
