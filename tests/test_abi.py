"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the header
declares, and validates arguments on the host (no GPU is touched by any call here)."""
import ctypes
import os
import re

import pytest
import torch

from twilight_amd import _lib
import twilight_amd.kernel as K

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_are_exported(hip_lib):
    hdr = open(os.path.join(ROOT, "include", "twilight_hip.h")).read()
    declared = set(re.findall(r"\b(twl_[a-z0-9_]+)\s*\(", hdr))
    declared -= {"twl_top_p_"}  # a prefix used in a comment, not a symbol
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(hip_lib, name), name
    assert hip_lib.twl_abi_version() == int(re.search(r"#define TWL_ABI_VERSION (\d+)", hdr).group(1)) == _lib.ABI_VERSION


def test_header_compiles_as_c():
    import subprocess, tempfile
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include "twilight_hip.h"\nint main(void){return sizeof(twl_layer_args)>0?0:1;}\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                        "-c", src, "-o", os.path.join(d, "t.o")], check=True)


def test_layer_struct_matches_header(hip_lib):
    import subprocess, tempfile
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include <stdio.h>\n#include <stddef.h>\n#include "twilight_hip.h"\n'
                             'int main(void){printf("%zu %zu %zu %zu", sizeof(twl_layer_args),'
                             'offsetof(twl_layer_args, sm_scale), offsetof(twl_layer_args, scores),'
                             'offsetof(twl_layer_args, out));return 0;}\n')
        exe = os.path.join(d, "t")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), src, "-o", exe], check=True)
        sizes = [int(x) for x in subprocess.run([exe], capture_output=True, text=True).stdout.split()]
    A = _lib.LayerArgs
    assert sizes == [ctypes.sizeof(A), A.sm_scale.offset, A.scores.offset, A.out.offset]


def test_strerror(hip_lib):
    assert _lib.strerror(0) == "ok"
    for rc in range(-7, 0):
        assert _lib.strerror(rc) and "unknown" not in _lib.strerror(rc)
    assert "unknown" in _lib.strerror(-99)


def test_c_level_validation_without_gpu(hip_lib):
    L = hip_lib
    fake = 0x1000  # never dereferenced: validation fails first
    assert L.twl_top_p_f32(0, fake, 0, 0, 0, 0.9, 1, 8, 8, 0, 0, 0, 0) == -1          # probs NULL
    assert L.twl_top_p_f32(fake, 0, 0, 0, 0, 0.9, 1, 8, 8, 0, 0, 0, 0) == -1          # no output
    assert L.twl_top_p_f32(fake, 0, fake, 0, 0, 0.9, 1, 8, 8, 0, 0, 0, 0) == -1       # idx without count
    assert L.twl_top_p_f32(fake, fake, 0, 0, 0, 0.9, 1, 0, 8, 0, 0, 0, 0) == -2       # d == 0
    assert L.twl_top_p_f32(fake, fake, 0, 0, 0, 0.9, 1, 40000, 8, 0, 0, 0, 0) == -2   # d too large
    assert L.twl_top_p_f32(fake, fake, 0, 0, 0, float("nan"), 1, 8, 8, 0, 0, 0, 0) == -2   # p NaN
    assert L.twl_softmax_top_p_f32(fake, 8, 0, 1, 8, 0, 0.0, 1, 0, 0, fake, 8, fake, 0, 0, 0) == -2   # p out of (0,1]
    assert L.twl_softmax_top_p_f32(fake, 8, 0, 1, 8, 0, 1.5, 1, 0, 0, fake, 8, fake, 0, 0, 0) == -2
    assert L.twl_top_p_f32(fake, fake, 0, 0, 0, 0.9, 1, 8, 8, 7, 0, 0, 0) == -2       # bad high_mode
    assert L.twl_top_p_f32(fake, 0, fake, fake, 0, 0.9, 1, 8, 4, 0, 0, 0, 0) == -2    # idx_stride < d
    assert L.twl_top_p_f32(fake + 2, fake, 0, 0, 0, 0.9, 1, 8, 8, 0, 0, 0, 0) == -4   # misaligned
    assert L.twl_top_p_f16(fake, 2, fake, 0, 0, 0, 0.9, 1, 8, 8, 0, 0, 0, 0) == -3    # dtype
    assert L.twl_gemv_int4(fake, 0, 0, 16, 0, fake, 0, 0, 0, fake, fake, fake, 1, 1, 1, 1, 1.0, 0) == -1
    assert L.twl_gemv_int4(fake, 2, fake, 16, 0, fake, 0, 0, 0, fake, fake, fake, 1, 1, 1, 1, 1.0, 0) == -3
    assert L.twl_gemv_int4(fake, 0, fake, 16, 0, fake, 0, 0, 0, fake, fake, fake, 1, 3, 2, 1, 1.0, 0) == -2
    assert L.twl_gemv_int4(fake, 0, fake, 8, 0, fake, 0, 0, 0, fake, fake, fake, 1, 1, 1, 1, 1.0, 0) == -2
    assert L.twl_gemv_int4(fake + 4, 0, fake, 16, 0, fake, 0, 0, 0, fake, fake, fake, 1, 1, 1, 1, 1.0, 0) == -4
    ws = L.twl_sparse_attn_workspace_bytes(1, 8)
    assert ws == 256 + 130 * 4 and L.twl_sparse_attn_workspace_bytes(256, 8192) == 2048 + 256 * 64 * 520
    assert L.twl_sparse_attn(fake, fake, 0, fake, fake, 4096, 256, 128, 0, 8, fake, fake, fake,
                             1, 1, 1, 1.0, 0, fake, ws, 0) == -1
    assert L.twl_sparse_attn(fake, fake, 0, fake, fake, 4096, 256, 130, fake, 8, fake, fake, fake,
                             1, 1, 1, 1.0, 0, fake, ws, 0) == -4
    assert L.twl_sparse_attn(fake, fake, 0, fake, fake, 4096, 256, 128, fake, 0, fake, fake, fake,
                             1, 1, 1, 1.0, 0, fake, ws, 0) == -2
    assert L.twl_sparse_attn(fake, fake, 0, fake, fake, 4096, 256, 128, fake, 8, fake, fake, fake,
                             1, 1, 1, 1.0, 0, fake, ws - 1, 0) == -2      # workspace too small
    assert L.twl_sparse_attn(fake, fake, 0, fake, fake, 4096, 256, 128, fake, 8, fake, fake, fake,
                             1, 1, 1, 1.0, 0, 0, ws, 0) == -1             # workspace NULL
    # the entry without a workspace argument: same checks, and a size limit (24 MiB of partials)
    assert L.twl_sparse_attn_static(fake, fake, 0, fake, fake, 4096, 256, 128, 0, 8, fake, fake,
                                    fake, 1, 1, 1, 1.0, 0, 0) == -1
    assert L.twl_sparse_attn_static(fake, fake, 0, fake, fake, 4096, 256, 130, fake, 8, fake, fake,
                                    fake, 1, 1, 1, 1.0, 0, 0) == -4
    assert L.twl_sparse_attn_workspace_bytes(512, 8192) <= _lib.STATIC_SCRATCH_BYTES
    assert L.twl_sparse_attn_static(fake, fake, 0, fake, fake, 4096, 256, 128, fake, 8192, fake,
                                    fake, fake, 128, 32, 32, 1.0, 0, 0) == -7   # 4096 rows: too big
    # the group GEMV: a page list is required, 2 / 4 / 8 q heads per kv head
    gg = lambda **kw: L.twl_gemv_int4_group(
        fake, 0, fake, kw.get("os", 64), 0, fake, kw.get("sel", fake), 0, 4, fake, fake, fake, 1,
        kw.get("hq", 4), kw.get("hkv", 1), 4, 1.0, 0)
    assert gg(sel=0) == -1 and gg(hq=3) == -2 and gg(hq=4, hkv=4) == -2 and gg(os=63) == -2
    # attention on given weights: weights and workspace required, V strides and sizes as above
    wat = lambda **kw: L.twl_sparse_attn_weighted(
        kw.get("out", fake), 0, fake, 4096, 256, kw.get("hs", 128), fake, kw.get("stride", 8), fake,
        kw.get("w", fake), fake, fake, 1, 1, 1, 0, kw.get("ws", fake), kw.get("wsb", ws), 0)
    assert wat(w=0) == -1 and wat(ws=0) == -1 and wat(out=0) == -1
    assert wat(hs=130) == -4 and wat(w=fake + 2) == -4
    assert wat(stride=0) == -2 and wat(wsb=ws - 1) == -2
    assert L.twl_quest_select(fake, 0, fake, fake, fake, 1, 1, 1, 0, 4, fake, 4, fake, fake, 4, 0) == -2
    assert L.twl_quest_select(fake, 0, fake, fake, fake, 1, 1, 1, 64, 4, fake, 2, fake, fake, 4, 0) == -2
    assert L.twl_quest_select(fake, 0, fake, fake, fake, 1, 1, 1, 64, 4, 0, 4, fake, fake, 4, 0) == -1
    assert L.twl_quest_topk_pages(fake, 4, fake, 1, 1, 64, 4, fake, 2, fake, 0) == -2
    assert L.twl_quest_page_scores(fake, 0, fake, fake, fake, 1, 1, 1, 4, 0, 4, 0) == -1
    assert L.twl_kv_shadow_build(fake, 0, 4096, 256, 128, 0, 0, 1, 1, 0, 0, 0) == -1
    assert L.twl_dequant_int4(fake, 0, fake, 0) == -2
    assert L.twl_decode_layer(None, 0) == -1
    # entry points added after the first ABI version
    f = fake
    gtp = lambda **kw: L.twl_gemv_top_p(
        kw.get("q", f), kw.get("dt", 0), f, kw.get("sel", f), f, kw.get("sel_stride", 4), f, f, f,
        1, kw.get("hq", 1), kw.get("hkv", 1), kw.get("k", 4), 1.0, 0, kw.get("p", 0.9),
        kw.get("high", 1), kw.get("idx", f), kw.get("idx_stride", 64), f, 0, 64, 0, 0, 0)
    assert gtp(sel=0) == -1 and gtp(idx=0) == -1
    assert gtp(dt=2) == -3
    assert gtp(hq=3, hkv=2) == -2 and gtp(k=0) == -2 and gtp(k=4096) == -2
    assert gtp(sel_stride=2) == -2 and gtp(idx_stride=32) == -2
    assert gtp(p=0.0) == -2 and gtp(high=5) == -2
    assert gtp(q=f + 8) == -4
    sep = lambda **kw: L.twl_select_estimate_prune(
        kw.get("q", f), kw.get("dt", 0), kw.get("meta", f), f, f, f, f, 1, kw.get("hq", 1),
        kw.get("hkv", 1), kw.get("budget", 64), kw.get("npg", 16), 1.0, 0, kw.get("p", 0.9), 1,
        kw.get("sel", f), kw.get("sel_stride", 4), f, f, kw.get("idx_stride", 64), f, 0, 0, 0, 64,
        0, kw.get("planes", 0), kw.get("cap", 0), kw.get("slots", 0), kw.get("nslots", 0), 0)
    assert sep(meta=0) == -1 and sep(sel=0) == -1
    assert sep(dt=5) == -3
    assert sep(budget=0) == -2 and sep(npg=0) == -2 and sep(npg=9000) == -2
    assert sep(sel_stride=3) == -2 and sep(idx_stride=63) == -2 and sep(p=2.0) == -2
    assert sep(hq=4, hkv=3) == -2
    assert sep(q=f + 4) == -4
    assert sep(meta=0, planes=f, cap=16) == -1            # the records are needed with planes too
    assert sep(planes=f, cap=8) == -2 and sep(planes=f, cap=20) == -2   # cap < pages, cap % 8
    assert sep(planes=f, cap=16, slots=f, nslots=0) == -2               # slot table, no slots
    app = lambda **kw: L.twl_kv_append(
        kw.get("k", f), f, kw.get("dt", 0), 256, 128, f, f, 4096, kw.get("ts", 256), 128, f, f,
        kw.get("last", f), kw.get("b", 1), 1, 0, 0, kw.get("planes", 0), kw.get("cap", 0),
        kw.get("slots", 0), kw.get("nslots", 0), 0)
    assert app(k=0) == -1 and app(last=0) == -1
    assert app(dt=2) == -3 and app(b=0) == -2 and app(ts=250) == -4 and app(k=f + 2) == -4
    assert app(planes=f, cap=12) == -2 and app(planes=f, cap=16, slots=f, nslots=0) == -2
    assert app(planes=f, cap=16) == -1                    # planes are written from the record
    pb = lambda **kw: L.twl_meta_planes_build(kw.get("meta", f), f, f, 1, 1, kw.get("npg", 8),
                                              kw.get("planes", f), kw.get("cap", 8),
                                              kw.get("slots", 0), kw.get("nslots", 0), 0)
    assert pb(meta=0) == -1 and pb(planes=0) == -1 and pb(slots=f, nslots=0) == -2
    assert pb(cap=12) == -2 and pb(npg=16) == -2 and pb(npg=0) == -2 and pb(planes=f + 8) == -4
    qk = lambda **kw: L.twl_qk_int8_lse(
        kw.get("q", f), f, f, f, kw.get("lse", f), 1, kw.get("hq", 1), kw.get("hkv", 1),
        kw.get("qo", 8), kw.get("kv", 8), kw.get("d", 128), 1024, 1024, kw.get("sqn", 128),
        1024, 1024, 128, 0)
    assert qk(q=0) == -1 and qk(lse=0) == -1
    assert qk(d=96) == -2 and qk(qo=0) == -2 and qk(kv=0) == -2 and qk(hq=3, hkv=2) == -2
    assert qk(sqn=100) == -4 and qk(q=f + 1) == -4


def test_python_ops_reject_cpu_and_malformed_tensors(hip_lib):
    # same conditions as CHECK_INPUT / CHECK_DIM (csrc/src/sampling.cu:25-27): RuntimeError
    p = torch.rand(2, 3, 1, 64)
    with pytest.raises(RuntimeError, match="CUDA"):
        K.top_p_fp32_return_mask(p, 0.9)
    with pytest.raises(RuntimeError, match="CUDA"):
        K.top_p_fp16_return_mask(p.half(), 0.9)
    with pytest.raises(RuntimeError):
        K.top_p_fp32_return_mask("nope", 0.9)
    with pytest.raises(RuntimeError, match="CUDA"):
        K.sparse_gemv_int4(torch.zeros(1, 1, 128).half(), torch.zeros(1, 1, 1280, dtype=torch.uint8),
                           torch.zeros(1, dtype=torch.int32), torch.zeros(2, dtype=torch.int32),
                           torch.ones(1, dtype=torch.int32), max_pages=1)
    with pytest.raises(RuntimeError, match="CUDA"):
        K.softmax_top_p(torch.zeros(1, 1, 16), 0.9)
    with pytest.raises(RuntimeError, match="CUDA"):
        K.quest_select(torch.zeros(1, 1, 128).half(), torch.zeros(1, 1, 512, dtype=torch.uint8),
                       torch.zeros(1, dtype=torch.int32), torch.zeros(2, dtype=torch.int32), 16, 1)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()


def test_sparse_config_parsing():
    from twilight_amd.layer import parse_sparse_config
    cfg = {"compressor": {"type": "none"},
           "selector": {"type": "quest", "token_budget": 8192, "chunk_size": 16},
           "weight_estimator": {"type": "min_max_quant", "quant_bit": 4},
           "weight_pruner": {"type": "top_p", "threshold": 0.85},
           "skip_first_two_layers": True, "use_estimated_weights_in_attn": False}
    assert parse_sparse_config(cfg) == {"token_budget": 8192, "top_p": 0.85, "sparsity_rate": -1,
                                        "use_estimated_weights": False}
    knobs = dict(cfg, use_estimated_weights_in_attn=True,
                 selector={"type": "quest", "sparsity_rate": 0.25, "chunk_size": 16})
    assert parse_sparse_config(knobs)["sparsity_rate"] == 0.25
    assert parse_sparse_config(knobs)["use_estimated_weights"] is True
    with pytest.raises(RuntimeError, match="sparsity_rate"):
        parse_sparse_config(dict(cfg, selector={"type": "quest", "sparsity_rate": 1.5}))
    bad = dict(cfg, selector={"type": "ds"})
    with pytest.raises(RuntimeError):
        parse_sparse_config(bad)
    with pytest.raises(RuntimeError):
        parse_sparse_config(dict(cfg, weight_estimator={"type": "min_max_quant", "quant_bit": 2}))
