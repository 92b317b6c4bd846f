"""The entry point that allocates nothing, ``twl_sparse_attn_static``, against ``twl_sparse_attn``
(which takes a caller's workspace): same kernels, so the outputs must be identical bit for bit.
Two calls in a row share the library's scratch array, the second on a smaller input. Runs through
the C ABI (ctypes), after every other GPU test and also alone in a fresh process."""
import math

import numpy as np
import pytest
import torch

from twilight_amd import _lib
from twilight_amd.cache import PagedKVCache
from twilight_amd.kernel._check import ptr, stream_of

pytestmark = pytest.mark.gpu


def _case(dev, B, H, N, lens, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, 128), generator=g).to(dtype)
    k = torch.randn((B, H, N, 128), generator=g).to(dtype)
    v = torch.randn((B, H, N, 128), generator=g).to(dtype)
    n_pages = B * ((N + 15) // 16)
    cache = PagedKVCache.from_dense(k, v, dev, page_perm=torch.randperm(n_pages, generator=g))
    idx = torch.zeros((B, H, N), dtype=torch.int32)
    cnt = torch.zeros((B, H), dtype=torch.int32)
    for r, n in enumerate(lens):
        b, h = divmod(r, H)
        idx[b, h, :n] = torch.sort(torch.randperm(N, generator=g)[:n]).values.int()
        cnt[b, h] = n
    return q.to(dev), cache, idx.to(dev), cnt.to(dev)


def _run(L, static, q, cache, idx, cnt, ws=None, out=None, lse=None):
    B, H, _ = q.shape
    if out is None:
        out = torch.full_like(q, float("nan"))
        lse = torch.full((B, H), float("nan"), dtype=torch.float32, device=q.device)
    ks = cache.k_cache.stride()
    code = _lib.TWL_F16 if q.dtype == torch.float16 else _lib.TWL_BF16
    head = (ptr(q), ptr(out), code, ptr(cache.k_cache), ptr(cache.v_cache), ks[0], ks[1], ks[2],
            ptr(idx), idx.size(2), ptr(cnt), ptr(cache.kv_page_indices), ptr(cache.kv_page_indptr),
            B, H, cache.k_cache.size(2), 1.0 / math.sqrt(128), ptr(lse))
    if static:
        rc = L.twl_sparse_attn_static(*head, stream_of(q))
    else:
        rc = L.twl_sparse_attn(*head, ptr(ws), ws.numel(), stream_of(q))
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    return out, lse


def test_static_scratch_entry_equals_workspace_entry(dev):
    L = _lib.lib()
    # first call: 16 rows, up to 3000 survivors (24 chunks); second: fewer, shorter rows whose
    # chunks land on partial-result slots and tickets that the first call used
    cases = [
        (2, 8, 3000, [1, 127, 128, 129, 256, 257, 1000, 3000, 0, 3000, 5, 640, 2, 1999, 384, 130],
         31, torch.float16),
        (1, 4, 700, [700, 129, 0, 300], 32, torch.bfloat16),
    ]
    for B, H, N, lens, seed, dtype in cases:
        q, cache, idx, cnt = _case(dev, B, H, N, lens, seed, dtype)
        ws = torch.zeros(int(L.twl_sparse_attn_workspace_bytes(B * H, N)), dtype=torch.uint8,
                         device=dev)
        ref_out, ref_lse = _run(L, False, q, cache, idx, cnt, ws)
        # one untimed call first: the address lookup of the first call on a device is set-up
        _run(L, True, q, cache, idx, cnt)
        out = torch.full_like(q, float("nan"))
        lse = torch.full((B, H), float("nan"), dtype=torch.float32, device=dev)
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        reserved0 = torch.cuda.memory_reserved()
        out, lse = _run(L, True, q, cache, idx, cnt, out=out, lse=lse)
        # neither torch's allocator nor the device lost memory to the call
        assert torch.cuda.memory_reserved() == reserved0
        assert torch.cuda.mem_get_info()[0] >= free0
        assert torch.equal(out.view(torch.int16), ref_out.view(torch.int16)), (B, H, N)
        assert torch.equal(lse.view(torch.int32), ref_lse.view(torch.int32)), (B, H, N)
        assert torch.isfinite(out.float()).all()
        # and once more on the same input: the array holds this call's own leftovers now
        out2, _ = _run(L, True, q, cache, idx, cnt)
        assert torch.equal(out2.view(torch.int16), ref_out.view(torch.int16))


def test_static_scratch_entry_rejects_what_does_not_fit(dev):
    L = _lib.lib()
    q, cache, idx, cnt = _case(dev, 1, 2, 64, [3, 4], 33, torch.float16)
    ks = cache.k_cache.stride()
    # 4096 rows x 8192 survivors would need 136 MB of partial results
    rc = L.twl_sparse_attn_static(ptr(q), ptr(q), 0, ptr(cache.k_cache), ptr(cache.v_cache), ks[0],
                                  ks[1], ks[2], ptr(idx), 8192, ptr(cnt),
                                  ptr(cache.kv_page_indices), ptr(cache.kv_page_indptr), 128, 32,
                                  32, 0.1, 0, 0)
    assert rc == -7 and "fit" in _lib.strerror(rc)
