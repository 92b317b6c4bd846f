"""GPU parity of the Double-Sparse label ops against the reference's own torch checks
(twilight/kernel/triton/channel.py:82-106, twilight/kernel/triton/bgemv_int8.py:78-134)."""
import pytest
import torch

from oracle import pyimpl_port as P
import twilight_amd.kernel as K

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16])
def test_get_label_tensor(dev, dt):
    # shapes of the reference's self-test (channel.py:84-93) and a larger strided case
    g = torch.Generator().manual_seed(0)
    for (L, H, D, r) in ((10, 3, 8, 4), (257, 32, 128, 16)):
        x = torch.randn((L, H, D), generator=g).to(dt)
        channel = torch.stack([torch.randperm(D, generator=g)[:r] for _ in range(H)]).to(torch.int64)
        out = torch.empty((L, H, r), dtype=dt, device=dev)
        K.get_label_tensor(x.to(dev), channel.to(dev), out, r)
        assert torch.equal(out.cpu(), P.get_label_tensor_ref(x, channel, r))     # a gather: exact
    # non-contiguous input view, as double_sparse.py:72-77 produces before .contiguous()
    xs = torch.randn((4, 50, 6, 128), generator=g).to(dt)                        # [B,N,H,D]
    xv = xs.to(dev).transpose(1, 2)[1].transpose(0, 1)                           # [N,H,D] strided
    out = torch.empty((50, 6, 8), dtype=dt, device=dev)
    ch = torch.stack([torch.randperm(128, generator=g)[:8] for _ in range(6)]).to(torch.int64)
    K.get_label_tensor(xv, ch.to(dev), out, 8)
    assert torch.equal(out.cpu(), P.get_label_tensor_ref(xs[1], ch, 8))


def test_bgemv_int8_reference_selftest_shape(dev):
    # the reference's own check: B = H = 32, N_CTX = 2048, r = 8, normal(0.1, 0.2), atol 1e-3 rtol 0
    # (bgemv_int8.py:98-134)
    B, H, N, r = 32, 32, 2048, 8
    g = torch.Generator().manual_seed(0)
    q = (torch.randn((B, H, r), generator=g) * 0.2 + 0.1).half()
    kf = (torch.randn((B * N, H, r), generator=g) * 0.2 + 0.1).half()
    scales = (kf.float().abs().max(-1)[0] / 127.0).half()                       # :107
    k8 = (kf.float() / scales.float()[:, :, None]).to(torch.int8)               # :108
    out = torch.empty((B, H, N), dtype=torch.float16, device=dev)
    ret = K.bgemv_int8(q.to(dev), k8.to(dev), scales.to(dev), out)
    assert ret is out
    ref = P.bgemv_int8_ref(q, k8, scales)
    assert torch.allclose(out.cpu().float(), ref, atol=1e-3, rtol=0)


@pytest.mark.parametrize("B,H,N,r", [
    (2, 32, 1000, 16),     # the Double-Sparse shape: 32 heads, 16 heavy channels; partial last tile
    (3, 8, 517, 32),       # two 16-byte pieces per head
    (1, 16, 2051, 64),     # four pieces per head
    (2, 64, 300, 8),       # 8-byte pieces, more pieces per token than threads
    (1, 4, 77, 16),        # fewer pieces per token than a wavefront
])
def test_bgemv_int8_dense_layout(dev, B, H, N, r):
    # dense operands take the streaming kernel (strided ones the general one): same numbers
    g = torch.Generator().manual_seed(B * N + r)
    q = torch.randn((B, H, r), generator=g).half()
    k8 = torch.randint(-128, 128, (B * N, H, r), generator=g, dtype=torch.int16).to(torch.int8)
    scales = (torch.rand((B * N, H), generator=g) * 0.01).half()
    out = torch.full((B, H, N), 5.0, dtype=torch.float16, device=dev)
    K.bgemv_int8(q.to(dev), k8.to(dev), scales.to(dev), out)
    ref = P.bgemv_int8_ref(q, k8, scales)
    assert torch.allclose(out.cpu().float(), ref, atol=2e-3, rtol=2e-3)
    # the same through strided views (general kernel)
    kpad = torch.zeros((B * N, H, r + 3), dtype=torch.int8)
    kpad[..., :r] = k8
    out2 = torch.empty((B, H, N), dtype=torch.float16, device=dev)
    K.bgemv_int8(q.to(dev), kpad.to(dev)[..., :r], scales.to(dev), out2)
    assert torch.allclose(out2.cpu().float(), out.cpu().float(), atol=1e-3, rtol=1e-3)


def test_bgemv_int8_ragged(dev):
    B, H, N, r = 3, 5, 131, 16
    g = torch.Generator().manual_seed(1)
    q = torch.randn((B, H, r), generator=g).half()
    k8 = torch.randint(-128, 128, (B * N, H, r), generator=g, dtype=torch.int16).to(torch.int8)
    scales = (torch.rand((B * N, H), generator=g) * 0.01).half()
    out = torch.empty((B, H, N), dtype=torch.float16, device=dev)
    K.bgemv_int8(q.to(dev), k8.to(dev), scales.to(dev), out)
    ref = P.bgemv_int8_ref(q, k8, scales)
    assert torch.allclose(out.cpu().float(), ref, atol=2e-3, rtol=2e-3)
    with pytest.raises(RuntimeError):
        K.bgemv_int8(q.to(dev), k8.to(dev), scales.to(dev), out[:, :, :-1])


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("b,h_qo,h_kv,qo_len,kv_len,d", [
    (2, 4, 2, 150, 100, 128),     # partial query block, partial key block (zero-padded tail), GQA
    (1, 2, 2, 1, 1000, 128),      # decode: one query row
    (1, 8, 1, 300, 257, 64),      # head_dim 64, MQA
    (1, 1, 1, 128, 64, 128),      # exactly one block each way
])
def test_qk_int8_per_block_lse(dev, layout, b, h_qo, h_kv, qo_len, kv_len, d):
    # twilight/kernel/triton/qk_int8_per_block.py:111-143: lse in base 2, first output all zeros
    g = torch.Generator().manual_seed(qo_len + kv_len)
    q = torch.randint(-127, 128, (b, h_qo, qo_len, d), generator=g, dtype=torch.int8)
    k = torch.randint(-127, 128, (b, h_kv, kv_len, d), generator=g, dtype=torch.int8)
    qs = torch.rand((b, h_qo, (qo_len + 127) // 128), generator=g) * 2e-3 + 5e-4
    ks = torch.rand((b, h_kv, (kv_len + 63) // 64), generator=g) * 2e-3 + 5e-4
    want = P.qk_int8_lse_ref(q, k, qs, ks)
    qd, kd = q.to(dev), k.to(dev)
    if layout == "NHD":
        qd, kd = qd.transpose(1, 2).contiguous(), kd.transpose(1, 2).contiguous()
    o, lse = K.qk_int8_per_block(qd, kd, qs.to(dev), ks.to(dev), tensor_layout=layout,
                                 output_dtype=torch.float16, return_lse=True)
    assert o.shape == qd.shape and o.dtype == torch.float16 and not o.any()
    # integer products are exact; exp2 / log2 and the summation order differ by a few ulps
    assert torch.allclose(lse.cpu(), want, rtol=1e-5, atol=2e-5), (lse.cpu() - want).abs().max()
    o2, lse2 = K.qk_int8_per_block(qd, kd, qs.to(dev), ks.to(dev), tensor_layout=layout)
    assert lse2.numel() == 0 and lse2.device.type == "cpu"


def test_qk_int8_per_block_errors(dev):
    q = torch.zeros((1, 2, 8, 128), dtype=torch.int8, device=dev)
    s = torch.ones((1, 2, 1), device=dev)
    with pytest.raises(ValueError):
        K.qk_int8_per_block(q, q, s, s, tensor_layout="XYZ")
    with pytest.raises(RuntimeError):
        K.qk_int8_per_block(q.float(), q, s, s, return_lse=True)
    with pytest.raises(RuntimeError):
        K.qk_int8_per_block(q[..., :96], q[..., :96], s, s, return_lse=True)   # head_dim 96
    with pytest.raises(RuntimeError):
        K.qk_int8_per_block(q, q, s[:, :1], s, return_lse=True)               # q_scale too short
