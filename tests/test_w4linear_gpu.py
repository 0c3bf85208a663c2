"""W4A16Linear: the quantiser on the CPU (round trip, exact zero points), the module's forward on the GPU."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from tilelang_amd import w4linear
from oracle import dq_oracle as orc


def _oracle_tile(packed, s, z):
    if z is None:
        return orc.dequant_u4_scale(packed, s.numpy(), 128)
    return orc.dequant_u4_scale_zeros(packed, s.numpy(), z.numpy(), 128, "original")


@pytest.mark.parametrize("with_zeros", [False, True])
def test_quantize_w4_round_trip(with_zeros):
    """Codes stay in a nibble, zero points are integers, and the dequantised weight is within half a step."""
    g = torch.Generator().manual_seed(3)
    W = torch.randn((48, 512), generator=g) * 0.05
    if with_zeros:
        W += 0.03  # off-centre groups are what zero points are for
    q, s, z = w4linear.quantize_w4(W, 128, with_zeros)
    assert q.dtype == torch.uint8 and int(q.max()) <= 15
    assert s.shape == (48, 4) and s.dtype == torch.float16
    if with_zeros:
        assert torch.equal(z, z.round()) and float(z.min()) >= 0 and float(z.max()) <= 15
    else:
        assert z is None and int(q.min()) >= 1
    Wd = w4linear.dequantize_w4_reference(q, s, z, 128).float()
    step = s.float().repeat_interleave(128, dim=1)
    assert torch.all((Wd - W).abs() <= 0.51 * step + 1e-3 * W.abs())
    # the same tile through the numpy oracle (quantization.py:298-307, 321-330)
    packed = tl.quantize.general_compress(q.to(torch.int8), 4).numpy()
    ref = _oracle_tile(packed, s, z)
    np.testing.assert_array_equal(Wd.half().numpy().view(np.uint16), ref.view(np.uint16))


def test_w4linear_rejects_bad_shapes():
    with pytest.raises(ValueError):
        tl.W4A16Linear(100, 64)
    with pytest.raises(ValueError):
        tl.W4A16Linear(256, 64, group_size=96)
    with pytest.raises(ValueError):
        w4linear.quantize_w4(torch.zeros(4, 100), 64)


@pytest.mark.gpu
@pytest.mark.parametrize("with_zeros", [False, True])
@pytest.mark.parametrize("batch", [(1,), (5,), (3, 20), (300,)])
def test_w4linear_forward(cuda, with_zeros, batch):
    """One launch whatever the batch (GEMV, small-batch and MFMA GEMM routes) against dequant + fp32 matmul."""
    in_f, out_f = 1024, 768
    rng = np.random.default_rng(len(batch) * 29 + int(with_zeros) + batch[0])
    W = (rng.standard_normal((out_f, in_f), dtype=np.float32) * 0.03 + (0.02 if with_zeros else 0.0)).astype(np.float32)
    bias = rng.standard_normal(out_f).astype(np.float16)
    x = rng.standard_normal(batch + (in_f,), dtype=np.float32).astype(np.float16)

    lin = torch.nn.Linear(in_f, out_f)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(W))
        lin.bias.copy_(torch.from_numpy(bias).float())
    layer = tl.W4A16Linear.from_linear(lin, group_size=128, with_zeros=with_zeros).to(cuda)
    out = layer(torch.from_numpy(x).to(cuda))
    torch.cuda.synchronize()
    assert out.shape == batch + (out_f,) and out.dtype == torch.float16

    q, s, z = w4linear.quantize_w4(torch.from_numpy(W), 128, with_zeros)
    packed = tl.quantize.general_compress(q.to(torch.int8), 4).numpy()
    assert np.array_equal(layer.qweight.cpu().numpy(), packed)
    Wd = _oracle_tile(packed, s, z).astype(np.float32)
    ref = x.reshape(-1, in_f).astype(np.float32) @ Wd.T + bias.astype(np.float32)[None, :]
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(-1, out_f), ref, rtol=1e-2, atol=1e-2)
    # a state_dict round trip keeps the packed weights
    clone = tl.W4A16Linear(in_f, out_f, group_size=128, with_zeros=with_zeros, bias=True).to(cuda)
    clone.load_state_dict(layer.state_dict())
    assert torch.equal(clone(torch.from_numpy(x).to(cuda)), out)
