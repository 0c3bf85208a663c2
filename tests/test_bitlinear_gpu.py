"""GPU parity of the BitLinear caller path: activation quantiser (bit-exact) and the module's forward."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from tilelang_amd import bitlinear
from oracle import dq_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,K", [(1, 128), (3, 8192), (64, 1024), (257, 4096), (5, 8 * 37), (2, 16384), (2, 16384 + 2048), (1500, 512)])
def test_activation_quant_bit_exact(cuda, M, K):
    """examples/bitnet-1.58b/utils_quant.py:156-163: int8 codes and fp32 scales identical to the restatement."""
    rng = np.random.default_rng(M * 131 + K)
    x = (rng.standard_normal((M, K), dtype=np.float32) * rng.uniform(0.01, 30.0, size=(M, 1)).astype(np.float32)).astype(np.float16)
    x[0, : min(K, 16)] = np.array([0.5, -0.5, 1.5, 2.5, -2.5, 0.0, 1e-4, -1e-4] * 2, dtype=np.float16)[: min(K, 16)]  # ties
    if M > 2:
        x[2, :] = 0  # all-zero row: the 1e-5 clamp decides the scale
    xq, s = tl.bitnet_activation_quant(M, K)(torch.from_numpy(x).to(cuda))
    torch.cuda.synchronize()
    ref_q, ref_s = orc.activation_quant(x)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), ref_s.reshape(-1).view(np.uint32))
    np.testing.assert_array_equal(xq.cpu().numpy(), ref_q)
    # and against torch's own ops, the way the reference computes it
    tq, ts = bitlinear.activation_quant_reference(torch.from_numpy(x))
    assert torch.equal(xq.cpu(), tq) and torch.equal(s.cpu(), ts.reshape(-1))


@pytest.mark.parametrize("interleave", [True, False])
@pytest.mark.parametrize("batch", [(1,), (7,), (2, 130)])
def test_bitlinear_forward(cuda, interleave, batch):
    """Module forward against forward_fp32_simulated of utils_quant.py:189-205 restated with the oracle."""
    in_f, out_f = 1024, 768
    rng = np.random.default_rng(len(batch) * 17 + int(interleave))
    W = (rng.standard_normal((out_f, in_f), dtype=np.float32) * 0.02).astype(np.float32)
    bias = rng.standard_normal(out_f).astype(np.float16)
    x = rng.standard_normal(batch + (in_f,), dtype=np.float32).astype(np.float16)

    layer = tl.BitLinear(in_f, out_f, interleave=interleave).to(cuda)
    layer.load_float_weight(torch.from_numpy(W), torch.from_numpy(bias))
    out = layer(torch.from_numpy(x).to(cuda))
    torch.cuda.synchronize()
    assert out.shape == batch + (out_f,) and out.dtype == torch.float16

    wq, sw = orc.weight_quant(W)
    xq, sa = orc.activation_quant(x.reshape(-1, in_f))
    acc = xq.astype(np.int64) @ wq.astype(np.int64).T
    ref = orc.post_quant_process(acc, sa, sw).astype(np.float32) + bias.astype(np.float32)[None, :]
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(-1, out_f), ref, rtol=1e-2, atol=1e-2)


def test_bitlinear_layer_on_fragment_ordered_weights(cuda):
    """``prefill_fragments=True``: the layer holds its weights in the matrix instruction's operand order ONLY (one
    packed copy) and every batch size reads it: the decode kernel (1 and 4 rows), the K-sliced kernel (8 and 256 rows),
    the tiled kernel (1300 rows); each must give the bits of the row-major layer."""
    in_f, out_f = 4096, 4096
    rng = np.random.default_rng(11)
    W = (rng.standard_normal((out_f, in_f), dtype=np.float32) * 0.02).astype(np.float32)
    plain = tl.BitLinear(in_f, out_f)
    frag = tl.BitLinear(in_f, out_f, prefill_fragments=True)
    for layer in (plain, frag):
        layer.load_float_weight(torch.from_numpy(W))
        layer.to(cuda)
    assert frag.prefill_fragments and frag.qweight.shape == (out_f // 32, in_f // 128, 64, 16) and frag.qweight.is_cuda
    assert plain.qweight.shape == (out_f, in_f // 4)
    assert sum(b.numel() for b in frag.buffers()) == sum(b.numel() for b in plain.buffers())  # one copy, same bytes
    assert torch.equal(frag.rowmajor_weight(), plain.qweight)
    for M in (1, 4, 8, 256, 1300):
        print(f"BitLinear on fragments: M={M}", flush=True)
        x = torch.from_numpy(rng.standard_normal((M, in_f), dtype=np.float32).astype(np.float16)).to(cuda)
        a, b = plain(x), frag(x)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # weights replaced through the state dict of another fragment-ordered layer
    W2 = (rng.standard_normal((out_f, in_f), dtype=np.float32) * 0.02).astype(np.float32)
    other = tl.BitLinear(in_f, out_f, prefill_fragments=True)
    other.load_float_weight(torch.from_numpy(W2))
    other.to(cuda)
    frag.load_state_dict(other.state_dict())
    plain.load_packed_weight(other.rowmajor_weight(), other.sw)
    assert frag._sw_value == plain._sw_value == other._sw_value
    x = torch.from_numpy(rng.standard_normal((256, in_f), dtype=np.float32).astype(np.float16)).to(cuda)
    a, b = plain(x), frag(x)
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert not tl.BitLinear(1024, 768, prefill_fragments=True).prefill_fragments  # in_features the kernels cannot slice


def test_bitlinear_decode_batches_on_a_large_layer(cuda):
    """An 8192 x 8192 layer on fragment-ordered weights at decode batches: the decode kernel reads the fragment order
    (M * K <= 32768: one to four rows at K = 8192) and gives the plain layer's bits."""
    in_f = out_f = 8192
    rng = np.random.default_rng(13)
    W = (rng.standard_normal((out_f, in_f), dtype=np.float32) * 0.02).astype(np.float32)
    plain = tl.BitLinear(in_f, out_f)
    frag = tl.BitLinear(in_f, out_f, prefill_fragments=True)
    for layer in (plain, frag):
        layer.load_float_weight(torch.from_numpy(W))
        layer.to(cuda)
    for M in (1, 2, 4):
        x = torch.from_numpy(rng.standard_normal((M, in_f), dtype=np.float32).astype(np.float16)).to(cuda)
        a, b = plain(x), frag(x)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
