"""GPU parity of the weight quantisers that produce the packed operands: MXFP4 (bit-exact codes and scale
bytes against the CPU oracle, and through the MXFP4 GEMM) and gen_quant4's layout through the W4A16 kernels."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from oracle import dq_oracle as orc

pytestmark = pytest.mark.gpu


def _bf16_tensor(x_f32: np.ndarray, cuda) -> torch.Tensor:
    """float32 values that are exactly representable in bf16 -> bf16 device tensor."""
    return torch.from_numpy(x_f32).to(cuda).to(torch.bfloat16)


@pytest.mark.parametrize("N,K", [(1, 32), (3, 64), (8, 8192), (257, 96), (64, 4096 + 32), (1000, 1024)])
@pytest.mark.parametrize("scale_bias", [127, 0])
def test_mxfp4_quantiser_bit_exact(cuda, N, K, scale_bias):
    rng = np.random.default_rng(N * 7 + K + scale_bias)
    x = rng.standard_normal((N, K), dtype=np.float32) * np.exp2(rng.integers(-10, 10, size=(N, 1))).astype(np.float32)
    x = orc.round_to_bf16(x)
    # special values: thresholds and their predecessors next to a 6 that pins the exponent, zeros, an all-zero
    # block, subnormals, the largest finite bf16
    row = x[0]
    row[:8] = [6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    if K >= 64:
        row[32:64] = 0.0
    if N > 1:
        x[1, :4] = [3.3895314e38, -1e-40, 9.18e-41, 0.0]
    if N > 2:
        x[2, :] = 0.0
        x[2, -1] = -2.0**-120
    x = orc.round_to_bf16(x)
    B, S = tl.quantize_bf16_mxfp4(N, K, scale_bias=scale_bias)(_bf16_tensor(x, cuda))
    torch.cuda.synchronize()
    assert B.shape == (N, K // 2) and B.dtype == torch.uint8 and S.shape == (N, K // 32) and S.dtype == torch.uint8
    ref_B, ref_S = orc.quantize_mxfp4(x, scale_bias=scale_bias)
    np.testing.assert_array_equal(S.cpu().numpy(), ref_S)
    np.testing.assert_array_equal(B.cpu().numpy(), ref_B)


@pytest.mark.parametrize("e", [0, -3, 5])
def test_mxfp4_quantiser_every_bf16_value_under_a_pinned_exponent(cuda, e):
    """Every bf16 bit pattern (both signs, subnormals included) whose magnitude does not exceed 6 * 2^e, 31 per block
    next to a 6 * 2^e that pins the block exponent: the element rule over its whole domain."""
    top = np.float32(6.0 * 2.0**e)
    top_bits = int(orc.f32_to_bf16_bits(np.array([top]))[0])
    mags = np.arange(0, top_bits + 1, dtype=np.uint16)
    vals = np.concatenate([orc.bf16_bits_to_f32(mags), orc.bf16_bits_to_f32(mags | 0x8000)])
    pad = (-len(vals)) % 31
    vals = np.concatenate([vals, np.zeros(pad, dtype=np.float32)]).reshape(-1, 31)
    blocks = np.concatenate([np.full((vals.shape[0], 1), top, dtype=np.float32), vals], axis=1)
    x = blocks.reshape(1, -1)
    B, S = tl.quantize_bf16_mxfp4(1, x.shape[1])(_bf16_tensor(x, cuda))
    torch.cuda.synchronize()
    ref_B, ref_S = orc.quantize_mxfp4(x)
    assert (ref_S == 127 + e).all()
    np.testing.assert_array_equal(S.cpu().numpy(), ref_S)
    np.testing.assert_array_equal(B.cpu().numpy(), ref_B)


def test_mxfp4_quantiser_full_size_properties(cuda):
    """At the benchmark's weight size (8192 x 8192): every block's maximum lands in e2m1's top binade, the
    quantiser is idempotent (quantise o dequantise o quantise = quantise) and the first rows match the oracle."""
    N = K = 8192
    g = torch.Generator(device=cuda).manual_seed(3)
    w = (torch.randn((N, K), generator=g, device=cuda, dtype=torch.float32) * 0.05).to(torch.bfloat16)
    quant = tl.quantize_bf16_mxfp4(N, K)
    B, S = quant(w)
    codes = torch.stack((B & 0xF, B >> 4), dim=-1).reshape(N, K)
    assert bool(((codes & 7).reshape(N, K // 32, 32).amax(dim=-1) >= 6).all())
    lut = torch.tensor(orc.E2M1_VALUES, device=cuda)
    deq = lut[codes.long()].reshape(N, K // 32, 32) * torch.exp2(S.to(torch.float32) - 127)[..., None]
    B2, S2 = quant(deq.reshape(N, K).to(torch.bfloat16))
    torch.cuda.synchronize()
    assert torch.equal(B2, B) and torch.equal(S2, S)
    ref_B, ref_S = orc.quantize_mxfp4(w[:16].float().cpu().numpy())
    np.testing.assert_array_equal(B[:16].cpu().numpy(), ref_B)
    np.testing.assert_array_equal(S[:16].cpu().numpy(), ref_S)


def test_mxfp4_quantise_then_gemm(cuda):
    """The quantiser's output is what the MXFP4 GEMM consumes: A @ dequant(quantise(W)).T against the oracle's
    ref_program on the same operands."""
    M, N, K = 64, 256, 512
    rng = np.random.default_rng(9)
    a = orc.round_to_bf16(rng.standard_normal((M, K), dtype=np.float32))
    w = orc.round_to_bf16(rng.standard_normal((N, K), dtype=np.float32) * 0.1)
    B, S = tl.quantize_bf16_mxfp4(N, K)(_bf16_tensor(w, cuda))
    kern = tl.matmul_bf16_mxfp4(M, N, K, weight_format="e2m1", with_bias=False, scale_bias=127)
    C = kern(_bf16_tensor(a, cuda), B, S, torch.zeros((M, N), dtype=torch.bfloat16, device=cuda))
    torch.cuda.synchronize()
    ref = orc.ref_mxfp4(orc.f32_to_bf16_bits(a), B.cpu().numpy(), S.cpu().numpy(), fmt="e2m1", scale_size=32, scale_bias=127)
    np.testing.assert_allclose(C.float().cpu().numpy(), orc.bf16_bits_to_f32(ref), rtol=1e-2, atol=1e-2)
    # and the quantised weights are close to the originals: within the e2m1 step of each block
    deq = orc.mxfp4_dequant(B.cpu().numpy(), S.cpu().numpy(), fmt="e2m1", scale_size=32, scale_bias=127)
    step = np.repeat(np.exp2(S.cpu().numpy().astype(np.float64) - 127), 32, axis=1)
    assert (np.abs(deq - w) <= 2.0 * step).all()


@pytest.mark.parametrize("groupsize", [128, -1])
def test_gen_quant4_through_the_w4a16_kernels(cuda, groupsize):
    """gen_quant4's (q, s), repacked into this library's layout, dequantise on the GPU to the reference's
    `linear.weight` bit for bit (elements whose code saturated at 15 aside) and give the same GEMV."""
    K, N = 1024, 256
    torch.manual_seed(0)
    original_w, linear, s, q = tl.quantize.gen_quant4(K, N, groupsize)
    ref_deq, ref_s, ref_q = orc.gen_quant4_quantize(original_w.numpy(), groupsize)
    np.testing.assert_array_equal(s.numpy(), ref_s)
    np.testing.assert_array_equal(q.numpy(), ref_q)
    np.testing.assert_array_equal(linear.weight.data.numpy(), ref_deq.T)
    with pytest.raises(ValueError):
        tl.quantize.pack_gen_quant4(q, s)          # a +8 exists in every group
    B, Scale = tl.quantize.pack_gen_quant4(q, s, saturate=True)
    group = K if groupsize == -1 else groupsize
    W = tl.dequantize_w4(N, K, group, source_format="int", with_scaling=True)(B.to(cuda), Scale.to(cuda))
    torch.cuda.synchronize()
    kept = (q.t() < 8).numpy()
    np.testing.assert_array_equal(W.cpu().numpy()[kept], linear.weight.data.numpy()[kept])
    sat = W.cpu().numpy()[~kept].astype(np.float32)
    np.testing.assert_array_equal(sat, (7 * np.repeat(s.t().numpy(), group, axis=1))[~kept].astype(np.float16).astype(np.float32))
    if groupsize == 128:
        x = torch.randn((1, K), dtype=torch.float16)
        C = torch.empty((1, N), dtype=torch.float16, device=cuda)
        tl.dequantize_gemv(1, N, K, group_size=128, source_format="int", with_scaling=True)(x.to(cuda), B.to(cuda), Scale.to(cuda), C)
        torch.cuda.synchronize()
        ref = (x.float() @ W.cpu().float().t()).half()
        np.testing.assert_allclose(C.cpu().float().numpy(), ref.float().numpy(), rtol=1e-2, atol=1e-2)
