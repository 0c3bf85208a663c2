"""GPU parity of the block-scaled MXFP4 x MXFP4 GEMM (through the C-ABI) against the CPU oracle.

Both operands are e2m1 codes with one E8M0 byte per 32 k; the kernel hands codes and scale bytes to the scaled
matrix instruction as they lie in memory.  Two bars:

* bit-exact bf16 output where every partial sum is exactly representable in fp32 (scale exponents in -1..1,
  K <= 2048: products are multiples of 2**-4 below 2**8, sums stay below 2**24 of those units), so that a wrong
  lane / k / scale-byte mapping cannot hide inside a tolerance;
* rtol = atol = 1e-2 for the general case (fp32 accumulation order and the final bf16 rounding differ from the
  oracle's float64 sum).
"""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from tilelang_amd import workloads
from oracle import dq_oracle as orc

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _dev(x, cuda):
    return torch.from_numpy(np.ascontiguousarray(x)).to(cuda)


def _run(cuda, d, M, N, K, bias_bits=None):
    kern = tl.matmul_mxfp4_mxfp4(M, N, K, with_bias=bias_bits is not None)
    Bias = _dev(bias_bits if bias_bits is not None else np.zeros((M, N), np.uint16), cuda).view(torch.bfloat16)
    C = kern(_dev(d["A"], cuda), _dev(d["B"], cuda), _dev(d["SFA"], cuda), _dev(d["SFB"], cuda), Bias)
    torch.cuda.synchronize()
    assert C.shape == (M, N) and C.dtype == torch.bfloat16
    return C.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (512, 256, 384), (256, 768, 2048), (32, 32, 512)])
def test_bit_exact_when_sums_are_exact(cuda, M, N, K):
    print(f"blockscaled exact M={M} N={N} K={K}", flush=True)
    d = workloads.mxfp4_mxfp4(M, N, K, seed=M + N + K, scale_exp_range=(-1, 1))
    got = _run(cuda, d, M, N, K)
    ref = orc.ref_mxfp4_mxfp4(d["A"], d["SFA"], d["B"], d["SFB"])
    np.testing.assert_array_equal(got, ref)


def test_every_scale_block_and_lane_half_matters(cuda):
    """One nonzero code per operand row and a distinct scale in every 32-k block: an output element is a single
    product, so a scale byte taken from the wrong block or the wrong lane half changes it by a power of two."""
    M = N = 256
    K = 512
    rng = np.random.default_rng(5)
    codes_a = np.zeros((M, K), np.uint8)
    codes_b = np.zeros((N, K), np.uint8)
    ka = rng.integers(0, K, size=M)
    codes_a[np.arange(M), ka] = rng.integers(1, 8, size=M)
    for n in range(N):  # B row n has a nonzero code wherever some A row has one, so every product is live
        codes_b[n, :] = rng.integers(1, 8, size=K)
    SA = (127 + (np.arange(K // 32)[None, :] % 7) - 3 + np.zeros((M, 1), np.int64)).astype(np.uint8)
    SB = (127 + (np.arange(K // 32)[None, :] * 3 % 5) - 2 + np.zeros((N, 1), np.int64)).astype(np.uint8)
    d = {"A": workloads.pack_nibbles(codes_a), "B": workloads.pack_nibbles(codes_b), "SFA": SA, "SFB": SB}
    got = _run(cuda, d, M, N, K)
    ref = orc.ref_mxfp4_mxfp4(d["A"], d["SFA"], d["B"], d["SFB"])
    np.testing.assert_array_equal(got, ref)


@pytest.mark.parametrize("M,N,K", [(512, 768, 1024), (256, 256, 8192), (1024, 512, 4096)])
def test_general_scales(cuda, M, N, K):
    print(f"blockscaled general M={M} N={N} K={K}", flush=True)
    d = workloads.mxfp4_mxfp4(M, N, K, seed=1, scale_exp_range=(-8, 0))
    got = orc.bf16_bits_to_f32(_run(cuda, d, M, N, K))
    ref = orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(d["A"], d["SFA"], d["B"], d["SFB"]))
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got, ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M,N,K", [(1, 256, 256), (100, 300, 384), (257, 255, 256), (300, 520, 640)])
def test_ragged_shapes(cuda, M, N, K):
    print(f"blockscaled ragged M={M} N={N} K={K}", flush=True)
    d = workloads.mxfp4_mxfp4(M, N, K, seed=2, scale_exp_range=(-1, 1))
    got = _run(cuda, d, M, N, K)
    ref = orc.ref_mxfp4_mxfp4(d["A"], d["SFA"], d["B"], d["SFB"])
    np.testing.assert_array_equal(got, ref)


def test_scale_byte_255_is_nan(cuda):
    """E8M0 has no infinity: byte 255 is NaN, and the instruction propagates it to every output of that row."""
    M = N = K = 256
    d = workloads.mxfp4_mxfp4(M, N, K, seed=6)
    d["SFA"][3, 1] = 255
    d["SFB"][200, 7] = 255
    got = orc.bf16_bits_to_f32(_run(cuda, d, M, N, K))
    ref = orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(d["A"], d["SFA"], d["B"], d["SFB"]))
    np.testing.assert_array_equal(np.isnan(got), np.isnan(ref))
    assert np.isnan(got[3]).all() and np.isnan(got[:, 200]).all() and np.isnan(got).sum() == M + N - 1
    ok = ~np.isnan(ref)
    np.testing.assert_allclose(got[ok], ref[ok], rtol=RTOL, atol=ATOL)


def test_full_size_properties(cuda):
    """M=4096, N=K=8192 (512 tiles, 64 K tiles each): a band of rows against the oracle, and two properties that
    hold bit for bit at any size: raising every scale byte of A by one doubles every output (a power of two moves no
    rounding), and swapping the operands transposes the result (the fp32 sums run in the same k order)."""
    M, N, K = 4096, 8192, 8192
    d = workloads.mxfp4_mxfp4(M, N, K, seed=9, scale_exp_range=(-6, 0))
    got = _run(cuda, d, M, N, K)
    rows = np.r_[0:8, 2040:2056, 4088:4096]
    ref = orc.ref_mxfp4_mxfp4(d["A"][rows], d["SFA"][rows], d["B"], d["SFB"])
    np.testing.assert_allclose(orc.bf16_bits_to_f32(got[rows]), orc.bf16_bits_to_f32(ref), rtol=RTOL, atol=ATOL)
    d2 = dict(d)
    d2["SFA"] = (d["SFA"] + 1).astype(np.uint8)
    doubled = _run(cuda, d2, M, N, K)
    np.testing.assert_array_equal(orc.bf16_bits_to_f32(doubled), 2.0 * orc.bf16_bits_to_f32(got))
    d3 = {"A": d["B"][:M], "SFA": d["SFB"][:M], "B": d["A"], "SFB": d["SFA"]}  # (B[:M] . A^T) = (A . B[:M]^T)^T
    swapped = _run(cuda, d3, M, M, K)
    np.testing.assert_array_equal(swapped, got[:, :M].T)


def test_bias(cuda):
    M, N, K = 300, 512, 512
    d = workloads.mxfp4_mxfp4(M, N, K, seed=3, scale_exp_range=(-4, 0))
    rng = np.random.default_rng(4)
    bias_bits = orc.f32_to_bf16_bits(rng.standard_normal((M, N), dtype=np.float32) * 4)
    got = orc.bf16_bits_to_f32(_run(cuda, d, M, N, K, bias_bits))
    ref = orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(d["A"], d["SFA"], d["B"], d["SFB"], bias_bits))
    np.testing.assert_allclose(got, ref, rtol=RTOL, atol=ATOL)


def test_operands_from_the_quantiser(cuda):
    """bf16 activations and weights through the library's MXFP4 quantiser, then the block-scaled GEMM: bit-exact
    against the oracle on the quantised operands, and close (cosine similarity, the reference example's own
    end-to-end measure, gemm_mxfp8_blockscaled_1d1d.py:622-626,716-720) to the unquantised product."""
    M, N, K = 512, 512, 1024
    g = torch.Generator(device="cpu").manual_seed(0)
    X = torch.randn((M, K), generator=g, dtype=torch.float32).to(torch.bfloat16)
    W = torch.randn((N, K), generator=g, dtype=torch.float32).to(torch.bfloat16)
    qa = tl.quantize_bf16_mxfp4(M, K, scale_bias=127)
    qb = tl.quantize_bf16_mxfp4(N, K, scale_bias=127)
    A, SA = qa(X.to(cuda))
    B, SB = qb(W.to(cuda))
    kern = tl.matmul_mxfp4_mxfp4(M, N, K)
    C = kern(A, B, SA, SB, torch.zeros((M, N), dtype=torch.bfloat16, device=cuda))
    torch.cuda.synchronize()
    got = C.float().cpu().numpy()
    ref = orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(A.cpu().numpy(), SA.cpu().numpy(), B.cpu().numpy(), SB.cpu().numpy()))
    np.testing.assert_allclose(got, ref, rtol=RTOL, atol=ATOL)
    full = (X.float() @ W.float().T).numpy()
    cos = float((got * full).sum() / (np.linalg.norm(got) * np.linalg.norm(full)))
    assert cos > 0.98, cos
