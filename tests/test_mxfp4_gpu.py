"""GPU parity of the MXFP4 x bf16 GEMM (through the C-ABI) against the CPU oracle.

bf16 outputs within rtol=1e-2, atol=1e-2 of ``A.float() @ (decode(B) * 2**(Scale - bias)).float().T -> bf16``
(the dequantised operand is exact in bf16, the only rounding is the fp32 accumulation and the final cast).
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


def _check(cuda, M, N, K, fmt, scale_bias, seed=0, with_bias=False, exp_range=(-8, 0)):
    d = workloads.mxfp4(M, N, K, seed=seed, scale_exp_range=exp_range, scale_bias=scale_bias)
    B = d["B"]
    if fmt == "twiddling":
        B = orc.twiddle_pack_fp4(orc.unpack_u4(B))
    kern = tl.matmul_bf16_mxfp4(M, N, K, weight_format=fmt, scale_bias=scale_bias, with_bias=with_bias)
    A = _dev(d["A"], cuda).view(torch.bfloat16)
    rng = np.random.default_rng(seed + 1)
    bias_bits = orc.f32_to_bf16_bits(rng.standard_normal((M, N), dtype=np.float32) * 4)
    Bias = _dev(bias_bits, cuda).view(torch.bfloat16)
    C = kern(A, _dev(B, cuda), _dev(d["Scale"], cuda), Bias)
    torch.cuda.synchronize()
    ref_bits = orc.ref_mxfp4(d["A"], B, d["Scale"], bias_bits if with_bias else None, fmt=fmt, scale_bias=scale_bias)
    ref = orc.bf16_bits_to_f32(ref_bits)
    got = C.float().cpu().numpy()
    assert got.shape == (M, N) and np.isfinite(got).all()
    np.testing.assert_allclose(got, ref, rtol=RTOL, atol=ATOL)
    return got


@pytest.mark.parametrize("fmt", ["e2m1", "twiddling", "simple"])
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (64, 64, 64), (128, 512, 128)])
def test_reference_test_shapes(cuda, fmt, M, N, K):
    """Shapes of testing/python/amd/test_tilelang_mxfp4_gfx950.py:111-222, but over all 16 codes
    and, like the reference programs, the raw unbiased exponent (2**Scale, Scale in 0..2)."""
    _check(cuda, M, N, K, fmt, scale_bias=0, exp_range=(0, 2))


@pytest.mark.parametrize("fmt", ["e2m1", "twiddling", "simple"])
def test_e8m0_scales(cuda, fmt):
    _check(cuda, 512, 768, 512, fmt, scale_bias=127)


@pytest.mark.parametrize("M,N,K", [(1, 256, 64), (100, 300, 192), (257, 255, 128), (300, 520, 320)])
def test_ragged_shapes(cuda, M, N, K):
    _check(cuda, M, N, K, "e2m1", scale_bias=127)


@pytest.mark.parametrize("fmt", ["e2m1", "twiddling", "simple"])
@pytest.mark.parametrize("with_bias", [False, True])
def test_many_tiles(cuda, fmt, with_bias):
    """Enough 256 x 256 tiles for the direct-to-LDS kernel (ragged edges, K of 2 and of 5 tiles), and the
    128 x 128 tile choice below it."""
    _check(cuda, 3581, 3589, 128, fmt, scale_bias=127, with_bias=with_bias)
    _check(cuda, 3584, 3584, 320, fmt, scale_bias=0, with_bias=with_bias, exp_range=(0, 4))
    _check(cuda, 1500, 2000, 192, fmt, scale_bias=127, with_bias=with_bias)
    # too few 256 x 256 tiles, 96 of 128 x 256: the direct-to-LDS kernel on its half-height tile (ragged both ways)
    _check(cuda, 1500, 2000, 256, fmt, scale_bias=127, with_bias=with_bias)
    _check(cuda, 1025, 3000, 384, fmt, scale_bias=127, with_bias=with_bias)
    if not with_bias:  # direct-to-LDS kernel with 4, 6 and 10 K tiles: prologue pair, steady pairs, tail
        for K in (256, 384, 640):
            _check(cuda, 3584, 3600, K, fmt, scale_bias=127)


@pytest.mark.parametrize("fmt", ["e2m1", "twiddling", "simple"])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 256, 128), (5, 300, 1024), (16, 1001, 2048), (8, 4100, 2176), (3, 64, 8192),
                                   (16, 9000, 5120), (17, 515, 1280), (40, 130, 4096), (64, 8200, 768), (12, 33, 6144),
                                   # K % 128 == 64: the last chunk of 128 k is half empty (2880: a hidden size in use)
                                   (4, 300, 2880), (16, 5763, 2880), (8, 100, 192), (20, 513, 4160), (3, 2880, 64),
                                   # K beyond 8192: slices of at most 6144 k, running sums in LDS between them
                                   (8, 300, 14336), (16, 4500, 8320), (5, 130, 28672), (24, 64, 12288),
                                   # K % 256 == 0: whole pairs of chunks per wave, runs of unequal length (7168 = 28 pairs, 256 = 1)
                                   (9, 700, 7168), (16, 130, 256), (2, 48, 3584),
                                   # one row up to K = 8192: the dot-product kernel (whole rows per wave, lanes beyond a row's end idle)
                                   (1, 300, 1024), (1, 1001, 2880), (1, 4100, 8192), (1, 513, 5120), (1, 5, 64), (1, 9000, 7168), (1, 31, 4160),
                                   # two rows: the same with the activations in LDS
                                   (2, 4100, 8192), (2, 1001, 5120), (2, 515, 1024), (2, 9000, 7168), (2, 7, 64),
                                   # one and two rows beyond K = 8192: chunks of four steps, activations padded to whole chunks in LDS
                                   (1, 300, 14336), (2, 1001, 16384), (1, 64, 28672), (2, 130, 8320), (1, 4100, 12288), (2, 33, 32768),
                                   (1, 40, 40960)])
def test_decode_batches(cuda, fmt, with_bias, M, N, K):
    """Decode batches with K a multiple of 64 (of 128 beyond 8192): the kernel that keeps the activations in registers
    and streams weights and scale bytes once per 16 rows.  Ragged N (last block of 16 weight rows, N % 4 != 0), K slices of unequal
    length over the eight waves (2176 = 17 chunks, 1280 = 10, 128 = 1), the eight-chunk form with parked activations
    (8192), passes of 16 rows (17, 40, 64), every format, with and without bias."""
    _check(cuda, M, N, K, fmt, scale_bias=127, seed=M + K, with_bias=with_bias)


def test_decode_batch_full_size_and_deterministic(cuda):
    """N = K = 8192 at 16 rows against the oracle, twice: the partial sums of the eight K slices are added in a
    fixed order."""
    a = _check(cuda, 16, 8192, 8192, "e2m1", scale_bias=127, seed=4)
    b = _check(cuda, 16, 8192, 8192, "e2m1", scale_bias=127, seed=4)
    np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("fmt", ["e2m1", "simple"])
def test_bias(cuda, fmt):
    _check(cuda, 384, 512, 256, fmt, scale_bias=127, with_bias=True)


def test_weight_values_exact(cuda):
    """A = identity picks single weights: C[i, n] must equal decode(B)[n, i] * 2**e exactly (bf16)."""
    N, K = 512, 256
    for fmt in ("e2m1", "twiddling", "simple"):
        d = workloads.mxfp4(K, N, K, seed=7, scale_bias=127)
        B = d["B"]
        # every byte value appears
        B[0, :] = np.arange(K // 2, dtype=np.uint8)
        B[1, :] = np.arange(K // 2, dtype=np.uint8)[::-1] + 128
        Bp = orc.twiddle_pack_fp4(orc.unpack_u4(B)) if fmt == "twiddling" else B
        eye = orc.f32_to_bf16_bits(np.eye(K, dtype=np.float32))
        kern = tl.matmul_bf16_mxfp4(K, N, K, weight_format=fmt, scale_bias=127)
        C = kern(_dev(eye, cuda).view(torch.bfloat16), _dev(Bp, cuda), _dev(d["Scale"], cuda),
                 torch.empty((K, N), dtype=torch.bfloat16, device=cuda))
        torch.cuda.synchronize()
        W = orc.mxfp4_dequant(Bp, d["Scale"], fmt, 32, 127)  # [N, K] float32, exact
        got = C.float().cpu().numpy()
        np.testing.assert_array_equal(got, W.T + np.float32(0.0))


def test_full_size_properties(cuda):
    """Benchmark configuration 4 (M=4096, N=K=8192), checked without a full CPU matmul: a sample of
    rows and columns against the oracle, and linearity in A."""
    M, N, K = 4096, 8192, 8192
    d = workloads.mxfp4(M, N, K, seed=0, scale_bias=127)
    kern = tl.matmul_bf16_mxfp4(M, N, K, weight_format="e2m1", scale_bias=127)
    A = _dev(d["A"], cuda).view(torch.bfloat16)
    B, S = _dev(d["B"], cuda), _dev(d["Scale"], cuda)
    bias = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
    C = kern(A, B, S, bias)
    torch.cuda.synchronize()
    rng = np.random.default_rng(1)
    rows = rng.choice(M, 48, replace=False)
    cols = rng.choice(N, 64, replace=False)
    Af = orc.bf16_bits_to_f32(d["A"][rows])
    W = orc.mxfp4_dequant(d["B"][cols], d["Scale"][cols], "e2m1", 32, 127)
    ref = orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(Af @ W.T))
    got = C[torch.from_numpy(rows).to(cuda)][:, torch.from_numpy(cols).to(cuda)].float().cpu().numpy()
    np.testing.assert_allclose(got, ref, rtol=RTOL, atol=ATOL)
    # whole-matrix check against a row sample: rows of C computed by an independent call on A[rows] (80 rows: the tiled
    # kernel again, whose sums do not depend on where in the matrix a row lies; up to 64 rows the decode kernel would
    # take the call and add the same products in another order)
    rows = rng.choice(M, 80, replace=False)
    kern_small = tl.matmul_bf16_mxfp4(len(rows), N, K, weight_format="e2m1", scale_bias=127)
    C_rows = kern_small(A[torch.from_numpy(rows).to(cuda)].contiguous(), B, S, bias[: len(rows)].contiguous())
    torch.cuda.synchronize()
    assert torch.equal(C_rows, C[torch.from_numpy(rows).to(cuda)])
    # and the decode kernel on 16 of those rows: within rounding of the same values
    kern_dec = tl.matmul_bf16_mxfp4(16, N, K, weight_format="e2m1", scale_bias=127)
    C_dec = kern_dec(A[torch.from_numpy(rows[:16]).to(cuda)].contiguous(), B, S, bias[:16].contiguous())
    torch.cuda.synchronize()
    np.testing.assert_allclose(C_dec.float().cpu().numpy(), C_rows[:16].float().cpu().numpy(), rtol=RTOL, atol=ATOL)
    # linearity: C(2A) == 2 C(A) exactly (power-of-two scaling commutes with every rounding)
    C2 = kern((A.float() * 2).to(torch.bfloat16), B, S, bias)
    torch.cuda.synchronize()
    assert torch.equal(C2.float(), C.float() * 2)


# ---- bf16 x fp4 without block scales (the example with kernel(A, qB)) ------------------------------------------------

@pytest.mark.parametrize("fast_dequant", [True, False])
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (100, 300, 192), (512, 1024, 2048), (1500, 2000, 256)])
def test_unscaled_bf16_fp4(cuda, fast_dequant, M, N, K):
    """examples/dequantize_gemm/example_dequant_gemm_bf16_fp4_hopper.py: main(256, 256, 256, fast_dequant) against
    ref_program_twiddling / ref_program_simple, here the oracle's restatement of them (block exponent 0)."""
    fmt = "twiddling" if fast_dequant else "simple"
    d = workloads.mxfp4(M, N, K, seed=11, scale_exp_range=(0, 0), scale_bias=0)
    B = orc.twiddle_pack_fp4(orc.unpack_u4(d["B"])) if fast_dequant else d["B"]
    kern = tl.matmul_bf16_fp4(M, N, K, "bfloat16", "bfloat16", "float32", num_bits=4, fast_dequant=fast_dequant,
                              block_M=256, block_N=128, block_K=128, num_stages=2, threads=256, split=1)
    C = kern(_dev(d["A"], cuda).view(torch.bfloat16), _dev(B, cuda))
    torch.cuda.synchronize()
    zero_scale = np.zeros((N, K // 32), np.uint8)
    ref = orc.bf16_bits_to_f32(orc.ref_mxfp4(d["A"], B, zero_scale, None, fmt=fmt, scale_bias=0))
    got = C.float().cpu().numpy()
    assert got.shape == (M, N) and np.isfinite(got).all()
    np.testing.assert_allclose(got, ref, rtol=RTOL, atol=ATOL)


def test_unscaled_bf16_fp4_reads_back_the_reference_vectors(cuda):
    """A = identity makes the GEMM return the dequantised operand itself, exactly: against what the reference's own
    torch_convert_bit_twiddling (all 65 536 byte pairs) and torch_convert (all 256 bytes) produce
    (tests/golden/reference_vectors.npz, written by tests/golden/make_vectors.py)."""
    import os

    v = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))
    for fast, qB, want_bits in ((True, v["twiddling_in"], v["twiddling_out_bits"]), (False, v["convert_in"], v["convert_out_bits"])):
        N, K = qB.shape[0], qB.shape[1] * 2
        kern = tl.matmul_bf16_fp4(K, N, K, fast_dequant=fast)
        eye = torch.eye(K, dtype=torch.bfloat16, device=cuda)
        C = kern(eye, _dev(qB, cuda))
        torch.cuda.synchronize()
        got = C.float().cpu().numpy().T  # [N, K]
        np.testing.assert_array_equal(got, orc.bf16_bits_to_f32(want_bits))
