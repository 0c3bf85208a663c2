"""GPU parity of the 2-bit and 1-bit cases of dequantize_gemv (fp16 activations, B[N, K * bits / 8]) through the C-ABI."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from oracle import dq_oracle as orc

pytestmark = pytest.mark.gpu


def _inputs(M, N, K, seed, integer_a=False):
    rng = np.random.default_rng(seed)
    if integer_a:
        A = rng.integers(-4, 5, size=(M, K)).astype(np.float16)
    else:
        A = rng.standard_normal((M, K)).astype(np.float16)
    packed = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    return A, packed


def _run(kernel, cuda, A, B, S=None):
    M, N = A.shape[0], B.shape[0]
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=cuda)
    args = [torch.from_numpy(A).to(cuda), torch.from_numpy(B.view(np.int8)).to(cuda)]
    if S is not None:
        args.append(torch.from_numpy(S).to(cuda))
    kernel(*args, C)
    torch.cuda.synchronize()
    return C.cpu().numpy()


@pytest.mark.parametrize("M,N,K", [(1, 1024, 1024), (1, 256, 128), (2, 1000, 4096), (1, 4096, 11008), (3, 517, 8192),
                                   (1, 64, 16384), (1, 96, 20480), (5, 33, 2048), (1, 7, 32768)])
@pytest.mark.parametrize("fast,fmt", [(False, "uint"), (True, "uint"), (True, "int")])
def test_w2a16_exact_integers(cuda, M, N, K, fast, fmt):
    """Small-integer activations: every product and partial sum is exact in fp32, so the result must be too
    (slow path = two's complement; fast paths = interleaved words, unsigned / minus two)."""
    A, packed = _inputs(M, N, K, seed=M * 7 + N + K + int(fast), integer_a=True)
    conv = "twos" if not fast else ("offset" if fmt == "int" else "unsigned")
    B = orc.interleave_weight(packed.view(np.int8), 2, "float16").view(np.uint8) if fast else packed
    kernel = tl.dequantize_gemv(M, N, K, "float16", "float16", "float32", num_bits=2, source_format=fmt, fast_decoding=fast)
    got = _run(kernel, cuda, A, B)
    acc = A.astype(np.int64) @ orc.decode_i2(packed, conv).astype(np.int64).T
    np.testing.assert_array_equal(got.astype(np.float64), acc.astype(np.float16).astype(np.float64))


@pytest.mark.parametrize("N", [1, 2, 7, 9, 31, 513, 4099, 7919, 57347])
@pytest.mark.parametrize("K", [512, 4096, 8192, 16384])
def test_w2a16_rows_split_over_workgroups(cuda, N, K):
    """The grid hands every workgroup an even share of the rows whatever N is (row counts that are odd, prime,
    smaller than a batch, or too many for 512 workgroups): each output row must come out once and exact, with K
    chosen so that a row takes a quarter of a wave, one wave, two waves and two chunks per thread."""
    A, packed = _inputs(1, N, K, seed=N + K, integer_a=True)
    B = orc.interleave_weight(packed.view(np.int8), 2, "float16").view(np.uint8)
    kernel = tl.dequantize_gemv(1, N, K, "float16", "float16", "float32", num_bits=2, source_format="int", fast_decoding=True)
    got = _run(kernel, cuda, A, B)
    acc = A.astype(np.int64) @ orc.decode_i2(packed, "offset").astype(np.int64).T
    np.testing.assert_array_equal(got.astype(np.float64), acc.astype(np.float16).astype(np.float64))


@pytest.mark.parametrize("M,N,K,group", [(1, 1024, 1024, 128), (1, 28672, 8192, 128), (2, 300, 4096, 64), (4, 1024, 8192, 8192),
                                         (1, 512, 11008, 64)])
@pytest.mark.parametrize("fast,fmt", [(False, "int"), (True, "int"), (True, "uint")])
def test_w2a16_scaled(cuda, M, N, K, group, fast, fmt):
    """Gaussian activations and group scales against dequantise + fp32 matmul, rtol = atol = 1e-2, no mismatches."""
    A, packed = _inputs(M, N, K, seed=N + K + group)
    S = np.random.default_rng(3).uniform(0.005, 0.02, size=(N, K // group)).astype(np.float16)
    conv = "twos" if not fast else ("offset" if fmt == "int" else "unsigned")
    B = orc.interleave_weight(packed.view(np.int8), 2, "float16").view(np.uint8) if fast else packed
    kernel = tl.dequantize_gemv(M, N, K, "float16", "float16", "float32", num_bits=2, source_format=fmt, fast_decoding=fast,
                                group_size=group, with_scaling=True)
    got = _run(kernel, cuda, A, B, S)
    ref = orc.ref_w2a16(A, packed, conv, S, group)
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=1e-2, atol=1e-2)


def test_w2a16_unscaled_gaussian_and_repeatable(cuda):
    """Unscaled, Gaussian activations; two launches give bit-identical results (fixed reduction order)."""
    M, N, K = 2, 4096, 8192
    A, packed = _inputs(M, N, K, seed=9)
    kernel = tl.dequantize_gemv(M, N, K, "float16", "float16", "float32", num_bits=2)
    got = _run(kernel, cuda, A, packed)
    again = _run(kernel, cuda, A, packed)
    np.testing.assert_array_equal(got.view(np.uint16), again.view(np.uint16))
    ref = orc.ref_w2a16(A, packed, "twos")
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=1e-2, atol=1e-2)


# ---- one bit, and the zero-point forms of both widths ---------------------------------------------------------


def _packed(N, K, bits, seed):
    return np.random.default_rng(seed).integers(0, 256, size=(N, K * bits // 8), dtype=np.uint8)


@pytest.mark.parametrize("M,N,K", [(1, 1024, 1024), (1, 256, 128), (2, 1000, 4096), (1, 512, 11008), (3, 517, 8192), (1, 40, 32768)])
@pytest.mark.parametrize("fast,fmt", [(False, "uint"), (True, "uint"), (True, "int")])
def test_w1a16_exact_integers(cuda, M, N, K, fast, fmt):
    """One bit per weight, small-integer activations: exact (two's complement -c; fast decoders c and 2c - 1 on
    words passed through the 1-bit interleave)."""
    A = np.random.default_rng(M + N + K).integers(-4, 5, size=(M, K)).astype(np.float16)
    packed = _packed(N, K, 1, seed=K + int(fast))
    conv = "twos" if not fast else ("offset" if fmt == "int" else "unsigned")
    B = orc.interleave_weight(packed.view(np.int8), 1, "float16").view(np.uint8) if fast else packed
    kernel = tl.dequantize_gemv(M, N, K, "float16", "float16", "float32", num_bits=1, source_format=fmt, fast_decoding=fast)
    got = _run(kernel, cuda, A, B)
    acc = A.astype(np.int64) @ orc.decode_lowbit(packed, 1, conv).astype(np.int64).T
    np.testing.assert_array_equal(got.astype(np.float64), acc.astype(np.float16).astype(np.float64))


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("M,N,K,group", [(1, 1024, 1024, 128), (1, 28672, 8192, 128), (2, 300, 4096, 256), (3, 64, 8192, 8192)])
@pytest.mark.parametrize("fast,fmt,zeros_mode", [(True, "uint", "original"), (True, "uint", "rescale"), (True, "int", "original"),
                                                 (False, "int", "rescale"), (True, "int", None)])
def test_lowbit_scale_and_zeros(cuda, bits, M, N, K, group, fast, fmt, zeros_mode):
    """Group scales and zero points (original: (w - z) s; rescale: w s - z) against dequantise + fp32 matmul."""
    rng = np.random.default_rng(bits * 1000 + N + K + group)
    A = rng.standard_normal((M, K)).astype(np.float16)
    packed = _packed(N, K, bits, seed=N + bits)
    S = rng.uniform(0.005, 0.02, size=(N, K // group)).astype(np.float16)
    if zeros_mode == "original":
        Z = rng.integers(0, 1 << bits, size=(N, K // group)).astype(np.float16)
    elif zeros_mode == "rescale":
        Z = (rng.uniform(0.0, 0.03, size=(N, K // group))).astype(np.float16)
    else:
        Z = None
    conv = "twos" if not fast else ("offset" if fmt == "int" else "unsigned")
    B = orc.interleave_weight(packed.view(np.int8), bits, "float16").view(np.uint8) if fast else packed
    kernel = tl.dequantize_gemv(M, N, K, "float16", "float16", "float32", num_bits=bits, source_format=fmt, fast_decoding=fast,
                                group_size=group, with_scaling=True, with_zeros=Z is not None,
                                zeros_mode=zeros_mode or "original")
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=cuda)
    args = [torch.from_numpy(A).to(cuda), torch.from_numpy(B.view(np.int8)).to(cuda), torch.from_numpy(S).to(cuda)]
    if Z is not None:
        args.append(torch.from_numpy(Z).to(cuda))
    kernel(*args, C)
    torch.cuda.synchronize()
    ref = orc.ref_lowbit(A, packed, bits, conv, S, Z, group, zeros_mode or "original")
    np.testing.assert_allclose(C.float().cpu().numpy(), ref.astype(np.float32), rtol=1e-2, atol=1e-2)


# ---- the integer branch of dequantize_gemv (int8 activations, int32 accumulation) --------------------------------


@pytest.mark.parametrize("M,N,K", [(1, 1024, 1024), (3, 520, 2048), (64, 256, 1024)])
@pytest.mark.parametrize("bits,fast,fmt", [(2, False, "uint"), (2, True, "int"), (2, True, "uint"), (4, False, "int"),
                                           (4, True, "uint"), (4, True, "int")])
def test_dequantize_gemv_int8_exact(cuda, M, N, K, bits, fast, fmt):
    """use_dp4a branch of the example (example_dequant_gemv_fp16xint4.py:47-48,126-133): exact int32."""
    rng = np.random.default_rng(M + N + K + bits)
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    packed = _packed(N, K, bits, seed=bits + int(fast))
    if bits == 2:
        conv = "twos" if not fast else ("offset" if fmt == "int" else "unsigned")
        W = orc.decode_i2(packed, conv).astype(np.int64)
        B = orc.interleave_weight(packed.view(np.int8), 2, "int8").view(np.uint8) if fast else packed
    elif fast:
        # decode_i4{u,s}_to_i8s over interleave_weight(., 4, "int8") words (lop3.py:999-1047): w = q, or q - 7
        B = orc.interleave_weight(packed.view(np.int8), 4, "int8").view(np.uint8)
        W = orc.decode_i4_fast_int8(B, signed=(fmt == "int")).astype(np.int64)
        assert np.array_equal(W, orc.unpack_u4(packed).astype(np.int64) - (7 if fmt == "int" else 0))
    else:
        W = orc.decode_i4_signed(packed).astype(np.int64)
        B = packed
    kernel = tl.dequantize_gemv(M, N, K, "int8", "int32", "int32", num_bits=bits, source_format=fmt, fast_decoding=fast)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    kernel(torch.from_numpy(A).to(cuda), torch.from_numpy(B.view(np.int8)).to(cuda), C)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy().astype(np.int64), A.astype(np.int64) @ W.T)


@pytest.mark.parametrize("M,N,K", [(1, 1024, 1024), (2, 520, 2048), (4, 300, 4096), (1, 4099, 8192), (3, 64, 11008),
                                   (4, 96, 16384), (1, 7, 128), (2, 33, 12288)])
@pytest.mark.parametrize("decode", ["twos", "fast_uint", "fast_int", "unsigned"])
def test_int8xint4_decode_gemv_exact(cuda, M, N, K, decode):
    """The streaming int8 x 4-bit decode kernel (M <= 4: v_dot4_i32_i8 over 16 bytes of B per lane, the decoder's
    constant applied through the sum of the activations): exact int32 against the oracle's decoders, shapes that take
    a quarter of a wave, one to four waves and two chunks per thread, ragged N; and bit for bit what the tiled GEMM
    gives on the same operands."""
    from tilelang_amd import _lib
    import ctypes

    rng = np.random.default_rng(M * 3 + N + K)
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    packed = _packed(N, K, 4, seed=K + len(decode))
    if decode == "twos":
        W, B, dec = orc.decode_i4_signed(packed).astype(np.int64), packed, 1
    elif decode == "unsigned":
        W, B, dec = orc.unpack_u4(packed).astype(np.int64), packed, 0
    else:
        B = orc.interleave_weight(packed.view(np.int8), 4, "int8").view(np.uint8)
        W = orc.decode_i4_fast_int8(B, signed=(decode == "fast_int")).astype(np.int64)
        dec = 3 if decode == "fast_int" else 2
    lib = _lib.get_library()
    Ad, Bd = torch.from_numpy(A).to(cuda), torch.from_numpy(B.view(np.int8)).to(cuda)
    outs = []
    for flag in (0, 32):  # the library's choice (the decode kernel), then the tiled GEMM by name
        C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
        rc = lib.call_gemm_int8xint4(ctypes.c_void_p(Ad.data_ptr()), ctypes.c_void_p(Bd.data_ptr()), ctypes.c_void_p(C.data_ptr()),
                                     M, N, K, dec, 0, flag, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.get_last_error().decode()
        torch.cuda.synchronize()
        outs.append(C.cpu().numpy())
    np.testing.assert_array_equal(outs[0].astype(np.int64), A.astype(np.int64) @ W.T)
    np.testing.assert_array_equal(outs[0], outs[1])


@pytest.mark.parametrize("M", [1, 4])
@pytest.mark.parametrize("decode", ["twos", "fast_int"])
def test_int8xint4_decode_gemv_full_size(cuda, M, decode):
    """N = 28672, K = 8192 (117 MB of weights): every int32 output."""
    N, K = 28672, 8192
    print(f"int8 x int4 decode GEMV full size: M={M} decode={decode}", flush=True)
    rng = np.random.default_rng(17 + M)
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    packed = _packed(N, K, 4, seed=23)
    fast = decode == "fast_int"
    if fast:
        B = orc.interleave_weight(packed.view(np.int8), 4, "int8").view(np.uint8)
        W = (orc.unpack_u4(packed).astype(np.int32) - 7)
    else:
        B, W = packed, orc.decode_i4_signed(packed).astype(np.int32)
    kernel = tl.dequantize_gemv(M, N, K, "int8", "int32", "int32", num_bits=4, source_format="int", fast_decoding=fast)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    kernel(torch.from_numpy(A).to(cuda), torch.from_numpy(B.view(np.int8)).to(cuda), C)
    torch.cuda.synchronize()
    ref = (A.astype(np.float64) @ W.T.astype(np.float64)).astype(np.int64)  # |sum| < 2^53: exact in fp64
    np.testing.assert_array_equal(C.cpu().numpy().astype(np.int64), ref)


@pytest.mark.parametrize("M,N,K", [(1, 1024, 1024), (2, 520, 4096), (3, 77, 8192), (4, 300, 16384), (1, 9, 128), (1, 40, 65536),
                                   (2, 4099, 2048)])
@pytest.mark.parametrize("fast,fmt", [(False, "uint"), (True, "uint"), (True, "int")])
def test_int8xint1_decode_gemv_exact(cuda, M, N, K, fast, fmt):
    """int8 x 1-bit (decode_i1{u,s}_to_i8s, lop3.py:893-948, over interleave_weight(., 1, "int8") words; the slow path
    sign-extends the one-bit field): exact int32."""
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    packed = _packed(N, K, 1, seed=5 + int(fast))
    if fast:
        B = orc.interleave_weight(packed.view(np.int8), 1, "int8").view(np.uint8)
        W = orc.decode_i1_fast_int8(B, signed=(fmt == "int")).astype(np.int64)
        assert np.array_equal(W, orc.decode_lowbit(packed, 1, "offset" if fmt == "int" else "unsigned").astype(np.int64))
    else:
        B, W = packed, orc.decode_lowbit(packed, 1, "twos").astype(np.int64)
    kernel = tl.dequantize_gemv(M, N, K, "int8", "int32", "int32", num_bits=1, source_format=fmt, fast_decoding=fast)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    kernel(torch.from_numpy(A).to(cuda), torch.from_numpy(B.view(np.int8)).to(cuda), C)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy().astype(np.int64), A.astype(np.int64) @ W.T)


def test_int8xint1_refuses_prefill_batches(cuda):
    with pytest.raises(ValueError, match="decode kernel"):
        tl.dequantize_gemv(8, 64, 1024, "int8", "int32", "int32", num_bits=1)


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (300, 520, 384), (1, 64, 1024), (1500, 2000, 256)])
def test_int4xint2_gemm_exact(cuda, M, N, K):
    """Packed int4 activations x 2-bit codes (the operands decode_i2{u,s}_to_i4s prepare for the int4 x int4 matrix
    instruction, lop3.py:1049-1089; both decoders leave the code unsigned): exact int32."""
    rng = np.random.default_rng(M + N)
    Ap = rng.integers(0, 256, size=(M, K // 2), dtype=np.uint8)
    Bp = _packed(N, K, 2, seed=9)
    # the reference decoder's own output, read back as unsigned nibbles: nibble e of word 2 j + i is code 2 e + i of word j
    i4 = orc.unpack_u4(orc.decode_i2_fast_int4(Bp)).reshape(N, K // 16, 2, 8)
    codes = orc.unpack_u2(Bp).reshape(N, K // 16, 8, 2)
    assert np.array_equal(i4.transpose(0, 1, 3, 2), codes)
    kernel = tl.matmul_nt_int4xint2(M, N, K)
    C = kernel(torch.from_numpy(Ap.view(np.int8)).to(cuda), torch.from_numpy(Bp.view(np.int8)).to(cuda))
    torch.cuda.synchronize()
    ref = orc.decode_i4_signed(Ap).astype(np.int64) @ orc.unpack_u2(Bp).astype(np.int64).T
    np.testing.assert_array_equal(C.cpu().numpy().astype(np.int64), ref)


@pytest.mark.parametrize("M", [1, 4, 20])
@pytest.mark.parametrize("qfmt", ["int16", "packed4"])
def test_w2a16_quantized_zeros(cuda, M, qfmt):
    """zeros_mode="quantized" for two bits (decode_i2u_to_f16_scale_zeros_quantized, lop3.py:638-677): integer zero
    points folded into the magic number, (1024 + c) + (0xe400 | qz) = c - qz exactly, times the scale once."""
    N, K, group = 520, 2048, 128
    rng = np.random.default_rng(31 + M)
    A = rng.standard_normal((M, K)).astype(np.float16)
    packed = _packed(N, K, 2, seed=3)
    S = rng.uniform(0.005, 0.02, size=(N, K // group)).astype(np.float16)
    qz = rng.integers(0, 4, size=(N, K // group)).astype(np.int16)
    Z = qz if qfmt == "int16" else (qz[:, 0::2] | (qz[:, 1::2] << 4)).astype(np.uint8)
    B = orc.interleave_weight(packed.view(np.int8), 2, "float16").view(np.uint8)
    kernel = tl.dequantize_gemv(M, N, K, "float16", "float16", "float32", num_bits=2, source_format="uint", fast_decoding=True,
                                group_size=group, with_scaling=True, with_zeros=True, zeros_mode="quantized", qzeros_format=qfmt)
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=cuda)
    kernel(torch.from_numpy(A).to(cuda), torch.from_numpy(B.view(np.int8)).to(cuda), torch.from_numpy(S).to(cuda),
           torch.from_numpy(Z).to(cuda), C)
    torch.cuda.synchronize()
    # the oracle's tile with the integers as fp16 zero points: c - qz is exact either way
    W = orc.dequant_lowbit(packed, 2, "unsigned", S, qz.astype(np.float16), group, "original").astype(np.float32)
    ref = (A.astype(np.float32) @ W.T).astype(np.float16).astype(np.float32)
    np.testing.assert_allclose(C.float().cpu().numpy(), ref, rtol=1e-2, atol=1e-2)
    with pytest.raises(ValueError, match="quantized"):
        tl.dequantize_gemv(M, N, K, num_bits=2, source_format="int", fast_decoding=True, group_size=group, with_scaling=True,
                           with_zeros=True, zeros_mode="quantized")
