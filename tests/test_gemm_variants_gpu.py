"""GPU parity of the remaining dequantize GEMMs (through the C-ABI) against the CPU oracle: integer
accumulations bit-exact, fp16 outputs within rtol=atol=1e-2."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from tilelang_amd import quantize, workloads
from oracle import dq_oracle as orc

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _dev(x, cuda):
    return torch.from_numpy(np.ascontiguousarray(x)).to(cuda)


@pytest.mark.parametrize("M,N,K", [(128, 256, 256), (512, 512, 512), (100, 130, 384), (1, 8, 128),
                                   (1500, 2000, 256), (3581, 3589, 128), (3581, 3589, 768),
                                   (3584, 3584, 256)])  # 128x128 tiles, 256x256 tiles, and twice the direct-to-LDS kernel
def test_w4a8_exact(cuda, M, N, K):
    """examples/dequantize_gemm/example_dequant_gemm_w4a8.py: Ct[N,M] int32, all byte values."""
    d = workloads.int8_int4(M, N, K, seed=M)
    Ct = tl.matmul_int8xint4(M, N, K)(_dev(d["A"], cuda), _dev(d["B"], cuda))
    torch.cuda.synchronize()
    assert Ct.shape == (N, M) and Ct.dtype == torch.int32
    np.testing.assert_array_equal(Ct.cpu().numpy(), orc.ref_w4a8(d["A"], d["B"]))


@pytest.mark.parametrize("decode", [2, 3])
@pytest.mark.parametrize("M,N,K", [(128, 256, 256), (100, 130, 384), (1500, 2000, 256), (3581, 3589, 768)])  # last: direct-to-LDS kernel
def test_int8xint4_fast_decode_exact(cuda, M, N, K, decode):
    """The int8 branch of the GEMV example with fast_decoding, at GEMM sizes, through the C-ABI: words passed through
    interleave_weight(., 4, "int8"), decode_i4u_to_i8s (w = q) / decode_i4s_to_i8s (w = q - 7),
    examples/dequantize_gemm/quantize/lop3.py:999-1047; exact int32, all byte values."""
    import ctypes

    from tilelang_amd import _lib

    d = workloads.int8_int4(M, N, K, seed=M + decode)
    Bil = orc.interleave_weight(d["B"].view(np.int8), 4, "int8").view(np.uint8)
    W = orc.decode_i4_fast_int8(Bil, signed=(decode == 3)).astype(np.int64)
    A, B = _dev(d["A"], cuda), _dev(Bil, cuda)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    lib = _lib.get_library()
    rc = lib.call_gemm_int8xint4(ctypes.c_void_p(A.data_ptr()), ctypes.c_void_p(B.data_ptr()), ctypes.c_void_p(C.data_ptr()),
                                 M, N, K, decode, 0, 0, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.get_last_error().decode()
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy().astype(np.int64), d["A"].astype(np.int64) @ W.T)


@pytest.mark.parametrize("M,N,K", [(1024, 1024, 1024), (16, 16, 128), (300, 200, 256), (1500, 2000, 256), (3584, 3590, 128)])
def test_int4xint4_exact(cuda, M, N, K):
    """examples/gemm_int4/example_tilelang_gemm_int4.py:70-103: rtol=0, atol=0."""
    d = workloads.int4_int4(M, N, K, seed=K)
    Ap = quantize.pack_int4(torch.from_numpy(d["A_logical"])).to(cuda)
    Bp = quantize.pack_int4(torch.from_numpy(d["B_logical"])).to(cuda)
    C = tl.matmul_nt_int4(M, N, K)(Ap, Bp)
    torch.cuda.synchronize()
    ref = d["A_logical"].astype(np.int64) @ d["B_logical"].astype(np.int64).T
    np.testing.assert_array_equal(C.cpu().numpy(), ref.astype(np.int32))
    np.testing.assert_array_equal(orc.ref_int4xint4(Ap.cpu().numpy(), Bp.cpu().numpy()), ref.astype(np.int32))


@pytest.mark.parametrize("in_dtype", ["float16", "int8"])
def test_fine_grained(cuda, in_dtype):
    """examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:425-428 shapes (256^3), random nibbles."""
    M = N = K = 256
    rng = np.random.default_rng(0)
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    kern = tl.matmul_w4_fine_grained(M, N, K, in_dtype=in_dtype)
    if in_dtype == "int8":
        A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
        C = kern(_dev(A, cuda), _dev(B, cuda).view(torch.int8))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(C.cpu().numpy(), orc.ref_u4_int8(A, B))
    else:
        A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
        C = kern(_dev(A, cuda), _dev(B, cuda).view(torch.int8))
        torch.cuda.synchronize()
        ref = orc.ref_w4a16(A, B, mode="unsigned")
        np.testing.assert_allclose(C.float().cpu().numpy(), ref.astype(np.float32), rtol=RTOL, atol=ATOL * 10)


def test_fine_grained_int8_many_tiles(cuda):
    """The unsigned-nibble int8 path with enough 256 x 256 tiles for the direct-to-LDS kernel, ragged edges."""
    M, N, K = 3581, 3589, 512
    rng = np.random.default_rng(4)
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    C = tl.matmul_w4_fine_grained(M, N, K, in_dtype="int8")(_dev(A, cuda), _dev(B, cuda).view(torch.int8))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy(), orc.ref_u4_int8(A, B))


@pytest.mark.parametrize("transposed", [True, False])
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (72, 200, 128), (1500, 2000, 128), (3581, 3589, 256)])  # last: direct-to-LDS kernel
def test_fp16_fp4(cuda, transposed, M, N, K):
    """examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py: Ct[N,M] fp16, all byte values."""
    rng = np.random.default_rng(1)
    A = (rng.standard_normal((M, K), dtype=np.float32) * 0.5).astype(np.float16)
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    out = tl.matmul_fp16_fp4(M, N, K, transposed_output=transposed)(_dev(A, cuda), _dev(B, cuda))
    torch.cuda.synchronize()
    ref = orc.ref_fp16xfp4(A, B)
    if not transposed:
        ref = ref.T
    np.testing.assert_allclose(out.float().cpu().numpy(), ref.astype(np.float32), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("transposed", [True, False])
@pytest.mark.parametrize("M,N,K,split", [(256, 256, 1024, 4), (128, 192, 2048, 8), (100, 72, 512, 2), (300, 520, 768, 3),
                                         (2048, 2048, 1024, 4)])  # last: direct-to-LDS kernel (256 tiles of 256 x 256 x 256)
def test_fp16_fp4_split_k(cuda, transposed, M, N, K, split):
    """main_split of examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:136-175: fp16 partial results per K
    slice, added in fp16 in slice order.  The same call twice gives the same bits (fixed order, no atomics)."""
    print(f"split-K M={M} N={N} K={K} split={split} transposed={transposed}", flush=True)
    rng = np.random.default_rng(2)
    A = (rng.standard_normal((M, K), dtype=np.float32) * 0.5).astype(np.float16)
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    kern = tl.matmul_fp16_fp4(M, N, K, split=split, transposed_output=transposed)
    Ad, Bd = _dev(A, cuda), _dev(B, cuda)
    out = kern(Ad, Bd)
    again = kern(Ad, Bd)
    torch.cuda.synchronize()
    assert out.shape == ((N, M) if transposed else (M, N))
    assert torch.equal(out, again)
    ref = orc.ref_fp16xfp4_splitk(A, B, split).astype(np.float32)
    # Every slice result and every running sum is rounded to fp16.  The kernel's fp32 slice sums differ from the
    # oracle's in the last bits (summation order), so each of those 2 * split roundings may land one fp16 ulp away:
    # where large slices cancel, that ulp (of the largest intermediate) exceeds 1e-2 of the small final value, so
    # it is added to the bar, element by element.
    W = orc.decode_fp4_simple_f16(B).astype(np.float32)
    kk = K // split
    parts = np.stack([A[:, z * kk:(z + 1) * kk].astype(np.float32) @ W[:, z * kk:(z + 1) * kk].T for z in range(split)])
    big = np.maximum(np.abs(parts).max(axis=0), np.abs(np.cumsum(parts, axis=0)).max(axis=0))
    ulp = np.exp2(np.floor(np.log2(np.maximum(big, 2.0 ** -14))) - 10)
    bound = RTOL * np.abs(ref) + ATOL + 2 * split * ulp
    got = out.float().cpu().numpy()
    if transposed:
        got = got.T
    assert (np.abs(got - ref) <= bound).all(), float((np.abs(got - ref) - bound).max())
    # and almost everywhere the plain 1e-2 bar holds
    assert np.isclose(got, ref, rtol=RTOL, atol=ATOL).mean() > 0.9999


def test_fp16_fp4_split_k_exact_when_slices_are_exact(cuda):
    """Small integers: every slice product is an exact fp16 value, so the split result must equal the oracle's bit
    for bit (a slice read from the wrong columns or written to the wrong partial buffer cannot hide)."""
    M, N, K, split = 64, 128, 512, 4
    rng = np.random.default_rng(3)
    A = rng.integers(-2, 3, size=(M, K)).astype(np.float16)
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8) & 0x33  # codes 0..3 of both signs... magnitudes 0.5 .. 1.5
    out = tl.matmul_fp16_fp4(M, N, K, split=split, transposed_output=False)(_dev(A, cuda), _dev(B, cuda))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), orc.ref_fp16xfp4_splitk(A, B, split))


def test_fp16_fp4_weights_exact(cuda):
    K, N = 128, 256
    B = np.tile(np.arange(256, dtype=np.uint8), (N, 1))[:, : K // 2].copy()
    B[1] = B[0][::-1] + 64
    eye = np.eye(K, dtype=np.float16)
    out = tl.matmul_fp16_fp4(K, N, K)(_dev(eye, cuda), _dev(B, cuda))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy().astype(np.float32), orc.decode_fp4_simple_f16(B).astype(np.float32))


@pytest.mark.parametrize("mode", ["scale", "original", "rescale", "signed", "folded"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("M,N,K", [(200, 320, 512), (1500, 2000, 256), (3581, 3589, 128), (3581, 3589, 768),
                                   (3584, 3584, 256)])  # 128x64, 128x128, 256x256 tiles; the last two: direct-to-LDS kernel
def test_w4a16_large_m(cuda, mode, interleaved, M, N, K):
    """W4A16 through the MFMA GEMM (M > 128): same tile-exact decoders as the decode kernel."""
    group = 128
    d = workloads.w4a16(M, N, K, group, seed=2, scale_range=(0.002, 0.01), zeros_range=(6, 10))
    kw = {"scale": dict(source_format="int"), "original": dict(source_format="uint", with_zeros=True),
          "rescale": dict(source_format="uint", with_zeros=True, zeros_mode="rescale"),
          "folded": dict(source_format="uint", with_zeros=True, zeros_mode="folded"),
          "signed": dict(with_scaling=False)}[mode]
    Bdev = _dev(d["B"], cuda).view(torch.int8)
    if interleaved:
        if mode == "signed":
            pytest.skip("the sign-extending decoder is the plain-layout slow path")
        Bdev = quantize.interleave_weight(Bdev, 4, "float16")
    kern = tl.matmul_w4a16(M, N, K, group_size=group, fast_decoding=interleaved, **kw)
    args = [_dev(d["A"], cuda), Bdev]
    if kw.get("with_scaling", True):
        args.append(_dev(d["Scale"], cuda))
    if kw.get("with_zeros"):
        args.append(_dev(d["Zeros"], cuda))
    C = torch.empty((M, N), dtype=torch.float16, device=cuda)
    kern(*args, C)
    torch.cuda.synchronize()
    ref = orc.ref_w4a16(d["A"], d["B"], d["Scale"], d["Zeros"], group, mode)
    np.testing.assert_allclose(C.float().cpu().numpy(), ref.astype(np.float32), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("group", [32, 64, 256, 512, -1])
@pytest.mark.parametrize("mode", ["scale", "original"])
@pytest.mark.parametrize("M,N", [(3584, 3584), (1100, 3500), (300, 320)])  # direct-to-LDS 256 x 256, 128 x 256; staged
def test_w4a16_large_m_group_sizes_tile_exact_through_identity(cuda, group, mode, M, N):
    """Group sizes other than 128 through the GEMM: the direct-to-LDS kernel brings a dword of scales per row (two
    groups) per the tiles it serves (one tile of 64 k at group 32, on the 128 x 256 tile only; eight tiles at 256); one group per row (-1) and odd
    group counts stay on the register-staged kernel.  Identity rows for A: C[k, n] = W[n, k], every bit."""
    K = 1024
    g = K if group == -1 else group
    d = workloads.w4a16(1, N, K, g, seed=13 + g, scale_range=(0.002, 0.02), zeros_range=(6, 10))
    B, S, Z = d["B"], d["Scale"], d["Zeros"]
    B[1, :] = np.arange(K // 2, dtype=np.uint8)
    Z[3, :] = Z[3, :] - np.float16(0.25)
    kw = {"scale": dict(source_format="int"), "original": dict(source_format="uint", with_zeros=True)}[mode]
    W = orc.dequant_u4_scale(B, S, g) if mode == "scale" else orc.dequant_u4_scale_zeros(B, S, Z, g, mode)
    rows = min(M, K)
    A = np.zeros((M, K), dtype=np.float16)
    A[np.arange(rows), np.arange(rows)] = 1.0
    kern = tl.matmul_w4a16(M, N, K, group_size=g, **kw)
    args = [_dev(A, cuda), _dev(B, cuda).view(torch.int8), _dev(S, cuda)] + ([_dev(Z, cuda)] if kw.get("with_zeros") else [])
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=cuda)
    kern(*args, C)
    torch.cuda.synchronize()
    got = C.cpu().numpy()
    np.testing.assert_array_equal(got[:rows].view(np.uint16), np.ascontiguousarray(W.T[:rows]).view(np.uint16))
    assert not got[rows:].any()


@pytest.mark.parametrize("mode", ["scale", "original", "rescale", "folded"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("N", [300, 3584])  # register-staged tiles / the direct-to-LDS kernel
def test_w4a16_large_m_tile_exact_through_identity(cuda, mode, interleaved, N):
    """An identity for A makes the GEMM write its dequantised tile: C[k, n] = W[n, k], every bit, with scales that
    exercise the rounding (and fractional, negative zero points)."""
    K, group = 512, 128
    M = 3584 if N == 3584 else K
    d = workloads.w4a16(1, N, K, group, seed=11, scale_range=(0.002, 0.02), zeros_range=(6, 10))
    B, S, Z = d["B"], d["Scale"], d["Zeros"]
    B[1, :] = np.arange(K // 2, dtype=np.uint8)
    S[2, :] = np.array([6.1e-5, 1.0, -0.013, 655.0], dtype=np.float16)
    Z[3, :] = np.array([7.5, -3.25, 0.0, 15.0], dtype=np.float16)
    kw = {"scale": dict(source_format="int"), "original": dict(source_format="uint", with_zeros=True),
          "rescale": dict(source_format="uint", with_zeros=True, zeros_mode="rescale"),
          "folded": dict(source_format="uint", with_zeros=True, zeros_mode="folded")}[mode]
    W = orc.dequant_u4_scale(B, S, group) if mode == "scale" else orc.dequant_u4_scale_zeros(B, S, Z, group, mode)
    A = np.zeros((M, K), dtype=np.float16)
    A[np.arange(K), np.arange(K)] = 1.0
    Bdev = _dev(B, cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 4, "float16")
    kern = tl.matmul_w4a16(M, N, K, group_size=group, fast_decoding=interleaved, **kw)
    args = [_dev(A, cuda), Bdev, _dev(S, cuda)] + ([_dev(Z, cuda)] if kw.get("with_zeros") else [])
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device=cuda)
    kern(*args, C)
    torch.cuda.synchronize()
    got = C.cpu().numpy()
    np.testing.assert_array_equal(got[:K].view(np.uint16), np.ascontiguousarray(W.T).view(np.uint16))
    assert not got[K:].any()


@pytest.mark.parametrize("convention", ["unsigned", "offset", "twos"])
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (1, 256, 256), (130, 300, 384), (1500, 2000, 256), (1300, 4000, 256), (3590, 3580, 128),
                                   (3590, 3580, 768)])  # the last one: direct-to-LDS kernel
@pytest.mark.parametrize("interleaved", [True, False])
def test_bitnet_gemm_int32_exact(cuda, convention, M, N, K, interleaved):
    """tilelang_bitnet_158_int8xint2_prefill.py:360-381 (256^3, B in {0,1}) generalised to all codes, exact;
    with the weights interleaved as the reference feeds them (fast_decoding) and plain."""
    rng = np.random.default_rng(M + K)
    A = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    C = torch.zeros((M, N), dtype=torch.int32, device=cuda)
    Bdev = _dev(B, cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 2, "int8")
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention=convention)(_dev(A, cuda), Bdev, C)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy(), orc.ref_bitnet_int(A, B, convention))


@pytest.mark.parametrize("M", [256, 1])
def test_bitnet_reference_example_inputs(cuda, M):
    """The reference's own check, with its own call sequence (prefill.py:360-381 at 256^3, decode.py:237-258 at
    1x256x256): A in [0,4), B in {0,1}, general_compress then interleave_weight(qw, 2, int8), default arguments."""
    N = K = 256
    torch.manual_seed(42)
    A = torch.randint(0, 4, (M, K), dtype=torch.int8)
    W = torch.randint(0, 2, (N, K), dtype=torch.int8)
    qw = quantize.interleave_weight(quantize.general_compress(W, source_bits=2), 2, "int8")
    C = torch.zeros((M, N), dtype=torch.int32, device=cuda)
    factory = tl.bitnet_158_int8xint2_prefill if M > 1 else tl.bitnet_158_int8xint2_decode
    factory(M, N, K, "int8", "int32", "int32")(A.to(cuda), qw.to(cuda), C)
    torch.cuda.synchronize()
    ref = torch.matmul(A.float(), W.float().T).to(torch.int32)
    assert torch.equal(C.cpu(), ref)


@pytest.mark.parametrize("M", [1, 256, 2048])
def test_bitlinear_config5(cuda, M):
    """Benchmark configuration 5 at N=K=1024 (oracle-sized): ternary weights stored as w+2, per-row activation
    scale, per-tensor weight scale, fp16 out = (acc / s_a) / s_w."""
    N = K = 1024
    d = workloads.bitnet(M, N, K, seed=M)
    out = tl.bitlinear_int8xint2(M, N, K, float(d["s_w"]))(_dev(d["A"], cuda), _dev(d["B"], cuda).view(torch.int8), _dev(d["s_a"], cuda))
    Bil = quantize.interleave_weight(_dev(d["B"], cuda).view(torch.int8), 2, "int8")
    out_il = tl.bitlinear_int8xint2(M, N, K, float(d["s_w"]), interleaved=True)(_dev(d["A"], cuda), Bil, _dev(d["s_a"], cuda))
    torch.cuda.synchronize()
    ref = orc.ref_bitnet(d["A"], d["B"], d["s_a"], d["s_w"], "offset")
    np.testing.assert_allclose(out.float().cpu().numpy(), ref.astype(np.float32), rtol=RTOL, atol=ATOL)
    assert torch.equal(out, out_il)
    acc = torch.zeros((M, N), dtype=torch.int32, device=cuda)
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=False, convention="offset")(_dev(d["A"], cuda), _dev(d["B"], cuda).view(torch.int8), acc)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(acc.cpu().numpy(), d["A"].astype(np.int64) @ d["W"].astype(np.int64).T)


@pytest.mark.parametrize("M", [256, 1024, 2048])
@pytest.mark.parametrize("interleaved", [True, False])
def test_bitnet_full_size_exact(cuda, M, interleaved):
    """Configuration 5 at full size (M in {256, 2048}, and 1024 for the small-tile kernel in between; N = K = 8192), in the interleaved packing the benchmark
    feeds and in the plain one: EVERY int32 entry against the integer oracle.  |A . w| <= 127 * 8192 < 2^24 and so
    is every partial sum, hence an fp32 BLAS matmul on the host gives the exact integers; a sample of entries is
    recomputed in int64 to pin that, and the fused BitLinear epilogue runs on the same inputs."""
    N = K = 8192
    print(f"bitnet full size: M={M} N={N} K={K} interleaved={interleaved}", flush=True)
    d = workloads.bitnet(M, N, K, seed=M)
    Bdev = _dev(d["B"], cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 2, "int8")
    acc = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention="offset")(_dev(d["A"], cuda), Bdev, acc)
    out = tl.bitlinear_int8xint2(M, N, K, float(d["s_w"]), interleaved=interleaved)(_dev(d["A"], cuda), Bdev, _dev(d["s_a"], cuda))
    torch.cuda.synchronize()
    got = acc.cpu().numpy()
    ref32 = d["A"].astype(np.float32) @ d["W"].astype(np.float32).T
    ref = ref32.astype(np.int32)
    rows, cols = np.arange(0, M, 37), np.arange(0, N, 211)
    np.testing.assert_array_equal(ref[np.ix_(rows, cols)], d["A"][rows].astype(np.int64) @ d["W"][cols].astype(np.int64).T)
    np.testing.assert_array_equal(got, ref)
    np.testing.assert_allclose(out.float().cpu().numpy(), orc.post_quant_process(ref, d["s_a"].reshape(-1, 1), d["s_w"]).astype(np.float32),
                               rtol=RTOL, atol=ATOL)
    if M == 256:  # the benchmark's other row at this size: the same weights re-ordered offline into operand order
        Bfrag = quantize.prepack_i2_fragments(Bdev)
        acc_f = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
        tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention="offset", weight_fragments=True)(_dev(d["A"], cuda), Bfrag, acc_f)
        out_f = tl.bitlinear_int8xint2(M, N, K, float(d["s_w"]), interleaved=interleaved, weight_fragments=True)(_dev(d["A"], cuda), Bfrag, _dev(d["s_a"], cuda))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(acc_f.cpu().numpy(), ref)
        assert torch.equal(out_f.view(torch.int16), out.view(torch.int16))


@pytest.mark.parametrize("convention", ["unsigned", "offset", "twos"])
@pytest.mark.parametrize("M,N,K", [(1, 256, 256), (1, 1000, 8192), (2, 130, 4096), (3, 64, 2048), (4, 4096, 8192), (1, 96, 16384), (2, 40, 16384)])
@pytest.mark.parametrize("interleaved", [True, False])
def test_bitnet_decode_gemv_exact(cuda, convention, M, N, K, interleaved):
    """tilelang_bitnet_158_int8xint2_decode.py:237-258 (1x256x256) generalised: all codes, int8 range, exact."""
    rng = np.random.default_rng(M * 7 + K)
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    Bdev = _dev(B, cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 2, "int8")
    tl.bitnet_158_int8xint2_decode(M, N, K, fast_decoding=interleaved, convention=convention)(_dev(A, cuda), Bdev, C)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy(), orc.ref_bitnet_int(A, B, convention))


def test_bitnet_decode_full_size(cuda):
    """Configuration 5, M=1, N=K=8192: exact against the integer oracle, plus the fp16 BitLinear epilogue."""
    M, N, K = 1, 8192, 8192
    d = workloads.bitnet(M, N, K, seed=1)
    C = torch.zeros((M, N), dtype=torch.int32, device=cuda)
    tl.bitnet_158_int8xint2_decode(M, N, K, fast_decoding=False, convention="offset")(_dev(d["A"], cuda), _dev(d["B"], cuda).view(torch.int8), C)
    out = tl.bitlinear_int8xint2(M, N, K, float(d["s_w"]))(_dev(d["A"], cuda), _dev(d["B"], cuda).view(torch.int8), _dev(d["s_a"], cuda))
    torch.cuda.synchronize()
    ref = d["A"].astype(np.int64) @ d["W"].astype(np.int64).T
    np.testing.assert_array_equal(C.cpu().numpy(), ref)
    np.testing.assert_allclose(out.float().cpu().numpy(), orc.post_quant_process(ref, d["s_a"].reshape(-1, 1), d["s_w"]).astype(np.float32),
                               rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("convention", ["unsigned", "offset", "twos"])
@pytest.mark.parametrize("M,N,K", [(64, 128, 4096), (130, 300, 4096), (256, 384, 8192), (70, 1001, 12288), (1, 8, 4096),
                                   # an odd number of block pairs per wave: one, three, seven
                                   (64, 130, 2048), (100, 257, 6144), (33, 128, 14336)])
@pytest.mark.parametrize("interleaved", [True, False])
def test_bitnet_k_sliced_kernel_exact(cuda, convention, M, N, K, interleaved):
    """The kernel that slices K over the waves of a workgroup (the library's choice at a few hundred rows), named
    explicitly so that small and ragged shapes reach it: every int32 entry against the integer oracle, all codes,
    the int8 range of A including -128, and the fused BitLinear epilogue against the tiled kernel's bits."""
    rng = np.random.default_rng(M + K)
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    s_a = torch.tensor(rng.uniform(0.5, 3.0, size=M).astype(np.float32), device=cuda)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    Bdev = _dev(B, cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 2, "int8")
    print(f"bitnet k-sliced: M={M} N={N} K={K} {convention} interleaved={interleaved}", flush=True)
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention=convention, kernel="ksliced")(_dev(A, cuda), Bdev, C)
    out = tl.bitlinear_int8xint2(M, N, K, 1.7, convention=convention, interleaved=interleaved, kernel="ksliced")(_dev(A, cuda), Bdev, s_a)
    out_tiled = tl.bitlinear_int8xint2(M, N, K, 1.7, convention=convention, interleaved=interleaved, kernel="tiled")(_dev(A, cuda), Bdev, s_a)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy(), orc.ref_bitnet_int(A, B, convention))
    assert torch.equal(out.view(torch.int16), out_tiled.view(torch.int16))


@pytest.mark.parametrize("convention", ["unsigned", "offset", "twos"])
@pytest.mark.parametrize("M,N,K", [(64, 128, 4096), (130, 300, 4096), (256, 384, 8192), (70, 1001, 12288), (90, 200, 6144),
                                   # decode kernel on fragments: one to four rows, one to eight blocks per wave, ragged N
                                   (1, 128, 4096), (1, 1001, 8192), (2, 300, 16384), (3, 77, 8192), (4, 4100, 8192), (1, 40, 32768),
                                   # direct-to-LDS tiled kernel on fragments: 256 x 256 and 128 x 256 tiles, ragged edges
                                   (3590, 3580, 4096), (1300, 4000, 4096)])
@pytest.mark.parametrize("interleaved", [True, False])
def test_bitnet_fragment_ordered_weights_exact(cuda, convention, M, N, K, interleaved):
    """Weights re-ordered offline into the matrix instruction's operand order (``prepack_i2_fragments``; N ragged, so
    the last block of 32 rows is padded) through whichever kernel the library picks for the shape (decode kernel,
    K-sliced kernel, direct-to-LDS tiled kernel): every int32 entry against the integer oracle, and the fused
    BitLinear epilogue against the bits of the row-major path."""
    rng = np.random.default_rng(M + K + 1)
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    s_a = torch.tensor(rng.uniform(0.5, 3.0, size=M).astype(np.float32), device=cuda)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    Bdev = _dev(B, cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 2, "int8")
    Bfrag = quantize.prepack_i2_fragments(Bdev)
    assert Bfrag.shape == ((N + 31) // 32, K // 128, 64, 16)
    assert torch.equal(quantize.unpack_i2_fragments(Bfrag, N), Bdev)
    print(f"bitnet fragments: M={M} N={N} K={K} {convention} interleaved={interleaved}", flush=True)
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention=convention, weight_fragments=True)(_dev(A, cuda), Bfrag, C)
    out = tl.bitlinear_int8xint2(M, N, K, 1.7, convention=convention, interleaved=interleaved, weight_fragments=True)(_dev(A, cuda), Bfrag, s_a)
    out_rows = tl.bitlinear_int8xint2(M, N, K, 1.7, convention=convention, interleaved=interleaved)(_dev(A, cuda), Bdev, s_a)
    torch.cuda.synchronize()
    # every product is at most 128 * 3 and every partial sum below 2^53 (2^24 when K * 384 < 2^24): a BLAS product in
    # floating point is exact, whatever its summation order, and far faster than an int64 one
    ft = np.float32 if K * 384 < (1 << 24) else np.float64
    ref = (A.astype(ft) @ orc.decode_i2(B, convention).astype(ft).T).astype(np.int64)
    rows, cols = np.arange(0, M, max(1, M // 7)), np.arange(0, N, max(1, N // 11))
    np.testing.assert_array_equal(ref[np.ix_(rows, cols)], A[rows].astype(np.int64) @ orc.decode_i2(B[cols], convention).astype(np.int64).T)
    np.testing.assert_array_equal(C.cpu().numpy().astype(np.int64), ref)
    assert torch.equal(out.view(torch.int16), out_rows.view(torch.int16))


def test_bitnet_fragment_ordered_weights_where_no_kernel_reads_them(cuda):
    """Through the C-ABI: a K that neither the K-sliced nor (for want of tiles) the tiled kernel takes, and the tiled
    kernel named on a problem with too few tiles for it."""
    lib = tl._lib.get_library()
    A = torch.zeros((200, 4096), dtype=torch.int8, device=cuda)
    B = torch.zeros((4, 32, 64, 16), dtype=torch.int8, device=cuda)
    C = torch.zeros((200, 128), dtype=torch.int32, device=cuda)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.call_gemm_int8xint2(A.data_ptr(), B.data_ptr(), C.data_ptr(), 200, 128, 1024, 1, 2, None, 1.0, 0, stream) == -1
    assert "no kernel takes" in tl._lib.last_error()
    assert lib.call_gemm_int8xint2(A.data_ptr(), B.data_ptr(), C.data_ptr(), 64, 128, 4096, 1, 2, None, 1.0, 32, stream) == -1
    assert "the tiled kernel reads fragment-ordered weights from" in tl._lib.last_error()


@pytest.mark.parametrize("convention", ["unsigned", "offset", "twos"])
@pytest.mark.parametrize("M,N,K", [(5, 128, 4096), (32, 300, 8192), (17, 1001, 2048), (8, 33, 256), (31, 64, 1280), (16, 4100, 6912),
                                   (1, 8, 512), (24, 9000, 2560), (32, 8300, 6144),
                                   # three and four blocks of 32 weight rows per workgroup: both sets of weight registers
                                   (9, 20000, 1024), (32, 28677, 8192),
                                   # more than 32 activation rows on a matrix of few rows: passes of 32
                                   (64, 300, 4096), (100, 1001, 2048), (128, 2560, 1280), (33, 5000, 512),
                                   # up to 16 rows: blocks of 16 weight rows, four sets of weight registers in turn
                                   (16, 28677, 8192), (3, 9000, 2560), (12, 16 * 256 * 6 + 5, 512), (16, 16 * 256 * 4, 1024),
                                   # the same form on small and ragged matrices (K >= 4096 at any N): fewer blocks than CUs, one or two per workgroup
                                   (16, 100, 4352), (7, 1000, 5120), (16, 4097, 7936), (12, 33, 8192), (9, 2048, 6144),
                                   # K beyond what the registers hold: chunks of K, running sums in LDS
                                   (8, 300, 11008), (32, 1001, 16384), (5, 9000, 28672), (17, 64, 8448), (64, 200, 12288)])
@pytest.mark.parametrize("interleaved", [True, False])
def test_bitnet_register_resident_kernel_exact(cuda, convention, M, N, K, interleaved):
    """The small-batch kernel that keeps the activations in registers (the library's choice from 5 to 32 rows up to
    K = 8192), named explicitly so that one row and ragged shapes reach it: K slices of unequal length over the eight
    waves (K = 1280: five pairs of 128-k blocks for eight waves; 256: one), every int32 entry against the
    integer oracle, all codes, the int8 range of A including -128; the fused BitLinear epilogue against the tiled
    kernel's bits; fragment-ordered weights where the factory takes them."""
    rng = np.random.default_rng(M + K + 2)
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    s_a = torch.tensor(rng.uniform(0.5, 3.0, size=M).astype(np.float32), device=cuda)
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    Bdev = _dev(B, cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 2, "int8")
    print(f"bitnet register-resident: M={M} N={N} K={K} {convention} interleaved={interleaved}", flush=True)
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention=convention, kernel="resident")(_dev(A, cuda), Bdev, C)
    out = tl.bitlinear_int8xint2(M, N, K, 1.7, convention=convention, interleaved=interleaved, kernel="resident")(_dev(A, cuda), Bdev, s_a)
    out_tiled = tl.bitlinear_int8xint2(M, N, K, 1.7, convention=convention, interleaved=interleaved, kernel="tiled")(_dev(A, cuda), Bdev, s_a)
    torch.cuda.synchronize()
    ft = np.float32 if K * 384 < (1 << 24) else np.float64  # exact in floating point, see the fragment test above
    ref = (A.astype(ft) @ orc.decode_i2(B, convention).astype(ft).T).astype(np.int64)
    rows, cols = np.arange(0, M, max(1, M // 5)), np.arange(0, N, max(1, N // 11))
    np.testing.assert_array_equal(ref[np.ix_(rows, cols)], A[rows].astype(np.int64) @ orc.decode_i2(B[cols], convention).astype(np.int64).T)
    np.testing.assert_array_equal(C.cpu().numpy().astype(np.int64), ref)
    assert torch.equal(out.view(torch.int16), out_tiled.view(torch.int16))
    if K % 2048 == 0:
        Bfrag = quantize.prepack_i2_fragments(Bdev)
        Cf = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
        tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention=convention, kernel="resident",
                                        weight_fragments=True)(_dev(A, cuda), Bfrag, Cf)
        out_f = tl.bitlinear_int8xint2(M, N, K, 1.7, convention=convention, interleaved=interleaved, kernel="resident",
                                       weight_fragments=True)(_dev(A, cuda), Bfrag, s_a)
        torch.cuda.synchronize()
        assert torch.equal(Cf, C)
        assert torch.equal(out_f.view(torch.int16), out.view(torch.int16))


def test_bitnet_register_resident_kernel_refuses_what_does_not_fit_its_registers(cuda):
    A = torch.zeros((129, 16384), dtype=torch.int8, device=cuda)
    B = torch.zeros((128, 4096), dtype=torch.int8, device=cuda)
    C = torch.zeros((129, 128), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="register-resident kernel needs"):
        tl.bitnet_158_int8xint2_prefill(129, 128, 4096, convention="offset", kernel="resident")(A[:, :4096].contiguous(), B[:, :1024].contiguous(), C)
    with pytest.raises(RuntimeError, match="register-resident kernel needs"):  # K % 256
        tl.bitnet_158_int8xint2_prefill(32, 128, 8320, convention="offset", kernel="resident")(
            A[:32, :8320].contiguous(), B[:, :2080].contiguous(), C[:32].contiguous())
    # 64 rows against 28672 weight rows: 1792 workgroup-blocks, far beyond two rounds
    A2 = torch.zeros((64, 256), dtype=torch.int8, device=cuda)
    B2 = torch.zeros((28672, 64), dtype=torch.int8, device=cuda)
    C2 = torch.zeros((64, 28672), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="register-resident kernel needs"):
        tl.bitnet_158_int8xint2_prefill(64, 28672, 256, convention="offset", kernel="resident")(A2, B2, C2)


def test_bitnet_k_sliced_kernel_refuses_what_it_cannot_slice(cuda):
    A = torch.zeros((64, 1024), dtype=torch.int8, device=cuda)
    B = torch.zeros((128, 256), dtype=torch.int8, device=cuda)
    C = torch.zeros((64, 128), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="K-sliced kernel needs"):
        tl.bitnet_158_int8xint2_prefill(64, 128, 1024, convention="offset", kernel="ksliced")(A, B, C)


@pytest.mark.parametrize("interleaved", [True, False])
def test_bitnet_default_dispatch_takes_the_k_sliced_kernel_on_ragged_shapes(cuda, interleaved):
    """165 tiles of 64 x 128 with K = 4096: the library's own choice is the K-sliced kernel; M and N are ragged and N is
    not a multiple of 8 (element-wise stores).  Every int32 entry against the oracle and the tiled kernel."""
    M, N, K = 300, 4100, 4096
    rng = np.random.default_rng(7)
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    Bdev = _dev(B, cuda).view(torch.int8)
    if interleaved:
        Bdev = quantize.interleave_weight(Bdev, 2, "int8")
    C = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    Ct = torch.full((M, N), -7, dtype=torch.int32, device=cuda)
    print(f"bitnet default dispatch: M={M} N={N} K={K} interleaved={interleaved}", flush=True)
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention="offset")(_dev(A, cuda), Bdev, C)
    tl.bitnet_158_int8xint2_prefill(M, N, K, fast_decoding=interleaved, convention="offset", kernel="tiled")(_dev(A, cuda), Bdev, Ct)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(C.cpu().numpy(), orc.ref_bitnet_int(A, B, "offset"))
    assert torch.equal(C, Ct)
