"""Plain GEMM (no dequantise step) on the MFMA tile the dequantize GEMMs share, through the C-ABI, against
``torch.matmul`` in fp32 on the host -- the check of testing/python/kernel/test_tilelang_kernel_gemm.py:51-104 at the
shapes of :107-260 and of testing/python/amd/test_tilelang_test_amd.py:112-157.  fp outputs rtol = atol = 1e-2 with
no allowance for mismatching elements; int8 -> int32 exact."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _run(cuda, M, N, K, trans_A, trans_B, in_dtype, out_dtype, seed=0):
    print(f"plain gemm M={M} N={N} K={K} trans_A={trans_A} trans_B={trans_B} {in_dtype}->{out_dtype}", flush=True)
    gen = torch.Generator().manual_seed(seed)
    it = getattr(torch, in_dtype)
    a_shape = (K, M) if trans_A else (M, K)
    b_shape = (N, K) if trans_B else (K, N)
    if it == torch.int8:
        A = torch.randint(-128, 128, a_shape, generator=gen, dtype=torch.int32).to(torch.int8)
        B = torch.randint(-128, 128, b_shape, generator=gen, dtype=torch.int32).to(torch.int8)
    else:
        A = torch.randn(a_shape, generator=gen).to(it)
        B = torch.randn(b_shape, generator=gen).to(it)
    kern = tl.matmul(M, N, K, 128, 128, 32, trans_A, trans_B, in_dtype, out_dtype, "int32" if it == torch.int8 else "float32")
    C = kern(A.to(cuda), B.to(cuda))
    torch.cuda.synchronize()
    assert C.shape == (M, N) and C.dtype == getattr(torch, out_dtype)
    a = A.T if trans_A else A      # [M, K]
    bt = B.T if trans_B else B     # [K, N]
    if it == torch.int8:
        # |sum| <= 128 * 128 * K < 2^24 for K <= 1024, and so is every partial sum: the fp32 BLAS matmul gives the
        # exact integers; a sample of rows is recomputed in int64 to pin that
        assert K <= 1024
        ref = torch.matmul(a.float(), bt.float()).to(torch.int32)
        rows = torch.arange(0, M, 61)
        assert torch.equal(ref[rows], (a[rows].to(torch.int64) @ bt.to(torch.int64)).to(torch.int32))
        assert torch.equal(C.cpu(), ref)
    else:
        ref = torch.matmul(a.float(), bt.float()).to(getattr(torch, out_dtype))
        np.testing.assert_allclose(C.float().cpu().numpy(), ref.float().numpy(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("trans_A,trans_B,in_dtype,out_dtype", [
    (False, False, "float16", "float16"),    # test_gemm_f16f16f16_nn
    (False, False, "float16", "float32"),    # test_gemm_f16f16f32_nn (fp32 accumulate; output kept in fp32 here)
    (False, False, "bfloat16", "bfloat16"),  # test_gemm_bf16bf16f32_nn
    (True, False, "float16", "float16"),     # test_gemm_f16f16f16_tn
    (False, True, "float16", "float16"),     # test_gemm_f16f16f16_nt
    (False, True, "int8", "int32"),          # test_gemm_i8i8i32_nt
    (True, False, "int8", "int32"),          # test_gemm_i8i8i32_tn
])
def test_reference_kernel_gemm_shapes(cuda, trans_A, trans_B, in_dtype, out_dtype):
    _run(cuda, 512, 1024, 768, trans_A, trans_B, in_dtype, out_dtype)


@pytest.mark.parametrize("trans_A,trans_B", [(False, False), (False, True), (True, True), (True, False)])
@pytest.mark.parametrize("in_dtype,out_dtype", [("float16", "float32"), ("bfloat16", "float32"), ("bfloat16", "bfloat16")])
def test_reference_amd_gemm_shapes(cuda, trans_A, trans_B, in_dtype, out_dtype):
    """testing/python/amd/test_tilelang_test_amd.py:112-157: 1024^3, every operand layout."""
    _run(cuda, 1024, 1024, 1024, trans_A, trans_B, in_dtype, out_dtype, seed=1)


@pytest.mark.parametrize("M,N,K,in_dtype,out_dtype", [
    (2048, 1536, 256, "float16", "float16"),   # 192 tiles of 128 x 128: the larger wave tile
    (2040, 1530, 128, "int8", "int32"),        # the same with ragged edges
    (100, 72, 64, "bfloat16", "float32"),      # one ragged tile, a single k-block
    (1, 8, 128, "float16", "float16"),
    (130, 257, 384, "int8", "int32"),
])
def test_tile_sizes_and_ragged_edges(cuda, M, N, K, in_dtype, out_dtype):
    _run(cuda, M, N, K, False, True, in_dtype, out_dtype, seed=2)
    _run(cuda, M, N, K, True, False, in_dtype, out_dtype, seed=3)


def test_identity_operand_pins_the_tile_layout(cuda):
    """A = I: C must equal B^T element for element (every A row, k index and output column lands where it should;
    a swapped fragment half or a mis-swizzled piece cannot cancel)."""
    M = K = 256
    N = 384
    B = torch.randn((N, K), generator=torch.Generator().manual_seed(4)).to(torch.float16)
    C = tl.matmul(M, N, K, trans_A=False, trans_B=True)(torch.eye(M, dtype=torch.float16, device=cuda), B.to(cuda))
    torch.cuda.synchronize()
    assert torch.equal(C.cpu(), B.T.contiguous())
    Bi = torch.randint(-128, 128, (N, K), generator=torch.Generator().manual_seed(5), dtype=torch.int32).to(torch.int8)
    Ci = tl.matmul(M, N, K, in_dtype="int8", out_dtype="int32")(torch.eye(M, dtype=torch.int8, device=cuda), Bi.to(cuda))
    torch.cuda.synchronize()
    assert torch.equal(Ci.cpu(), Bi.T.to(torch.int32).contiguous())


def test_bad_arguments(cuda):
    with pytest.raises(ValueError, match="does not go with"):
        tl.matmul(64, 64, 128, in_dtype="int8", out_dtype="float16")
    with pytest.raises(ValueError, match="multiple of 128"):
        tl.matmul(64, 64, 192, in_dtype="int8", out_dtype="int32")
    kern = tl.matmul(64, 64, 128)
    with pytest.raises(ValueError, match="Static shape mismatch"):
        kern(torch.zeros((64, 64), dtype=torch.float16, device=cuda), torch.zeros((64, 128), dtype=torch.float16, device=cuda))
