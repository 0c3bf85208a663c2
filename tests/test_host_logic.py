"""Host-side logic that needs no GPU: the C-ABI library loads and exports what include/dqgemm.h declares,
the adapter validates arguments like the reference's wrapper, the packing helpers agree with the oracle."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from tilelang_amd import _lib, quantize, workloads
from tilelang_amd.adapter import KernelAdapter, KernelParam
from oracle import dq_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dqgemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"^\s*(?:int|size_t|const char\*)\s+(\w+)\s*\(", text, flags=re.M)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load_library()
    names = _declared_symbols()
    assert "init" in names and "get_last_error" in names and len(names) >= 4
    for n in names:
        assert getattr(lib, n) is not None
    # every declared entry point has a bound signature, and nothing undeclared is bound
    assert sorted(set(_lib.SIGNATURES) | set(_lib.SIZE_QUERIES) | {"get_last_error"}) == names
    assert lib.get_last_error().decode() == "" or isinstance(lib.get_last_error(), bytes)


def test_w4a16_workspace_query():
    """How much room the small-batch kernel asks for to cut K over workgroups: nothing where the rows alone fill the
    chip, where there is one row or K is short; otherwise a whole number of [M, N] fp32 slices, at most 16."""
    q = _lib.load_library().dq_w4a16_workspace_bytes
    assert q(16, 28672, 8192, 128, 5) == 0          # 448 workgroups of 64 rows
    assert q(1, 4096, 14336, 128, 5) == 0           # the GEMV takes one row
    assert q(16, 1536, 1024, 128, 5) == 0           # four steps of 256 k: nothing to cut
    assert q(3, 1023, 8192, 128, 5) == 0            # M * N not a multiple of four: the slices' rows would be misaligned
    assert q(2048, 4096, 14336, 128, 5) == 0        # the tiled GEMM's
    for (M, N, K, group, mode) in ((4, 4096, 14336, 128, 5), (64, 4096, 11008, 128, 5), (256, 4096, 14336, 128, 5),
                                   (32, 512, 8192, 32, 3), (16, 1024, 4096, 4096, 5), (24, 1024, 6144, 128, 0)):
        nbytes = q(M, N, K, group, mode)
        assert nbytes > 0 and nbytes % (M * N * 4) == 0 and 2 <= nbytes // (M * N * 4) <= 16
        assert K // 256 // (nbytes // (M * N * 4)) >= 4  # every slice at least 1024 k long


def test_entry_points_reject_bad_arguments_before_any_launch():
    """NULL pointers and impossible sizes return -1 with a message; no GPU is touched."""
    lib = _lib.load_library()
    vp = ctypes.c_void_p
    assert lib.call_dequantize_gemv_w4a16(vp(0), vp(0), vp(0), vp(0), vp(0), 1, 64, 256, 128, 3, 0, -1, vp(0)) == -1
    assert "non-NULL data pointer" in lib.get_last_error().decode()
    buf = ctypes.create_string_buffer(4096 + 64)
    a = vp((ctypes.addressof(buf) + 63) & ~63)
    assert lib.call_dequantize_gemv_w4a16(a, a, a, vp(0), a, 1, 64, 200, 128, 3, 0, -1, vp(0)) == -1
    assert "multiple" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_w4a16(a, a, a, vp(0), a, 1, 64, 384, 96, 3, 0, -1, vp(0)) == -1
    assert "group" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_w4a16(a, a, vp(0), vp(0), a, 1, 64, 256, 128, 3, 0, -1, vp(0)) == -1
    assert "Scale is expected to have non-NULL" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_w4a16(a, a, a, vp(0), a, 1, 64, 256, 128, 99, 0, -1, vp(0)) == -1
    assert "unknown mode" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_w4a16(vp(a.value + 2), a, a, vp(0), a, 1, 64, 256, 128, 3, 0, -1, vp(0)) == -1
    assert "aligned" in lib.get_last_error().decode()
    assert lib.call_dequant_gemm_bf16_mxfp4(a, a, a, vp(0), a, 64, 64, 100, 32, 0, 127, vp(0)) == -1
    assert "multiple of 64" in lib.get_last_error().decode()
    assert lib.call_dequant_gemm_bf16_mxfp4(a, a, a, vp(0), a, 64, 64, 128, 16, 0, 127, vp(0)) == -1
    assert "scale_size" in lib.get_last_error().decode()
    assert lib.call_gemm_int8xint2(a, a, a, 8, 64, 256, 0, 7, vp(0), 1.0, 0, vp(0)) == -1
    assert "unknown weight layout" in lib.get_last_error().decode()
    assert lib.call_gemm_int8xint2(a, a, a, 8, 64, 256, 5, 0, vp(0), 1.0, 0, vp(0)) == -1
    assert "unknown code convention" in lib.get_last_error().decode()
    assert lib.call_bitnet_activation_quant(a, a, vp(0), 4, 256, vp(0)) == -1
    assert "S is expected to have non-NULL" in lib.get_last_error().decode()
    assert lib.call_bitnet_activation_quant(a, a, a, 4, 100, vp(0)) == -1
    assert "multiple of 8" in lib.get_last_error().decode()
    assert lib.call_quantize_bf16_mxfp4(a, vp(0), a, 4, 64, 127, vp(0)) == -1
    assert "B is expected to have non-NULL" in lib.get_last_error().decode()
    assert lib.call_quantize_bf16_mxfp4(a, a, a, 4, 48, 127, vp(0)) == -1
    assert "multiple of 32" in lib.get_last_error().decode()
    assert lib.call_quantize_bf16_mxfp4(a, a, a, 4, 64, 300, vp(0)) == -1
    assert "scale_bias" in lib.get_last_error().decode()
    assert lib.call_dequant_gemm_fp16_fp4_splitk(a, a, vp(0), a, 64, 64, 256, 2, 1, vp(0)) == -1
    assert "SplitC is expected to have non-NULL" in lib.get_last_error().decode()
    assert lib.call_dequant_gemm_fp16_fp4_splitk(a, a, a, a, 64, 64, 256, 3, 1, vp(0)) == -1
    assert "64 * split" in lib.get_last_error().decode()
    assert lib.call_dequant_gemm_fp16_fp4_splitk(a, a, a, a, 3, 5, 256, 2, 1, vp(0)) == -1
    assert "multiple of 8" in lib.get_last_error().decode()
    assert lib.call_gemm_mxfp4_mxfp4(a, a, vp(0), a, vp(0), a, 64, 64, 256, vp(0)) == -1
    assert "ScaleA is expected to have non-NULL" in lib.get_last_error().decode()
    assert lib.call_gemm_mxfp4_mxfp4(a, a, a, a, vp(0), a, 64, 64, 320, vp(0)) == -1
    assert "multiple of 128" in lib.get_last_error().decode()
    assert lib.call_gemm_mxfp4_mxfp4(a, a, a, a, vp(0), a, 64, 64, 128, vp(0)) == -1
    assert "at least 256" in lib.get_last_error().decode()
    assert lib.call_gemm_mxfp4_mxfp4(a, a, a, vp(a.value + 2), vp(0), a, 64, 64, 256, vp(0)) == -1
    assert "4-byte aligned" in lib.get_last_error().decode()
    # low-bit GEMV: (A, B, Scale, Zeros, C, M, N, K, group, bits, convention, layout, zeros_rescale, stream)
    assert lib.call_dequantize_gemv_lowbit(a, a, vp(0), vp(0), a, 1, 64, 256, 256, 3, 0, 0, 0, vp(0)) == -1
    assert "bits must be 1 or 2" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_lowbit(a, vp(0), vp(0), vp(0), a, 1, 64, 256, 256, 2, 0, 0, 0, vp(0)) == -1
    assert "B is expected to have non-NULL" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_lowbit(a, a, vp(0), vp(0), a, 65, 64, 256, 256, 2, 0, 0, 0, vp(0)) == -1
    assert "decode batch" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_lowbit(a, a, vp(0), vp(0), a, 1, 64, 192, 192, 1, 0, 0, 0, vp(0)) == -1
    assert "multiple of 128" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_lowbit(a, a, a, vp(0), a, 1, 64, 256, 32, 2, 0, 0, 0, vp(0)) == -1
    assert "group" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_lowbit(a, a, vp(0), a, a, 1, 64, 256, 256, 2, 0, 0, 0, vp(0)) == -1
    assert "Zeros without Scale" in lib.get_last_error().decode()
    assert lib.call_dequantize_gemv_lowbit(a, a, vp(0), vp(0), a, 1, 64, 256, 256, 2, 4, 0, 0, vp(0)) == -1
    assert "unknown code convention" in lib.get_last_error().decode()


def test_bitlinear_weight_packing_matches_oracle():
    """BitLinear.load_float_weight: ternary codes w + 2, four per byte, interleaved for the fast decoder; decoding
    the packed buffer with the oracle gives back weight_quant(W) (utils_quant.py:149-154)."""
    import numpy as np
    from oracle import dq_oracle as orc
    from tilelang_amd import bitlinear

    rng = np.random.default_rng(3)
    W = (rng.standard_normal((48, 256), dtype=np.float32) * 0.05).astype(np.float32)
    wq_ref, sw_ref = orc.weight_quant(W)
    assert torch.equal(bitlinear.weight_quant(torch.from_numpy(W)), torch.from_numpy(wq_ref))
    for interleave in (False, True):
        layer = bitlinear.BitLinear(256, 48, interleave=interleave)
        layer.load_float_weight(torch.from_numpy(W))
        packed = layer.qweight.numpy().view(np.uint8)
        if interleave:
            words = np.ascontiguousarray(packed).view(np.uint32)
            dec = orc.fast_decode_i2_to_i8(words, signed=True).reshape(48, 256)
        else:
            dec = orc.decode_i2(packed, "offset")
        np.testing.assert_array_equal(dec, wq_ref)
        assert abs(float(layer.sw) - float(sw_ref)) <= 1e-6 * float(sw_ref)


# ---- adapter ----------------------------------------------------------------------------------------

def _cpu_adapter(result_idx=()):
    calls = []

    def launch(ptrs, stream):
        calls.append(([p.value for p in ptrs], stream))
        return 0

    params = [KernelParam("A", torch.float16, (2, 8)), KernelParam("B", torch.int8, (4, 4), packed=True),
              KernelParam("C", torch.float16, (2, 4))]
    return KernelAdapter("k", params, list(result_idx), launch, lambda: "boom", device_type="cpu"), calls


def test_adapter_passes_pointers_and_stream():
    k, calls = _cpu_adapter()
    A, B, C = torch.zeros(2, 8, dtype=torch.float16), torch.zeros(4, 4, dtype=torch.uint8), torch.zeros(2, 4, dtype=torch.float16)
    assert k(A, B, C) is None
    assert calls[0][0] == [A.data_ptr(), B.data_ptr(), C.data_ptr()] and calls[0][1] == 0
    k(A, B, C, stream=1234)
    assert calls[1][1] == 1234
    k(A, None, C)
    assert calls[2][0][1] is None or calls[2][0][1] == 0


def test_adapter_out_idx_allocates_outputs():
    k, calls = _cpu_adapter(result_idx=[-1])
    A, B = torch.zeros(2, 8, dtype=torch.float16), torch.zeros(4, 4, dtype=torch.int8)
    C = k(A, B)
    assert C.shape == (2, 4) and C.dtype == torch.float16 and calls[0][0][2] == C.data_ptr()


@pytest.mark.parametrize("case,match", [
    ("count", r"Expected 3 inputs, got 2 with 2 inputs and 0 outputs"),
    ("dtype", r"Buffer dtype mismatch for parameter A: expected torch.float16, got torch.float32"),
    ("ndim", r"Static shape mismatch for parameter A: expected 2 dimensions, got 1"),
    ("shape", r"Static shape mismatch for parameter A: expected 8 at index 1, got 16"),
    ("stride", r"Static stride mismatch for parameter C"),
    ("device", r"Buffer device mismatch for parameter A"),
])
def test_adapter_validation_errors(case, match):
    """Same classes as the reference wrapper (tilelang/jit/adapter/cython/cython_wrapper.pyx:78-156,172-175)."""
    k, calls = _cpu_adapter()
    A, B, C = torch.zeros(2, 8, dtype=torch.float16), torch.zeros(4, 4, dtype=torch.int8), torch.zeros(2, 4, dtype=torch.float16)
    with pytest.raises(ValueError, match=match):
        if case == "count":
            k(A, B)
        elif case == "dtype":
            k(A.float(), B, C)
        elif case == "ndim":
            k(A.reshape(-1), B, C)
        elif case == "shape":
            k(torch.zeros(2, 16, dtype=torch.float16), B, C)
        elif case == "stride":
            k(A, B, torch.zeros(4, 2, dtype=torch.float16).t())
        elif case == "device":
            k(A.to("meta"), B, C)
    assert not calls
    if case != "count":
        # validation can be skipped like in the reference
        args = {"dtype": (A.float(), B, C), "ndim": (A.reshape(-1), B, C)}.get(case)
        if args:
            k(*args, skip_tensor_validation=True)
            assert len(calls) == 1


def test_adapter_error_code_raises_runtime_error():
    params = [KernelParam("A", torch.float16, (1, 8))]
    k = KernelAdapter("k", params, [], lambda ptrs, s: -1, lambda: "boom", device_type="cpu")
    with pytest.raises(RuntimeError, match="Kernel call failed: boom"):
        k(torch.zeros(1, 8, dtype=torch.float16))


def test_kernels_refuse_cpu_tensors_and_bad_factory_arguments():
    kern = tl.dequantize_gemv(1, 64, 256, group_size=128, source_format="int", with_scaling=True)
    A, B = torch.zeros(1, 256, dtype=torch.float16), torch.zeros(64, 128, dtype=torch.int8)
    S, C = torch.zeros(64, 2, dtype=torch.float16), torch.zeros(1, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="Buffer device mismatch for parameter A: expected cuda"):
        kern(A, B, S, C)
    with pytest.raises(ValueError, match="multiple of 128"):
        tl.dequantize_gemv(1, 64, 200)
    with pytest.raises(ValueError, match="group_size"):
        tl.dequantize_gemv(1, 64, 256, group_size=48, with_scaling=True)
    with pytest.raises(ValueError, match="multiple of 64"):
        tl.matmul_bf16_mxfp4(64, 64, 96)
    with pytest.raises(ValueError, match="multiple of 64"):
        tl.matmul_bf16_fp4(64, 64, 96)
    with pytest.raises(ValueError, match="must be bfloat16"):
        tl.matmul_bf16_fp4(64, 64, 64, in_dtype="float16")
    kern = tl.matmul_bf16_fp4(64, 32, 128)  # kernel(A, qB) -> C
    assert [p.name for p in kern.params] == ["A", "B", "C"] and kern.result_idx == [2]
    assert kern.params[1].shape == (32, 64)
    with pytest.raises(AssertionError):
        tl.dequantize_gemv(1, 64, 256, trans_A=True)
    with pytest.raises(ValueError, match="kernel must be None, 'ksliced', 'tiled' or 'resident'"):
        tl.bitnet_158_int8xint2_prefill(256, 8192, 8192, kernel="sliced")
    with pytest.raises(ValueError, match="kernel must be None, 'ksliced', 'tiled' or 'resident'"):
        tl.bitlinear_int8xint2(256, 8192, 8192, 1.0, kernel="both")


# ---- packing helpers against the oracle ---------------------------------------------------------------

@pytest.mark.parametrize("bits", [1, 2, 4])
def test_general_compress_matches_oracle(bits):
    rng = np.random.default_rng(bits)
    x = rng.integers(0, 1 << bits, size=(6, 64)).astype(np.int8)
    got = quantize.general_compress(torch.from_numpy(x), bits).numpy()
    np.testing.assert_array_equal(got, orc.general_compress(x, bits))
    assert got.dtype == np.int8


@pytest.mark.parametrize("nbits,target", [(4, "float16"), (2, "int8"), (2, "float16"), (1, "int8"), (1, "float16"), (4, "int8")])
def test_interleave_weight_matches_oracle(nbits, target):
    rng = np.random.default_rng(nbits)
    raw = rng.integers(-128, 128, size=(8, 32)).astype(np.int8)
    got = quantize.interleave_weight(torch.from_numpy(raw), nbits, target).numpy()
    np.testing.assert_array_equal(got, orc.interleave_weight(raw, nbits, target))
    assert got.dtype == np.int8 and got.shape == raw.shape


def test_pack_and_fp4_helpers_match_oracle():
    rng = np.random.default_rng(0)
    x = rng.integers(-8, 8, size=(4, 32)).astype(np.int8)
    np.testing.assert_array_equal(quantize.pack_int4(torch.from_numpy(x)).numpy(), orc.pack_int4(x))
    with pytest.raises(TypeError):
        quantize.pack_int4(torch.zeros(2, 4, dtype=torch.int32))
    with pytest.raises(ValueError):
        quantize.pack_int4(torch.zeros(2, 3, dtype=torch.int8))
    v = (rng.standard_normal((3, 64)) * 3).astype(np.float32)
    v[0, :8] = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25]  # the rounding thresholds
    codes = quantize.encode_fp4_e2m1_values(torch.from_numpy(v))
    np.testing.assert_array_equal(codes.numpy(), orc.encode_fp4_e2m1_values(v))
    packed = quantize.pack_fp4_e2m1_codes(codes)
    np.testing.assert_array_equal(packed.numpy().view(np.uint8), orc.pack_fp4_e2m1_codes(codes.numpy()))
    np.testing.assert_array_equal(quantize.decode_packed_fp4_e2m1(packed).numpy(), orc.decode_fp4_e2m1(packed.numpy()))
    values = torch.tensor([[0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.5, -1.0]])
    assert quantize.encode_fp4_e2m1_values(values).tolist() == [[0, 1, 2, 3, 4, 5, 6, 7, 9, 10]]


def test_workload_generators_are_seeded_and_shaped():
    a, b = workloads.w4a16(1, 64, 256, 128, seed=3), workloads.w4a16(1, 64, 256, 128, seed=3)
    for k in a:
        np.testing.assert_array_equal(a[k], b[k])
    assert a["B"].shape == (64, 128) and a["Scale"].shape == (64, 2) and a["Scale"].dtype == np.float16
    assert 0.005 <= a["Scale"].min() and a["Scale"].max() <= 0.02
    z = workloads.w4a16(4, 32, 256, 128, seed=1, zeros_range=(6, 10))["Zeros"]
    assert set(np.unique(z)).issubset({6, 7, 8, 9, 10})
    m = workloads.mxfp4(8, 16, 128, seed=0)
    assert m["Scale"].min() >= 119 and m["Scale"].max() <= 127 and m["A"].dtype == np.uint16
    bn = workloads.bitnet(2, 8, 64, seed=0)
    np.testing.assert_array_equal(orc.decode_i2(bn["B"], "offset"), bn["W"])
    # algorithmic byte counts of the benchmark configurations
    assert workloads.w4a16_bytes(1, 28672, 8192) == 121184256
    assert workloads.w4a16_bytes(64, 28672, 8192, zeros=True) == 129499136
    assert workloads.mxfp4_bytes(4096, 8192, 8192) == 169869312
    assert workloads.bitnet_bytes(2048, 8192, 8192) == 67117060
    assert workloads.flops(4096, 8192, 8192) == 549755813888


def test_lowbit_gemv_factory_rejections():
    """Shape and option checks of dequantize_gemv(num_bits=2 / 1) fire before any launch (no GPU needed)."""
    with pytest.raises(ValueError):
        tl.dequantize_gemv(1, 64, 1024, "float16", "float16", "float32", num_bits=2, with_scaling=True, with_zeros=True,
                           zeros_mode="quantized", group_size=128)
    with pytest.raises(ValueError):
        tl.dequantize_gemv(1, 64, 1024, "float16", "float16", "float32", num_bits=1, with_scaling=True, group_size=64)
    with pytest.raises(ValueError):
        tl.dequantize_gemv(1, 64, 1024, "float16", "float16", "float32", num_bits=2, with_scaling=True, group_size=32)
    with pytest.raises(ValueError):
        tl.dequantize_gemv(128, 64, 1024, "float16", "float16", "float32", num_bits=2)
    with pytest.raises(ValueError):
        tl.dequantize_gemv(1, 64, 1024, "float16", "float16", "float32", num_bits=3)
    with pytest.raises(ValueError):
        tl.dequantize_gemv(1, 64, 1024, "int8", "float16", "int32", num_bits=2)
    # int8 x int4 with fast_decoding is built (decode_i4{u,s}_to_i8s over interleave_weight(., 4, "int8") words)
    assert tl.dequantize_gemv(1, 64, 1024, "int8", "int32", "int32", num_bits=4, fast_decoding=True).name == "dequantize_gemv"
    with pytest.raises(ValueError, match="qzeros_format"):
        tl.dequantize_gemv(1, 64, 1024, with_scaling=True, with_zeros=True, zeros_mode="quantized", group_size=128,
                           qzeros_format="int3")
    k = tl.dequantize_gemv(1, 64, 1024, with_scaling=True, with_zeros=True, zeros_mode="quantized", group_size=128)
    assert [p.dtype for p in k.params if p.name == "Zeros"] == [torch.int16] and k.workspace_idx == [len(k.params) - 1]
    k = tl.dequantize_w4(64, 1024, 128, source_format="uint", with_zeros=True, zeros_mode="quantized", qzeros_format="packed4")
    assert [p.shape for p in k.params if p.name == "Zeros"] == [(64, 4)]
    with pytest.raises(ValueError):
        tl.dequantize_gemv(1, 64, 1024, "int8", "int32", "int32", num_bits=2, with_scaling=True, group_size=128)


def test_fragment_prepack_matches_the_oracle_and_inverts():
    """quantize.prepack_w4_fragments against the oracle's index formula, its inverse, and the factory's shape rules."""
    rng = np.random.default_rng(3)
    B = rng.integers(0, 256, size=(80, 192), dtype=np.uint8)  # N = 80, K = 384
    frag = quantize.prepack_w4_fragments(torch.from_numpy(B))
    assert frag.shape == (5, 3, 64, 16)
    np.testing.assert_array_equal(frag.numpy(), orc.prepack_w4_fragments(B))
    np.testing.assert_array_equal(quantize.unpack_w4_fragments(frag).numpy(), B)
    with pytest.raises(ValueError, match="N % 16 == 0"):
        quantize.prepack_w4_fragments(torch.zeros(24, 64, dtype=torch.uint8))
    kern = tl.dequantize_gemv(4, 64, 2048, group_size=128, source_format="int", with_scaling=True, weight_fragments=True)
    assert kern.params[1].shape == (4, 16, 64, 16)
    for bad in (dict(M=17), dict(K=1024), dict(group_size=64)):
        args = dict(M=4, N=64, K=2048, group_size=128)
        args.update(bad)
        with pytest.raises(ValueError, match="fragment-ordered weights"):
            tl.dequantize_gemv(args["M"], args["N"], args["K"], group_size=args["group_size"], source_format="int",
                               with_scaling=True, weight_fragments=True)



def test_i2_fragment_addresses_of_the_decode_and_tiled_kernels():
    """The byte offsets the decode kernel and the direct-to-LDS tiled kernel compute for fragment-ordered 2-bit
    weights (block (nb, kb) at ((nb * K/128) + kb) * 1024, lane 32 h + r at + 16 lane) against the prepack itself:
    lane (h, r) of block (nb, kb) must hold bytes 32 kb + 16 h .. + 15 of row 32 nb + r, for a ragged N."""
    from tilelang_amd import quantize

    N, K = 70, 1024
    rng = np.random.default_rng(3)
    B = torch.from_numpy(rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8))
    flat = quantize.prepack_i2_fragments(B).reshape(-1).numpy()
    KB, row_blocks = K // 128, (N + 31) // 32
    for nb in range(row_blocks):
        for kb in range(KB):
            for lane in range(64):
                h, r = lane >> 5, lane & 31
                off = (nb * KB + kb) * 1024 + lane * 16  # dq_gemv_int.hip: issue(); dq_gemm_core.h: b_voff + kb * 1024
                got = flat[off:off + 16]
                row = 32 * nb + r
                want = B[row, 32 * kb + 16 * h:32 * kb + 16 * h + 16].numpy() if row < N else np.zeros(16, np.uint8)
                assert np.array_equal(got, want), (nb, kb, lane)
    assert flat.size == row_blocks * KB * 1024


def test_i2_fragment_prepack_matches_the_oracle_and_inverts():
    """quantize.prepack_i2_fragments against the oracle's index formula (N ragged: the last block of 32 rows is padded
    with zeros), its inverse, and the factories' shape rules."""
    rng = np.random.default_rng(5)
    B = rng.integers(0, 256, size=(70, 96), dtype=np.uint8)  # N = 70, K = 384
    frag = quantize.prepack_i2_fragments(torch.from_numpy(B))
    assert frag.shape == (3, 3, 64, 16)
    np.testing.assert_array_equal(frag.numpy(), orc.prepack_i2_fragments(B))
    np.testing.assert_array_equal(quantize.unpack_i2_fragments(frag, 70).numpy(), B)
    assert quantize.unpack_i2_fragments(frag).shape == (96, 96)
    with pytest.raises(ValueError, match="K % 128 == 0"):
        quantize.prepack_i2_fragments(torch.zeros(32, 48, dtype=torch.uint8))
    with pytest.raises(ValueError, match="does not fit"):
        quantize.unpack_i2_fragments(frag, 64)
    kern = tl.bitnet_158_int8xint2_prefill(256, 1001, 8192, weight_fragments=True)
    assert kern.params[1].shape == (32, 64, 64, 16)
    assert tl.bitlinear_int8xint2(256, 128, 4096, 1.0, weight_fragments=True).params[1].shape == (4, 32, 64, 16)
    assert tl.bitnet_158_int8xint2_prefill(256, 128, 6144, weight_fragments=True).params[1].shape == (4, 48, 64, 16)
    with pytest.raises(ValueError, match="K % 2048 == 0"):
        tl.bitnet_158_int8xint2_prefill(256, 128, 1024, weight_fragments=True)
    # the tiled kernel may be named together with the flag: the library decides whether the problem has tiles enough
    assert tl.bitlinear_int8xint2(256, 128, 4096, 1.0, kernel="tiled", weight_fragments=True).params[1].shape == (4, 32, 64, 16)
