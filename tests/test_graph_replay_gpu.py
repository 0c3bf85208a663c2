"""HIP graph capture of the entry points: the library never allocates or synchronises and sets kernel attributes
only on a kernel's first (eager) launch, so its launches can be captured; every replay must reproduce the eager
result bit for bit."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from tilelang_amd import workloads

pytestmark = pytest.mark.gpu


def _dev(x, cuda):
    return torch.from_numpy(np.ascontiguousarray(x)).to(cuda)


def test_graph_replays_match_eager(cuda):
    M1, N1, K1 = 1, 2048, 4096
    d1 = workloads.w4a16(M1, N1, K1, 128, seed=1)
    gemv = tl.dequantize_gemv(M1, N1, K1, group_size=128, source_format="int", with_scaling=True)
    A1, B1, S1 = _dev(d1["A"], cuda), _dev(d1["B"], cuda).view(torch.int8), _dev(d1["Scale"], cuda)
    C1 = torch.empty((M1, N1), dtype=torch.float16, device=cuda)

    M2, N2, K2 = 16, 1024, 2048
    d2 = workloads.w4a16(M2, N2, K2, 128, seed=2, zeros_range=(6, 10))
    batch = tl.dequantize_gemv(M2, N2, K2, group_size=128, source_format="uint", with_scaling=True, with_zeros=True)
    A2, B2, S2, Z2 = _dev(d2["A"], cuda), _dev(d2["B"], cuda).view(torch.int8), _dev(d2["Scale"], cuda), _dev(d2["Zeros"], cuda)
    C2 = torch.empty((M2, N2), dtype=torch.float16, device=cuda)

    M3, N3, K3 = 256, 512, 512
    d3 = workloads.mxfp4(M3, N3, K3, seed=3, scale_bias=127)
    gemm = tl.matmul_bf16_mxfp4(M3, N3, K3, weight_format="e2m1", scale_bias=127)
    A3, B3, S3 = _dev(d3["A"], cuda).view(torch.bfloat16), _dev(d3["B"], cuda), _dev(d3["Scale"], cuda)
    bias = torch.empty((M3, N3), dtype=torch.bfloat16, device=cuda)

    M4, N4, K4 = 8, 512, 1024
    d4 = workloads.bitnet(M4, N4, K4, seed=4)
    quant = tl.bitnet_activation_quant(M4, K4)
    lin = tl.bitlinear_int8xint2(M4, N4, K4, float(d4["s_w"]))
    X4 = torch.randn((M4, K4), dtype=torch.float16, device=cuda)
    B4 = _dev(d4["B"], cuda).view(torch.int8)

    def run():
        gemv(A1, B1, S1, C1)
        batch(A2, B2, S2, Z2, C2)
        c3 = gemm(A3, B3, S3, bias)
        xq, sa = quant(X4)
        return c3, lin(xq, B4, sa)

    c3_e, o4_e = run()  # eager: first launches set the kernel attributes
    torch.cuda.synchronize()
    eager = [C1.clone(), C2.clone(), c3_e.clone(), o4_e.clone()]

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            c3_g, o4_g = run()
    for _ in range(3):
        C1.fill_(float("nan"))
        C2.fill_(float("nan"))
        c3_g.fill_(float("nan"))
        o4_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip([C1, C2, c3_g, o4_g], eager):
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_graph_replays_match_eager_batch_kernels(cuda):
    """The K-sliced batch kernel (a voting barrier and 159 KiB of dynamic LDS), the register-resident kernel on
    fragment-ordered weights, the unscaled bf16 x fp4 GEMM and the K-sliced BitNet GEMM under capture."""
    M1, N1, K1 = 40, 16 * 1400, 2048
    d1 = workloads.w4a16(M1, N1, K1, 128, seed=5, zeros_range=(6, 10))
    ks = tl.dequantize_gemv(M1, N1, K1, group_size=128, source_format="uint", with_scaling=True, with_zeros=True)
    A1, B1, S1, Z1 = _dev(d1["A"], cuda), _dev(d1["B"], cuda).view(torch.int8), _dev(d1["Scale"], cuda), _dev(d1["Zeros"], cuda)
    C1 = torch.empty((M1, N1), dtype=torch.float16, device=cuda)

    M2, N2, K2 = 4, 1024, 4096
    d2 = workloads.w4a16(M2, N2, K2, 128, seed=6)
    fr = tl.dequantize_gemv(M2, N2, K2, group_size=128, source_format="int", with_scaling=True, weight_fragments=True)
    A2, S2 = _dev(d2["A"], cuda), _dev(d2["Scale"], cuda)
    B2 = tl.quantize.prepack_w4_fragments(_dev(d2["B"], cuda).view(torch.int8))
    C2 = torch.empty((M2, N2), dtype=torch.float16, device=cuda)

    M3, N3, K3 = 256, 256, 256
    d3 = workloads.mxfp4(M3, N3, K3, seed=7, scale_bias=0)
    f4 = tl.matmul_bf16_fp4(M3, N3, K3, fast_dequant=False)
    A3, B3 = _dev(d3["A"], cuda).view(torch.bfloat16), _dev(d3["B"], cuda)

    # BitLinear at 64 tiles of 64 x 128 with a long K: the kernel that slices K over the waves (128 KiB of LDS, loads
    # counted by hand)
    M5, N5, K5 = 64, 8192, 4096
    d5 = workloads.bitnet(M5, N5, K5, seed=8)
    bl = tl.bitlinear_int8xint2(M5, N5, K5, float(d5["s_w"]))
    A5, B5, sa5 = _dev(d5["A"], cuda), _dev(d5["B"], cuda).view(torch.int8), _dev(d5["s_a"], cuda)

    def run():
        ks(A1, B1, S1, Z1, C1)
        fr(A2, B2, S2, C2)
        return f4(A3, B3), bl(A5, B5, sa5)

    c3_e, c5_e = run()
    torch.cuda.synchronize()
    eager = [C1.clone(), C2.clone(), c3_e.clone(), c5_e.clone()]
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            c3_g, c5_g = run()
    for _ in range(3):
        for t in (C1, C2, c3_g, c5_g):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip([C1, C2, c3_g, c5_g], eager):
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_graph_replays_match_eager_decode_and_half_tile_kernels(cuda):
    """The integer decode GEMVs (4-bit and 1-bit weights; 2-bit weights in fragment order, whose kernel stages the
    activations in LDS), the streaming batch kernel with the folded zero point, the direct-to-LDS GEMM on its
    half-height tile (MXFP4) and on fragment-ordered BitNet weights, under capture."""
    from tilelang_amd import quantize

    rng = np.random.default_rng(21)
    M1, N1, K1 = 2, 1000, 4096
    A1 = _dev(rng.integers(-128, 128, size=(M1, K1), dtype=np.int8), cuda)
    B1 = _dev(rng.integers(0, 256, size=(N1, K1 // 2), dtype=np.uint8), cuda).view(torch.int8)
    g4 = tl.dequantize_gemv(M1, N1, K1, "int8", "int32", "int32", num_bits=4, source_format="int")
    C1 = torch.empty((M1, N1), dtype=torch.int32, device=cuda)
    B1b = _dev(rng.integers(0, 256, size=(N1, K1 // 8), dtype=np.uint8), cuda).view(torch.int8)
    g1 = tl.dequantize_gemv(M1, N1, K1, "int8", "int32", "int32", num_bits=1, source_format="int", fast_decoding=True)
    C1b = torch.empty((M1, N1), dtype=torch.int32, device=cuda)

    M2, N2, K2 = 2, 1001, 8192
    A2 = _dev(rng.integers(-128, 128, size=(M2, K2), dtype=np.int8), cuda)
    B2 = quantize.prepack_i2_fragments(_dev(rng.integers(0, 256, size=(N2, K2 // 4), dtype=np.uint8), cuda).view(torch.int8))
    gf = tl.bitnet_158_int8xint2_prefill(M2, N2, K2, fast_decoding=False, convention="offset", weight_fragments=True)
    C2 = torch.empty((M2, N2), dtype=torch.int32, device=cuda)

    M3, N3, K3 = 64, 300, 1536
    d3 = workloads.w4a16(M3, N3, K3, 128, seed=9, zeros_range=(6, 10))
    st = tl.dequantize_gemv(M3, N3, K3, group_size=128, source_format="uint", with_scaling=True, with_zeros=True)
    A3, B3, S3, Z3 = _dev(d3["A"], cuda), _dev(d3["B"], cuda).view(torch.int8), _dev(d3["Scale"], cuda), _dev(d3["Zeros"], cuda)
    C3 = torch.empty((M3, N3), dtype=torch.float16, device=cuda)

    M4, N4, K4 = 1500, 2000, 256  # 96 tiles of 128 x 256
    d4 = workloads.mxfp4(M4, N4, K4, seed=10, scale_bias=127)
    mx = tl.matmul_bf16_mxfp4(M4, N4, K4, weight_format="e2m1", scale_bias=127)
    A4, B4, S4 = _dev(d4["A"], cuda).view(torch.bfloat16), _dev(d4["B"], cuda), _dev(d4["Scale"], cuda)
    bias = torch.empty((M4, N4), dtype=torch.bfloat16, device=cuda)

    M5, N5, K5 = 1300, 4000, 4096  # 176 tiles of 128 x 256, fragment-ordered weights
    A5 = _dev(rng.integers(-128, 128, size=(M5, K5), dtype=np.int8), cuda)
    B5 = quantize.prepack_i2_fragments(_dev(rng.integers(0, 256, size=(N5, K5 // 4), dtype=np.uint8), cuda).view(torch.int8))
    tf = tl.bitnet_158_int8xint2_prefill(M5, N5, K5, fast_decoding=True, convention="offset", weight_fragments=True)
    C5 = torch.empty((M5, N5), dtype=torch.int32, device=cuda)

    def run():
        g4(A1, B1, C1)
        g1(A1, B1b, C1b)
        gf(A2, B2, C2)
        st(A3, B3, S3, Z3, C3)
        tf(A5, B5, C5)
        return mx(A4, B4, S4, bias)

    c4_e = run()
    torch.cuda.synchronize()
    outs = [C1, C1b, C2, C3, C5]
    eager = [t.clone() for t in outs] + [c4_e.clone()]
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            c4_g = run()
    for _ in range(3):
        for t in outs:
            t.fill_(-7)
        c4_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs + [c4_g], eager):
            assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))


def test_graph_replays_match_eager_mxfp4_decode_kernels(cuda):
    """The MXFP4 dot-product kernels (one row; two rows with the activations in LDS; K beyond 8192 in chunks), the
    register-resident MXFP4 kernel at 16 rows and the 16-row BitNet form on a small matrix, under capture."""
    cases = [(1, 1001, 4096), (2, 515, 8192), (1, 300, 16384), (2, 130, 12288), (16, 1000, 8192)]
    runs = []
    for i, (M, N, K) in enumerate(cases):
        d = workloads.mxfp4(M, N, K, seed=30 + i, scale_bias=127)
        kern = tl.matmul_bf16_mxfp4(M, N, K, weight_format="e2m1", scale_bias=127)
        A, B, S = _dev(d["A"], cuda).view(torch.bfloat16), _dev(d["B"], cuda), _dev(d["Scale"], cuda)
        bias = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
        runs.append((kern, (A, B, S, bias)))
    M5, N5, K5 = 16, 1000, 4096
    d5 = workloads.bitnet(M5, N5, K5, seed=40)
    bl = tl.bitlinear_int8xint2(M5, N5, K5, float(d5["s_w"]))
    A5, B5, sa5 = _dev(d5["A"], cuda), _dev(d5["B"], cuda).view(torch.int8), _dev(d5["s_a"], cuda)

    def run():
        return [k(*a) for k, a in runs] + [bl(A5, B5, sa5)]

    eager = [t.clone() for t in run()]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            outs = run()
    for _ in range(3):
        for t in outs:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
