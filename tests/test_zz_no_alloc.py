"""The split-K entry point that allocates nothing (``call_dequant_gemm_fp16_fp4_splitk_static``) against the
entry point that takes the caller's partial-result buffer, through the C-ABI: same bits, on two calls in a row,
the second with a smaller input (the library's own scratch buffer then still holds the first call's partial
results), and a clear error when the partial results would not fit."""

import ctypes

import numpy as np
import pytest
import torch

from tilelang_amd import _lib
from oracle import dq_oracle as orc

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 16 << 20  # DQ_STATIC_SCRATCH_BYTES of include/dqgemm.h


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, cuda, M, N, K, split, transposed, seed):
    print(f"no-alloc split-K: M={M} N={N} K={K} split={split} transposed={transposed} seed={seed}", flush=True)
    rng = np.random.default_rng(seed)
    A = torch.from_numpy((rng.standard_normal((M, K), dtype=np.float32) * 0.5).astype(np.float16)).to(cuda)
    B = torch.from_numpy(rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)).to(cuda)
    shape = (N, M) if transposed else (M, N)
    parts = torch.empty((split,) + shape, dtype=torch.float16, device=cuda)
    want = torch.full(shape, float("nan"), dtype=torch.float16, device=cuda)
    got = torch.full(shape, float("nan"), dtype=torch.float16, device=cuda)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.call_dequant_gemm_fp16_fp4_splitk(_ptr(A), _ptr(B), _ptr(parts), _ptr(want), M, N, K, split, int(transposed), stream)
    assert rc == 0, lib.get_last_error().decode()
    # device-wide free memory, not torch's own counter: a hipMalloc inside the library would show here
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    rc = lib.call_dequant_gemm_fp16_fp4_splitk_static(_ptr(A), _ptr(B), _ptr(got), M, N, K, split, int(transposed), stream)
    assert rc == 0, lib.get_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.isfinite(got).all()
    assert torch.equal(got, want)


def test_static_scratch_matches_caller_buffer_twice(cuda):
    lib = _lib.get_library()
    # first call: 8 slices of 512 x 768 fill 6 MiB of the scratch buffer
    _both(lib, cuda, 512, 768, 2048, 8, False, seed=11)
    # second call, smaller and with another shape: stale partial results of the first call lie all around it
    _both(lib, cuda, 64, 128, 512, 4, False, seed=12)
    # ... and the smaller call is also right in absolute terms (small integers: every slice product is exact in fp16)
    rng = np.random.default_rng(13)
    Ai = rng.integers(-2, 3, size=(64, 512)).astype(np.float16)
    Bi = rng.integers(0, 256, size=(128, 256), dtype=np.uint8) & 0x33
    out = torch.empty((64, 128), dtype=torch.float16, device=cuda)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    Ad, Bd = torch.from_numpy(Ai).to(cuda), torch.from_numpy(Bi).to(cuda)
    rc = lib.call_dequant_gemm_fp16_fp4_splitk_static(_ptr(Ad), _ptr(Bd), _ptr(out), 64, 128, 512, 4, 0, stream)
    assert rc == 0, lib.get_last_error().decode()
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), orc.ref_fp16xfp4_splitk(Ai, Bi, 4))
    # transposed output, ragged tiles, then again a smaller one
    _both(lib, cuda, 300, 520, 768, 3, True, seed=14)
    _both(lib, cuda, 100, 72, 512, 2, True, seed=15)


def test_static_scratch_under_graph_capture(cuda):
    """The callers the entry point is for: captured into a graph after one eager call (an allocation during capture
    would raise), replayed several times with eager work and synchronisations in between, every replay bit-identical
    to the eager result."""
    lib = _lib.get_library()
    M, N, K, split = 256, 384, 1024, 4
    rng = np.random.default_rng(21)
    A = torch.from_numpy((rng.standard_normal((M, K), dtype=np.float32) * 0.5).astype(np.float16)).to(cuda)
    B = torch.from_numpy(rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)).to(cuda)
    eager = torch.full((M, N), float("nan"), dtype=torch.float16, device=cuda)
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device=cuda)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.call_dequant_gemm_fp16_fp4_splitk_static(_ptr(A), _ptr(B), _ptr(eager), M, N, K, split, 0, stream)
    assert rc == 0, lib.get_last_error().decode()
    torch.cuda.synchronize()
    print("no-alloc split-K: graph capture", flush=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.call_dequant_gemm_fp16_fp4_splitk_static(_ptr(A), _ptr(B), _ptr(out), M, N, K, split, 0,
                                                              ctypes.c_void_p(side.cuda_stream))
    assert rc == 0, lib.get_last_error().decode()
    torch.cuda.synchronize()
    for i in range(3):
        out.fill_(float("nan"))
        # eager work between the replays, on the same scratch buffer, with another shape
        small = torch.empty((64, 128), dtype=torch.float16, device=cuda)
        rc = lib.call_dequant_gemm_fp16_fp4_splitk_static(_ptr(A), _ptr(B), _ptr(small), 64, 128, 512, 2, 0, stream)
        assert rc == 0, lib.get_last_error().decode()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i} differs from the eager result"


def test_static_scratch_rejects_what_does_not_fit(cuda):
    lib = _lib.get_library()
    M, N, K, split = 2048, 2048, 1024, 4  # 4 * 2048 * 2048 * 2 bytes = 32 MiB
    assert split * M * N * 2 > SCRATCH_BYTES
    A = torch.zeros((M, K), dtype=torch.float16, device=cuda)
    B = torch.zeros((N, K // 2), dtype=torch.uint8, device=cuda)
    C = torch.zeros((M, N), dtype=torch.float16, device=cuda)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.call_dequant_gemm_fp16_fp4_splitk_static(_ptr(A), _ptr(B), _ptr(C), M, N, K, split, 0, stream)
    assert rc == -1
    msg = lib.get_last_error().decode()
    assert "static scratch buffer holds" in msg and str(SCRATCH_BYTES) in msg
    # split == 1 needs no scratch at all and goes through
    rc = lib.call_dequant_gemm_fp16_fp4_splitk_static(_ptr(A), _ptr(B), _ptr(C), M, N, K, 1, 0, stream)
    assert rc == 0, lib.get_last_error().decode()
    torch.cuda.synchronize()
