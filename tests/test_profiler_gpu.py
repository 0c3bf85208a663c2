"""``do_bench`` backends and result modes (tilelang/profiler/bench.py:68-272) on a real kernel, and the adapter's
handling of an explicit stream."""

import numpy as np
import pytest
import torch

import tilelang_amd as tl
from tilelang_amd import profiler, workloads

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gemv(cuda):
    M, N, K = 1, 4096, 4096
    d = workloads.w4a16(M, N, K, 128, seed=0)
    kern = tl.dequantize_gemv(M, N, K, group_size=128, source_format="int", with_scaling=True)
    args = [torch.from_numpy(d["A"]).to(cuda), torch.from_numpy(d["B"]).to(cuda).view(torch.int8),
            torch.from_numpy(d["Scale"]).to(cuda), torch.empty((M, N), dtype=torch.float16, device=cuda)]
    return kern, args


@pytest.mark.parametrize("backend", ["event", "cudagraph", "cupti"])
def test_backends_agree_on_a_memory_bound_kernel(gemv, backend):
    """Every backend times the same launches: a 4096 x 4096 decode GEMV (8.4 MB of weights) takes a few microseconds;
    the event backend adds the host's launch cost on top of the device time the other two see."""
    kern, args = gemv
    print(f"do_bench backend={backend}", flush=True)
    ms = profiler.do_bench(lambda: kern(*args), warmup=5, rep=20, backend=backend)
    assert isinstance(ms, float) and 1e-3 < ms < 0.2, ms


def test_result_modes_and_quantiles(gemv):
    kern, args = gemv
    fn = lambda: kern(*args)  # noqa: E731
    lo = profiler.do_bench(fn, _n_warmup=3, _n_repeat=40, return_mode="min")
    hi = profiler.do_bench(fn, _n_warmup=3, _n_repeat=40, return_mode="max")
    med = profiler.do_bench(fn, _n_warmup=3, _n_repeat=40, return_mode="median")
    assert 0 < lo <= hi and 0 < med
    q = profiler.do_bench(fn, _n_warmup=3, _n_repeat=40, quantiles=[0.2, 0.5, 0.8])
    assert isinstance(q, list) and len(q) == 3 and q[0] <= q[1] <= q[2]
    assert isinstance(profiler.do_bench(fn, _n_warmup=3, _n_repeat=10, quantiles=[0.5]), float)
    g = profiler.do_bench(fn, _n_warmup=3, _n_repeat=20, backend="cudagraph", quantiles=[0.5, 0.9])
    assert len(g) == 2 and g[0] <= g[1]
    # an estimate beyond the baseline is returned as it is
    early = profiler.do_bench(fn, early_stop_baseline=1e-9)
    assert early > 1e-9
    assert profiler.do_bench(fn, early_stop_baseline=1e-9, quantiles=[0.1, 0.9]) == pytest.approx([early] * 2, rel=2.0)
    assert profiler.do_bench(fn, _n_warmup=1, _n_repeat=5, device=0) > 0
    with pytest.raises(ValueError, match="Unknown profiler backend"):
        profiler.do_bench(fn, backend="nvtx")
    with pytest.raises(ValueError, match="Invalid return_mode"):
        profiler.do_bench(fn, return_mode="mode")


def test_explicit_stream_gets_its_own_outputs(cuda):
    """``kernel(..., stream=handle)`` with a stream that is not torch's current one: the output is allocated under that
    stream (a block freed early cannot be handed to work on the current stream) and the result is right."""
    M, N, K = 256, 256, 256
    d = workloads.mxfp4(M, N, K, seed=1, scale_bias=127)
    kern = tl.matmul_bf16_mxfp4(M, N, K, weight_format="e2m1", scale_bias=127)
    A = torch.from_numpy(d["A"]).to(cuda).view(torch.bfloat16)
    B, S = torch.from_numpy(d["B"]).to(cuda), torch.from_numpy(d["Scale"]).to(cuda)
    bias = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
    torch.cuda.synchronize()
    expect = kern(A, B, S, bias)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    outs = []
    for _ in range(4):
        outs.append(kern(A, B, S, bias, stream=side.cuda_stream))
        # churn on the current stream: were the output a current-stream block, dropping it here could hand it on
        junk = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=cuda)
        del junk
    side.synchronize()
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o, expect)
    assert len({o.data_ptr() for o in outs}) == 4


@pytest.mark.parametrize("dtype, peak", [("bfloat16", 2.5e15), ("float16", 2.5e15), ("int8", 5.0e15), ("fp4", 10.1e15)])
def test_mfma_sustained_rate_is_a_plausible_ceiling(cuda, dtype, peak):
    """``call_mfma_rate`` through ``profiler.mfma_sustained_rate``: the matrix pipe alone, on random operands, runs at
    a sizeable fraction of the published peak and never above it (the count of operations per launch is right)."""
    m = profiler.mfma_sustained_rate(dtype, launch_ms=1.0, settle_ms=5.0, launches=3, device=cuda)
    assert 0.35 * peak < m["ops_per_s"] < 1.02 * peak, m


def test_mfma_rate_rejects_what_it_cannot_run(cuda):
    from tilelang_amd import _lib

    lib = _lib.get_library()
    buf = torch.zeros(65536, dtype=torch.int8, device=cuda)
    sink = torch.zeros(256, dtype=torch.float32, device=cuda)
    assert lib.call_mfma_rate(buf.data_ptr(), sink.data_ptr(), 3, 1, 1, None) == -1
    assert "in_dtype" in _lib.last_error()
    assert lib.call_mfma_rate(None, sink.data_ptr(), 1, 1, 1, None) == -1
    assert "non-NULL" in _lib.last_error()
    assert lib.call_mfma_rate(buf.data_ptr(), sink.data_ptr(), 1, 0, 1, None) == -1
    assert "workgroups" in _lib.last_error()
