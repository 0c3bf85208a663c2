"""Checking and timing helpers with the reference profiler's policy.

``Profiler.assert_allclose`` / ``do_bench`` follow tilelang/profiler/__init__.py:104-162,
tilelang/profiler/bench.py:172-272 and tilelang/utils/tensor.py:42-118,205-293: inputs are
drawn per parameter from a ``TensorSupplyType``, outputs are compared with
``rtol=atol=1e-2`` (here with no allowance for mismatching elements unless asked), and
timing is the mean over event-bracketed calls with a 256 MiB buffer zeroed before each one
so the kernel starts from a cold L2.
"""

from __future__ import annotations

from enum import Enum
from typing import Callable

import torch


class TensorSupplyType(Enum):
    Integer = 1
    Uniform = 2
    Normal = 3
    Randn = 4
    Zero = 5
    One = 6
    Auto = 7


def get_tensor_supply(supply_type: TensorSupplyType = TensorSupplyType.Integer, device="cuda"):
    """Per-parameter random input, same distributions as tilelang/utils/tensor.py:42-118."""

    def get_tensor(param) -> torch.Tensor:
        dtype, shape = param.dtype, list(param.shape)
        unsigned = dtype == torch.uint8
        is_float = dtype in (torch.float16, torch.float32, torch.bfloat16)
        if supply_type == TensorSupplyType.Auto:
            if unsigned:
                return torch.randint(0, 3, shape, device=device, dtype=dtype)
            if is_float:
                return torch.empty(*shape, device=device, dtype=dtype).uniform_(-1.0, 1.0)
            return torch.randint(-2, 3, shape, device=device, dtype=dtype)
        if dtype == torch.int8 and supply_type in (TensorSupplyType.Uniform, TensorSupplyType.Normal):
            return torch.ones(*shape, device=device, dtype=dtype)
        if supply_type == TensorSupplyType.Integer:
            if unsigned:
                return torch.randint(0, 3, shape, device=device, dtype=dtype)
            return torch.randint(-2, 3, shape, device=device, dtype=dtype)
        if supply_type == TensorSupplyType.Uniform:
            return torch.empty(*shape, device=device, dtype=torch.float32).uniform_(-1.0, 1.0).to(dtype)
        if supply_type == TensorSupplyType.Normal:
            return torch.empty(*shape, device=device, dtype=torch.float32).normal_(-1.0, 1.0).to(dtype)
        if supply_type == TensorSupplyType.Randn:
            return torch.randn(*shape, device=device).to(dtype)
        if supply_type == TensorSupplyType.Zero:
            return torch.zeros(*shape, device=device, dtype=dtype)
        if supply_type == TensorSupplyType.One:
            return torch.ones(*shape, device=device, dtype=dtype)
        raise NotImplementedError(supply_type)

    return get_tensor


def torch_assert_close(a, b, rtol=1e-2, atol=1e-2, max_mismatched_ratio=0.0, base_name="LHS", ref_name="RHS"):
    """``isclose`` count against an allowed ratio (tilelang/utils/tensor.py:205-293); default allows none."""
    if a.shape != b.shape:
        raise AssertionError(f"shape mismatch: {tuple(a.shape)} vs {tuple(b.shape)}")
    if a.dtype != b.dtype:
        raise AssertionError(f"dtype mismatch: {a.dtype} vs {b.dtype}")
    if a.dtype in (torch.float16, torch.bfloat16):
        a, b = a.float(), b.float()
    bad = ~torch.isclose(a, b, rtol=rtol, atol=atol, equal_nan=True)
    n_bad, total = int(bad.sum().item()), a.numel()
    allowed = int(total * max_mismatched_ratio)
    if n_bad > allowed:
        idx = int(torch.argmax(bad.reshape(-1).int()).item())
        av, bv = a.reshape(-1)[idx].item(), b.reshape(-1)[idx].item()
        diff = (a.double() - b.double()).abs()
        raise AssertionError(
            f"Too many mismatched elements: {n_bad} > {allowed} of {total}. First mismatch at flat index {idx}: "
            f"{base_name}={av}, {ref_name}={bv}. Greatest absolute difference: {diff.max().item()}"
        )
    return True


def _summarise(times_ms: "torch.Tensor", quantiles, return_mode: str):
    """One number (mean / median / min / max) or the requested quantiles of the per-call times."""
    if quantiles is not None:
        q = torch.quantile(times_ms, torch.tensor(list(quantiles), dtype=torch.float)).tolist()
        return q[0] if len(q) == 1 else q
    return getattr(torch, return_mode)(times_ms).item()


def _time_with_events(fn, flush, n_repeat):
    """One event pair around every call, the cache flushed in front of each."""
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_repeat)]
    for begin, finish in pairs:
        flush()
        begin.record()
        fn()
        finish.record()
    torch.cuda.synchronize()
    return torch.tensor([b.elapsed_time(f) for b, f in pairs], dtype=torch.float)


def _time_with_graph(fn, flush, n_repeat, replays: int = 10):
    """``n_repeat`` calls captured back to back into one graph on a side stream (default priority), the graph
    replayed ``replays`` times with the cache flushed in front of every replay: per-call time without the host's
    launch cost.  The flush cannot be part of the graph, so calls after the first of a replay may hit the cache."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(n_repeat):
                fn()
        torch.cuda.synchronize()
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(replays)]
        for begin, finish in pairs:
            flush()
            begin.record()
            graph.replay()
            finish.record()
        torch.cuda.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    return torch.tensor([b.elapsed_time(f) / n_repeat for b, f in pairs], dtype=torch.float)


_FLUSH_RANGE = "tilelang_amd::cache_flush"


def _time_with_trace(fn, flush, n_repeat):
    """Device time of the kernels themselves from torch's kernel trace (the reference's ``backend="cupti"``; on
    ROCm the trace comes from the runtime's tracer): everything the GPU ran during the measured step minus what ran
    inside the annotated flush range, divided by the number of calls.  One number: the trace has no per-call split."""
    import warnings

    from torch.profiler import ProfilerActivity, profile, record_function, schedule

    with warnings.catch_warnings():
        warnings.simplefilter("ignore", UserWarning)  # "won't be using warmup", "clears events at the end of each cycle"
        plan = schedule(wait=1, warmup=0, active=1, repeat=1)
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA], schedule=plan) as prof:
            for _ in range(2):  # the first step is the schedule's wait step
                for _ in range(n_repeat):
                    with record_function(_FLUSH_RANGE):
                        flush()
                    fn()
                torch.cuda.synchronize()
                prof.step()
    kernels_us = flush_us = 0.0
    for ev in prof.events():
        if getattr(getattr(ev, "device_type", None), "name", "") != "CUDA":
            continue
        if ev.is_user_annotation:
            if ev.key == _FLUSH_RANGE:
                flush_us += ev.self_device_time_total
        else:
            kernels_us += ev.self_device_time_total
    return torch.tensor([(kernels_us - flush_us) / n_repeat * 1e-3], dtype=torch.float)


def do_bench(
    fn: Callable,
    warmup: float = 25,
    rep: float = 100,
    _n_warmup: int = 0,
    _n_repeat: int = 0,
    quantiles=None,
    fast_flush: bool = True,
    backend: str = "event",
    return_mode: str = "mean",
    device=None,
    cache_size: int = 256,
    early_stop_baseline: float | None = None,
):
    """Milliseconds per call of ``fn`` with the last-level cache flushed between calls.  Twin of ``do_bench`` of
    tilelang/profiler/bench.py:68-272 (same arguments and result conventions).

    ``warmup`` / ``rep``: target milliseconds of untimed and timed calls (the counts follow from a five-call
    estimate; ``_n_warmup`` / ``_n_repeat`` override them).  ``backend``: ``"event"`` (an event pair per call),
    ``"cudagraph"`` (the calls captured into one graph, replayed ten times) or ``"cupti"`` (device time from the
    kernel trace; ``"profiler"`` is accepted as a name for it).  ``return_mode`` (mean, median, min, max) or
    ``quantiles`` (a list of fractions; one fraction returns a float) pick the summary; ``early_stop_baseline``
    returns the estimate at once when it already exceeds that many milliseconds.  ``device``: a device index or
    ``torch.device`` to run on (default: the current one).
    """
    if return_mode not in ("min", "max", "mean", "median"):
        raise ValueError(f"Invalid return_mode: {return_mode}")
    if backend not in ("event", "cudagraph", "cupti", "profiler"):
        raise ValueError(f"Unknown profiler backend: {backend}")
    if device is not None:
        dev = torch.device("cuda", device) if isinstance(device, int) else torch.device(device)
        if dev.type != "cuda":
            raise ValueError(f"do_bench device must be a CUDA device, got {dev}")
        with torch.cuda.device(dev):
            return do_bench(fn, warmup, rep, _n_warmup, _n_repeat, quantiles, fast_flush, backend, return_mode, None,
                            cache_size, early_stop_baseline)

    fn()
    torch.cuda.synchronize()
    nbytes = cache_size * 1024 * 1024
    cache = torch.empty(nbytes // 4 if fast_flush else nbytes, dtype=torch.int if fast_flush else torch.int8, device="cuda")
    flush = cache.zero_

    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    first.record()
    for _ in range(5):
        flush()
        fn()
    last.record()
    torch.cuda.synchronize()
    estimate_ms = max(first.elapsed_time(last) / 5, 1e-4)
    if early_stop_baseline is not None and estimate_ms > early_stop_baseline:
        return [estimate_ms] * len(quantiles) if quantiles is not None else estimate_ms

    n_warmup = min(_n_warmup if _n_warmup > 0 else max(1, int(warmup / estimate_ms)), 1000)
    n_repeat = min(_n_repeat if _n_repeat > 0 else max(1, int(rep / estimate_ms)), 1000)
    for _ in range(n_warmup):
        fn()
    if backend == "event":
        times = _time_with_events(fn, flush, n_repeat)
    elif backend == "cudagraph":
        times = _time_with_graph(fn, flush, n_repeat)
    else:
        return _time_with_trace(fn, flush, n_repeat).item()
    return _summarise(times, quantiles, return_mode)


class Profiler:
    """``kernel.get_profiler()`` twin (tilelang/jit/kernel.py:494-508, tilelang/profiler/__init__.py)."""

    def __init__(self, adapter, supply_type: TensorSupplyType = TensorSupplyType.Auto):
        self.adapter = adapter
        self.supply = get_tensor_supply(supply_type)
        self.result_idx = adapter.result_idx

    def _get_inputs(self, with_output: bool = False):
        return [self.supply(p) for i, p in enumerate(self.adapter.params) if with_output or i not in self.result_idx]

    def run_once(self):
        return self.adapter(*self._get_inputs())

    def assert_allclose(self, reference_program: Callable, input_tensors=None, atol=1e-2, rtol=1e-2, max_mismatched_ratio=0.0):
        ins = self._get_inputs() if input_tensors is None else input_tensors
        ref = reference_program(*ins)
        torch.cuda.synchronize()
        out = self.adapter(*ins)
        torch.cuda.synchronize()
        refs = list(ref) if isinstance(ref, (list, tuple)) else [ref]
        outs = list(out) if isinstance(out, (list, tuple)) else [out]
        assert len(refs) == len(outs), "len(lib_outs) not equals to len(ref_outs) !"
        for lhs, rhs in zip(outs, refs):
            if lhs is not None and rhs is not None:
                torch_assert_close(lhs, rhs, rtol=rtol, atol=atol, max_mismatched_ratio=max_mismatched_ratio,
                                   base_name="tilelang_amd", ref_name="ref")

    def assert_consistent(self, repeat: int = 10):
        """Bit-identical outputs over repeated runs on the same inputs (tilelang/profiler/__init__.py:195-212)."""
        ins = self._get_inputs()
        first = self.adapter(*ins)
        firsts = [t.clone() for t in (first if isinstance(first, (list, tuple)) else [first])]
        for _ in range(repeat - 1):
            out = self.adapter(*ins)
            outs = out if isinstance(out, (list, tuple)) else [out]
            for a, b in zip(firsts, outs):
                assert torch.equal(a, b), "outputs differ between runs"

    def do_bench(self, func: Callable | None = None, warmup: int = 25, rep: int = 100, input_tensors=None, **kw) -> float:
        ins = self._get_inputs() if input_tensors is None else input_tensors
        fn = (lambda: func(*ins)) if func is not None else (lambda: self.adapter(*ins))
        return do_bench(fn, warmup=warmup, rep=rep, **kw)


_MFMA_RATE_DTYPES = {"float16": (0, 16), "bfloat16": (1, 16), "int8": (2, 32), "fp4": (5, 64)}


def mfma_sustained_rate(dtype: str = "bfloat16", launch_ms: float = 5.0, settle_ms: float = 60.0, launches: int = 8,
                        device=None) -> dict:
    """Operations per second the matrix pipe of the device sustains on random operands, with nothing else running
    beside the matrix instructions (``call_mfma_rate``): one workgroup of four waves per compute unit, each issuing
    the 16 instructions of a 128 x 128 wave tile over and over.  The published peak assumes the top clock; operands
    that toggle like real data hold the chip at its power limit below it, so this is the rate a GEMM kernel on this
    device can approach.  Untimed launches for ``settle_ms`` first (the clock settles), then the median of
    ``launches`` launches of about ``launch_ms`` each, timed with events on the current stream.

    No counterpart in the reference (its benchmarks quote the vendor's peak)."""
    from . import _lib

    code, k = _MFMA_RATE_DTYPES[dtype]
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(dev):
        lib = _lib.get_library(dev.index)
        gen = torch.Generator(device="cpu").manual_seed(0)
        if dtype in ("int8", "fp4"):  # every byte is a valid operand: an int8, or two e2m1 codes
            operands = torch.randint(-128, 128, (65536,), generator=gen, dtype=torch.int8).to(dev)
        else:
            operands = torch.randn(32768, generator=gen).to(getattr(torch, dtype)).to(dev)
        workgroups = torch.cuda.get_device_properties(dev).multi_processor_count
        sink = torch.empty(workgroups * 256, dtype=torch.float32, device=dev)
        ops_per_iter = workgroups * 4 * 16 * 2 * 32 * 32 * k
        stream = torch.cuda.current_stream(dev)

        def launch(iters):
            if lib.call_mfma_rate(operands.data_ptr(), sink.data_ptr(), code, workgroups, iters, stream.cuda_stream) != 0:
                raise RuntimeError(_lib.last_error())

        def timed(iters):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            launch(iters)
            b.record(stream)
            b.synchronize()
            return a.elapsed_time(b)

        iters = 2000
        ms = timed(iters)
        iters = max(1000, int(iters * launch_ms / max(ms, 1e-3)))
        spent = 0.0
        while spent < settle_ms:
            spent += timed(iters)
        times = sorted(timed(iters) for _ in range(launches))
        ms = times[len(times) // 2]
    return {"ops_per_s": ops_per_iter * iters / (ms * 1e-3), "ms_per_launch": ms, "iters": iters,
            "workgroups": workgroups, "dtype": dtype}
