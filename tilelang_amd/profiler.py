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


def do_bench(
    fn: Callable,
    warmup: float = 25,
    rep: float = 100,
    _n_warmup: int = 0,
    _n_repeat: int = 0,
    return_mode: str = "mean",
    cache_size: int = 256,
) -> float:
    """Mean (or min/max/median) milliseconds per call, event-timed, L2 flushed before each call."""
    fn()
    torch.cuda.synchronize()
    cache = torch.empty(cache_size * 1024 * 1024 // 4, dtype=torch.int, device="cuda")
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        cache.zero_()
        fn()
    end.record()
    torch.cuda.synchronize()
    estimate_ms = max(start.elapsed_time(end) / 5, 1e-4)
    n_warmup = _n_warmup if _n_warmup > 0 else max(1, int(warmup / estimate_ms))
    n_repeat = _n_repeat if _n_repeat > 0 else max(1, int(rep / estimate_ms))
    n_warmup, n_repeat = min(n_warmup, 1000), min(n_repeat, 1000)
    for _ in range(n_warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for i in range(n_repeat):
        cache.zero_()
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([s.elapsed_time(e) for s, e in zip(starts, ends)], dtype=torch.float)
    return getattr(torch, return_mode)(times).item()


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
