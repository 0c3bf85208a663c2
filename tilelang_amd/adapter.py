"""Kernel adapter: the callable a kernel factory returns.

Mirrors the call contract of the reference's adapter for JIT kernels
(tilelang/jit/adapter/cython/cython_wrapper.pyx:164-287, tilelang/jit/kernel.py:195-211):

* ``kernel(*inputs)``; parameters listed in ``result_idx`` are allocated here with
  ``torch.empty`` on the first input's device and returned (``out_idx`` semantics);
* before the launch: argument count, device, dtype, shape, strides, contiguity are
  checked (``skip_tensor_validation=True`` skips them); errors are ``ValueError`` with
  the reference's wording;
* tensors are passed as raw ``data_ptr()``; ``None`` becomes a NULL pointer;
* the launch goes to torch's current stream unless ``stream=`` is given; it is
  asynchronous and never synchronises;
* a non-zero return code raises ``RuntimeError("Kernel call failed: <get_last_error()>")``.
"""

from __future__ import annotations

import contextlib
import ctypes
from dataclasses import dataclass
from typing import Callable, Sequence

import torch


@dataclass(frozen=True)
class KernelParam:
    name: str
    dtype: torch.dtype
    shape: tuple
    #: packed sub-byte storage: the strict dtype check accepts int8 and uint8 alike
    packed: bool = False


def current_stream_handle(device_type: str = "cuda") -> int:
    """Raw handle of torch's current stream (tilelang/jit/adapter/cython/cython_wrapper.pyx:178-185)."""
    if device_type == "cuda" and torch.cuda.is_available():
        try:
            return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())
        except (ImportError, AttributeError):
            return torch.cuda.current_stream().cuda_stream
    return 0


class KernelAdapter:
    def __init__(
        self,
        name: str,
        params: Sequence[KernelParam],
        result_idx: Sequence[int],
        launch: Callable[[list, int], int],
        get_last_error: Callable[[], str],
        device_type: str = "cuda",
        workspace_idx: Sequence[int] = (),
    ):
        self.name = name
        self.params = list(params)
        n = len(self.params)
        self.result_idx = [i if i >= 0 else n + i for i in result_idx]
        # parameters the kernel uses as scratch (the reference's T.alloc_buffer globals): allocated here for every
        # call, passed to the library, never returned.  torch's caching allocator hands a freed block back to the
        # stream it was allocated under only (__call__ allocates under the stream it launches on), so calls on
        # different streams never share a scratch buffer.
        self.workspace_idx = [i if i >= 0 else n + i for i in workspace_idx]
        self._launch = launch
        self._get_last_error = get_last_error
        self.device_type = device_type

    # -- validation, same order and wording as the reference ------------------------------
    def _check(self, tensors: list):
        for p, t in zip(self.params, tensors):
            if not isinstance(t, torch.Tensor):
                continue
            if t.device.type != self.device_type:
                raise ValueError(
                    f"Buffer device mismatch for parameter {p.name}: expected {self.device_type}, got {t.device}"
                )
        for p, t in zip(self.params, tensors):
            if not isinstance(t, torch.Tensor):
                continue
            ok = t.dtype == p.dtype or (p.packed and t.dtype in (torch.int8, torch.uint8))
            if not ok:
                raise ValueError(f"Buffer dtype mismatch for parameter {p.name}: expected {p.dtype}, got {t.dtype}")
        for p, t in zip(self.params, tensors):
            if not isinstance(t, torch.Tensor):
                continue
            if t.dim() != len(p.shape):
                raise ValueError(
                    f"Static shape mismatch for parameter {p.name}: expected {len(p.shape)} dimensions, got {t.dim()}"
                )
            for i, e in enumerate(p.shape):
                if e != -1 and t.shape[i] != e:
                    raise ValueError(
                        f"Static shape mismatch for parameter {p.name}: expected {e} at index {i}, got {t.shape[i]}"
                    )
        for p, t in zip(self.params, tensors):
            if not isinstance(t, torch.Tensor):
                continue
            expected = 1
            for i in range(len(p.shape) - 1, -1, -1):
                if t.shape[i] != 1 and t.stride(i) != expected:
                    raise ValueError(
                        f"Static stride mismatch for parameter {p.name}: expected {expected} at index {i}, got {t.stride(i)}"
                    )
                expected *= t.shape[i]
        for p, t in zip(self.params, tensors):
            if isinstance(t, torch.Tensor) and not t.is_contiguous():
                raise ValueError(f"Expected parameter {p.name} to be a contiguous tensor")

    def __call__(self, *inputs, stream: int = -1, skip_tensor_validation: bool = False):
        n_params, n_in, n_out = len(self.params) - len(self.workspace_idx), len(inputs), len(self.result_idx)
        if n_params != n_in + n_out:
            raise ValueError(
                f"Expected {n_params} inputs, got {n_in + n_out} with {n_in} inputs and {n_out} outputs"
            )
        device = None
        for t in inputs:
            if isinstance(t, torch.Tensor):
                device = t.device
                break
        if device is None:
            device = torch.device(self.device_type)
        on_gpu = device.type == "cuda" and torch.cuda.is_available()
        # the library launches on the CURRENT device: make the operands' device current for the length of the call
        guard = contextlib.nullcontext()
        if on_gpu and device.index is not None and device.index != torch.cuda.current_device():
            guard = torch.cuda.device(device)
        with guard:
            current = current_stream_handle(self.device_type)
            if stream == -1:
                stream = current
            # Outputs and scratch come from torch's caching allocator, which hands a freed block back to work on
            # the stream it was allocated under only.  With an explicit stream= that is not torch's current one,
            # allocate under that stream, so that a block freed while this launch still runs cannot go to an op on
            # another stream.
            alloc_ctx = contextlib.nullcontext()
            if on_gpu and stream != current and (self.result_idx or self.workspace_idx):
                alloc_ctx = torch.cuda.stream(torch.cuda.ExternalStream(stream, device=device))
            tensors, it = [], iter(inputs)
            with alloc_ctx:
                for i, p in enumerate(self.params):
                    if i in self.workspace_idx or i in self.result_idx:
                        tensors.append(torch.empty(*p.shape, dtype=p.dtype, device=device))
                    else:
                        tensors.append(next(it))
            return self._run(tensors, stream, skip_tensor_validation, n_out)

    def _run(self, tensors, stream, skip_tensor_validation, n_out):
        ptrs = []
        for t in tensors:
            if isinstance(t, torch.Tensor):
                ptrs.append(ctypes.c_void_p(t.data_ptr()))
            elif t is None:
                ptrs.append(ctypes.c_void_p(0))
            elif isinstance(t, int):
                ptrs.append(ctypes.c_void_p(t))
            else:
                raise ValueError(f"Unsupported tensor type: {type(t)}")

        if not skip_tensor_validation:
            self._check(tensors)

        rc = self._launch(ptrs, stream)
        if rc != 0:
            raise RuntimeError(f"Kernel call failed: {self._get_last_error()}")

        if n_out == 0:
            return None
        if n_out == 1:
            return tensors[self.result_idx[0]]
        return [tensors[i] for i in self.result_idx]

    # conveniences mirroring tilelang/jit/kernel.py:494-520
    def get_profiler(self, tensor_supply_type=None):
        from .profiler import Profiler, TensorSupplyType

        return Profiler(self, tensor_supply_type or TensorSupplyType.Auto)
