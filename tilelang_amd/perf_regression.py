"""Perf-regression harness with the shape of the reference's (tilelang/testing/perf_regression.py:16-165).

A benchmark module defines ``regression_<case>()`` functions; each calls :func:`process_func` on one or more
callables that return a latency; :func:`regression` runs every such function of the calling module in name
order and emits the results the way the reference's collectors expect: one ``name: latency`` line per result,
or, with ``TL_PERF_REGRESSION_FORMAT=json``, one marker line ``__TILELANG_PERF_RESULTS_JSON__=[{"name", "latency",
"case"}, ...]``.  ``TL_PERF_REGRESSION_ONLY`` (JSON list or comma-separated glob / substring patterns, case
insensitive) selects cases.  ``python -m tilelang_amd.perf_regression`` runs the dequantize-GEMM cases of
examples/dequantize_gemm/regression_example_dequantize_gemm.py on this library's kernels.
"""

from __future__ import annotations

import fnmatch
import inspect
import json
import os
import sys
import time
import warnings
from dataclasses import dataclass

RESULTS_JSON_PREFIX = "__TILELANG_PERF_RESULTS_JSON__="
MAX_RETRIES = 5
_CASE_PREFIX = "regression_"


@dataclass(frozen=True)
class PerfResult:
    name: str
    latency: float
    case: str | None = None

    def as_json_item(self) -> dict:
        item = {"name": self.name, "latency": self.latency}
        if self.case is not None:
            item["case"] = self.case
        return item


class _Recorder:
    """What one run of :func:`regression` collects: the results so far and the case they belong to."""

    def __init__(self):
        self.items: list[PerfResult] = []
        self.case: str | None = None

    def add(self, name: str, latency: float) -> None:
        self.items.append(PerfResult(name, latency, self.case))

    def write(self, stream) -> None:
        as_json = os.environ.get("TL_PERF_REGRESSION_FORMAT", "text").strip().lower() == "json"
        if as_json:
            payload = json.dumps([r.as_json_item() for r in self.items], separators=(",", ":"))
            print(RESULTS_JSON_PREFIX + payload, file=stream)
        else:
            for r in self.items:
                print(f"{r.name}: {r.latency}", file=stream)


_recorder = _Recorder()


def results() -> list[PerfResult]:
    """The results recorded since the last :func:`regression` started."""
    return list(_recorder.items)


def _strip_prefix(name: str) -> str:
    return name[len(_CASE_PREFIX):] if name.startswith(_CASE_PREFIX) else name


def _case_selector():
    """Predicate on a case's function name built from ``TL_PERF_REGRESSION_ONLY``: a JSON list (or one JSON string)
    or a comma-separated list of patterns; a pattern selects a case when it is a glob match or a substring of the
    function name or of the name without ``regression_``, case-insensitively.  No patterns: every case."""
    spec = os.environ.get("TL_PERF_REGRESSION_ONLY", "").strip()
    patterns: list[str] = []
    if spec:
        try:
            decoded = json.loads(spec)
        except json.JSONDecodeError:
            decoded = spec.split(",")
        if isinstance(decoded, str):
            decoded = [decoded]
        if isinstance(decoded, list):
            patterns = [text.lower() for text in (str(x).strip() for x in decoded) if text]

    def wanted(func_name: str) -> bool:
        if not patterns:
            return True
        for candidate in (func_name.lower(), _strip_prefix(func_name).lower()):
            for pat in patterns:
                if pat in candidate or fnmatch.fnmatch(candidate, pat):
                    return True
        return False

    return wanted


def process_func(func, name: str | None = None, /, **kwargs) -> None:
    """Run ``func(**kwargs)``, which returns a latency (any unit; only ratios matter), and record it under ``name``
    (default: the function's module, without a leading ``regression_``).  A non-positive latency is measured again,
    up to five more times, then dropped with a warning."""
    label = _strip_prefix(name if name is not None else getattr(func, "__module__", "<unknown>"))
    latency = 0.0
    for _attempt in range(1 + MAX_RETRIES):
        latency = float(func(**kwargs))
        if latency > 0.0:
            _recorder.add(label, latency)
            return
    warnings.warn(f"{label} has latency {latency} <= 0. Please verify the profiling results.", RuntimeWarning, 1)


def emit_results(stream=None) -> None:
    _recorder.write(stream or sys.stdout)


def regression(prefixes=("regression_",), verbose: bool = True, namespace: dict | None = None) -> None:
    """Run the ``regression_*`` callables of the calling module (or of ``namespace``), in name order, and emit the
    results.  Warnings raised inside a case are muted; a progress line per case goes to stdout when ``verbose``."""
    if namespace is None:
        namespace = inspect.currentframe().f_back.f_globals
    wanted = _case_selector()
    todo = [name for name in sorted(namespace)
            if callable(namespace[name]) and name.startswith(tuple(prefixes)) and wanted(name)]
    _recorder.items.clear()
    for position, func_name in enumerate(todo, start=1):
        _recorder.case = _strip_prefix(func_name)
        if verbose:
            print(f"  ├─ [{position}/{len(todo)}] {_recorder.case}", end="", flush=True)
        started = time.perf_counter()
        try:
            with warnings.catch_warnings():
                warnings.simplefilter("ignore")
                namespace[func_name]()
            if verbose:
                print(f" ({time.perf_counter() - started:.2f}s)", flush=True)
        finally:
            _recorder.case = None
    emit_results()


# ---- the dequantize-GEMM cases (examples/dequantize_gemm/regression_example_dequantize_gemm.py:10-26) --------------
# Each mirrors the example's run_regression_perf: same shapes and options, latency in ms from the profiler twin.


def _latency(kernel) -> float:
    # the examples' own calls: profiler.do_bench(backend="cupti"), device time from the kernel trace
    # (examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_hopper.py:559)
    return kernel.get_profiler().do_bench(backend="cupti")


def regression_example_dequant_gemv_fp16xint4():
    """example_dequant_gemv_fp16xint4.py:220-263: M=1, N=K=8192, unsigned fast decode, no scaling."""
    from . import kernels

    def run():
        return _latency(kernels.dequantize_gemv(1, 8192, 8192, "float16", "float16", "float16", 4, "int8", "uint", 4, 32,
                                                True, False, True, -1, False))

    run.__module__ = "example_dequant_gemv_fp16xint4"
    process_func(run)


def regression_example_dequant_gemm_fp4_hopper():
    """example_dequant_gemm_fp4_hopper.py:267-272: fp16 x fp4, 4096^3, Ct[N, M]."""
    from . import kernels

    def run(m=4096, n=4096, k=4096):
        return _latency(kernels.matmul_fp16_fp4(m, n, k, "float16", "float16", "float32", num_bits=4))

    run.__module__ = "example_dequant_gemm_fp4_hopper"
    process_func(run)


def regression_example_dequant_gemm_bf16_fp4_hopper():
    """example_dequant_gemm_bf16_fp4_hopper.py:437-455: bf16 x fp4 (twiddled layout), 4096^3, no scale: the example's
    own ``kernel(A, qB)``."""
    from . import kernels

    def run(m=4096, n=4096, k=4096, fast_dequant=True):
        return _latency(kernels.matmul_bf16_fp4(m, n, k, fast_dequant=fast_dequant))

    run.__module__ = "example_dequant_gemm_bf16_fp4_hopper"
    process_func(run)


def regression_example_dequant_gemm_bf16_mxfp4_hopper():
    """example_dequant_gemm_bf16_mxfp4_hopper.py:539-560: MXFP4 x bf16, 4096^3, scale_size 32."""
    from . import kernels

    def run(m=4096, n=4096, k=4096, scale_size=32, fast_dequant=True, with_bias=False):
        return _latency(kernels.matmul_bf16_mxfp4(m, n, k, scale_size=scale_size, fast_dequant=fast_dequant,
                                                  with_bias=with_bias, scale_bias=0))

    run.__module__ = "example_dequant_gemm_bf16_mxfp4_hopper"
    process_func(run)


def regression_example_dequant_gemm_w4a8():
    """example_dequant_gemm_w4a8.py:184-199: int8 x int4, 4096^3, Ct[N, M] int32."""
    from . import kernels

    def run(m=4096, n=4096, k=4096):
        return _latency(kernels.matmul_int8xint4(m, n, k, "int8", "int32", "int32", num_bits=4))

    run.__module__ = "example_dequant_gemm_w4a8"
    process_func(run)


if __name__ == "__main__":
    regression()
