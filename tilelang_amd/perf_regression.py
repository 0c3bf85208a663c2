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


@dataclass(frozen=True)
class PerfResult:
    name: str
    latency: float
    case: str | None = None


_results: list[PerfResult] = []
_current_case: str | None = None


def results() -> list[PerfResult]:
    """The results recorded since the last :func:`regression` started."""
    return list(_results)


def _only_filters() -> list[str]:
    raw = os.environ.get("TL_PERF_REGRESSION_ONLY", "").strip()
    if not raw:
        return []
    try:
        parsed = json.loads(raw)
    except json.JSONDecodeError:
        parsed = raw.split(",")
    if isinstance(parsed, str):
        parsed = [parsed]
    if not isinstance(parsed, list):
        return []
    return [str(p).strip() for p in parsed if str(p).strip()]


def _selected(case: str, filters: list[str]) -> bool:
    if not filters:
        return True
    names = (case.lower(), ("regression_" + case).lower())
    return any(fnmatch.fnmatch(n, f.lower()) or f.lower() in n for f in filters for n in names)


def process_func(func, name: str | None = None, /, **kwargs) -> None:
    """Run ``func(**kwargs)``, which returns a latency (any unit; only ratios matter), and record it under ``name``
    (default: the function's module, without a leading ``regression_``).  A non-positive latency is measured again,
    up to five times, then dropped with a warning."""
    label = getattr(func, "__module__", "<unknown>") if name is None else name
    if label.startswith("regression_"):
        label = label[len("regression_"):]
    latency = float(func(**kwargs))
    for _ in range(MAX_RETRIES):
        if latency > 0.0:
            break
        latency = float(func(**kwargs))
    if latency <= 0.0:
        warnings.warn(f"{label} has latency {latency} <= 0. Please verify the profiling results.", RuntimeWarning, 1)
        return
    _results.append(PerfResult(label, latency, _current_case))


def emit_results(stream=None) -> None:
    stream = stream or sys.stdout
    if os.environ.get("TL_PERF_REGRESSION_FORMAT", "text").strip().lower() == "json":
        items = []
        for r in _results:
            item = {"name": r.name, "latency": r.latency}
            if r.case is not None:
                item["case"] = r.case
            items.append(item)
        print(RESULTS_JSON_PREFIX + json.dumps(items, separators=(",", ":")), file=stream)
        return
    for r in _results:
        print(f"{r.name}: {r.latency}", file=stream)


def regression(prefixes=("regression_",), verbose: bool = True, namespace: dict | None = None) -> None:
    """Run the ``regression_*`` callables of the calling module (or of ``namespace``) and emit the results."""
    global _current_case
    if namespace is None:
        namespace = inspect.currentframe().f_back.f_globals
    _results.clear()
    filters = _only_filters()
    cases = sorted((k, v) for k, v in namespace.items() if callable(v) and any(k.startswith(p) for p in prefixes))
    cases = [(k, v) for k, v in cases if _selected(k[len("regression_"):] if k.startswith("regression_") else k, filters)]
    for idx, (name, fn) in enumerate(cases, 1):
        _current_case = name[len("regression_"):] if name.startswith("regression_") else name
        if verbose:
            print(f"  ├─ [{idx}/{len(cases)}] {_current_case}", end="", flush=True)
        t0 = time.perf_counter()
        try:
            with warnings.catch_warnings():
                warnings.simplefilter("ignore")
                fn()
            if verbose:
                print(f" ({time.perf_counter() - t0:.2f}s)", flush=True)
        finally:
            _current_case = None
    emit_results()


# ---- the dequantize-GEMM cases (examples/dequantize_gemm/regression_example_dequantize_gemm.py:10-26) --------------
# Each mirrors the example's run_regression_perf: same shapes and options, latency in ms from the profiler twin.


def _latency(kernel) -> float:
    return kernel.get_profiler().do_bench()


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
    """example_dequant_gemm_bf16_fp4_hopper.py:437-455: bf16 x fp4 (twiddled layout), 4096^3, no scale: run as the
    MXFP4 kernel with an all-zero exponent."""
    from . import kernels

    def run(m=4096, n=4096, k=4096, fast_dequant=True):
        return _latency(kernels.matmul_bf16_mxfp4(m, n, k, fast_dequant=fast_dequant, scale_bias=0))

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
