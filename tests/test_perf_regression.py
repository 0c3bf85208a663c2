"""The perf-regression harness: result format, case selection and retry policy of
tilelang/testing/perf_regression.py:16-165 (CPU), and one real case on the GPU."""

import io
import json
from contextlib import redirect_stdout

import pytest

from tilelang_amd import perf_regression as pr


def _run(namespace, monkeypatch, fmt=None, only=None):
    if fmt is None:
        monkeypatch.delenv("TL_PERF_REGRESSION_FORMAT", raising=False)
    else:
        monkeypatch.setenv("TL_PERF_REGRESSION_FORMAT", fmt)
    if only is None:
        monkeypatch.delenv("TL_PERF_REGRESSION_ONLY", raising=False)
    else:
        monkeypatch.setenv("TL_PERF_REGRESSION_ONLY", only)
    out = io.StringIO()
    with redirect_stdout(out):
        pr.regression(verbose=False, namespace=namespace)
    return out.getvalue()


def _namespace():
    calls = {"flaky": 0}

    def bench_a():
        return 1.5

    bench_a.__module__ = "regression_example_a"

    def flaky():
        calls["flaky"] += 1
        return 0.0 if calls["flaky"] < 3 else 2.0

    def never():
        return -1.0

    def regression_b_case():
        pr.process_func(flaky, "b")
        pr.process_func(never, "dropped")

    def regression_a_case():
        pr.process_func(bench_a)
        pr.process_func(lambda x=0: 0.25 * x, "a_kw", x=2)

    return {"regression_b_case": regression_b_case, "regression_a_case": regression_a_case, "helper": bench_a,
            "not_callable": 3}, calls


def test_text_format_order_names_and_retry(monkeypatch):
    ns, calls = _namespace()
    text = _run(ns, monkeypatch)
    # cases run in name order; the module name loses its regression_ prefix; a non-positive latency is measured
    # again (up to five more times) and dropped with a warning if it never turns positive
    assert text.splitlines() == ["example_a: 1.5", "a_kw: 0.5", "b: 2.0"]
    assert calls["flaky"] == 3
    assert [(r.name, r.case) for r in pr.results()] == [("example_a", "a_case"), ("a_kw", "a_case"), ("b", "b_case")]


def test_json_marker_line(monkeypatch):
    ns, _ = _namespace()
    text = _run(ns, monkeypatch, fmt="json")
    lines = text.splitlines()
    assert len(lines) == 1 and lines[0].startswith("__TILELANG_PERF_RESULTS_JSON__=")
    items = json.loads(lines[0].split("=", 1)[1])
    assert items == [{"name": "example_a", "latency": 1.5, "case": "a_case"}, {"name": "a_kw", "latency": 0.5, "case": "a_case"},
                     {"name": "b", "latency": 2.0, "case": "b_case"}]


@pytest.mark.parametrize("only,expected", [("b_case", ["b"]), ('["A_*"]', ["example_a", "a_kw"]), ("regression_b*", ["b"]),
                                           ("nothing", []), ("a_case, b_case", ["example_a", "a_kw", "b"])])
def test_case_selection(monkeypatch, only, expected):
    ns, _ = _namespace()
    text = _run(ns, monkeypatch, only=only)
    assert [line.split(":")[0] for line in text.splitlines()] == expected


def test_the_dequantize_gemm_cases_are_the_examples(monkeypatch):
    """Same case names as examples/dequantize_gemm/regression_example_dequantize_gemm.py:10-26."""
    cases = sorted(k for k, v in vars(pr).items() if k.startswith("regression_example_") and callable(v))
    assert cases == ["regression_example_dequant_gemm_bf16_fp4_hopper", "regression_example_dequant_gemm_bf16_mxfp4_hopper",
                     "regression_example_dequant_gemm_fp4_hopper", "regression_example_dequant_gemm_w4a8",
                     "regression_example_dequant_gemv_fp16xint4"]


@pytest.mark.gpu
def test_one_case_on_the_gpu(cuda, monkeypatch):
    text = _run(vars(pr), monkeypatch, only="gemv_fp16xint4")
    name, latency = text.strip().split(": ")
    assert name == "example_dequant_gemv_fp16xint4" and 0.0 < float(latency) < 1.0   # ms
