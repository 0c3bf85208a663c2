#!/usr/bin/env python3
"""Benchmark of the dequantize-GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--all-shapes]

A step is one pass of the headline kernel, the M=1 W4A16 decode GEMV at N=28672, K=8192
(group 128, w=(q-8)*s), over one weight matrix already resident in HBM.  Steps rotate over
several distinct copies of the weights (more than the 256 MiB of last-level cache in total) so
every step streams its weights from HBM.  Prints ONE JSON line: the GEMV time as `value`, its
HBM roofline, the per-configuration table (us, GB/s, TFLOP/s, fraction of the binding
roofline) and the CPU baseline (the torch restatement of the reference's ref_program, timed on
the host cores on a bounded sample).
"""

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12        # B/s
MFMA_BF16_PEAK = 2.5e15  # FLOP/s dense
MFMA_I8_PEAK = 5.0e15    # OP/s dense
MFMA_FP4_PEAK = 10.1e15  # FLOP/s dense, block-scaled fp4
# HBM bytes per launch of the headline GEMV: counters need the profiler, so this script cannot measure them; it READS
# them from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary (scaled there by what the same counters read
# for a plain 128 MiB copy kernel: 2 KiB and 1 KiB per count).  The row is looked up by workload and must name the
# kernel this script launches, otherwise `traffic` is null: a figure of another kernel is never printed as this one's.
GEMV_TRAFFIC_PROFILE = "profiles/bench_all_configs_hbm_traffic.md"
GEMV_KERNEL = "w4a16_gemv_kernel<1,1,4,1,0,1,0,1>"  # MROWS, NP, R, HAS_SCALE, HAS_ZEROS, G128, FLIP, WIDE


def gemv_hbm_traffic():
    """(bytes per launch or None, source) of the headline GEMV from the committed counter summary."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), GEMV_TRAFFIC_PROFILE)
    try:
        with open(path) as f:
            for line in f:
                cells = [c.strip() for c in line.split("|")]
                if len(cells) >= 6 and "(headline)" in cells[2] and GEMV_KERNEL in cells[1]:
                    return int(round(float(cells[3]) * 2048 + float(cells[4]) * 1024)), GEMV_TRAFFIC_PROFILE
    except (OSError, ValueError):
        pass
    return None, None


#: False (--no-graph): time plain back-to-back launches.  For runs under a profiler that collects hardware counters: it
#: serialises the kernels itself, and a replayed graph whose calls are two dependent kernels did not come back under it
#: (that row, the K split over workgroups, is left out of such runs altogether).
USE_GRAPH = True


def _time_launches(torch, fns, steps, warmup, min_launches=120, max_launches=None, settle_ms=50.0, replays=30):
    """Median device time per call of fns[i % len(fns)], independent of `steps`.

    `steps` launches (repeated for whole rounds until the graph holds at least `min_launches`) are captured
    into one HIP graph: the kernels are microseconds long and replaying a graph keeps the host out of the
    measurement.  The graph is replayed untimed until `settle_ms` of device time have passed, so the clocks
    have ramped, then `replays` times with an event pair of its own around every replay, all on the stream
    the kernels run on (per-iteration events as in tilelang/profiler/bench.py:172-272).  Returns the median
    over the replays of (replay time / launches in the graph), with the minimum and the mean beside it.
    Falls back to plain back-to-back launches if capture is refused.
    """
    for i in range(max(warmup, len(fns))):
        fns[i % len(fns)]()
    torch.cuda.synchronize()
    rounds = max(1, -(-min_launches // max(steps, 1)))
    launches = steps * rounds
    if max_launches is not None:
        launches = min(launches, max_launches)
    stream = torch.cuda.Stream()
    graph = None
    try:
        if not USE_GRAPH:
            raise RuntimeError("--no-graph")
        with torch.cuda.stream(stream):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(launches):
                    fns[i % len(fns)]()
            graph = g
    except Exception as exc:  # pragma: no cover - depends on the runtime
        print(f"[bench] graph capture refused ({exc}); timing direct launches", file=sys.stderr)
        torch.cuda.synchronize()

    def once():
        if graph is not None:
            graph.replay()
        else:
            for i in range(launches):
                fns[i % len(fns)]()

    with torch.cuda.stream(stream):
        settled, n_settle = 0.0, 0
        while settled < settle_ms and n_settle < 10000:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            once()
            b.record(stream)
            b.synchronize()
            settled += a.elapsed_time(b)
            n_settle += 1
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(replays)]
        for a, b in pairs:
            a.record(stream)
            once()
            b.record(stream)
        stream.synchronize()
    torch.cuda.synchronize()
    per = sorted(a.elapsed_time(b) / launches for a, b in pairs)
    stats = {"graph": graph is not None, "launches_per_replay": launches, "replays": replays,
             "us_min": per[0] * 1e3, "us_mean": sum(per) / len(per) * 1e3, "settle_replays": n_settle}
    return float(np.median(per)), stats


def _copies(nbytes, min_total=640 << 20, lo=2, hi=24):
    return int(min(hi, max(lo, -(-min_total // max(nbytes, 1)))))


def bench_w4a16(torch, tl, workloads, M, N, K, zeros, steps, warmup, dev, interleaved=False, fragments=False,
                zeros_mode="original", **tk):
    group = 128
    d = workloads.w4a16(M, N, K, group, seed=0, scale_range=(0.002, 0.01) if zeros else (0.005, 0.02),
                        zeros_range=(6, 10) if zeros else None)
    nbytes = workloads.w4a16_bytes(M, N, K, group, zeros=zeros)
    nc = _copies(nbytes)
    A = torch.from_numpy(d["A"]).to(dev)
    b0 = torch.from_numpy(d["B"]).view(torch.int8)
    if interleaved:
        # the word permutation the example applies before its fast decoder (example_dequant_gemv_fp16xint4.py:201-204)
        from tilelang_amd import quantize

        b0 = quantize.interleave_weight(b0, 4, "float16")
    if fragments:
        # offline re-ordering into the matrix instruction's operand order (the role of the reference's ladder weight
        # transform, example_dequant_gemm_fine_grained.py:136-354)
        from tilelang_amd import quantize

        b0 = quantize.prepack_w4_fragments(b0)
    Bs = [b0.to(dev).clone() for _ in range(nc)]
    Ss = [torch.from_numpy(d["Scale"]).to(dev).clone() for _ in range(nc)]
    Zs = [torch.from_numpy(d["Zeros"]).to(dev).clone() for _ in range(nc)] if zeros else None
    C = torch.empty((M, N), dtype=torch.float16, device=dev)
    kern = tl.dequantize_gemv(M, N, K, group_size=group, source_format="uint" if zeros else "int",
                              with_scaling=True, with_zeros=zeros, fast_decoding=interleaved, weight_fragments=fragments,
                              zeros_mode=zeros_mode)
    if zeros:
        fns = [(lambda i=i: kern(A, Bs[i], Ss[i], Zs[i], C, skip_tensor_validation=True)) for i in range(nc)]
    else:
        fns = [(lambda i=i: kern(A, Bs[i], Ss[i], C, skip_tensor_validation=True)) for i in range(nc)]
    ms, graphed = _time_launches(torch, fns, steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": nbytes, "flops": workloads.flops(M, N, K), "timing": graphed,
            "inputs": d, "out": C}


def bench_w2a16(torch, tl, M, N, K, steps, warmup, dev, fast=True, **tk):
    """The 2-bit case of dequantize_gemv: codes uniform over 0..3 (interleaved words, w = (c - 2) * s), group 128."""
    from tilelang_amd import quantize

    group = 128
    rng = np.random.default_rng(0)
    A = torch.from_numpy(rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)).to(dev)
    nbytes = N * K // 4 + 2 * N * K // group + 2 * M * K + 2 * M * N
    nc = _copies(nbytes)
    Bs = []
    for _ in range(nc):
        b = torch.from_numpy(rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)).view(torch.int8)
        Bs.append((quantize.interleave_weight(b, 2, "float16") if fast else b).to(dev).contiguous())
    Ss = [torch.from_numpy(rng.uniform(0.005, 0.02, size=(N, K // group)).astype(np.float16)).to(dev) for _ in range(nc)]
    C = torch.empty((M, N), dtype=torch.float16, device=dev)
    kern = tl.dequantize_gemv(M, N, K, num_bits=2, source_format="int", fast_decoding=fast, group_size=group, with_scaling=True)
    fns = [(lambda i=i: kern(A, Bs[i], Ss[i], C, skip_tensor_validation=True)) for i in range(nc)]
    ms, graphed = _time_launches(torch, fns, steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": nbytes, "flops": 2 * M * N * K, "timing": graphed}


def bench_mxfp4(torch, tl, workloads, M, N, K, steps, warmup, dev, **tk):
    d = workloads.mxfp4(M, N, K, seed=0, scale_bias=127)
    A = torch.from_numpy(d["A"]).to(dev).view(torch.bfloat16)
    # rotate over enough copies of the weights that A + the copies + C exceed the 256 MiB last-level cache: the
    # cold-cache policy of the reference's do_bench (tilelang/profiler/bench.py:190-195), as for the GEMV rows
    nc = max(3, -(-(256 << 20) // max(1, N * K // 2)) - 3)
    Bs = [torch.from_numpy(d["B"]).to(dev).clone() for _ in range(nc)]
    S = torch.from_numpy(d["Scale"]).to(dev)
    bias = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    kern = tl.matmul_bf16_mxfp4(M, N, K, weight_format="e2m1", scale_bias=127)
    out = [None]

    def mk(i):
        def f():
            out[0] = kern(A, Bs[i], S, bias, skip_tensor_validation=True)
        return f

    ms, graphed = _time_launches(torch, [mk(i) for i in range(nc)], steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": workloads.mxfp4_bytes(M, N, K), "flops": workloads.flops(M, N, K), "timing": graphed,
            "inputs": d, "out": out[0]}


def bench_mxfp4_blockscaled(torch, tl, workloads, M, N, K, steps, warmup, dev, **tk):
    """Both operands MXFP4 (e2m1 codes + one E8M0 byte per 32 k), block-scaled matrix instruction."""
    d = workloads.mxfp4_mxfp4(M, N, K, seed=0)
    nbytes = workloads.mxfp4_mxfp4_bytes(M, N, K)
    nc = _copies(nbytes, hi=12)
    A = torch.from_numpy(d["A"]).to(dev)
    SA = torch.from_numpy(d["SFA"]).to(dev)
    Bs = [torch.from_numpy(d["B"]).to(dev).clone() for _ in range(nc)]
    SBs = [torch.from_numpy(d["SFB"]).to(dev).clone() for _ in range(nc)]
    bias = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    kern = tl.matmul_mxfp4_mxfp4(M, N, K)
    out = [None]

    def mk(i):
        def f():
            out[0] = kern(A, Bs[i], SA, SBs[i], bias, skip_tensor_validation=True)
        return f

    ms, graphed = _time_launches(torch, [mk(i) for i in range(nc)], steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": nbytes, "flops": workloads.flops(M, N, K), "timing": graphed}


def bench_bitnet(torch, tl, workloads, M, N, K, steps, warmup, dev, interleaved=True, kernel=None, fragments=False, **tk):
    """BitLinear forward on quantised operands: int8 x 2-bit (offset-binary ternary), fused acc/s_a/s_w epilogue.

    ``interleaved``: the packed words went through ``interleave_weight(qw, 2, "int8")`` on the host, once, as in
    the reference's kernel benchmarks (examples/bitnet-1.58b/kernel_benchmark/
    tilelang_bitnet_158_int8xint2_prefill.py:372-373, ..._decode.py:249-250); False: the plain packing.
    ``fragments``: the words then re-ordered offline into the matrix instruction's operand order."""
    d = workloads.bitnet(M, N, K, seed=0)
    nbytes = workloads.bitnet_bytes(M, N, K)
    nc = _copies(nbytes, hi=40)
    A = torch.from_numpy(d["A"]).to(dev)
    B0 = torch.from_numpy(d["B"]).view(torch.int8)
    if interleaved:
        B0 = tl.quantize.interleave_weight(B0, 2, "int8")
    if fragments:
        B0 = tl.quantize.prepack_i2_fragments(B0)
    Bs = [B0.to(dev).clone() for _ in range(nc)]
    s_a = torch.from_numpy(np.asarray(d["s_a"], dtype=np.float32)).to(dev)
    kern = tl.bitlinear_int8xint2(M, N, K, float(d["s_w"]), convention="offset", interleaved=interleaved, kernel=kernel,
                                  weight_fragments=fragments)
    out = [None]

    def mk(i):
        def f():
            out[0] = kern(A, Bs[i], s_a, skip_tensor_validation=True)
        return f

    ms, graphed = _time_launches(torch, [mk(i) for i in range(nc)], steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": nbytes, "flops": workloads.flops(M, N, K), "timing": graphed}


def bench_activation_quant(torch, tl, M, K, steps, warmup, dev, **tk):
    """BitLinear activation quantiser (fp16 rows -> int8 + fp32 scale), the step before the W2A8 GEMM."""
    nc = _copies(3 * M * K, hi=12)
    gen = torch.Generator(device="cpu").manual_seed(0)
    xs = [torch.randn((M, K), generator=gen, dtype=torch.float32).to(torch.float16).to(dev) for _ in range(nc)]
    kern = tl.bitnet_activation_quant(M, K)
    out = [None]

    def mk(i):
        def f():
            out[0] = kern(xs[i], skip_tensor_validation=True)
        return f

    ms, graphed = _time_launches(torch, [mk(i) for i in range(nc)], steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": 3 * M * K + 4 * M, "flops": 2 * M * K, "timing": graphed}


def bench_mxfp4_quant(torch, tl, N, K, steps, warmup, dev, **tk):
    """MXFP4 weight quantiser (bf16 -> e2m1 codes + one scale byte per 32), the producer of the GEMM's B and Scale."""
    nbytes = 2 * N * K + N * K // 2 + N * K // 32
    nc = _copies(nbytes, hi=6)
    gen = torch.Generator(device="cpu").manual_seed(0)
    ws = [(torch.randn((N, K), generator=gen, dtype=torch.float32) * 0.05).to(torch.bfloat16).to(dev) for _ in range(nc)]
    kern = tl.quantize_bf16_mxfp4(N, K)
    out = [None]

    def mk(i):
        def f():
            out[0] = kern(ws[i], skip_tensor_validation=True)
        return f

    ms, graphed = _time_launches(torch, [mk(i) for i in range(nc)], steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": nbytes, "flops": 2 * N * K, "timing": graphed}


def bench_int4(torch, tl, workloads, M, N, K, a_packed, steps, warmup, dev, **tk):
    """W4A8 (int8 x int4, Ct[N,M] int32) or int4 x int4 (C[M,N] int32), exact."""
    if a_packed:
        from tilelang_amd import quantize

        d = workloads.int4_int4(M, N, K, seed=0)
        kern = tl.matmul_nt_int4(M, N, K)
        nbytes = M * K // 2 + N * K // 2 + 4 * M * N
        A = quantize.pack_int4(torch.from_numpy(d["A_logical"])).to(dev)
        B = quantize.pack_int4(torch.from_numpy(d["B_logical"])).to(dev)
    else:
        d = workloads.int8_int4(M, N, K, seed=0)
        kern = tl.matmul_int8xint4(M, N, K)
        nbytes = M * K + N * K // 2 + 4 * M * N
        A = torch.from_numpy(d["A"]).to(dev)
        B = torch.from_numpy(d["B"]).to(dev)
    out = [None]

    def f():
        out[0] = kern(A, B, skip_tensor_validation=True)

    ms, graphed = _time_launches(torch, [f], steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": nbytes, "flops": workloads.flops(M, N, K), "timing": graphed}


def bench_int8_gemv(torch, tl, M, N, K, bits, steps, warmup, dev, **tk):
    """The integer branch of dequantize_gemv (int8 activations, int32 out) with the fast decoder: 4-bit words through
    interleave_weight(., 4, "int8"), w = q - 7 (decode_i4s_to_i8s)."""
    from tilelang_amd import quantize

    rng = np.random.default_rng(0)
    A = torch.from_numpy(rng.integers(-127, 128, size=(M, K), dtype=np.int8)).to(dev)
    nbytes = N * K * bits // 8 + M * K + 4 * M * N
    nc = _copies(nbytes)
    Bs = []
    for _ in range(nc):
        b = torch.from_numpy(rng.integers(0, 256, size=(N, K * bits // 8), dtype=np.uint8)).view(torch.int8)
        Bs.append(quantize.interleave_weight(b, bits, "int8").to(dev).contiguous())
    C = torch.empty((M, N), dtype=torch.int32, device=dev)
    kern = tl.dequantize_gemv(M, N, K, "int8", "int32", "int32", num_bits=bits, source_format="int", fast_decoding=True)
    fns = [(lambda i=i: kern(A, Bs[i], C, skip_tensor_validation=True)) for i in range(nc)]
    ms, graphed = _time_launches(torch, fns, steps, warmup, **tk)
    return {"us": ms * 1e3, "bytes": nbytes, "flops": 2 * M * N * K, "timing": graphed}


def _row(config, r, bound, peak):
    sec = r["us"] * 1e-6
    row = {"config": config, "us": r["us"], "us_min": r["timing"]["us_min"], "GB/s": r["bytes"] / sec / 1e9, "TFLOP/s": r["flops"] / sec / 1e12, "bound": bound}
    row["frac"] = (r["bytes"] / sec / HBM_PEAK) if bound == "hbm" else (r["flops"] / sec / peak)
    # progress on stderr (stdout carries the one JSON line): a row at a time, so that a run under a profiler, which
    # takes minutes, is seen to be alive
    print(f"[bench] {config}: {r['us']:.1f} us", file=sys.stderr, flush=True)
    return row


def _median_time(fn, budget_s, min_runs=3, max_runs=25):
    fn()  # warm-up
    times, t_start = [], time.perf_counter()
    while len(times) < max_runs and (len(times) < min_runs or time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times)), len(times)


def cpu_baselines(budget_s=16.0):
    """The reference's ``ref_program`` of every benchmark configuration restated in torch, on CPU tensors and all
    host cores: dequantise and matmul timed separately (median of at least 3 runs each).  Configurations whose
    CPU time is seconds are timed on the first rows of the weight matrix and scaled; `sample` says which.
    Returns (headline entry, per-configuration list)."""
    import torch

    from oracle import ref_torch
    from tilelang_amd import workloads

    torch.set_num_threads(os.cpu_count() or 1)
    cores = torch.get_num_threads()
    rows_out = []

    def leg(name, n_full, n_rows, make, dequant, matmul, share):
        d = make(n_rows)
        t_deq, r1 = _median_time(lambda: dequant(d), share / 2)
        W = dequant(d)
        t_mm, r2 = _median_time(lambda: matmul(d, W), share / 2)
        f = n_full / n_rows
        rows_out.append({"config": name, "dequant_us": t_deq * f * 1e6, "matmul_us": t_mm * f * 1e6,
                         "us": (t_deq + t_mm) * f * 1e6, "cores": cores,
                         "sample": (f"all {n_full} weight rows" if n_rows == n_full else
                                    f"first {n_rows} of {n_full} weight rows x {f:.0f}") + f", median of {r1}/{r2} runs"})
        return rows_out[-1]

    def w4(M, N, K, zeros, rows, share, tag):
        def make(n):
            d = workloads.w4a16(M, n, K, 128, seed=0, scale_range=(0.002, 0.01) if zeros else (0.005, 0.02),
                                zeros_range=(6, 10) if zeros else None)
            return {k: torch.from_numpy(v) for k, v in d.items()}
        return leg(f"{tag} M={M} N={N} K={K}", N, rows, make,
                   lambda d: ref_torch.dequant_w4a16(d["B"], d["Scale"], d.get("Zeros")),
                   lambda d, W: ref_torch.matmul_f32(d["A"], W, torch.half), share)

    unit = budget_s / 24.0
    w4(1, 1024, 1024, False, 1024, 0.5 * unit, "w4a16_gemv (the CPU-path configuration)")
    head = w4(1, 28672, 8192, False, 28672, 4 * unit, "w4a16_gemv")
    for (n, k) in [(11008, 4096), (4096, 11008), (4096, 4096)]:
        w4(1, n, k, False, n, 1 * unit, "w4a16_gemv")
    for m in (4, 16, 64):
        w4(m, 28672, 8192, True, 28672, 2 * unit, "w4a16_zeros")

    def mx_make(n):
        d = workloads.mxfp4(4096, n, 8192, seed=0, scale_bias=127)
        return {"A": torch.from_numpy(d["A"]).view(torch.bfloat16), "B": torch.from_numpy(d["B"]), "Scale": torch.from_numpy(d["Scale"])}
    leg("mxfp4_gemm M=4096 N=8192 K=8192", 8192, 1024, mx_make,
        lambda d: ref_torch.dequant_mxfp4_e2m1(d["B"], d["Scale"], 127),
        lambda d, W: ref_torch.matmul_f32(d["A"], W, torch.bfloat16), 3 * unit)

    for m, rows in ((1, 8192), (256, 8192), (2048, 2048)):
        def bn_make(n, m=m):
            d = workloads.bitnet(m, n, 8192, seed=0)
            return {"A": torch.from_numpy(d["A"]), "B": torch.from_numpy(d["B"]),
                    "s_a": torch.from_numpy(np.asarray(d["s_a"], dtype=np.float32)), "s_w": float(d["s_w"])}
        leg(f"bitnet_w2a8 M={m} N=8192 K=8192", 8192, rows, bn_make,
            lambda d: ref_torch.dequant_bitnet(d["B"]),
            lambda d, W: ref_torch.bitnet_epilogue(torch.matmul(d["A"].float(), W.T), d["s_a"], d["s_w"]), 2 * unit)

    cpu = {
        "value": head["us"], "unit": "us", "cores": cores, "kind": "port",
        "dequant_us": head["dequant_us"], "matmul_us": head["matmul_us"],
        "sample": "torch-CPU ref_program (unpack, (q-8)*s in fp16; fp32 matmul) of the headline GEMV, " + head["sample"],
        "note": "the reference's other CPU path, TileLang's LLVM CPU backend, cannot be built here (it needs the TVM "
                "submodule and LLVM, both absent), so the baseline is the torch restatement of ref_program only",
        "configs": rows_out,
    }
    return cpu


def check_timed_outputs(head, mx):
    """What the timed launches left in their output buffers against the torch-CPU ``ref_program`` (rtol = atol = 1e-2,
    the tolerance the reference's own checks use), after the timing and outside it: every output of the headline
    GEMV; for the MXFP4 GEMM the columns of 64 weight rows spread over N.  Returns ``(gemv, gemm)`` dictionaries
    ``{"checked": bool, "max_abs_err": float, "compared": int}``."""
    import torch

    from oracle import ref_torch

    def verdict(got, ref):
        got, ref = got.float(), ref.float()
        ok = bool(torch.isfinite(got).all()) and bool(torch.allclose(got, ref, rtol=1e-2, atol=1e-2))
        return {"checked": ok, "max_abs_err": float((got - ref).abs().max()), "compared": got.numel()}

    d = {k: torch.from_numpy(v) for k, v in head["inputs"].items()}
    gemv = verdict(head["out"].cpu(), ref_torch.ref_w4a16(d["A"], d["B"], d["Scale"], d.get("Zeros")))
    gemm = None
    if mx is not None:
        d = mx["inputs"]
        n_rows = d["B"].shape[0]
        rows = torch.arange(0, n_rows, max(1, n_rows // 64))[:64]
        ref = ref_torch.ref_mxfp4_e2m1(torch.from_numpy(d["A"]).view(torch.bfloat16), torch.from_numpy(d["B"])[rows],
                                       torch.from_numpy(d["Scale"])[rows], 127)
        gemm = verdict(mx["out"].cpu()[:, rows], ref)
    return gemv, gemm


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=12)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--headline-only", action="store_true", help="skip the per-configuration table")
    ap.add_argument("--no-graph", action="store_true",
                    help="time plain launches instead of replaying a HIP graph (for counter runs under rocprofv3 --pmc)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain elementwise copy of 128 MiB a few times: under `rocprofv3 --pmc FETCH_SIZE` / "
                         "`WRITE_SIZE` its counters give the factor that turns counter units into bytes")
    args = ap.parse_args()
    global USE_GRAPH
    USE_GRAPH = not args.no_graph
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (the path would shard by output rows N, "
                 "each GPU holding its rows of the weights and a replica of the activations, with no communication)")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import tilelang_amd as tl
    from tilelang_amd import workloads

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # ---- headline: M=1 W4A16 GEMV at N=28672, K=8192 ------------------------------------------
    M, N, K = 1, 28672, 8192
    S, W = args.steps, args.warmup
    head = bench_w4a16(torch, tl, workloads, M, N, K, False, S, W, dev)
    us = head["us"]
    gbs = head["bytes"] / (us * 1e-6) / 1e9
    traffic, traffic_source = gemv_hbm_traffic()
    roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": gbs * 1e9 / HBM_PEAK,
            "traffic": traffic, "traffic_source": traffic_source,
            "kernel": GEMV_KERNEL, "algorithmic_bytes": head["bytes"],
            "us_min": head["timing"]["us_min"], "us_mean": head["timing"]["us_mean"]}

    if args.copy_calibration:
        src = torch.full((128 << 20,), 3, dtype=torch.uint8, device=dev).view(torch.int32)
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.add(src, 1, out=dst)  # reads 128 MiB, writes 128 MiB
        torch.cuda.synchronize()
        del src, dst

    shapes = []
    mx_run = None
    if not args.headline_only:
        gemm = {"min_launches": 24, "max_launches": 48}  # launches of hundreds of microseconds: a replay is milliseconds
        for (m, n, kk) in [(1, 1024, 1024), (1, 11008, 4096), (1, 4096, 11008), (1, 4096, 4096)]:
            r = bench_w4a16(torch, tl, workloads, m, n, kk, False, S, W, dev)
            shapes.append(_row(f"w4a16_gemv M={m} N={n} K={kk}", r, "hbm", MFMA_BF16_PEAK))
        for m in (4, 16, 64):
            r = bench_w4a16(torch, tl, workloads, m, 28672, 8192, True, S, W, dev)
            row = _row(f"w4a16_zeros M={m} N=28672 K=8192", r, "hbm", MFMA_BF16_PEAK)
            row["frac_mfma"] = r["flops"] / (r["us"] * 1e-6) / MFMA_BF16_PEAK
            shapes.append(row)
        # a matrix of few rows and a long K: K split over workgroups, fp32 partial sums in a workspace.  Left out of
        # counter runs (--no-graph): under `rocprofv3 --pmc` this row's pair of dependent kernels has stalled, as a
        # replayed graph and once as plain launches, while tests, timing and the kernel trace run it without trouble.
        if USE_GRAPH:
            r = bench_w4a16(torch, tl, workloads, 16, 4096, 14336, True, S, W, dev)
            shapes.append(_row("w4a16_zeros M=16 N=4096 K=14336", r, "hbm", MFMA_BF16_PEAK))
        for m in (4, 16):
            r = bench_w4a16(torch, tl, workloads, m, 28672, 8192, True, S, W, dev, fragments=True)
            shapes.append(_row(f"w4a16_zeros M={m} N=28672 K=8192 (weights re-ordered offline into the matrix instruction's operand order)",
                               r, "hbm", MFMA_BF16_PEAK))
        r = bench_w2a16(torch, tl, 1, 28672, 8192, S, W, dev)
        shapes.append(_row("w2a16_gemv M=1 N=28672 K=8192 (num_bits=2, interleaved words, (c-2)*s)", r, "hbm", MFMA_BF16_PEAK))
        r = bench_int8_gemv(torch, tl, 1, 28672, 8192, 4, S, W, dev)
        shapes.append(_row("w4a8_gemv M=1 N=28672 K=8192 (int8 activations, interleaved words, q - 7, int32 out)", r, "hbm", MFMA_I8_PEAK))
        r = bench_mxfp4(torch, tl, workloads, 4096, 8192, 8192, S, W, dev, **gemm)
        mx_run = r
        shapes.append(_row("mxfp4_gemm M=4096 N=8192 K=8192", r, "mfma", MFMA_BF16_PEAK))
        # MXFP4 weights at one row, the headline matrix's shape: the dot-product kernel (no matrix instruction)
        r = bench_mxfp4(torch, tl, workloads, 1, 28672, 8192, S, W, dev)
        shapes.append(_row("mxfp4_gemv M=1 N=28672 K=8192", r, "hbm", MFMA_BF16_PEAK))
        # the same weights at a decode batch: activations resident in registers, weights streamed once
        r = bench_mxfp4(torch, tl, workloads, 16, 8192, 8192, S, W, dev)
        shapes.append(_row("mxfp4_gemm M=16 N=8192 K=8192", r, "hbm", MFMA_BF16_PEAK))
        for m in (1, 16, 256, 2048):
            r = bench_bitnet(torch, tl, workloads, m, 8192, 8192, S, W, dev, **({} if m <= 16 else gemm))
            shapes.append(_row(f"bitnet_w2a8 M={m} N=8192 K=8192", r, "hbm" if m <= 16 else "mfma", MFMA_I8_PEAK))
        # 17 to 32 rows: the register-resident form on blocks of 32 weight rows (up to 16 rows: blocks of 16, the row above)
        r = bench_bitnet(torch, tl, workloads, 32, 28672, 8192, S, W, dev)
        shapes.append(_row("bitnet_w2a8 M=32 N=28672 K=8192", r, "hbm", MFMA_I8_PEAK))
        r = bench_bitnet(torch, tl, workloads, 256, 8192, 8192, S, W, dev, fragments=True, **gemm)
        shapes.append(_row("bitnet_w2a8 M=256 N=8192 K=8192 (weights re-ordered offline into the matrix instruction's operand order)",
                           r, "mfma", MFMA_I8_PEAK))
        r = bench_bitnet(torch, tl, workloads, 2048, 8192, 8192, S, W, dev, interleaved=False, **gemm)
        shapes.append(_row("bitnet_w2a8 M=2048 N=8192 K=8192 (plain packing, not interleaved)", r, "mfma", MFMA_I8_PEAK))
        r = bench_w4a16(torch, tl, workloads, 4096, 8192, 8192, True, S, W, dev, **gemm)
        shapes.append(_row("w4a16_zeros_gemm M=4096 N=8192 K=8192", r, "mfma", MFMA_BF16_PEAK))
        r = bench_w4a16(torch, tl, workloads, 4096, 8192, 8192, True, S, W, dev, interleaved=True, **gemm)
        shapes.append(_row("w4a16_zeros_gemm M=4096 N=8192 K=8192 (interleaved words, the example's fast-decode layout)", r, "mfma", MFMA_BF16_PEAK))
        r = bench_w4a16(torch, tl, workloads, 4096, 8192, 8192, True, S, W, dev, zeros_mode="folded", **gemm)
        shapes.append(_row("w4a16_zeros_gemm M=4096 N=8192 K=8192 (zeros_mode folded: fma(q, s, -rne16(z s)), the library's cheaper form)", r, "mfma", MFMA_BF16_PEAK))
        r = bench_mxfp4_quant(torch, tl, 8192, 8192, S, W, dev, **gemm)
        shapes.append(_row("mxfp4_quantize N=8192 K=8192", r, "hbm", MFMA_BF16_PEAK))
        r = bench_activation_quant(torch, tl, 2048, 8192, S, W, dev)
        shapes.append(_row("bitnet_activation_quant M=2048 K=8192", r, "hbm", MFMA_I8_PEAK))
        r = bench_int4(torch, tl, workloads, 4096, 4096, 4096, False, S, W, dev, **gemm)
        shapes.append(_row("w4a8_gemm M=4096 N=4096 K=4096 (Ct int32)", r, "mfma", MFMA_I8_PEAK))
        r = bench_int4(torch, tl, workloads, 4096, 4096, 4096, True, S, W, dev, **gemm)
        shapes.append(_row("int4xint4_gemm M=4096 N=4096 K=4096", r, "mfma", MFMA_I8_PEAK))
        r = bench_mxfp4_blockscaled(torch, tl, workloads, 4096, 8192, 8192, S, W, dev, **gemm)
        shapes.append(_row("mxfp4_x_mxfp4_blockscaled_gemm M=4096 N=8192 K=8192", r, "mfma", MFMA_FP4_PEAK))
        # what a launch costs before any byte moves: the same timing of the smallest problem the library takes
        r = bench_w4a16(torch, tl, workloads, 1, 16, 1024, False, S, W, dev)
        shapes.append({"config": "launch floor: w4a16_gemv M=1 N=16 K=1024 (back-to-back launches in a graph, 10 KB of work)",
                       "us": r["us"], "us_min": r["timing"]["us_min"], "bound": "launch"})

    # the metric's second half: the M=4096 MXFP4-weight GEMM against the dense bf16 MFMA peak
    roof_gemm = None
    for row in shapes:
        if row["config"].startswith("mxfp4_gemm M=4096"):
            roof_gemm = {"bound": "mfma", "achieved": row["TFLOP/s"], "peak": MFMA_BF16_PEAK / 1e12, "unit": "TFLOP/s",
                         "frac": row["frac"], "us": row["us"], "kernel": "gemm_kernel_dma<MxPolicy<e2m1>,4,4>",
                         "workload": "A bf16 [4096,8192] x e2m1 [8192,8192] with e8m0 scales per 32, bf16 out",
                         "algorithmic_flops": 2 * 4096 * 8192 * 8192}
    # What the matrix pipe sustains on random operands with nothing beside it, measured now on this device: the
    # published peak assumes the top clock, which operands that toggle like real data do not hold.
    from tilelang_amd import profiler as tl_profiler

    sustained = {}
    for dt in ("bfloat16", "float16", "int8", "fp4"):
        m = tl_profiler.mfma_sustained_rate(dt, device=dev)
        sustained[dt] = {"T(FL)OP/s": m["ops_per_s"] / 1e12, "ms_per_launch": m["ms_per_launch"],
                         "frac_of_published_peak": m["ops_per_s"] / {"int8": MFMA_I8_PEAK, "fp4": MFMA_FP4_PEAK}.get(dt, MFMA_BF16_PEAK)}
    for row in shapes:  # every matrix-pipe row also against the matrix-only rate of its operand type
        if row.get("bound") == "mfma" and "TFLOP/s" in row:
            cfg = row["config"]
            dt = ("fp4" if cfg.startswith("mxfp4_x_mxfp4") else "bfloat16" if cfg.startswith("mxfp4_gemm") else
                  "float16" if cfg.startswith("w4a16") else "int8")
            row["frac_of_sustained"] = row["TFLOP/s"] / sustained[dt]["T(FL)OP/s"]
    if roof_gemm is not None:
        roof_gemm["sustained_mfma_only"] = sustained["bfloat16"]["T(FL)OP/s"]
        roof_gemm["frac_of_sustained"] = roof_gemm["achieved"] / sustained["bfloat16"]["T(FL)OP/s"]
    cpu = None
    if not args.no_cpu:
        # the CPU leg also looks at what was timed: a kernel that regressed to wrong results must not print a figure
        gemv_check, gemm_check = check_timed_outputs(head, mx_run)
        roof.update(gemv_check)
        if roof_gemm is not None and gemm_check is not None:
            roof_gemm.update(gemm_check)
        if not gemv_check["checked"] or (gemm_check is not None and not gemm_check["checked"]):
            sys.exit(f"bench.py: the timed kernels' outputs do not match the CPU ref_program: gemv {gemv_check}, gemm {gemm_check}")
        cpu = cpu_baselines()

    line = {
        "metric": "M=1 W4A16 GEMV us + %HBM peak; M=4096 dequant GEMM TFLOP/s + %MFMA peak",
        "value": us,
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": us / 1e3,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "W4A16 decode GEMV M=1 N=28672 K=8192 group=128 w=(q-8)*s, fp32 accumulate, fp16 out",
                   "weights_rotated_over_copies": _copies(head["bytes"]), "timed_with": ("hip graph replay" if head["timing"]["graph"] else "direct launches")
                   + f", median of {head['timing']['replays']} event-bracketed replays of {head['timing']['launches_per_replay']} launches"
                     f" after {head['timing']['settle_replays']} untimed replays (at least 50 ms)"},
        "roofline": roof,
        "roofline_gemm": roof_gemm,
        "mfma_sustained": {"what": "call_mfma_rate: 16 matrix instructions of a 128 x 128 wave tile in a loop on random operands, one "
                                   "workgroup of four waves per CU, no memory / LDS / decode work; median of 8 launches of about 5 ms "
                                   "after 60 ms of untimed launches", **sustained},
        "cpu_baseline": cpu,
        "shapes": shapes,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
