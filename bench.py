#!/usr/bin/env python3
"""Headline benchmark of the GGUF quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  ``value`` is the whole-job throughput of the batch-1 Q4_K
decode GEMV (BASELINE config 2) in algorithmic GB/s: one *step* runs
``ops.ggml_mul_mat_vec_a8`` once on each of the three Llama-3-8B-like
projections [4096,4096], [14336,4096], [4096,14336] (activation quantisation
included), rotating over distinct weight copies that together exceed the 256 MB
Infinity Cache, with every input resident in HBM before the clock starts.

Beside it:
  roofline      the GEMV kernel against the 8 TB/s HBM peak, timed per launch with HIP events over at least 100 launches
  mmq           the second half of the metric: Q6_K prefill GEMM at M=512 (BASELINE config 3) in TOPS against the
                5.03 POPS dense int8 MFMA peak, on the operator's default engine: exact int8 dot products on
                v_mfma_i32_32x32x32_i8 with fp32 block scales, the reference's arithmetic.  The opt-in engine that
                multiplies dequantized operands on half-precision MFMA is timed beside it as ``half_engine``
  other_configs the remaining BASELINE configurations (1: Q8_0 small, 2: batch sweep, 4: codebook formats, 5: MoE layer)
  cpu_baseline  the reference's CPU path (block dequantize + fp32 matmul) restated in numpy/torch,
                timed on one host core on a bounded sample of the same workload
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
INT8_PEAK_TOPS = 5033.0        # dense int8 MFMA, double-K shapes v_mfma_i32_32x32x32_i8 / 16x16x64_i8 (256 CU x 8192 op/clk x 2.4 GHz)
INT8_LEGACY_PEAK_TOPS = 2516.0 # the legacy-K shapes (v_mfma_i32_32x32x16_i8, 16x16x32_i8) run at half of it
# the matrix instruction the integer engine issues per format: formats whose weight scale changes every 16 values
# multiply 16 values at a time
MMQ_INSTRUCTION = {14: "v_mfma_i32_32x32x16_i8", 11: "v_mfma_i32_32x32x16_i8"}
F16_PEAK_TFLOPS = 2516.0       # dense half-precision MFMA
Q4_K, Q6_K = 12, 14
CFG2_SHAPES = [(4096, 4096), (14336, 4096), (4096, 14336)]
CFG3_SHAPES = [(18944, 3584), (3584, 18944)]
ROTATE_BYTES = 640 << 20       # distinct weight bytes walked per rotation (> 2x the 256 MB cache)
MIN_LAUNCHES = 100             # every reported per-launch time is an average over at least this many launches
# HBM bytes per launch cannot be read from inside this process: they come from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# runs of `bench.py --profile`, each counter scaled by what it reads for a 256 MiB device copy.  The summary of those runs
# carries one `traffic_bytes_per_launch <key> = <bytes>` line per kernel; without the file the figure is null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "pmc_hbm_traffic_mmvq_q4_k_mmq_q6_k.txt")


def _traffic(key):
    try:
        text = open(TRAFFIC_FILE).read()
    except OSError:
        return None
    m = re.search(rf"^traffic_bytes_per_launch\s+{re.escape(key)}\s*=\s*([0-9.eE+]+)", text, re.M)
    return float(m.group(1)) if m else None


def _events_ms(fn, iters):
    """Average milliseconds per call of ``fn`` over ``iters`` back-to-back calls, by HIP events on torch's
    current stream (the stream the kernels are launched on)."""
    import torch

    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(iters):
        fn(i)
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def _graph_ms(fn, calls, replays):
    """Same, with the calls captured once into a HIP graph and replayed, so host launch cost is excluded."""
    import torch

    for i in range(min(calls, 3)):
        fn(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(calls):
            fn(i)
    g.replay()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        g.replay()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / (replays * calls)


def _timed_ms(fn, calls, eager=False):
    """Milliseconds per call over at least MIN_LAUNCHES calls: graph-timed where the calls can be captured (and
    ``eager`` is not asked for), event-timed otherwise."""
    import torch

    replays = -(-MIN_LAUNCHES // calls)
    if not eager:
        try:
            return _graph_ms(fn, calls, replays)
        except Exception:  # a call that cannot be captured: time the eager launches
            torch.cuda.synchronize()
    for i in range(3):
        fn(i)
    return _events_ms(fn, calls * replays)


def _other_configs(rng, dev, w_14336x4096):
    """The BASELINE configurations the headline does not cover, each as time per call and the rate its roofline names."""
    import torch

    from vllm_gguf_plugin_prism_amd import dispatch, ops, synth

    Q8_0, Q4_0, IQ2_XXS, IQ4_XS = 8, 2, 16, 23
    res = {}

    def gemv_bytes(qt, n, k, m):
        qk, bs = ops.quant_sizes(qt)
        return n * (k // qk) * bs + 2 * m * k + 2 * m * n

    def xs(m, k):
        return torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(torch.float16).to(dev)

    # config 1: Q8_0 [3072,1024] dequantize and batch-1 GEMV (3.3 MB: launch-bound)
    n, k = 3072, 1024
    w = torch.from_numpy(synth.make_weights(rng, Q8_0, n, k)).to(dev)
    x = xs(1, k)
    ms = _timed_ms(lambda i: ops.ggml_dequantize(w, Q8_0, n, k, torch.float16), 20)
    res["config1_q8_0_dequant_fp16"] = {"us": ms * 1e3, "GBps": (w.numel() + 2 * n * k) / (ms * 1e-3) / 1e9}
    ms = _timed_ms(lambda i: ops.ggml_mul_mat_vec_a8(w, x, Q8_0, n), 20)
    res["config1_q8_0_gemv_bs1"] = {"us": ms * 1e3, "GBps": gemv_bytes(Q8_0, n, k, 1) / (ms * 1e-3) / 1e9}

    # config 2: batch sweep on [14336,4096]; the reference's policy sends batch 4 and 8 at this N to the tile GEMM
    n, k = 14336, 4096
    copies = [torch.from_numpy(w_14336x4096).to(dev)]
    copies += [copies[0].clone() for _ in range(19)]          # 20 x 33 MB, walked in turn
    for b in (1, 2, 4, 8, 16, 32):      # (the baseline names 1, 2, 4, 8; 16 and 32 show the few-row tile route)
        x = xs(b, k)
        path = dispatch.select_mul_mat_path(Q4_K, b, n)
        ms = _timed_ms(lambda i: dispatch.fused_mul_mat_gguf(x, copies[i % 20], Q4_K), 20)
        res[f"config2_q4_k_14336x4096_bs{b}"] = {"path": path, "us": ms * 1e3,
                                                "GBps": gemv_bytes(Q4_K, n, k, b) / (ms * 1e-3) / 1e9}
        if path != "mmvq" and b <= 8:
            ms = _timed_ms(lambda i: ops.ggml_mul_mat_vec_a8(copies[i % 20], x, Q4_K, n), 20)
            res[f"config2_q4_k_14336x4096_bs{b}_gemv"] = {"path": "mmvq (forced)", "us": ms * 1e3,
                                                         "GBps": gemv_bytes(Q4_K, n, k, b) / (ms * 1e-3) / 1e9}
    del copies

    # config 4: codebook formats, raw valid blocks
    for qt, name, n, k in ((IQ4_XS, "iq4_xs", 5120, 5120), (IQ2_XXS, "iq2_xxs", 17408, 5120)):
        nc = 16
        base = torch.from_numpy(synth.random_blocks(rng, qt, n, k)).to(dev)
        cp = [base] + [base.clone() for _ in range(nc - 1)]
        x = xs(1, k)
        ms = _timed_ms(lambda i: ops.ggml_mul_mat_vec_a8(cp[i % nc], x, qt, n), nc)
        res[f"config4_{name}_gemv_bs1"] = {"us": ms * 1e3, "GBps": gemv_bytes(qt, n, k, 1) / (ms * 1e-3) / 1e9}
        x = xs(256, k)
        ms = _timed_ms(lambda i: dispatch.fused_mul_mat_gguf(x, base, qt), 10)
        res[f"config4_{name}_m256_dequant_then_gemm"] = {"us": ms * 1e3, "TFLOPS": 2.0 * 256 * n * k / (ms * 1e-3) / 1e12}
        ms = _timed_ms(lambda i: ops.ggml_mul_mat_a8(base, x, qt, n), 10)
        res[f"config4_{name}_m256_a8_gemm"] = {"us": ms * 1e3, "TOPS": 2.0 * 256 * n * k / (ms * 1e-3) / 1e12}
        del cp, base

    # config 5: 64-expert top-8 Q4_0 MoE layer, whole layer (two expert GEMMs, gated activation, weighted sum)
    E, H, I, top_k = 64, 2048, 1024, 8
    w13 = torch.from_numpy(np.stack([synth.random_blocks(rng, Q4_0, 2 * I, H) for _ in range(E)])).to(dev)
    w2 = torch.from_numpy(np.stack([synth.random_blocks(rng, Q4_0, H, I) for _ in range(E)])).to(dev)
    expert_bytes = (w13.numel() + w2.numel()) // E
    for t in (1, 64, 512):
        x = xs(t, H)
        tw, ids = torch.topk(torch.softmax(torch.randn(t, E, device=dev), 1), top_k)
        ids = ids.to(torch.int32).contiguous()   # (the routing weights stay fp32, as vLLM's fused_topk returns them)
        ms = _timed_ms(lambda i: dispatch.fused_moe_gguf(x, w13, w2, tw, ids, Q4_0, Q4_0, "silu"), 5)
        distinct = int(torch.unique(ids).numel())
        res[f"config5_moe_q4_0_T{t}"] = {"path": dispatch.select_moe_path(Q4_0, Q4_0, t), "us": ms * 1e3,
                                         "TOPS": 2.0 * t * top_k * 3 * I * H / (ms * 1e-3) / 1e12,
                                         "distinct_expert_GBps": distinct * expert_bytes / (ms * 1e-3) / 1e9}
    # every entry against the roofline its operator is bound by: HBM for dequantize / GEMV / per-pair MoE (algorithmic
    # bytes; for the MoE layer each distinct expert once), int8 MFMA for the a8 tile GEMMs, half-precision MFMA for the
    # library GEMM of the dequantize-then-GEMM route
    for v in res.values():
        if "GBps" in v:
            v["roofline"] = {"bound": "hbm", "peak_GBps": HBM_PEAK_GBS, "frac": v["GBps"] / HBM_PEAK_GBS}
        elif v.get("path") == "vec" and "distinct_expert_GBps" in v:   # the per-pair MoE operator: weights read, each distinct expert once
            v["roofline"] = {"bound": "hbm (distinct experts once)", "peak_GBps": HBM_PEAK_GBS, "frac": v["distinct_expert_GBps"] / HBM_PEAK_GBS}
        elif "TOPS" in v:
            v["roofline"] = {"bound": "mfma int8", "peak_TOPS": INT8_PEAK_TOPS, "frac": v["TOPS"] / INT8_PEAK_TOPS}
        elif "TFLOPS" in v:
            v["roofline"] = {"bound": "mfma f16", "peak_TFLOPS": F16_PEAK_TFLOPS, "frac": v["TFLOPS"] / F16_PEAK_TFLOPS}
    return res


def _errors(got, want):
    """max-abs, rel-L2 and max-rel (over elements whose reference exceeds 1e-3 of the largest) of got against want."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = np.abs(got - want)
    big = np.abs(want) >= 1e-3 * np.abs(want).max()
    return {"max_abs": float(d.max()), "rel_l2": float(np.linalg.norm(got - want) / np.linalg.norm(want)),
            "max_rel": float((d[big] / np.abs(want[big])).max())}


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _probes(rng, dev):
    """What one launch can reach on this machine before any arithmetic, and where the GEMV kernel's time goes.

    Prints a text report (the profiles/ summaries are made from it).  Uses libgguf_probes.so: plain streaming reads by
    launch geometry over rotating matrix-sized buffers in one HIP graph, and the library's streaming GEMV kernel built
    with its phase trace on."""
    import ctypes

    import torch

    from vllm_gguf_plugin_prism_amd import build as _build, synth

    if not _build.PROBES_LIB.exists():
        raise RuntimeError(f"{_build.PROBES_LIB} is missing: python -m vllm_gguf_plugin_prism_amd.build")
    h = ctypes.CDLL(str(_build.PROBES_LIB))
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    h.gguf_probe_read.argtypes = [vp, i64, ci, ci, ci, ci, vp, vp]
    h.gguf_probe_mmvq_q4_k.argtypes = [vp, vp, vp, i64, i64, vp]
    h.gguf_probe_mmvq_trace.argtypes = [vp, ci]
    stream = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    print("== plain streaming read of one matrix-sized buffer per launch, 20 distinct buffers per HIP graph (660 MB walked)")
    print("   (a launch reads the buffer once, 16 bytes per lane and load; best of 3 graph replays)")
    for nbytes in (33030144, 9437184):
        bufs = [torch.full((nbytes,), i + 1, dtype=torch.uint8, device=dev) for i in range(20)]
        rows = []
        for threads, per_cu in ((256, 1), (256, 2), (256, 4), (256, 8), (256, 32), (512, 1), (512, 2), (512, 4), (1024, 1), (1024, 2)):
            for unroll in (2, 4, 8):
                for nt in (0, 1):
                    def call(i, threads=threads, per_cu=per_cu, unroll=unroll, nt=nt):
                        rc = h.gguf_probe_read(bufs[i % 20].data_ptr(), nbytes, threads, 256 * per_cu, unroll, nt, sink.data_ptr(), stream())
                        assert rc == 0
                    ms = min(_graph_ms(call, 20, 1) for _ in range(3))
                    rows.append((ms * 1e3, threads, per_cu, unroll, nt))
        rows.sort()
        print(f"-- {nbytes / 1e6:.1f} MB per launch: fastest and slowest geometries of {len(rows)}")
        for us, threads, per_cu, unroll, nt in rows[:6] + rows[-2:]:
            print(f"   {us:6.2f} us  {nbytes / us / 1e6:5.2f} TB/s  ({100 * nbytes / us / 1e6 / 8.0:4.1f} % of 8 TB/s)  {threads:4d} threads x {per_cu:2d} workgroups per CU, "
                  f"{unroll} loads in flight per lane, {'non-temporal' if nt else 'plain'} loads")
        del bufs

    print("== streaming GEMV kernel, Q4_K batch 1 fp16: wall-clock times of eight points, microseconds after the first wave")
    print("   of the launch entered (median over workgroups; first wave / last wave of a workgroup); 10 ns clock;")
    print("   the launch traced is the last of a HIP graph of back-to-back launches over rotating weight copies")
    for n, k in CFG2_SHAPES:
        ws = [torch.from_numpy(np.concatenate([synth.make_weights(rng, Q4_K, min(2048, n - r), k) for r in range(0, n, 2048)], axis=0)).to(dev)]
        ws += [ws[0].clone() for _ in range(int(700e6 // ws[0].numel()))]
        x = torch.from_numpy(rng.standard_normal((1, k)).astype(np.float32)).to(torch.float16).to(dev)
        y = torch.empty((1, n), dtype=torch.float16, device=dev)

        def launch(i):
            rc = h.gguf_probe_mmvq_q4_k(ws[i % len(ws)].data_ptr(), x.data_ptr(), y.data_ptr(), n, k, stream())
            assert rc == 0

        # back-to-back launches over all copies in one HIP graph; the trace buffer holds the last launch of a replay
        for i in range(3):
            launch(i)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(len(ws)):
                launch(i)
        acc = []
        nwg = 256
        for rep in range(12):
            g.replay()
            torch.cuda.synchronize()
            buf = (ctypes.c_ulonglong * (nwg * 16))()
            assert h.gguf_probe_mmvq_trace(buf, nwg) == 0
            t = np.frombuffer(buf, dtype=np.uint64).reshape(nwg, 2, 8)[:, :, [0, 5, 6, 7, 1, 2, 3, 4]].astype(np.int64)
            if rep >= 2:
                acc.append((t - t[:, :, 0].min()) * 0.01)
        t = np.median(np.stack(acc), axis=0)          # [workgroup][first/last wave][point], median over launches
        names = ("entered", "kernel arguments read", "activation requests out", "first weight requests out",
                 "own activations quantized", "all activations in LDS", "own rows walked", "results stored")
        print(f"-- [{n},{k}], {n * (k // 256) * 144 / 1e6:.1f} MB")
        for p, name in enumerate(names):
            a, b = np.median(t[:, 0, p]), np.median(t[:, 1, p])
            print(f"   {name:28s} {a:6.2f} / {b:6.2f}   (latest workgroup {t[:, :, p].max():6.2f})")
        del ws


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-mmq", action="store_true", help="skip the Q6_K MMQ leg")
    ap.add_argument("--no-other", action="store_true",
                    help="skip the other BASELINE configurations (1: Q8_0, 2: batch sweep, 4: i-quants, 5: MoE layer), "
                         "which otherwise go into an 'other_configs' object (about half a minute)")
    ap.add_argument("--profile", action="store_true",
                    help="counter-collection mode: eager launches only (no HIP graph), no CPU leg, no other configurations, "
                         "M=512 only for the MMQ leg, and one 256 MiB device copy at the end to calibrate byte counters")
    ap.add_argument("--probes", action="store_true",
                    help="print the measurement probes instead of the benchmark line: the plain-read ceiling of one launch "
                         "by geometry, and the phase timeline of the streaming GEMV kernel")
    args = ap.parse_args()
    if args.profile:
        args.no_cpu = args.no_other = True
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the operators shard by "
              "rows/columns of W with no communication). Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    from vllm_gguf_plugin_prism_amd import ops, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(0)
    torch.manual_seed(0)           # the MoE routing of the other configurations is drawn with torch
    if args.probes:
        _probes(rng, dev)
        return 0

    # ---------------------------------------------------------------- config 2: Q4_K batch-1 GEMV
    mats = []
    total_copy_bytes = sum(n * (k // 256) * 144 for n, k in CFG2_SHAPES)
    ncopies = max(2, -(-ROTATE_BYTES // total_copy_bytes))
    host_w = {}
    for n, k in CFG2_SHAPES:
        w = np.concatenate([synth.make_weights(rng, Q4_K, min(2048, n - r), k) for r in range(0, n, 2048)], axis=0)
        host_w[(n, k)] = w
        base = torch.from_numpy(w).to(dev)
        copies = [base] + [base.clone() for _ in range(ncopies - 1)]
        x = torch.from_numpy(rng.standard_normal((1, k)).astype(np.float32)).to(torch.float16).to(dev)
        mats.append((n, k, copies, x))
    step_bytes = sum(n * (k // 256) * 144 + 2 * k + 2 * n for n, k in CFG2_SHAPES)

    def step(i):
        for n, k, copies, x in mats:
            ops.ggml_mul_mat_vec_a8(copies[i % ncopies], x, Q4_K, n)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    # the same eager steps through torch.ops._C_gguf, i.e. through the compiled binding where it has been built
    from vllm_gguf_plugin_prism_amd import _C_gguf
    torch_op = torch.ops._C_gguf.ggml_mul_mat_vec_a8
    for i in range(args.warmup):
        for n, k, copies, x in mats:
            torch_op(copies[i % ncopies], x, Q4_K, n)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        for n, k, copies, x in mats:
            torch_op(copies[i % ncopies], x, Q4_K, n)
    torch.cuda.synchronize()
    eager_torch_ops_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    # the same steps as one HIP graph of a full rotation over the weight copies, replayed: host launch cost out of the
    # timed region.  At least K steps and at least MIN_LAUNCHES kernel launches are timed whatever K is.
    replays = max(-(-args.steps // ncopies), -(-MIN_LAUNCHES // (len(CFG2_SHAPES) * ncopies)))
    graph_ms = eager_ms if args.profile else _graph_ms(step, ncopies, replays)
    ms_per_step = min(eager_ms, eager_torch_ops_ms, graph_ms)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # per-launch duration of one matrix at a time (roofline of the dominant kernel)
    per_shape = {}
    for n, k, copies, x in mats:
        one = lambda i, n=n, copies=copies, x=x: ops.ggml_mul_mat_vec_a8(copies[i % ncopies], x, Q4_K, n)  # noqa: E731
        ms = _timed_ms(one, ncopies * 4, eager=args.profile)
        b = n * (k // 256) * 144 + 2 * k + 2 * n
        per_shape[f"{n}x{k}"] = {"us_per_call": ms * 1e3, "GBps": b / (ms * 1e-3) / 1e9, "bytes": b,
                                 "launches_timed": ncopies * 4 * -(-MIN_LAUNCHES // (ncopies * 4))}
    big = per_shape["14336x4096"]
    roofline = {"bound": "hbm", "achieved": big["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": big["GBps"] / HBM_PEAK_GBS, "traffic": _traffic("mmvq_q4_k_14336x4096_bs1"),
                "algorithmic_bytes": big["bytes"],
                "kernel": "mmvq Q4_K [14336,4096] bs1 (one kernel per call: activation quantisation fused into the GEMV)",
                "per_shape": per_shape}

    out = {
        "metric": "Q4_K GEMV HBM GB/s (% peak) @bs1; Q6_K MMQ int8 TOPS (% peak) @M=512",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot products, fp32 accumulate, fp16 in/out",
        "data": "synthetic (seeded N(0,0.02) weights quantized to Q4_K, N(0,1) fp16 activations)",
        "config": {"workload": "BASELINE config 2: Q4_K batch-1 MMVQ over [4096,4096],[14336,4096],[4096,14336]",
                   "weight_copies_rotated": ncopies, "rotated_bytes": ncopies * total_copy_bytes,
                   "eager_ms_per_step": eager_ms, "graph_ms_per_step": graph_ms,
                   "eager_ms_per_step_torch_ops": eager_torch_ops_ms,
                   "torch_ops_binding": "compiled (_C_gguf_native.so)" if _C_gguf.NATIVE else "python (torch.library + ctypes)",
                   "graph_steps_timed": 0 if args.profile else replays * ncopies,
                   "pct_of_hbm_peak": 100.0 * value / HBM_PEAK_GBS},
        "roofline": roofline,
    }

    # ---------------------------------------------------------------- config 3: Q6_K MMQ at M=512
    if not args.no_mmq:
        tables = {"auto": {}, "half": {}}
        for n, k in CFG3_SHAPES:
            w = np.concatenate([synth.make_weights(rng, Q6_K, min(2048, n - r), k) for r in range(0, n, 2048)], axis=0)
            wd = torch.from_numpy(w).to(dev)
            for m in ((512,) if args.profile else (128, 512, 2048)):
                x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(torch.float16).to(dev)
                for engine, table in tables.items():
                    call = lambda i, engine=engine: ops.ggml_mul_mat_a8(wd, x, Q6_K, n, engine=engine)  # noqa: E731
                    ms = _timed_ms(call, 20, eager=args.profile)
                    tops = 2.0 * m * n * k / (ms * 1e-3) / 1e12
                    table[f"{n}x{k}@M{m}"] = {"ms": ms, "TOPS": tops, "frac_int8_peak": tops / INT8_PEAK_TOPS,
                                              "frac_int8_legacy_k_peak": tops / INT8_LEGACY_PEAK_TOPS}
            del wd
        ops_total = sum(2.0 * 512 * n * k for n, k in CFG3_SHAPES)

        def at_m512(table):
            t_total = sum(v["ms"] for key, v in table.items() if key.endswith("@M512")) * 1e-3
            return ops_total / t_total / 1e12

        tops512, half512 = at_m512(tables["auto"]), at_m512(tables["half"])
        out["mmq"] = {
            "metric": "Q6_K MMQ int8 TOPS @M=512", "value": tops512, "unit": "TOPS",
            "engine": "gguf_mmq's default: exact int8 dot products per block on int8 MFMA, fp32 block scales",
            "matrix_instruction": MMQ_INSTRUCTION.get(Q6_K, "v_mfma_i32_32x32x32_i8")
                                  + " (Q6_K's weight scale changes every 16 values: the legacy-K shape, whose own peak is half the chip's)",
            "dtype": "int8 products, int32 sums per block, fp32 accumulation",
            "roofline": {"bound": "mfma", "achieved": tops512, "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                         "frac": tops512 / INT8_PEAK_TOPS,
                         "denominators": {"double_k_int8_peak_TOPS": INT8_PEAK_TOPS, "frac_of_double_k_peak": tops512 / INT8_PEAK_TOPS,
                                          "legacy_k_int8_peak_TOPS": INT8_LEGACY_PEAK_TOPS,
                                          "frac_of_legacy_k_peak": tops512 / INT8_LEGACY_PEAK_TOPS,
                                          "used_for_frac": "double_k_int8_peak_TOPS (the chip's dense int8 peak)"},
                         "traffic": {f"{n}x{k}": _traffic(f"mmqi_q6_k_{n}x{k}_m512") for n, k in CFG3_SHAPES}},
            "per_shape": tables["auto"],
            "half_engine": {"value": half512, "unit": "TOPS", "frac_of_f16_mfma_peak": half512 / F16_PEAK_TFLOPS,
                            "per_shape": tables["half"],
                            "note": "engine='half', opt-in: dequantized operands on v_mfma_f32_32x32x16_f16; not the "
                                    "reference's arithmetic (operands rounded to half), so not the headline"},
            "note": "time per call = activation quantisation kernel + GEMM kernel (+ the partial-sum kernel where K is split), "
                    "averaged over 100 calls",
        }

    # ---------------------------------------------------------------- CPU baseline (bounded sample)
    if not args.no_cpu:
        from oracle import gguf_oracle as oracle  # the checker, timed as the reference's CPU path

        n, k = CFG2_SHAPES[0]
        w = host_w[(n, k)]
        x16 = torch.from_numpy(rng.standard_normal((1, k)).astype(np.float32)).to(torch.float16)
        x32 = x16.float()
        threads_before = torch.get_num_threads()
        torch.set_num_threads(1)           # numpy's block decode is one thread; the matmul leg is held to the same
        best = None
        t_end = time.perf_counter() + 20.0
        reps = 0
        while reps < 6 or (time.perf_counter() < t_end and reps < 8):
            t0 = time.perf_counter()
            wd = oracle.dequantize(w, Q4_K, "f32", flavour="f32").reshape(n, k)
            t1 = time.perf_counter()
            y_cpu = x32 @ torch.from_numpy(wd).T
            t2 = time.perf_counter()
            if reps > 0 and (best is None or t2 - t0 < best[0]):
                best = (t2 - t0, t1 - t0, t2 - t1)
            reps += 1
        torch.set_num_threads(threads_before)
        qbytes = n * (k // 256) * 144
        # the GPU result on the same bytes against this CPU result (unquantized activations: q8_1 noise, about 5e-3
        # expected) and against the a8 oracle (the same q8_1 activations, exact integer dots)
        y_gpu = ops.ggml_mul_mat_vec_a8(torch.from_numpy(w).to(dev), x16.to(dev), Q4_K, n).float().cpu().numpy()
        y_a8 = oracle.mul_mat_a8(w, x32.numpy(), Q4_K, n, "mmvq")
        print(f"CPU baseline on 1 of {os.cpu_count()} cores ({_cpu_model()}; torch threads {threads_before} -> 1 for the timed leg)",
              file=sys.stderr)
        out["cpu_baseline"] = {
            "value": qbytes / best[0] / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"Q4_K [{n},{k}] batch 1 on one thread: numpy fp32 block dequantize ({best[1] * 1e3:.1f} ms) + torch fp32 "
                      f"matmul ({best[2] * 1e3:.1f} ms), best of {reps - 1} after 1 warm-up",
            "t_dequant_ms": best[1] * 1e3, "t_matmul_ms": best[2] * 1e3, "t_total_ms": best[0] * 1e3,
            "effective_GOPS": 2.0 * n * k / best[0] / 1e9,
            "cpu_model": _cpu_model(), "os_cpu_count": os.cpu_count(), "torch_num_threads": threads_before,
            "gpu_vs_cpu_unquantized_activations": _errors(y_gpu, y_cpu.numpy()),
            "gpu_vs_a8_oracle": _errors(y_gpu, y_a8),
        }

    if not args.no_other:
        out["other_configs"] = _other_configs(rng, dev, host_w[(14336, 4096)])

    if args.profile:
        # one plain device-to-device copy of known size: its FETCH_SIZE / WRITE_SIZE readings give the scale of
        # those counters on this machine (268435456 bytes read, 268435456 bytes written)
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        out["config"]["calibration_copy_bytes"] = 256 << 20

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
