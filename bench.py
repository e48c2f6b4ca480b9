"""Benchmark of the quantized-linear hot path on one MI355X.

Headline workload (``config.workload``): every int8 weight-only decode GEMV of a
Qwen3.5-4B-shaped model at M=1 -- 32 layers of {qkv 2560->6144, o 4096->2560,
gate_up 2560->19456, down 9728->2560} (q/k/v and gate/up fused along N exactly
as their callers fuse them) plus lm_head 2560->151936 -- 129 launches over
3.6 GB of distinct weights per step, so neither the L2s nor the 256 MB
Infinity Cache can serve a weight twice.  A step is replayed as one HIP graph
(``--no-graph`` launches eagerly through the C ABI instead).

``value`` is algorithmic bytes per step / step time, weights resident in HBM
before the clock starts.  One JSON line is printed; ``extra`` carries the other
configurations (M=4/8/16, W4A8 GEMV, W8A8/W4A8 prefill GEMM, the quantiser).
"""

from __future__ import annotations

import argparse
import ctypes
import json
import statistics
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published
INT8_PEAK_TOPS = 5033.0       # MI355X dense int8 MFMA, published (256 CU x 8192 op/clk x 2.4 GHz)
LAYERS = 32

METRIC = "decode GEMV HBM GB/s (% of peak) + W8A8 prefill int8 TOPS, Qwen3.5-4B shapes"


#: Summary of the rocprofv3 FETCH_SIZE / WRITE_SIZE runs of the default workload (M=1: the two
#: instantiation families gemv_w8a16_kernel and gemv_w8a16_wholerow_kernel); it carries the
#: line "roofline.traffic bytes per launch: <integer>", which is what `roofline.traffic` reports.
TRAFFIC_PROFILE = ROOT / "profiles" / "gemv_w8a16_decode_model_M1.md"


def measured_traffic_bytes_per_launch():
    """HBM bytes per launch from the committed counter summary, or None when it is absent."""
    import re
    try:
        m = re.search(r"roofline\.traffic bytes per launch:\s*([0-9][0-9,_]*)", TRAFFIC_PROFILE.read_text())
    except OSError:
        return None
    return int(m.group(1).replace(",", "").replace("_", "")) if m else None


def cpu_model() -> str:
    try:
        for line in Path("/proc/cpuinfo").read_text().splitlines():
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(budget_s: float, synth, torch) -> dict:
    """The reference's CPU path on one decode layer (7 int8 weight-only GEMVs, M = 1, 101.1 MB), timed
    on the host cores: torch eager evaluating backends/reference/__init__.py:93-95 --
    ``dense = (wq.float() * scale[:, None]).to(bf16)``; ``y = F.linear(x, dense)`` -- *faithful*
    (the dequantisation inside every call, as the reference does) and *hoisted* (dequantised once,
    outside the clock), each at all cores and at one thread.  Median of up to 25 calls after up to 2
    warm-ups per shape, fewer when the time budget (a quarter of ``budget_s`` per variant) runs
    out.  The C oracle of the same path is reported beside it as a labelled extra."""
    import statistics
    import torch.nn.functional as F
    gen = synth.generator(1234)
    layer = []
    for _, n_, k_ in synth.DECODE_LAYER:
        q = synth.int8_weight(n_, k_, gen)
        layer.append((q.wq, q.scale, synth.activations(1, k_, gen), synth.gemv_bytes(1, n_, k_)))
    layer_bytes = sum(nb for *_, nb in layer)
    all_cores = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or (os.cpu_count() or 1))))
    prev_threads = torch.get_num_threads()

    def leg(threads: int, hoisted: bool, budget: float):
        torch.set_num_threads(threads)
        t_start = time.perf_counter()
        total, calls = 0.0, 0
        for wq, sc, x, _ in layer:
            dense = (wq.float() * sc[:, None]).to(torch.bfloat16) if hoisted else None
            times = []
            for i in range(27):
                t0 = time.perf_counter()
                d = dense if hoisted else (wq.float() * sc[:, None]).to(torch.bfloat16)
                F.linear(x, d)
                dt = time.perf_counter() - t0
                if i >= 2 or time.perf_counter() - t_start > budget:
                    times.append(dt)
                if time.perf_counter() - t_start > budget and times:
                    break
            total += statistics.median(times)
            calls += len(times)
        return {"layer_ms": round(total * 1e3, 3), "GBps": round(layer_bytes / total / 1e9, 3), "threads": threads,
                "timed_calls": calls}

    per = budget_s / 4.0
    variants = {}
    for name, threads, hoisted in (("faithful_all_cores", all_cores, False), ("hoisted_all_cores", all_cores, True),
                                   ("faithful_1_thread", 1, False), ("hoisted_1_thread", 1, True)):
        variants[name] = leg(threads, hoisted, per)
    torch.set_num_threads(prev_threads)

    # the C oracle of the same path (fp64 inner loop, full dequantisation per call, OpenMP)
    from oracle import oracle as orc
    orc.set_num_threads(min(orc.num_threads(), all_cores))
    ops = [(wq.numpy(), sc.numpy(), orc.bits(x)) for wq, sc, x, _ in layer]
    orc.linear_qweight(*ops[1])
    t0 = time.perf_counter()
    for wq, sc, xb in ops:
        orc.linear_qweight(wq, sc, xb)
    c_dt = time.perf_counter() - t0

    head = variants["faithful_all_cores"]
    return {
        "value": head["GBps"],
        "unit": "GB/s",
        "cores": head["threads"],
        "kind": "port",
        "sample": "one decode layer (q, k, v, o, gate, up, down: 7 int8 weight-only GEMVs, M=1, "
                  f"{layer_bytes / 1e6:.1f} MB algorithmic) through torch eager restating the reference's CPU path "
                  "(weight dequantised to bf16 inside every call, then F.linear), median per shape of "
                  f"{head['timed_calls']} timed calls, all host cores",
        "cpu_model": cpu_model(),
        "os_cpu_count": os.cpu_count(),
        "torch": torch.__version__,
        "variants": variants,
        "c_oracle_port": {"layer_ms": round(c_dt * 1e3, 3), "GBps": round(layer_bytes / c_dt / 1e9, 3),
                          "threads": min(orc.num_threads(), all_cores),
                          "note": "C restatement with an fp64 accumulator, dequantisation per call"},
    }


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    # 20 untimed steps (16 ms): with 3 the clocks have not settled and the timed steps read 0.816-0.826 ms
    # from run to run instead of 0.810-0.811
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rows", type=int, default=1, help="activation rows M of the headline workload")
    ap.add_argument("--mfma", action="store_true",
                    help="headline workload through cmi_gemv_w8a16_mfma (the verify / short-prefill kernel) "
                         "instead of the dot-product GEMV; meant for --rows 3..16")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="time only the W8A8 prefill GEMM (M=2048 and 8192, N=9728, K=2560): the profiling "
                         "target for that kernel; prints its own JSON line")
    ap.add_argument("--w4a8-prefill-only", action="store_true",
                    help="time only the W4A8 prefill GEMM (M=1024, N=25600, K=5120): the profiling target "
                         "for that kernel; prints its own JSON line")
    ap.add_argument("--prequantised", action="store_true",
                    help="with --w4a8-decode-only: activations arrive as int8 rows + scales")
    ap.add_argument("--table-entries", action="store_true",
                    help="with --w4a8-decode-only: drive the step through the table entries of the backend "
                         "(rms_norm / add_rms_norm / silu_mul in front of linear), with and without the "
                         "producers handing over their quantised rows")
    ap.add_argument("--w4a8-decode-only", action="store_true",
                    help="time only the W4A8 decode step (32 layers + lm_head at one row, one "
                         "cmi_linear_w4a8_bf16 call per projection): the profiling target for the W4A8 decode "
                         "kernels and the quantiser; prints its own JSON line")
    ap.add_argument("--quant-only", action="store_true",
                    help="time only the per-token quantiser (8192 x 2560, 2048 x 9728, 16 x 9728 and 1 x 2560 rows): "
                         "the profiling target for quant_act_i8; prints its own JSON line")
    ap.add_argument("--tile-choice-check", action="store_true",
                    help="W8A8 GEMM: time the library's own kernel choice against every forced block tile on cold "
                         "weights over a set of layer shapes and batch sizes; prints the regret per shape.  The "
                         "choice is made by cost models fitted to this machine: run this after a driver, "
                         "compiler or clock change to see whether they still hold")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (known traffic, for scaling HBM counters)")
    return ap.parse_args()


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; the path needs no collectives and "
              "--gpus above 1 is not supported", file=sys.stderr)
        return 2

    import torch
    from coffin_amd import _native, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    lib = _native.load()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    vp = ctypes.c_void_p

    def ptr(t):
        return vp(t.data_ptr())

    def cur_stream():
        return vp(torch.cuda.current_stream().cuda_stream)

    def timed(fn, iters: int, warm: int = 2) -> float:
        """Seconds per call of fn(), HIP events on the launch stream."""
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / iters

    gen = synth.generator(1234, dev)

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    if args.tile_choice_check:
        tiles = (64, 128, 192, 128192, 256, 320, 321, 322, 6464)
        shapes_ = [(m, n_, k_) for (n_, k_) in ((9728, 2560), (4096, 2560), (2560, 9728), (6144, 2560), (2560, 4096))
                   for m in (64, 256, 512, 2048, 8192)] + [(4096, 9728, 2560), (8192, 19456, 2560)]
        rows_, worst, sum_auto, sum_best = {}, 0.0, 0.0, 0.0
        for m, n_, k_ in shapes_:
            x = synth.activations(m, k_, gen, outliers=True)
            xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
            xs = torch.empty(m, dtype=torch.float32, device=dev)
            y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
            lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream())
            copies = min(24, -(-600_000_000 // (n_ * k_)))
            cold_w = [synth.int8_weight(n_, k_, gen) for _ in range(copies)]
            def cold():
                st = cur_stream()
                for c in cold_w:
                    lib.cmi_gemm_w8a8(ptr(xq), ptr(c.wq), ptr(xs), ptr(c.scale), ptr(y), vp(0), m, n_, k_, n_, st)
            # every choice captured first, then replayed in turn, five rounds, median: a launch's time
            # depends on what ran before it (the clock a long 256 x 320 launch leaves behind costs the
            # next measurement 3-7 %), so no choice may always follow the same neighbour's warm-up only
            graphs_ = {}
            for tile in (0,) + tiles:
                if lib.cmi_set_option(b"gemm_tile", tile):
                    continue
                cold()
                torch.cuda.synchronize()
                g_ = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g_):
                    cold()
                graphs_[tile] = g_
            lib.cmi_set_option(b"gemm_tile", 0)
            samples = {tile: [] for tile in graphs_}
            for _ in range(5):
                for tile, g_ in graphs_.items():
                    samples[tile].append(timed(g_.replay, 3, warm=1) / copies * 1e6)
            t_by = {tile: statistics.median(v) for tile, v in samples.items()}
            del graphs_
            best = min((t, tl) for tl, t in t_by.items() if tl)
            regret = t_by[0] / best[0] - 1.0
            worst, sum_auto, sum_best = max(worst, regret), sum_auto + t_by[0], sum_best + best[0]
            rows_[f"M{m}_N{n_}_K{k_}"] = {"auto_us": round(t_by[0], 2), "best_forced_us": round(best[0], 2),
                                        "best_forced_tile": best[1], "regret": round(regret, 4),
                                        "by_tile_us": {str(tl): round(t, 2) for tl, t in t_by.items() if tl}}
            del cold_w
        print(json.dumps({"metric": "W8A8 GEMM kernel choice against the best forced tile (cold weights)", "unit": "us",
                          "total_auto_us": round(sum_auto, 1), "total_best_forced_us": round(sum_best, 1),
                          "total_regret": round(sum_auto / sum_best - 1.0, 4), "worst_regret": round(worst, 4),
                          "shapes": rows_}))
        return 0

    if args.prefill_only:
        out = {}
        for m, n_, k_ in ((2048, 9728, 2560), (8192, 9728, 2560)):
            q = synth.int8_weight(n_, k_, gen)
            x = synth.activations(m, k_, gen, outliers=True)
            xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
            xs = torch.empty(m, dtype=torch.float32, device=dev)
            y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
            lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream())
            t = timed(lambda: lib.cmi_gemm_w8a8(ptr(xq), ptr(q.wq), ptr(xs), ptr(q.scale), ptr(y), vp(0),
                                                m, n_, k_, n_, cur_stream()), args.steps, args.warmup)
            tops = synth.gemm_ops(m, n_, k_) / t / 1e12
            out[f"M{m}_N{n_}_K{k_}"] = {"gemm_us": round(t * 1e6, 2), "tops": round(tops, 1),
                                        "frac_of_int8_peak": round(tops / INT8_PEAK_TOPS, 4)}
        print(json.dumps({"metric": "W8A8 prefill GEMM int8 TOPS", "unit": "TOP/s", "w8a8_prefill_gemm": out}))
        return 0

    if args.w4a8_prefill_only:
        m, n_, k_ = 1024, 25600, 5120
        w = synth.int4_weight(n_, k_, gen)
        d4 = torch.empty((n_, k_ // 2), dtype=torch.uint8, device=dev)
        ds = torch.empty((n_, k_ // 128), dtype=torch.float32, device=dev)
        lib.cmi_w4_repack(ptr(w.packed), ptr(w.scale), ptr(d4), ptr(ds), n_, k_, 128, cur_stream())
        x = synth.activations(m, k_, gen)
        xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
        xs = torch.empty(m, dtype=torch.float32, device=dev)
        y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
        lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream())
        t = timed(lambda: lib.cmi_gemm_w4a8(ptr(d4), ptr(ds), ptr(xq), ptr(xs), ptr(y), vp(0), m, n_, k_, 128,
                                            cur_stream()), args.steps, args.warmup)
        tops = synth.gemm_ops(m, n_, k_) / t / 1e12
        print(json.dumps({"metric": "W4A8 prefill GEMM int8 TOPS", "unit": "TOP/s",
                          "w4a8_prefill_gemm_M1024_N25600_K5120": {
                              "us": round(t * 1e6, 2), "tops": round(tops, 1),
                              "frac_of_int8_peak": round(tops / INT8_PEAK_TOPS, 4)}}))
        return 0

    def w4a8_decode_step(rows: int, use_graph: bool, iters: int, prequantised: bool = False):
        """The decode step of the same model with int4 group-128 weights (32 x {qkv, o, gate_up,
        down} + lm_head, 1.84 GB of distinct packed weights), one cmi_linear_w4a8_bf16 call per
        projection: the quantiser folded into the GEMV where that is the faster route, else two
        launches.  ``prequantised``: the activations arrive as int8 rows + scales, as they do
        behind cmi_rms_norm_i8 / cmi_silu_mul_quant (the producer has quantised them), and every
        projection is one cmi_gemv_w4a8 call.  Returns the result block for ``extra``."""
        proj = []
        xs_ = {k_: synth.activations(16, k_, gen) for k_ in (2560, 4096, 9728)}
        for layer in range(LAYERS + 1):
            for _, n_, k_ in (synth.DECODE_LAYER_FUSED if layer < LAYERS else (synth.LM_HEAD,)):
                w = synth.int4_weight(n_, k_, gen)
                d4 = torch.empty((n_, k_ // 2), dtype=torch.uint8, device=dev)
                ds = torch.empty((n_, k_ // 128), dtype=torch.float32, device=dev)
                _native.check(lib.cmi_w4_repack(ptr(w.packed), ptr(w.scale), ptr(d4), ptr(ds), n_, k_, 128,
                                                cur_stream()), "repack")
                torch.cuda.synchronize()
                del w
                proj.append((d4, ds, xs_[k_], torch.empty((16, n_), dtype=torch.bfloat16, device=dev), n_, k_))
        nbytes = int(lib.cmi_linear_workspace_bytes(16, 9728))
        work = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        xq_ = {}
        if prequantised:
            for k_, x in xs_.items():
                q_ = torch.empty((16, k_), dtype=torch.int8, device=dev)
                s_ = torch.empty(16, dtype=torch.float32, device=dev)
                _native.check(lib.cmi_quant_act_i8(ptr(x), ptr(q_), ptr(s_), 16, k_, cur_stream()), "quant")
                xq_[k_] = (q_, s_)

        def step():
            st = cur_stream()
            for d4, ds, x, y, n_, k_ in proj:
                if prequantised:
                    rc = lib.cmi_gemv_w4a8(ptr(d4), ptr(ds), ptr(xq_[k_][0]), ptr(xq_[k_][1]), ptr(y), vp(0), rows, n_, k_,
                                           128, st)
                else:
                    rc = lib.cmi_linear_w4a8_bf16(ptr(d4), ptr(ds), ptr(x), ptr(y), rows, n_, k_, 128, ptr(work), nbytes, st)
                if rc:
                    _native.check(rc, "w4a8 projection")

        runner, mode = step, "eager"
        if use_graph:
            step()
            torch.cuda.synchronize()
            want = [p_[3][:rows].clone() for p_ in proj[:4]] + [proj[-1][3][:rows].clone()]
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            for _ in range(2):
                for p_ in proj:
                    p_[3][:rows].zero_()
                graph.replay()
                torch.cuda.synchronize()
                got = [p_[3][:rows] for p_ in proj[:4]] + [proj[-1][3][:rows]]
                if not all(bool((a.view(torch.int16) == b_.view(torch.int16)).all()) for a, b_ in zip(want, got)):
                    raise RuntimeError("HIP graph replay of the W4A8 step differs from the eager step")
            runner, mode = graph.replay, "hipgraph"
        t = timed(runner, iters, warm=2)
        # pre-quantised rows are one byte per element plus a scale per row instead of two bytes
        alg = sum(synth.w4_gemv_bytes(rows, n_, k_) - (rows * k_ - 4 * rows if prequantised else 0) for *_, n_, k_ in proj)
        gbps = alg / t / 1e9
        return {"ms_per_step": round(t * 1e3, 4), "GBps": round(gbps, 1), "launch": mode, "rows": rows,
                "activations": "int8 rows + scales (quantised upstream)" if prequantised else "bf16 (quantised inside the call)",
                "projections_per_step": len(proj), "algorithmic_bytes_per_step": alg,
                "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                             "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None,
                             "avg_projection_us": round(t / len(proj) * 1e6, 3),
                             "algorithmic_bytes_per_projection": round(alg / len(proj))}}

    def w4a8_step_through_table_entries(rows: int, iters: int):
        """The W4A8 decode step driven the way the reference drives it, through the table entries of
        coffin_amd.backend: per layer rms_norm -> linear(qkv), linear(o) on plain bf16 rows (the
        attention output: no producer of this backend in front of it), add_rms_norm -> linear(gate_up),
        silu_mul -> linear(down); rms_norm -> linear(lm_head) at the end (ops/norm.py:87,135,
        models/qwen35/blocks.py:69,97, ops/gemv.py:75,93).  Captured in a graph.  Measured with the
        producers handing their quantised rows to the projection behind them and without, and the
        producers alone (97 launches), so that "projections only" = sequence - producers."""
        from coffin_amd import backend as B
        from coffin_amd.weights import W4A8Weight as W4
        layers = []
        for _ in range(LAYERS):
            ws = []
            for _, n_, k_ in synth.DECODE_LAYER_FUSED:
                w = synth.int4_weight(n_, k_, gen)
                ws.append(W4(w.packed, w.scale, k=k_))
            layers.append(ws)
        _, n_, k_ = synth.LM_HEAD
        w = synth.int4_weight(n_, k_, gen)
        head = W4(w.packed, w.scale, k=k_)
        hidden, inter = 2560, 9728
        gain = (1.0 + 0.1 * torch.randn(hidden, generator=gen, device=dev)).to(torch.bfloat16)
        resid = synth.activations(rows, hidden, gen)
        attn = synth.activations(rows, 4096, gen)
        mix = synth.activations(rows, hidden, gen)
        normed = torch.empty((rows, hidden), dtype=torch.bfloat16, device=dev)
        gu_fixed = synth.activations(rows, 2 * inter, gen)
        one = rows == 1
        proj = B.linear if one else B.linear_m

        def row(t):                                   # a single sequence hands [K] to linear, as ops/gemv.py:75 does
            return t.view(-1) if one else t

        def sequence(projections: bool = True):
            x = resid.clone()
            for qkv, o, gate_up, down in layers:
                h = B.rms_norm(x, gain)
                if projections:
                    proj(qkv, row(h))
                    proj(o, row(attn))
                B.add_rms_norm(x, mix, gain, normed)
                gu = proj(gate_up, row(normed)) if projections else row(gu_fixed)
                gate, up = (gu[:inter], gu[inter:]) if one else (gu[:, :inter], gu[:, inter:])
                act = B.silu_mul(gate, up, up)
                if projections:
                    proj(down, act)
            h = B.rms_norm(x, gain)
            if projections:
                proj(head, row(h))

        out = {"rows": rows}
        alg = sum(synth.w4_gemv_bytes(rows, w_.n, w_.k) for ws in layers for w_ in ws) + synth.w4_gemv_bytes(rows, head.n, head.k)
        for label, handover, projections in (("handed_rows", True, True), ("bf16_rows", False, True),
                                             ("producers_only", False, False)):
            B.configure(handover=handover)
            sequence(projections)                     # warm-up: re-layouts, scratch, the consumer-seen flag
            sequence(projections)
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                sequence(projections)
            t = timed(gr.replay, iters, warm=2)
            out[label + "_ms"] = round(t * 1e3, 4)
            del gr
        B.configure(handover=True)
        for label in ("handed_rows", "bf16_rows"):
            t = (out[label + "_ms"] - out["producers_only_ms"]) * 1e-3
            out[label + "_projections_only_ms"] = round(t * 1e3, 4)
            out[label + "_projections_only_GBps"] = round(alg / t / 1e9, 1)
        out["launches"] = {"projections": 4 * LAYERS + 1, "producers": 3 * LAYERS + 1}
        out["algorithmic_bytes_of_the_projections"] = alg
        return out

    if args.quant_only:
        out = {}
        for m, k_ in ((8192, 2560), (2048, 9728), (16, 9728), (1, 2560)):
            x = synth.activations(m, k_, gen, outliers=True)
            xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
            xs = torch.empty(m, dtype=torch.float32, device=dev)
            t = timed(lambda: lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream()), args.steps, args.warmup)
            gbps = synth.quant_bytes(m, k_) / t / 1e9
            out[f"M{m}_K{k_}"] = {"us": round(t * 1e6, 2), "GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
                                  "algorithmic_bytes": synth.quant_bytes(m, k_)}
        print(json.dumps({"metric": "per-token int8 quantiser HBM GB/s", "unit": "GB/s", "quant_act_i8": out}))
        return 0

    if args.w4a8_decode_only and args.table_entries:
        print(json.dumps({"metric": "W4A8 decode step through the table entries", "unit": "ms",
                          "w4a8_decode_step": {f"M{args.rows}_through_table_entries":
                                               w4a8_step_through_table_entries(args.rows, args.steps)}}))
        return 0
    if args.w4a8_decode_only:
        key = f"M{args.rows}" + ("_prequantised" if args.prequantised else "")
        out = {key: w4a8_decode_step(args.rows, not args.no_graph, args.steps, args.prequantised)}
        print(json.dumps({"metric": "W4A8 decode step HBM GB/s", "unit": "GB/s", "w4a8_decode_step": out}))
        return 0

    # ------------------------------------------------------------ headline: decode GEMVs
    M = args.rows
    shapes = list(synth.DECODE_LAYER_FUSED)
    launches = []       # (wq, scale, x, y, M, N, K)
    x_by_k = {}
    for k in sorted({k for _, _, k in shapes} | {synth.LM_HEAD[2]}):
        x_by_k[k] = synth.activations(16, k, gen)
    for _layer in range(LAYERS):
        for _, n, k in shapes:
            q = synth.int8_weight(n, k, gen)
            y = torch.empty((16, n), dtype=torch.bfloat16, device=dev)
            launches.append((q.wq, q.scale, x_by_k[k], y, n, k))
    _, n, k = synth.LM_HEAD
    q = synth.int8_weight(n, k, gen)
    launches.append((q.wq, q.scale, x_by_k[k], torch.empty((16, n), dtype=torch.bfloat16, device=dev), n, k))
    weight_bytes = sum(w.numel() for w, *_ in launches)

    def step_bytes(m):
        return sum(synth.gemv_bytes(m, n_, k_) for *_, n_, k_ in launches)

    def run_step(m, mfma=False):
        # mfma: the matrix-pipe GEMV that verify and short prefill chunks take (rows of a batch
        # independent of each other, not bit-identical to the single-row call); otherwise the
        # dot-product GEMV of linear / linear_m
        st = cur_stream()
        fn = lib.cmi_gemv_w8a16_mfma if mfma else lib.cmi_gemv_w8a16
        for wq, sc, x, y, n_, k_ in launches:
            rc = fn(ptr(wq), ptr(sc), ptr(x), ptr(y), m, n_, k_, st)
            if rc:
                _native.check(rc, "cmi_gemv_w8a16")

    def make_runner(m, mfma=False):
        """Eager launcher, or a HIP graph of one step checked against the eager result."""
        def step_fn(rows):
            run_step(rows, mfma)
        if args.no_graph:
            return (lambda: step_fn(m)), "eager"
        step_fn(m)
        torch.cuda.synchronize()
        want = [y[:m].clone() for *_, y, _, _ in launches[:4]] + [launches[-1][3][:m].clone()]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step_fn(m)
        for _ in range(3):
            for *_, y, _, _ in launches:
                y[:m].zero_()
            graph.replay()
            torch.cuda.synchronize()
            got = [y[:m] for *_, y, _, _ in launches[:4]] + [launches[-1][3][:m]]
            if not all(bool((a.view(torch.int16) == b.view(torch.int16)).all()) for a, b in zip(want, got)):
                raise RuntimeError("HIP graph replay differs from the eager step")
        return graph.replay, "hipgraph"

    runner, launch_mode = make_runner(M, args.mfma)
    for _ in range(args.warmup):
        runner()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    wall0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        runner()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    step_s = e0.elapsed_time(e1) * 1e-3 / args.steps
    bytes_per_step = step_bytes(M)
    value = bytes_per_step / step_s / 1e9
    n_launch = len(launches)

    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 weights x bf16 activations, fp32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": f"int8 weight-only decode GEMVs of a Qwen3.5-4B-shaped model, M={M}: "
                        f"{LAYERS} layers x (qkv 2560->6144, o 4096->2560, gate_up 2560->19456, "
                        f"down 9728->2560) + lm_head 2560->151936",
            "rows": M,
            "launches_per_step": n_launch,
            "weight_bytes": weight_bytes,
            "algorithmic_bytes_per_step": bytes_per_step,
            "launch": launch_mode,
            "wall_ms_per_step": round(wall / args.steps * 1e3, 4),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(value, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(value / HBM_PEAK_GBPS, 4),
            # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this same
            # command (summary under profiles/); it only describes the default workload
            "traffic": measured_traffic_bytes_per_launch() if (M == 1 and not args.no_graph and not args.mfma) else None,
            "kernel": "gemv_w8a16_rows16_kernel" if args.mfma else ("gemv_w8a16_kernel + gemv_w8a16_wholerow_kernel" if M == 1 else "gemv_w8a16_kernel"),
            "avg_launch_us": round(step_s / n_launch * 1e6, 3),
            "algorithmic_bytes_per_launch": round(bytes_per_step / n_launch),
        },
    }

    # ------------------------------------------------------------------ secondary configs
    if not args.no_extra:
        extra = {}
        for m in (1, 4, 8, 16):
            if m == M:
                extra[f"decode_gemv_int8_M{m}_GBps"] = round(value, 1)
                continue
            r, _ = make_runner(m)
            t = timed(r, max(3, args.steps // 2), warm=2)
            extra[f"decode_gemv_int8_M{m}_GBps"] = round(step_bytes(m) / t / 1e9, 1)
        # the same step through the matrix-pipe GEMV (linear_m_verify, short linear_prefill chunks)
        family = {"dot": {}, "mfma": {}}
        for m in (1, 4, 8, 16):
            r, _ = make_runner(m, True)
            t = timed(r, max(3, args.steps // 2), warm=2)
            if m > 1:
                extra[f"verify_gemv_int8_mfma_M{m}_GBps"] = round(step_bytes(m) / t / 1e9, 1)
            family["mfma"][f"M{m}"] = {"ms_per_step": round(t * 1e3, 4), "GBps": round(step_bytes(m) / t / 1e9, 1),
                                       "frac_of_hbm_peak": round(step_bytes(m) / t / 1e9 / HBM_PEAK_GBPS, 4)}
            g_ = extra[f"decode_gemv_int8_M{m}_GBps"]
            family["dot"][f"M{m}"] = {"ms_per_step": round(step_bytes(m) / g_ / 1e6, 4), "GBps": g_,
                                      "frac_of_hbm_peak": round(g_ / HBM_PEAK_GBPS, 4)}
        # Static-batch decode owes "row r of a batch == the single-row call" (models/qwen35/batch.py:19-22),
        # which holds inside either kernel family as long as every call on a weight uses the same one
        # (coffin_amd.backend.configure(batch_family=...), or the weight's batch_family attribute): the
        # whole decode step at 1 / 4 / 8 / 16 rows in both, so the trade is a measured table.
        extra["static_batch_decode_by_family"] = family
        # per-shape kernel time, weights rotated through > 1 GB so HBM serves them
        per_shape = {}
        for name, n_, k_ in shapes + [synth.LM_HEAD]:
            group = [l for l in launches if (l[4], l[5]) == (n_, k_)]
            def one(group=group):
                st = cur_stream()
                for wq, sc, x, y, nn, kk in group:
                    lib.cmi_gemv_w8a16(ptr(wq), ptr(sc), ptr(x), ptr(y), 1, nn, kk, st)
            t = timed(one, 5) / len(group)
            per_shape[name] = {"us": round(t * 1e6, 2),
                               "GBps": round(synth.gemv_bytes(1, n_, k_) / t / 1e9, 1)}
        extra["decode_gemv_int8_M1_per_shape_eager"] = per_shape

        # What each projection costs the replayed step: per shape, the same launches as a dependent
        # chain of their own in a captured graph (the 32 layers' weights of that shape, cold; four
        # copies of lm_head), time / launches = start-to-start interval of that shape in steady
        # state.  A kernel trace cannot show this: the profiler serialises dispatches and adds about
        # 3 us between them (the traced step takes 1.2 ms).  The intervals, weighted by how often
        # each shape occurs, must add up to ms_per_step.
        if M == 1 and not args.no_graph and not args.mfma:
            chain = {}
            total = 0.0
            for name, n_, k_ in shapes + [synth.LM_HEAD]:
                group = [l for l in launches if (l[4], l[5]) == (n_, k_)]
                count = len(group)
                extra_w = []
                if count < 4:   # lm_head: one weight in the model; three more so that none is answered from cache
                    extra_w = [synth.int8_weight(n_, k_, gen) for _ in range(3)]
                    group = group + [(q_.wq, q_.scale, group[0][2], group[0][3], n_, k_) for q_ in extra_w]
                def one(group=group):
                    st = cur_stream()
                    for wq, sc, x, y, nn, kk in group:
                        lib.cmi_gemv_w8a16(ptr(wq), ptr(sc), ptr(x), ptr(y), 1, nn, kk, st)
                one()
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr):
                    one()
                t = timed(gr.replay, 10, warm=3) / len(group)
                chain[name] = {"interval_us": round(t * 1e6, 3), "per_step": count,
                               "GBps": round(synth.gemv_bytes(1, n_, k_) / t / 1e9, 1)}
                total += count * t
                del gr, extra_w
            chain["sum_of_intervals_ms"] = round(total * 1e3, 4)
            chain["ms_per_step"] = round(step_s * 1e3, 4)
            extra["decode_gemv_int8_M1_per_shape_hipgraph_chain"] = chain

        # the same 129 projections through the table entry (backend.linear: Python adapter + ctypes +
        # a fresh output tensor per call), eager and as a captured graph: what the host side costs
        from coffin_amd import backend as _adapters
        from coffin_amd.weights import QWeight as _QW
        qws = [(_QW(wq, sc), x[0]) for wq, sc, x, *_ in launches]
        def adapter_step():
            for qw, x1 in qws:
                _adapters.linear(qw, x1)
        adapter_step()
        torch.cuda.synchronize()
        w0 = time.perf_counter()
        for _ in range(5):
            adapter_step()
        host_s = (time.perf_counter() - w0) / 5          # enqueue time: the launches run behind it
        t_eager = timed(adapter_step, 5)
        ag = torch.cuda.CUDAGraph()
        with torch.cuda.graph(ag):
            adapter_step()
        t_graph = timed(ag.replay, max(3, args.steps // 2))
        extra["decode_step_through_backend_linear_M1"] = {
            "eager_ms": round(t_eager * 1e3, 4), "eager_GBps": round(step_bytes(1) / t_eager / 1e9, 1),
            "host_enqueue_us_per_call": round(host_s / len(qws) * 1e6, 2),
            "hipgraph_ms": round(t_graph * 1e3, 4), "hipgraph_GBps": round(step_bytes(1) / t_graph / 1e9, 1)}
        del qws, ag

        # q, k and v as three projections (2560 -> 4096 / 1024 / 1024) instead of the fused qkv: the
        # 1024-row GEMVs are the smallest launches of the configuration
        unf = {}
        for name, n_, k_ in (("q_proj", 4096, 2560), ("k_proj", 1024, 2560), ("gate_proj", 9728, 2560)):
            copies = max(8, int(1.2e9 // (n_ * k_)))
            ws_ = [synth.int8_weight(n_, k_, gen) for _ in range(copies)]
            y1 = torch.empty((1, n_), dtype=torch.bfloat16, device=dev)
            def one(ws_=ws_, y1=y1, n_=n_, k_=k_):
                st = cur_stream()
                for q in ws_:
                    lib.cmi_gemv_w8a16(ptr(q.wq), ptr(q.scale), ptr(x_by_k[k_]), ptr(y1), 1, n_, k_, st)
            one()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                one()
            t = timed(gr.replay, 5) / copies
            unf[name] = {"us": round(t * 1e6, 2), "GBps": round(synth.gemv_bytes(1, n_, k_) / t / 1e9, 1)}
            del ws_, gr
        extra["decode_gemv_int8_M1_unfused_shapes_hipgraph"] = unf
        launches.clear()
        torch.cuda.empty_cache()

        # W4A8 decode step (int4 weights, per-token int8 activations), one and sixteen rows
        extra["w4a8_decode_step"] = {f"M{m}": w4a8_decode_step(m, True, max(3, args.steps // 2)) for m in (1, 16)}
        torch.cuda.empty_cache()
        extra["w4a8_decode_step"]["M1_prequantised"] = w4a8_decode_step(1, True, max(3, args.steps // 2), True)
        torch.cuda.empty_cache()
        extra["w4a8_decode_step"]["M16_prequantised"] = w4a8_decode_step(16, True, max(3, args.steps // 2), True)
        torch.cuda.empty_cache()
        for m in (1, 16):
            extra["w4a8_decode_step"][f"M{m}_through_table_entries"] = w4a8_step_through_table_entries(m, max(3, args.steps // 2))
            torch.cuda.empty_cache()

        # W4A8 decode GEMV (quantiser + GEMV, as the adapter issues them)
        w4 = {}
        for n_, k_ in ((9728, 2560), (2560, 9728)):
            copies = 40
            ws_ = []
            for _ in range(copies):
                w = synth.int4_weight(n_, k_, gen)
                d4 = torch.empty((n_, k_ // 2), dtype=torch.uint8, device=dev)
                ds = torch.empty((n_, k_ // 128), dtype=torch.float32, device=dev)
                _native.check(lib.cmi_w4_repack(ptr(w.packed), ptr(w.scale), ptr(d4), ptr(ds), n_, k_, 128,
                                                cur_stream()), "repack")
                ws_.append((d4, ds))
            torch.cuda.synchronize()
            for m in (1, 16):
                x = synth.activations(m, k_, gen)
                xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
                xs = torch.empty(m, dtype=torch.float32, device=dev)
                y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
                def one(m=m, x=x, xq=xq, xs=xs, y=y, ws_=ws_, n_=n_, k_=k_):
                    st = cur_stream()
                    for d4, ds in ws_:
                        lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, st)
                        lib.cmi_gemv_w4a8(ptr(d4), ptr(ds), ptr(xq), ptr(xs), ptr(y), vp(0), m, n_, k_, 128, st)
                t = timed(one, 5) / copies
                w4[f"{k_}->{n_}_M{m}"] = {"us": round(t * 1e6, 2),
                                          "GBps": round(synth.w4_gemv_bytes(m, n_, k_) / t / 1e9, 1)}
                if m <= 4:
                    def fused(m=m, x=x, y=y, ws_=ws_, n_=n_, k_=k_):
                        st = cur_stream()
                        for d4, ds in ws_:
                            lib.cmi_gemv_w4a8_bf16(ptr(d4), ptr(ds), ptr(x), ptr(y), vp(0), vp(0), vp(0),
                                                   m, n_, k_, 128, st)
                    t = timed(fused, 5) / copies
                    w4[f"{k_}->{n_}_M{m}_fused"] = {"us": round(t * 1e6, 2),
                                                    "GBps": round(synth.w4_gemv_bytes(m, n_, k_) / t / 1e9, 1)}
            del ws_
        extra["w4a8_gemv_quant_plus_gemv"] = w4
        torch.cuda.empty_cache()

        # W8A8 prefill GEMM (GEMM kernel alone, and quantiser + GEMM)
        mm = {}
        for m, n_ in ((2048, 9728), (2048, 4096), (512, 9728), (512, 4096), (8192, 9728), (8192, 4096)):
            k_ = 2560
            q = synth.int8_weight(n_, k_, gen)
            x = synth.activations(m, k_, gen, outliers=True)
            xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
            xs = torch.empty(m, dtype=torch.float32, device=dev)
            y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
            lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream())
            def gemm():
                lib.cmi_gemm_w8a8(ptr(xq), ptr(q.wq), ptr(xs), ptr(q.scale), ptr(y), vp(0), m, n_, k_, n_, cur_stream())
            def both():
                lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream())
                gemm()
            tg, tb = timed(gemm, 20), timed(both, 20)
            # the same GEMM as a prefill meets it, the weight not in any cache: rotated through
            # copies of 600 MB in total (Infinity Cache: 256 MB), the calls captured once
            copies = min(64, -(-600_000_000 // (n_ * k_)))
            cold_w = [synth.int8_weight(n_, k_, gen) for _ in range(copies)]
            def cold():
                st = cur_stream()
                for c in cold_w:
                    lib.cmi_gemm_w8a8(ptr(xq), ptr(c.wq), ptr(xs), ptr(c.scale), ptr(y), vp(0), m, n_, k_, n_, st)
            cold()
            torch.cuda.synchronize()
            cold_graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(cold_graph):
                cold()
            tc = timed(cold_graph.replay, 5) / copies
            del cold_graph, cold_w
            tops = synth.gemm_ops(m, n_, k_) / tg / 1e12
            mm[f"M{m}_N{n_}_K{k_}"] = {"gemm_us": round(tg * 1e6, 2), "tops": round(tops, 1),
                                      "frac_of_int8_peak": round(tops / INT8_PEAK_TOPS, 4),
                                      "quant_plus_gemm_us": round(tb * 1e6, 2),
                                      "gemm_cold_weight_us": round(tc * 1e6, 2)}
        extra["w8a8_prefill_gemm"] = mm
        extra["w8a8_prefill_int8_TOPS_M2048_N9728"] = mm["M2048_N9728_K2560"]["tops"]

        # W8A8 on a verify-sized batch (16 rows): quantiser + the read-once kernel, weights rotated
        # through enough copies that none is answered from cache
        vf = {}
        for name, n_, k_ in shapes:
            copies = max(2, int(6e8 // (n_ * k_)))
            ws_ = [synth.int8_weight(n_, k_, gen) for _ in range(copies)]
            m = 16
            x = synth.activations(m, k_, gen)
            xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
            xs = torch.empty(m, dtype=torch.float32, device=dev)
            y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
            def verify(ws_=ws_, x=x, xq=xq, xs=xs, y=y, m=m, n_=n_, k_=k_):
                st = cur_stream()
                for q in ws_:
                    lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, st)
                    lib.cmi_gemm_w8a8(ptr(xq), ptr(q.wq), ptr(xs), ptr(q.scale), ptr(y), vp(0), m, n_, k_, n_, st)
            t = timed(verify, 5) / copies
            vf[name] = {"us": round(t * 1e6, 2), "GBps": round(n_ * k_ / t / 1e9, 1)}
            del ws_
        extra["w8a8_verify_M16_quant_plus_gemm"] = vf

        # 64 and 128 rows (between the GEMV and the tile pipeline) on the two MLP shapes, the three
        # weight formats as the adapter issues them: weight-only on the matrix-pipe GEMV (64 rows per
        # call), cmi_linear_w8a8_bf16 and cmi_linear_w4a8_bf16 (quantiser + GEMM) on the adapter's workspace
        # and a 512-row prefill chunk (a chat-sized prompt) on the four layer shapes, W8A8 and W4A8
        for m in (64, 128, 512):
            mid = {}
            shapes = ((9728, 2560), (2560, 9728)) if m < 512 else ((6144, 2560), (2560, 4096), (19456, 2560), (2560, 9728))
            for n_, k_ in shapes:
                copies = max(12, -(-300_000_000 // (n_ * k_)))
                w8 = [synth.int8_weight(n_, k_, gen) for _ in range(copies)]
                w4_ = []
                for _ in range(copies):
                    w = synth.int4_weight(n_, k_, gen)
                    d4 = torch.empty((n_, k_ // 2), dtype=torch.uint8, device=dev)
                    ds = torch.empty((n_, k_ // 128), dtype=torch.float32, device=dev)
                    lib.cmi_w4_repack(ptr(w.packed), ptr(w.scale), ptr(d4), ptr(ds), n_, k_, 128, cur_stream())
                    w4_.append((d4, ds))
                torch.cuda.synchronize()
                x = synth.activations(m, k_, gen)
                xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
                xs = torch.empty(m, dtype=torch.float32, device=dev)
                y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
                rows_per_call = 64
                def weight_only():
                    st = cur_stream()
                    for q in w8:
                        for lo in range(0, m, rows_per_call):
                            lib.cmi_gemv_w8a16_mfma(ptr(q.wq), ptr(q.scale), vp(x.data_ptr() + lo * k_ * 2),
                                                    vp(y.data_ptr() + lo * n_ * 2), rows_per_call, n_, k_, st)
                work = torch.empty(int(lib.cmi_linear_w8a8_workspace_bytes(m, n_, k_)), dtype=torch.uint8, device=dev)
                def w8a8():
                    st = cur_stream()
                    for q in w8:
                        lib.cmi_linear_w8a8_bf16(ptr(x), ptr(q.wq), ptr(q.scale), ptr(y), m, n_, k_, n_,
                                                 ptr(work), work.numel(), st)
                def w4a8():
                    st = cur_stream()
                    for d4, ds in w4_:
                        lib.cmi_linear_w4a8_bf16(ptr(d4), ptr(ds), ptr(x), ptr(y), m, n_, k_, 128,
                                                 ptr(work), work.numel(), st)
                def replayed(fn):  # the calls on `copies` cold weights, captured once
                    fn()
                    torch.cuda.synchronize()
                    gr = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(gr):
                        fn()
                    return timed(gr.replay, 5) / copies
                routes = (("weight_only_us", weight_only), ("w8a8_us", w8a8), ("w4a8_us", w4a8))
                mid[f"{k_}->{n_}"] = {name: round(replayed(fn) * 1e6, 2) for name, fn in routes[(0 if m < 512 else 1):]}
                del w8, w4_
            extra[f"mid_batch_M{m}" if m < 512 else f"prefill_chunk_M{m}_quant_plus_gemm"] = mid
        torch.cuda.empty_cache()
        torch.cuda.empty_cache()

        # W4A8 prefill GEMM, larger dense shape
        m, n_, k_ = 1024, 25600, 5120
        w = synth.int4_weight(n_, k_, gen)
        d4 = torch.empty((n_, k_ // 2), dtype=torch.uint8, device=dev)
        ds = torch.empty((n_, k_ // 128), dtype=torch.float32, device=dev)
        lib.cmi_w4_repack(ptr(w.packed), ptr(w.scale), ptr(d4), ptr(ds), n_, k_, 128, cur_stream())
        x = synth.activations(m, k_, gen)
        xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
        xs = torch.empty(m, dtype=torch.float32, device=dev)
        y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
        lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream())
        def w4gemm():
            lib.cmi_gemm_w4a8(ptr(d4), ptr(ds), ptr(xq), ptr(xs), ptr(y), vp(0), m, n_, k_, 128, cur_stream())
        t = timed(w4gemm, 10)
        tops = synth.gemm_ops(m, n_, k_) / t / 1e12
        extra["w4a8_prefill_gemm_M1024_N25600_K5120"] = {
            "us": round(t * 1e6, 2), "tops": round(tops, 1), "frac_of_int8_peak": round(tops / INT8_PEAK_TOPS, 4)}

        # W4A8 larger dense shape, both directions, M = 1 / 64 / 1024 (quantiser + GEMV or GEMM, as
        # the adapter issues them); a few distinct weights per shape so that no call finds its
        # weight in a cache
        sweep = {}
        for n_, k_ in ((25600, 5120), (5120, 25600)):
            ws_ = []
            for _ in range(4):
                w = synth.int4_weight(n_, k_, gen)
                d4 = torch.empty((n_, k_ // 2), dtype=torch.uint8, device=dev)
                ds = torch.empty((n_, k_ // 128), dtype=torch.float32, device=dev)
                lib.cmi_w4_repack(ptr(w.packed), ptr(w.scale), ptr(d4), ptr(ds), n_, k_, 128, cur_stream())
                ws_.append((d4, ds))
            torch.cuda.synchronize()
            for m in (1, 64, 1024):
                x = synth.activations(m, k_, gen)
                xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
                xs = torch.empty(m, dtype=torch.float32, device=dev)
                y = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
                fn = lib.cmi_gemv_w4a8 if m <= 16 else lib.cmi_gemm_w4a8
                def both(m=m, x=x, xq=xq, xs=xs, y=y, ws_=ws_, n_=n_, k_=k_, fn=fn):
                    st = cur_stream()
                    for d4, ds in ws_:
                        lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, st)
                        fn(ptr(d4), ptr(ds), ptr(xq), ptr(xs), ptr(y), vp(0), m, n_, k_, 128, st)
                t = timed(both, 5) / len(ws_)
                sweep[f"{k_}->{n_}_M{m}"] = {
                    "us": round(t * 1e6, 2), "GBps": round(synth.w4_gemv_bytes(m, n_, k_) / t / 1e9, 1),
                    "tops": round(synth.gemm_ops(m, n_, k_) / t / 1e12, 1)}
            del ws_
        extra["w4a8_large_shape_quant_plus_linear"] = sweep
        torch.cuda.empty_cache()

        # quantiser alone at prefill size
        m, k_ = 8192, 2560
        x = synth.activations(m, k_, gen)
        xq = torch.empty((m, k_), dtype=torch.int8, device=dev)
        xs = torch.empty(m, dtype=torch.float32, device=dev)
        t = timed(lambda: lib.cmi_quant_act_i8(ptr(x), ptr(xq), ptr(xs), m, k_, cur_stream()), 20)
        extra["quant_act_i8_M8192_K2560"] = {"us": round(t * 1e6, 2),
                                             "GBps": round(synth.quant_bytes(m, k_) / t / 1e9, 1)}
        torch.cuda.empty_cache()

        # fused producers, embedding gather and W4A16: algorithmic bytes / time against the HBM peak
        def hbm_line(t, nbytes):
            return {"us": round(t * 1e6, 2), "GBps": round(nbytes / t / 1e9, 1),
                    "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBPS, 4)}
        prod = {}

        def graph_time(calls):
            """Mean time of one call: the calls (each on operands of its own) captured once, replayed."""
            for c in calls:
                c()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                for c in calls:
                    c()
            return timed(gr.replay, 5) / len(calls)

        for m in (1, 2048, 8192):
            copies = 16 if m == 1 else 6
            kk = 9728      # silu(gate) * up over the two halves of a fused gate_up row -> bf16 + int8 + scale
            sets = []
            for _ in range(copies):
                gu = synth.activations(m, 2 * kk, gen)
                sets.append((gu, gu[:, kk:], torch.empty((m, kk), dtype=torch.bfloat16, device=dev),
                             torch.empty((m, kk), dtype=torch.int8, device=dev),
                             torch.empty(m, dtype=torch.float32, device=dev)))
            t = graph_time([lambda s_=s_: lib.cmi_silu_mul_quant(ptr(s_[0]), ptr(s_[1]), ptr(s_[2]), ptr(s_[3]), ptr(s_[4]),
                                                                  m, kk, 2 * kk, 2 * kk, kk, cur_stream()) for s_ in sets])
            prod[f"silu_mul_quant_M{m}_K{kk}"] = hbm_line(t, m * kk * 7 + 4 * m)
            t = graph_time([lambda s_=s_: lib.cmi_silu_mul_quant(ptr(s_[0]), ptr(s_[1]), None, ptr(s_[3]), ptr(s_[4]),
                                                                  m, kk, 2 * kk, 2 * kk, kk, cur_stream()) for s_ in sets])
            prod[f"silu_mul_quant_int8_only_M{m}_K{kk}"] = hbm_line(t, m * kk * 5 + 4 * m)
            del sets
            torch.cuda.empty_cache()
            nn = 2560      # RMSNorm (and residual add + RMSNorm, residual written back) -> int8 row + scale
            gain = synth.activations(1, nn, gen)[0].contiguous()
            sets = [(synth.activations(m, nn, gen), synth.activations(m, nn, gen),
                     torch.empty((m, nn), dtype=torch.int8, device=dev),
                     torch.empty(m, dtype=torch.float32, device=dev)) for _ in range(copies)]
            t = graph_time([lambda s_=s_: lib.cmi_rms_norm_i8(ptr(s_[0]), ptr(gain), None, ptr(s_[2]), ptr(s_[3]), m, nn,
                                                               nn, nn, 1e-6, cur_stream()) for s_ in sets])
            prod[f"rms_norm_i8_M{m}_N{nn}"] = hbm_line(t, m * nn * 3 + 2 * nn + 4 * m)
            t = graph_time([lambda s_=s_: lib.cmi_add_rms_norm_i8(ptr(s_[0]), ptr(s_[1]), ptr(gain), None, ptr(s_[2]),
                                                                   ptr(s_[3]), m, nn, nn, nn, nn, 1e-6, cur_stream())
                            for s_ in sets])
            prod[f"add_rms_norm_i8_M{m}_N{nn}"] = hbm_line(t, m * nn * 7 + 2 * nn + 4 * m)
            t = graph_time([lambda s_=s_: lib.cmi_quant_act_i8(ptr(s_[0]), ptr(s_[2]), ptr(s_[3]), m, nn, cur_stream())
                            for s_ in sets])
            prod[f"quant_act_i8_M{m}_K{nn}"] = hbm_line(t, m * nn * 3 + 4 * m)
            del sets, gain
            torch.cuda.empty_cache()
        extra["fused_producers"] = prod
        torch.cuda.empty_cache()

        emb = {}
        q = synth.int8_weight(151936, 2560, gen)
        for tkn in (1, 2048):
            sets = [(torch.randint(0, 151936, (tkn,), device=dev, dtype=torch.int64),
                     torch.empty((tkn, 2560), dtype=torch.bfloat16, device=dev)) for _ in range(8)]
            t = graph_time([lambda s_=s_: lib.cmi_embed_rows_i8(ptr(q.wq), ptr(q.scale), ptr(s_[0]), ptr(s_[1]), tkn,
                                                                 151936, 2560, cur_stream()) for s_ in sets])
            emb[f"int8_T{tkn}_K2560"] = hbm_line(t, tkn * (2560 * 3 + 12))
            del sets
        del q
        extra["embed_rows"] = emb
        torch.cuda.empty_cache()

        w16 = {}
        for n_, k_ in ((9728, 2560), (2560, 9728), (5120, 25600)):
            copies = 16 if k_ <= 10240 else 6
            ws4 = []
            for _ in range(copies):
                w = synth.int4_weight(n_, k_, gen)
                d4 = torch.empty((n_, k_ // 2), dtype=torch.uint8, device=dev)
                ds = torch.empty((n_, k_ // 128), dtype=torch.float32, device=dev)
                _native.check(lib.cmi_w4_repack(ptr(w.packed), ptr(w.scale), ptr(d4), ptr(ds), n_, k_, 128, cur_stream()), "repack")
                ws4.append((d4, ds))
                del w
            xv = synth.activations(1, k_, gen)
            yv = torch.empty((1, n_), dtype=torch.bfloat16, device=dev)
            def one(ws4=ws4, xv=xv, yv=yv, n_=n_, k_=k_):
                st = cur_stream()
                for d4, ds in ws4:
                    lib.cmi_gemv_w4a16(ptr(d4), ptr(ds), ptr(xv), ptr(yv), n_, k_, 128, st)
            one()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                one()
            t = timed(gr.replay, 5) / copies
            w16[f"{k_}->{n_}"] = hbm_line(t, synth.w4_gemv_bytes(1, n_, k_))
            del ws4, gr
        extra["w4a16_gemv_M1_hipgraph"] = w16
        torch.cuda.empty_cache()

        # weight rows longer than two rounds of registers (K = 25600, the long side of the int4 model,
        # as an int8 weight): both weight-only families at 1..64 rows, cold weights (4 x 131 MB)
        n_, k_ = 5120, 25600
        long_w = [synth.int8_weight(n_, k_, gen) for _ in range(4)]
        long_rows = {}
        for m in (1, 4, 16, 64):
            xv = synth.activations(m, k_, gen)
            yv = torch.empty((m, n_), dtype=torch.bfloat16, device=dev)
            turn = [0]
            def mfma_family():
                c = long_w[turn[0] % 4]
                turn[0] += 1
                _native.check(lib.cmi_linear_w8a16(ptr(c.wq), ptr(c.scale), ptr(xv), ptr(yv), m, n_, k_, 1, cur_stream()), "linear_w8a16")
            def dot_family():
                c = long_w[turn[0] % 4]
                turn[0] += 1
                _native.check(lib.cmi_linear_w8a16(ptr(c.wq), ptr(c.scale), ptr(xv), ptr(yv), m, n_, k_, 0, cur_stream()), "linear_w8a16")
            long_rows[f"M{m}"] = {"mfma_us": round(timed(mfma_family, 8) * 1e6, 1), "dot_us": round(timed(dot_family, 8) * 1e6, 1)}
        extra["w8a16_long_rows_25600_to_5120_by_family"] = long_rows
        del long_w
        result["extra"] = extra

    # ------------------------------------------------------------------ CPU baseline leg
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_baseline(args.cpu_seconds, synth, torch)

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
