#!/usr/bin/env python3
"""Benchmark of the op path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Prints ONE JSON line.  The headline workload is BASELINE.json's config 2 at its largest size: mmul bf16,
M = N = K = 4096, entries ~ N(0, 1/sqrt(K)) from seed 2002, output bf16, fp32 accumulation; one "step" is one
execCustomOp2(matmul) call through the C ABI with the operands already resident in HBM.
`value` = 2*M*N*K*steps / wall time of the timed region.  The `roofline` object prices the dominant kernel
against the dense bf16 MFMA peak; `cpu_baseline` times the CPU oracle (a restatement of the reference's
nd4j-native path) on a bounded sample of the same product on the host cores.  The `ops` list carries the other
BASELINE configs (legacy chain, row ops, attention) measured the same way, each with its own roofline entry and its
own cpu_baseline.

Memory-bound lines are measured COLD: the op rotates over several disjoint sets of input / output arrays whose
total footprint exceeds 600 MB, so no launch finds its operands in the 256 MB last-level cache; `roofline.frac` is
that figure, `frac_warm` the one from re-running on a single set (an upper bound: the set may sit in the cache).
Each cpu_baseline has two modes: "port" = the oracle's loops with the reference's per-element coordinate
arithmetic, on all host threads ("faithful"), and `fast` = the same arithmetic as dense vectorised numpy calls
(OpenBLAS for fp32 GEMM), both on a bounded sample of the op's input.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_PEAK = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}   # dense TFLOP/s

# HBM-side bytes per launch of the kernel behind each line, measured once with `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` (separate runs of this script) and scaled by what the same counters read for the plain copy
# kernel; the summary of those runs sits under profiles/.  Static figures: they are not re-measured here.
TRAFFIC_MB = {
    "mmul bf16 4096": 235.2, "mmul f16 4096": 235.2, "mmul f32 4096^3": 862.9, "mmul f32 4096^3 transposeB": 861.4,
    "mmul f32 1024": 29.5, "mmul f16 1024": 14.8, "mmul bf16 1024": 14.8,
    "copy fp32": 268.4, "pairwise_add fp32": 402.6, "transform_tanh fp32": 268.4, "reduce_sum": 134.5, "argmax dim1": 134.5,
    "layer_norm fp32": 100.8, "gelu fp32": 100.7, "softmax fp32": 1610.6, "layer_norm bf16": 50.4, "gelu bf16": 50.4,
    "softmax bf16": 805.3, "dot_product_attention_v2": 50.5, "dot_product_attention_v2 f32": 110.9,
    "reduce_cols": 101.0, "index_cols": 101.2, "transpose_tiled": 201.2, "cast_contig": 150.9, "softmax_block_regs": 205.8,
    "mmul unaligned": 913.8, "mmul ragged tb": 903.1, "mmul ragged bf16 500": 12.6, "mmul ragged bf16 2000": 58.9, "mmul ragged f32 2000": 115.5,
}


def traffic_of(label):
    best = None
    for k, v in TRAFFIC_MB.items():
        if label.startswith(k) and (best is None or len(k) > len(best[0])):
            best = (k, v)
    return None if best is None else int(best[1] * 1e6)


SETTLE_S = 0.06   # untimed run of an op before its warmup steps, see settle()


def settle(L, fn, seconds=None):
    """Untimed launches of fn for `seconds` of wall time.  The GPU's clock governor needs about 30 ms of sustained load to
    reach its steady state: the first launches after an idle period run 20-80 % longer (a 4096^3 bf16 GEMM: 195 us for
    the first hundred launches, 101 us from the third hundred on), so a figure timed right after a handful of warmup
    steps says more about the governor's ramp than about the kernel.  Every timed region here starts from that steady state."""
    seconds = SETTLE_S if seconds is None else seconds
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(25):
            fn()
        L.streamSynchronize(None)


def timed(ex, L, fn, steps, warmup, settled=True):
    """Run fn() warmup + steps times; returns (wall ms per step, event ms per step on the execution stream)."""
    if settled:
        settle(L, fn)
    for _ in range(warmup):
        fn()
    L.streamSynchronize(None)
    e0, e1 = L.nd4jhipCreateTimingEvent(), L.nd4jhipCreateTimingEvent()
    t0 = time.perf_counter()
    L.registerEvent(e0, None)
    for _ in range(steps):
        fn()
    L.registerEvent(e1, None)
    L.streamSynchronize(None)
    t1 = time.perf_counter()
    ev = L.nd4jhipEventElapsedMs(e0, e1)
    L.destroyEvent(e0)
    L.destroyEvent(e1)
    return (t1 - t0) * 1e3 / steps, ev / steps


def timed_rotating(ex, L, fns, steps, warmup):
    """Like timed(), cycling through the callables of `fns` (one per disjoint operand set)."""
    k = len(fns)
    n_pre = [0]

    def cycle():
        fns[n_pre[0] % k]()
        n_pre[0] += 1

    settle(L, cycle)
    for i in range(max(warmup, k)):
        fns[i % k]()
    L.streamSynchronize(None)
    e0, e1 = L.nd4jhipCreateTimingEvent(), L.nd4jhipCreateTimingEvent()
    t0 = time.perf_counter()
    L.registerEvent(e0, None)
    for i in range(steps):
        fns[i % k]()
    L.registerEvent(e1, None)
    L.streamSynchronize(None)
    t1 = time.perf_counter()
    ev = L.nd4jhipEventElapsedMs(e0, e1)
    L.destroyEvent(e0)
    L.destroyEvent(e1)
    return (t1 - t0) * 1e3 / steps, ev / steps


COLD_FOOTPRINT = 640e6     # bytes the rotating sets must cover together (the last-level cache holds 256 MB)


def n_sets(bytes_per_call):
    return max(3, int(math.ceil(COLD_FOOTPRINT / bytes_per_call)))


def hbm_entry(bytes_per_launch, ev_ms, label="", warm_ms=None, sets=None):
    ach = bytes_per_launch / (ev_ms * 1e-3) / 1e9
    e = {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
         "traffic": traffic_of(label)}
    if warm_ms is not None:
        e["frac_warm"] = round(bytes_per_launch / (warm_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        e["cold_sets"] = sets
    return e


def best_time(fn, reps=2):
    best = None
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    return best


def cpu_entry(work, unit_scale, unit, faithful, fast, sample, fast_how, fast_cores=1):
    """cpu_baseline object of one op: `work` algorithmic bytes or flops of the sample; faithful / fast are callables."""
    from oracle import oracle as O
    tf = best_time(faithful, 1)
    e = {"value": round(work / tf / unit_scale, 4), "unit": unit, "cores": O.get_threads(), "kind": "port",
         "sample": "%s, %.2f s" % (sample, tf)}
    if fast is not None:
        tq = best_time(fast)
        e["fast"] = {"value": round(work / tq / unit_scale, 4), "unit": unit, "cores": fast_cores, "how": fast_how}
    return e


def mfma_entry(flops, ev_ms, dtype, label=""):
    ach = flops / (ev_ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(ach, 2), "peak": MFMA_PEAK[dtype], "unit": "TFLOP/s", "frac": round(ach / MFMA_PEAK[dtype], 4),
            "traffic": traffic_of(label)}


def clock_study(ex, L):
    """The 4096^3 product under a sampled clock.  The published matrix peak assumes the top shader clock; under a sustained
    matrix load the package power limit decides the clock, and the power depends on the operand VALUES (bits that toggle in the
    multipliers), not only on the instruction stream.  Same kernel, same launch count per case; what changes is the data."""
    import subprocess
    import threading
    from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32, HALF, NDArray
    n = 4096
    rng = np.random.default_rng(2002)
    base_a = rng.normal(0, 1 / math.sqrt(n), (n, n)).astype(np.float32)
    base_b = rng.normal(0, 1 / math.sqrt(n), (n, n)).astype(np.float32)
    data = {"N(0,1/sqrt(K)) (the BASELINE operands)": (base_a, base_b), "all zeros": (np.zeros_like(base_a), np.zeros_like(base_b)),
            "all ones / 64": (np.full_like(base_a, 1 / 64), np.full_like(base_b, 1 / 64))}
    samples, stop = [], [False]

    def sampler():
        while not stop[0]:
            try:
                out = subprocess.run(["/opt/rocm/bin/rocm-smi", "--showpower", "--showclocks", "--json"], capture_output=True, text=True, timeout=10).stdout
                samples.append((time.perf_counter(), out))
            except Exception as exc:   # the tool is not there: the timings still stand
                samples.append((time.perf_counter(), "ERR %r" % (exc,)))
            time.sleep(0.25)

    def digits(v):
        m = "".join(ch for ch in str(v) if ch.isdigit() or ch == ".")
        return float(m) if m else None

    cases, first_sample = [], []
    for dt, dtn, launches in ((BFLOAT16, "bf16", 12000), (HALF, "f16", 12000), (FLOAT32, "f32", 1500)):
        for label, (a, b) in data.items():
            if dt == HALF:
                A, B = NDArray.from_numpy(a.astype(np.float16), dt), NDArray.from_numpy(b.astype(np.float16), dt)
            else:
                A, B = NDArray.from_numpy(a, dt), NDArray.from_numpy(b, dt)
            Z = NDArray.empty((n, n), dt)
            A.sync_to_device(); B.sync_to_device()
            fn = ex.bind_custom("matmul", [A, B], [Z])
            settle(L, fn, 0.3)
            del samples[:]
            stop[0] = False
            th = threading.Thread(target=sampler)
            th.start()
            t_start = time.perf_counter()
            per_launch = []
            for _ in range(3):
                _, e = timed(ex, L, fn, launches, 0, settled=False)
                per_launch.append(e * 1e3)
            t_end = time.perf_counter()
            stop[0] = True
            th.join()
            sclk, power = [], []
            for ts, out in samples:
                if not (t_start + 0.3 <= ts <= t_end):
                    continue
                try:
                    card = json.loads(out)
                    card = card[sorted(card.keys())[0]]
                    if not first_sample:
                        first_sample.append(card)
                    for k, v in card.items():
                        kl = k.lower()
                        if "sclk" in kl and "clock speed" in kl:
                            sclk.append(digits(str(v).split("(")[-1]))
                        elif "power" in kl and ("socket" in kl or "average" in kl or "package" in kl):
                            power.append(digits(v))
                except Exception:
                    pass
            us = sorted(per_launch)[1]
            cases.append({"dtype": dtn, "operands": label, "kernel": L.nd4jhipLastGemmKernel().decode(), "us_per_launch": [round(v, 2) for v in per_launch],
                          "tflops": round(2.0 * n ** 3 / (us * 1e-6) / 1e12, 1),
                          "sclk_mhz": {"samples": len(sclk), "min": min(sclk) if sclk else None, "median": sorted(sclk)[len(sclk) // 2] if sclk else None, "max": max(sclk) if sclk else None},
                          "power_w": {"samples": len(power), "median": sorted(power)[len(power) // 2] if power else None, "max": max(power) if power else None}})
            print("[clock-study] %s" % json.dumps(cases[-1]), file=sys.stderr, flush=True)
            del A, B, Z, fn
    print(json.dumps({"clock_study": cases, "one_raw_sample": first_sample[:1], "launches_per_case": "3 x 12000 (16-bit) / 3 x 1500 (fp32), back to back; the middle figure is quoted",
                      "sampling": "rocm-smi --showpower --showclocks --json every 0.25 s while the launches run (the first 0.3 s dropped)"}))


def main():
    global SETTLE_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--skip-ops", action="store_true", help="leave out the per-op lines of BASELINE configs 1-4")
    ap.add_argument("--configs", default="1,2,3,4,x", help="which BASELINE configs the per-op lines cover (comma-separated; for profiling one op class); "
                                                           "x = the kernels for shapes outside the configs (column reductions, transposing copies, long softmax rows, casts)")
    ap.add_argument("--skip-cpu", action="store_true", help="leave out the cpu_baseline leg")
    ap.add_argument("--skip-decode", action="store_true", help="leave out the GPT-2-shaped decode (tens of thousands of launches)")
    ap.add_argument("--settle", type=float, default=SETTLE_S,
                    help="seconds of untimed launches of an op before its warmup steps (0 for counter-collection runs under rocprofv3)")
    ap.add_argument("--no-graphs", action="store_true",
                    help="time the decode op by op only (for runs under rocprofv3: its kernel tracing aborts the queue on graph replays)")
    ap.add_argument("--decode-batches", default="1,32", help="batch sizes of the decode leg (comma-separated)")
    ap.add_argument("--clock-study", action="store_true",
                    help="instead of the benchmark: run the 4096^3 product for a few seconds per case (bf16 / f16 / f32; the BASELINE data, all-zero "
                         "operands, constant operands) while rocm-smi samples the shader clock and the package power; prints one JSON object")
    ap.add_argument("--replay-kernels", action="store_true",
                    help="decode: time only the replay that launches each recorded, merged step kernel by kernel (no graph launch: for a kernel trace of the merged step)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend is built and measured on one GPU; --gpus %d is not supported (no collectives are part of the op path)" % args.gpus)

    from deeplearning4j_amd.executioner import Executioner, IndexReduce, Pairwise, ReduceSame, TransformSame, TransformStrict
    from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32, HALF, NDArray, f32_to_bf16_bits

    ex = Executioner()
    L = ex.L
    L.nd4jhipSetSyncAfterCustomOp(0)     # the timed loop synchronises once at its end
    steps, warmup = args.steps, args.warmup
    SETTLE_S = args.settle

    if args.clock_study:
        clock_study(ex, L)
        return

    # ---- headline: mmul bf16 4096^3 ----------------------------------------------------------------------------
    n = 4096
    rng = np.random.default_rng(2002)
    a = rng.normal(0, 1 / math.sqrt(n), (n, n)).astype(np.float32)
    b = rng.normal(0, 1 / math.sqrt(n), (n, n)).astype(np.float32)
    A, B = NDArray.from_numpy(a, BFLOAT16), NDArray.from_numpy(b, BFLOAT16)
    Z = NDArray.empty((n, n), BFLOAT16)
    A.sync_to_device()
    B.sync_to_device()
    flops = 2.0 * n * n * n
    mm = ex.bind_custom("matmul", [A, B], [Z])
    # the very first launches, with the GPU coming out of idle, for the record; then the steady state `value` is quoted on
    _, ev_first = timed(ex, L, mm, 20, 0, settled=False)
    wall_ms, ev_ms = timed(ex, L, mm, steps, warmup)
    value = flops / (wall_ms * 1e-3) / 1e12
    _, ev200 = timed(ex, L, mm, 200, 5)
    result = {
        "metric": "mmul TFLOP/s (bf16, M=N=K=4096, fp32 accumulate)", "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "mmul bf16 A[4096,4096] x B[4096,4096] (BASELINE config 2), N(0,1/sqrt(K)) seed 2002, via execCustomOp2(matmul)"},
        "roofline": mfma_entry(flops, ev_ms, "bf16", "mmul bf16 4096"),
        "value_is": "wall time over the %d timed steps, after %.2f s of untimed launches of the same op and the %d warmup steps (steady clocks)" % (steps, SETTLE_S, warmup),
        "tflops_by_state": {"first_20_launches_out_of_idle": round(flops / (ev_first * 1e-3) / 1e12, 1), "steady_200_steps": round(flops / (ev200 * 1e-3) / 1e12, 1)},
    }

    # ---- cpu baseline: the oracle's usualGemm restatement on a bounded sample ------------------------------------
    if not args.skip_cpu:
        print("[bench] cpu baseline leg (about 15 s)", file=sys.stderr, flush=True)
        from oracle import oracle as O
        ab, bb = f32_to_bf16_bits(a), f32_to_bf16_bits(b)
        rows = 64
        oa = O.Arr(ab[:rows], O.BFLOAT16)
        ob = O.Arr(bb, O.BFLOAT16)
        oz = O.Arr(np.zeros((rows, n), np.uint16), O.BFLOAT16)
        t0 = time.perf_counter()
        O.matmul(oa, ob, oz, accumulate=0)    # multiply/accumulate in the output type, as the reference's CPU loop does
        probe = time.perf_counter() - t0
        rows2 = int(min(n, max(rows, rows * 15.0 / max(probe, 1e-3))))
        rows2 -= rows2 % 8
        oa = O.Arr(ab[:rows2], O.BFLOAT16)
        oz = O.Arr(np.zeros((rows2, n), np.uint16), O.BFLOAT16)
        t0 = time.perf_counter()
        O.matmul(oa, ob, oz, accumulate=0)
        dt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": round(2.0 * rows2 * n * n / dt / 1e12, 5), "unit": "TFLOP/s", "cores": O.get_threads(), "kind": "port",
                                  "sample": "first %d of 4096 rows of A against the full B (bf16 usualGemm restatement, accumulation in bf16), %.1f s" % (rows2, dt)}

    # ---- the other BASELINE configs ------------------------------------------------------------------------------------
    ops = []
    cfgs = {int(c) for c in args.configs.split(",") if c.strip() and c.strip() != "x"}
    extras = "x" in [c.strip() for c in args.configs.split(",")]
    if not args.skip_ops:
        print("[bench] per-op leg", file=sys.stderr, flush=True)
        del A, B, Z
        from deeplearning4j_amd.ndarray import INT64, bf16_bits_to_f32
        cpu = not args.skip_cpu
        if cpu:
            from oracle import oracle as O

        def hbm_line(name, label, nbytes, make_call, cpu_fn=None):
            """make_call(i) -> zero-argument callable on operand set i.  Cold = rotating over the sets, warm = set 0 only."""
            k = n_sets(nbytes)
            calls = [make_call(i) for i in range(k)]
            _, e_warm = timed(ex, L, calls[0], steps, warmup)
            w, e = timed_rotating(ex, L, calls, max(steps, 2 * k), warmup)   # last, so that a trace ends on the cold steps
            line = {"op": name, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(nbytes, e, label, e_warm, k)}
            if cpu and cpu_fn is not None:
                line["cpu_baseline"] = cpu_fn()
            ops.append(with_copy_fraction(line, nbytes))

        # What a cold launch of a given size reaches at all on this chip: the plain copy kernel (transform_same Copy, fp32) at
        # the total traffic of each memory-bound line below, timed the same way (cold over rotating sets, then warm).  Every
        # memory-bound line then carries `frac_of_copy` = its rate over the rate of the copy of the nearest size.
        copy_rate = {}      # total bytes per launch -> (cold GB/s, warm GB/s)
        if cfgs & {1, 3}:
            sizes = []
            if 1 in cfgs:
                sizes += [134217728, 268435456, 402653184]
            if 3 in cfgs:
                sizes += [50331648, 100663296, 805306368, 1610612736]
            for total in sorted(sizes):
                ne_c = total // 8
                kc = 1 if total >= 600e6 else n_sets(total // 2)   # inputs alone past the cache footprint, as the op lines below rotate them
                Cin = [NDArray.empty((ne_c,), FLOAT32) for _ in range(kc)]
                Cout = [NDArray.empty((ne_c,), FLOAT32) for _ in range(min(kc, 3))]
                for arr in Cin + Cout:
                    L.dbAllocateSpecialBuffer(arr.buffer.ptr)
                    L.dbTickDeviceWrite(arr.buffer.ptr)           # contents do not matter: no upload
                calls = [(lambda i: (lambda: ex.exec_transform_same(TransformSame.Copy, Cin[i], Cout[i % len(Cout)])))(i) for i in range(kc)]
                w_warm, e_warm = timed(ex, L, calls[0], steps, warmup)
                if kc > 1:
                    w, e = timed_rotating(ex, L, calls, max(steps, 2 * kc), warmup)
                else:
                    w, e = w_warm, e_warm     # one call streams past the cache by itself
                copy_rate[total] = (total / (e * 1e-3) / 1e9, total / (e_warm * 1e-3) / 1e9)
                ops.append({"op": "copy fp32, %.1f MB in + %.1f MB out (calibration: what a cold launch of this size reaches)" % (total / 2e6, total / 2e6),
                            "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(total, e, "", e_warm if kc > 1 else None, kc if kc > 1 else None)})
                del Cin, Cout, calls

        def with_copy_fraction(line, nbytes):
            if copy_rate:
                near = min(copy_rate, key=lambda t: abs(math.log(t / nbytes)))
                line["roofline"]["frac_of_copy"] = round(line["roofline"]["achieved"] / copy_rate[near][0], 4)
                line["roofline"]["copy_of_bytes"] = near
            return line

        if 1 in cfgs:
            # config 1: legacy chain, fp32 [8192, 4096]
            rng = np.random.default_rng(1001)
            shp = (8192, 4096)
            ne = shp[0] * shp[1]
            xh = rng.uniform(-1, 1, shp).astype(np.float32)
            yh = rng.uniform(-1, 1, shp).astype(np.float32)
            K1 = n_sets(4 * ne)        # the reductions read 128 MiB per call: they need the most sets
            Xs = [NDArray.from_numpy(xh) for _ in range(K1)]
            Ys = [NDArray.from_numpy(yh) for _ in range(3)]
            Ss = [NDArray.empty(shp, FLOAT32) for _ in range(3)]
            Rs = [NDArray.empty((shp[0],), FLOAT32) for _ in range(K1)]
            AMs = [NDArray.empty((shp[0],), INT64) for _ in range(K1)]
            for arr in Xs + Ys:
                arr.sync_to_device()
            rows_s = 1024                                     # CPU sample: the first 1024 rows (4 Mi elements)
            xs_, ys_ = xh[:rows_s].copy(), yh[:rows_s].copy()
            zs_ = np.zeros_like(xs_)
            samp = "first %d of 8192 rows" % rows_s
            GB = 1e9
            hbm_line("copy fp32 [8192,4096] (transform_same Copy; calibrates HBM counters)", "copy fp32", 2 * 4 * ne,
                     lambda i: (lambda: ex.exec_transform_same(TransformSame.Copy, Xs[i], Ss[i % 3])),
                     lambda: cpu_entry(2 * 4 * xs_.size, GB, "GB/s", lambda: O.transform_same(15, xs_, zs_), lambda: np.copyto(zs_, xs_), samp, "numpy copyto"))
            hbm_line("pairwise_add fp32 [8192,4096]", "pairwise_add fp32", 3 * 4 * ne,
                     lambda i: (lambda: ex.exec_pairwise(Pairwise.Add, Xs[i], Ys[i % 3], Ss[i % 3])),
                     lambda: cpu_entry(3 * 4 * xs_.size, GB, "GB/s", lambda: O.pairwise(0, xs_, ys_, zs_), lambda: np.add(xs_, ys_, out=zs_), samp, "numpy add"))
            hbm_line("transform_tanh fp32 [8192,4096]", "transform_tanh fp32", 2 * 4 * ne,
                     lambda i: (lambda: ex.exec_transform_strict(TransformStrict.Tanh, Xs[i], Ss[i % 3])),
                     lambda: cpu_entry(2 * 4 * xs_.size, GB, "GB/s", lambda: O.transform_strict(29, xs_, zs_), lambda: np.tanh(xs_, out=zs_), samp, "numpy tanh"))
            r_ = np.zeros(rows_s, np.float32)
            i_ = np.zeros(rows_s, np.int64)
            hbm_line("reduce_sum dim1 fp32 [8192,4096]", "reduce_sum", 4 * ne + 4 * shp[0],
                     lambda i: (lambda: ex.exec_reduce_same(ReduceSame.Sum, Xs[i], [1], z=Rs[i])),
                     lambda: cpu_entry(4 * xs_.size, GB, "GB/s", lambda: O.reduce_same(0, xs_, r_, [1]), lambda: np.sum(xs_, axis=1, out=r_), samp, "numpy sum"))
            hbm_line("argmax dim1 fp32 [8192,4096]", "argmax dim1", 4 * ne + 8 * shp[0],
                     lambda i: (lambda: ex.exec_index_reduce(IndexReduce.IndexMax, Xs[i], [1], z=AMs[i])),
                     lambda: cpu_entry(4 * xs_.size, GB, "GB/s", lambda: O.index_reduce(0, xs_, i_, [1]), lambda: np.argmax(xs_, axis=1, out=i_), samp, "numpy argmax"))
            del Xs, Ys, Ss, Rs, AMs, xh, yh
        if 3 in cfgs:
            # config 3: row ops on [16, 1024, 768] and softmax on [16, 12, 1024, 1024]
            rng = np.random.default_rng(3003)
            for dt, dtn, es in [(FLOAT32, "fp32", 4), (BFLOAT16, "bf16", 2)]:
                xs = (16, 1024, 768)
                nx = 16 * 1024 * 768
                xr = rng.normal(0, 1, xs).astype(np.float32)
                gh, bh = rng.normal(1, 0.02, 768).astype(np.float32), rng.normal(0, 0.02, 768).astype(np.float32)
                K3 = n_sets(2 * es * nx)
                Xr = [NDArray.from_numpy(xr, dt) for _ in range(K3)]
                Zr = [NDArray.empty(xs, dt) for _ in range(K3)]
                G, Bv = NDArray.from_numpy(gh, dt), NDArray.from_numpy(bh, dt)
                for arr in Xr + [G, Bv]:
                    arr.sync_to_device()
                # CPU sample: the first 2 of 16 batch entries
                conv = (lambda v: O.Arr(f32_to_bf16_bits(v), O.BFLOAT16)) if dt == BFLOAT16 else (lambda v: O.Arr(np.ascontiguousarray(v, np.float32)))
                sx = xr[:2].reshape(-1, 768)

                def ln_cpu():
                    ox, og, ob, oz = conv(sx), conv(gh), conv(bh), conv(np.zeros_like(sx))
                    def fast():
                        m = sx.mean(-1, keepdims=True); v = sx.var(-1, keepdims=True)
                        return (sx - m) / np.sqrt(v + 1e-5) * gh + bh
                    return cpu_entry(2 * es * sx.size, GB, "GB/s", lambda: O.layer_norm(ox, og, ob, oz, [1], channels_first=False), fast,
                                     "first 2 of 16 batch entries", "numpy mean/var/normalise in fp32")

                def gelu_cpu():
                    ox, oz = conv(sx), conv(np.zeros_like(sx))
                    return cpu_entry(2 * es * sx.size, GB, "GB/s", lambda: O.transform_strict(53, ox, oz), lambda: sx / (1.0 + np.exp(-1.702 * sx)),
                                     "first 2 of 16 batch entries", "numpy x * sigmoid(1.702 x) in fp32")

                binds = [ex.bind_custom("layer_norm", [Xr[i], G, Bv], [Zr[i]], i_args=[2], b_args=[False]) for i in range(K3)]
                hbm_line("layer_norm %s [16,1024,768]" % dtn, "layer_norm %s" % dtn, 2 * es * nx + 2 * es * 768, lambda i: binds[i], ln_cpu)
                hbm_line("gelu %s [16,1024,768]" % dtn, "gelu %s" % dtn, 2 * es * nx,
                         lambda i: (lambda: ex.exec_transform_strict(TransformStrict.GELU, Xr[i], Zr[i])), gelu_cpu)
                del Xr, Zr, binds
                ls = (16, 12, 1024, 1024)
                nl = 16 * 12 * 1024 * 1024
                # logits are generated in the permuted storage layout [16, 1024, 12, 1024]; the dense case uses the same numbers.
                # One call moves 1.6 GB (0.8 GB in bf16), several times the last-level cache, so every call is cold by itself.
                raw = rng.normal(0, 2, (16, 1024, 12, 1024)).astype(np.float32)
                Lg = NDArray.from_numpy(raw, dt)
                srow = raw[0, :64].reshape(-1, 1024).copy()        # CPU sample: 768 rows
                del raw
                Lg.sync_to_device()
                Zs = NDArray.empty(ls, dt)

                def sm_cpu():
                    ox, oz = conv(srow), conv(np.zeros_like(srow))
                    def fast():
                        e = np.exp(srow - srow.max(-1, keepdims=True))
                        return e / e.sum(-1, keepdims=True)
                    return cpu_entry(2 * es * srow.size, GB, "GB/s", lambda: O.softmax(ox, oz, 1), fast, "768 of 196,608 rows", "numpy max/exp/sum/divide in fp32")

                dense = Lg.reshape(16, 12, 1024, 1024)
                w, e = timed(ex, L, ex.bind_custom("softmax", [dense], [Zs], i_args=[3]), steps, warmup)
                line = {"op": "softmax %s [16,12,1024,1024]" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(2 * es * nl, e, "softmax %s" % dtn)}
                if cpu:
                    line["cpu_baseline"] = sm_cpu()
                ops.append(with_copy_fraction(line, 2 * es * nl))
                view = Lg.permute(0, 2, 1, 3)
                w, e = timed(ex, L, ex.bind_custom("softmax", [view], [Zs], i_args=[3]), steps, warmup)
                line2 = {"op": "softmax %s permuted[0,2,1,3] view" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(2 * es * nl, e, "softmax %s" % dtn)}
                if cpu:
                    line2["cpu_baseline"] = dict(line["cpu_baseline"], sample=line["cpu_baseline"]["sample"] + " (dense rows; the view changes addresses only)")
                ops.append(with_copy_fraction(line2, 2 * es * nl))
                del Lg, Zs, dense, view
        if extras:
            # kernels for shapes no BASELINE config uses, measured the same way (cold over rotating sets, then warm)
            rng = np.random.default_rng(77)
            GBx = 1e9
            rc_shape = (6144, 4096)
            xc = rng.normal(0, 1, rc_shape).astype(np.float32)
            Kx = n_sets(4 * xc.size)
            Xc = [NDArray.from_numpy(xc) for _ in range(Kx)]
            for arr in Xc:
                arr.sync_to_device()
            Rc = [NDArray.empty((rc_shape[1],), FLOAT32) for _ in range(Kx)]
            Ic = [NDArray.empty((rc_shape[1],), INT64) for _ in range(Kx)]
            hbm_line("reduce_sum dim0 fp32 [6144,4096] (column sums: reduce_cols)", "reduce_cols", 4 * xc.size + 4 * rc_shape[1],
                     lambda i: (lambda: ex.exec_reduce_same(ReduceSame.Sum, Xc[i], [0], z=Rc[i])))
            hbm_line("argmax dim0 fp32 [6144,4096] (index_cols)", "index_cols", 4 * xc.size + 8 * rc_shape[1],
                     lambda i: (lambda: ex.exec_index_reduce(IndexReduce.IndexMax, Xc[i], [0], z=Ic[i])))
            Tc = [NDArray.empty((rc_shape[1], rc_shape[0]), FLOAT32) for _ in range(3)]
            Xt = [x_.permute(1, 0) for x_ in Xc]
            hbm_line("assign of a transposed view fp32 [6144,4096] -> [4096,6144] (transpose_tiled)", "transpose_tiled", 2 * 4 * xc.size,
                     lambda i: (lambda: ex.exec_assign(Xt[i], Tc[i % 3])))
            Bc = [NDArray.empty(rc_shape, BFLOAT16) for _ in range(3)]
            hbm_line("cast fp32 -> bf16 [6144,4096] (cast_contig)", "cast_contig", 6 * xc.size,
                     lambda i: (lambda: ex.exec_assign(Xc[i], Bc[i % 3])))
            del Xc, Xt, Rc, Ic, Tc, Bc, xc
            lv = rng.normal(0, 2, (500, 50257)).astype(np.float32)
            Kl = n_sets(2 * 4 * lv.size)
            Lv = [NDArray.from_numpy(lv) for _ in range(Kl)]
            for arr in Lv:
                arr.sync_to_device()
            Zl = [NDArray.empty(lv.shape, FLOAT32) for _ in range(3)]
            sm_binds = [ex.bind_custom("softmax", [Lv[i]], [Zl[i % 3]], i_args=[1]) for i in range(Kl)]
            hbm_line("softmax fp32 [500,50257] (vocabulary-length rows: softmax_block_regs)", "softmax_block_regs", 2 * 4 * lv.size, lambda i: sm_binds[i])
            del Lv, Zl, sm_binds, lv
            # a product against a row-major matrix whose rows do not start on 16-byte boundaries (the [768, 50257] embedding
            # without the transpose flag): element-aligned vector loads in the bounds-handling tile kernel
            ue = rng.normal(0, 768 ** -0.5, (768, 50257)).astype(np.float32)
            ua = rng.normal(0, 1, (4096, 768)).astype(np.float32)
            Ua, Ue, Uz = NDArray.from_numpy(ua, BFLOAT16), NDArray.from_numpy(ue, BFLOAT16), NDArray.empty((4096, 50257), BFLOAT16)
            Ua.sync_to_device(); Ue.sync_to_device()
            w, e = timed(ex, L, ex.bind_custom("matmul", [Ua, Ue], [Uz]), max(steps // 5, 3), max(warmup // 5, 1))
            ops.append({"op": "mmul bf16 [4096,768] x [768,50257] (row length not a multiple of 8: %s)" % L.nd4jhipLastGemmKernel().decode(),
                        "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": mfma_entry(2.0 * 4096 * 50257 * 768, e, "bf16", "mmul unaligned")})
            # the same product against the k-contiguous [50257, 768] matrix (a tied embedding, transposeB): rows aligned, N not a
            # whole number of tiles -- the edge instantiation of the two-stage direct-load kernel
            Uet = NDArray.from_numpy(np.ascontiguousarray(ue.T), BFLOAT16)
            Uet.sync_to_device()
            w, e = timed(ex, L, ex.bind_custom("matmul", [Ua, Uet], [Uz], i_args=[0, 1, 0]), max(steps // 5, 3), max(warmup // 5, 1))
            ops.append({"op": "mmul bf16 [4096,768] x [50257,768]^T (transposeB, N not a whole number of tiles: %s)" % L.nd4jhipLastGemmKernel().decode(),
                        "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": mfma_entry(2.0 * 4096 * 50257 * 768, e, "bf16", "mmul ragged tb")})
            del Ua, Ue, Uet, Uz, ua, ue
            # ragged products of a few hundred to a few thousand rows and columns (a 500-token prompt's projections): the
            # direct-load kernels' edge instantiations
            for dt, nm, (rm, rn, rk) in ((BFLOAT16, "bf16", (500, 2304, 768)), (BFLOAT16, "bf16", (2000, 2000, 2048)), (FLOAT32, "f32", (2000, 2000, 2048))):
                ra = rng.normal(0, 1, (rm, rk)).astype(np.float32)
                rb = rng.normal(0, rk ** -0.5, (rk, rn)).astype(np.float32)
                Ra = NDArray.from_numpy(ra, dt) if dt != FLOAT32 else NDArray.from_numpy(ra)
                Rb = NDArray.from_numpy(rb, dt) if dt != FLOAT32 else NDArray.from_numpy(rb)
                Rz = NDArray.empty((rm, rn), dt)
                Ra.sync_to_device(); Rb.sync_to_device()
                w, e = timed(ex, L, ex.bind_custom("matmul", [Ra, Rb], [Rz]), steps, warmup)
                ops.append({"op": "mmul %s %d x %d x %d (ragged: %s)" % (nm, rm, rn, rk, L.nd4jhipLastGemmKernel().decode()),
                            "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": mfma_entry(2.0 * rm * rn * rk, e, nm, "mmul ragged %s %d" % (nm, rm))})
                del Ra, Rb, Rz, ra, rb
        if 2 in cfgs:
            # config 2, the remaining sizes/dtypes
            plain_cpu = {}     # (dtype, size) -> cpu_baseline of the plain-B product: the CPU loops do not depend on the layout flag
            for dt, dtn, peak in [(FLOAT32, "f32", "f32"), (HALF, "f16", "f16"), (BFLOAT16, "bf16", "bf16")]:
                for m in (1024, 4096):
                    for transb in (False, True):
                        if dt == BFLOAT16 and m == 4096 and not transb:
                            continue   # the headline
                        rng = np.random.default_rng(2002)
                        a = rng.normal(0, 1 / math.sqrt(m), (m, m)).astype(np.float32)
                        b = rng.normal(0, 1 / math.sqrt(m), (m, m)).astype(np.float32)
                        if dt == HALF:
                            a, b = a.astype(np.float16), b.astype(np.float16)
                        Am, Bm = NDArray.from_numpy(a, dt), NDArray.from_numpy(b, dt)
                        Zm = NDArray.empty((m, m), dt)
                        Am.sync_to_device(); Bm.sync_to_device()
                        ia = [0, 1] if transb else []
                        w, e = timed(ex, L, ex.bind_custom("matmul", [Am, Bm], [Zm], i_args=ia), steps, warmup)
                        line = {"op": "mmul %s %d^3%s" % (dtn, m, " transposeB" if transb else ""), "ms": round(e, 4), "wall_ms": round(w, 4),
                                "roofline": mfma_entry(2.0 * m * m * m, e, peak, "mmul %s %d^3%s" % (dtn, m, " transposeB" if transb else ""))}
                        if cpu and not transb:
                            # faithful: the reference's own loop for this type (fp32 goes to BLAS there, so the port of its plain loop is
                            # the lower bound and OpenBLAS sgemm through numpy the figure to compare with); 16-bit: usualGemm in the type
                            rows = 64 if dt == FLOAT32 else 32
                            a32, b32 = np.asarray(a, np.float32), np.asarray(b, np.float32)
                            if dt == BFLOAT16:
                                oa, ob, oz = O.Arr(f32_to_bf16_bits(a32[:rows]), O.BFLOAT16), O.Arr(f32_to_bf16_bits(b32), O.BFLOAT16), O.Arr(np.zeros((rows, m), np.uint16), O.BFLOAT16)
                            else:
                                oa, ob, oz = O.Arr(np.ascontiguousarray(a[:rows])), O.Arr(np.ascontiguousarray(b)), O.Arr(np.zeros((rows, m), a.dtype))
                            line["cpu_baseline"] = cpu_entry(2.0 * rows * m * m, 1e12, "TFLOP/s", lambda: O.matmul(oa, ob, oz, accumulate=0 if dt != FLOAT32 else 1),
                                                             lambda: a32 @ b32, "first %d of %d rows of A against the full B (plain loop in the array type)" % (rows, m),
                                                             "numpy fp32 sgemm (bundled OpenBLAS, all cores) on the whole %d^3 product%s" % (m, "" if dt == FLOAT32 else ", inputs widened to fp32"),
                                                             fast_cores=os.cpu_count())
                            # the fast figure is for the whole product, not the sample
                            tq = best_time(lambda: a32 @ b32)
                            line["cpu_baseline"]["fast"]["value"] = round(2.0 * m * m * m / tq / 1e12, 4)
                        elif cpu:
                            src = plain_cpu.get((dtn, m)) or result.get("cpu_baseline")   # bf16 4096: the headline's own measurement
                            line["cpu_baseline"] = dict(src, sample=src["sample"] + " (the plain-B measurement; the CPU loops do not depend on the layout flag)")
                        if cpu and not transb:
                            plain_cpu[(dtn, m)] = line["cpu_baseline"]
                        ops.append(line)
                        del Am, Bm, Zm
        if 4 in cfgs:
            # config 4: attention prefill, causal
            for dt, dtn in [(HALF, "f16"), (BFLOAT16, "bf16")] + ([(FLOAT32, "f32")] if extras else []):
                rng = np.random.default_rng(4004)
                qs = (96, 1024, 64)
                mk = lambda: rng.normal(0, 1, qs).astype(np.float32)
                q, k, v = mk(), mk(), mk()
                if dt == HALF:
                    q, k, v = q.astype(np.float16), k.astype(np.float16), v.astype(np.float16)
                Q, K_, V = NDArray.from_numpy(q, dt), NDArray.from_numpy(k, dt), NDArray.from_numpy(v, dt)
                O_ = NDArray.empty(qs, dt)
                for arr in (Q, K_, V):
                    arr.sync_to_device()
                w, e = timed(ex, L, ex.bind_custom("dot_product_attention_v2", [Q, V, K_], [O_], t_args=[0.125, 0.0], b_args=[True, False]),
                             max(steps // 5, 3), max(warmup // 5, 1))
                dense_flops = 4.0 * 96 * 1024 * 1024 * 64
                # what the kernel executes: a block owns 128 queries and walks the 64-key tiles up to its last query's diagonal
                executed_flops = 96 * sum(4.0 * 64 * 128 * min(1024, 64 * math.ceil(128 * (blk + 1) / 64)) for blk in range(8))
                useful_flops = 4.0 * 96 * 64 * (1024 * 1025 / 2)       # the scores on and below the diagonal
                rf = mfma_entry(dense_flops, e, dtn, "dot_product_attention_v2 f32" if dt == FLOAT32 else "dot_product_attention_v2")
                rf["achieved_executed"] = round(executed_flops / (e * 1e-3) / 1e12, 2)
                rf["frac_executed"] = round(rf["achieved_executed"] / MFMA_PEAK[dtn], 4)
                rf["achieved_causal_useful"] = round(useful_flops / (e * 1e-3) / 1e12, 2)
                if dt == FLOAT32:
                    # the dense count divided by the time exceeds the fp32 matrix peak (the kernel skips the tiles above the diagonal):
                    # the fraction of this line is the executed one, the dense figure is kept beside it
                    rf["achieved_dense"], rf["achieved"], rf["frac"] = rf["achieved"], rf["achieved_executed"], rf["frac_executed"]
                line = {"op": "dot_product_attention_v2 %s causal [96,1024,64] (output only)" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4),
                        "roofline": rf,
                        "note": ("achieved / frac count the executed flops here, achieved_dense the dense 4*B*T*T*D flops (25.77 GFLOP); " if dt == FLOAT32 else
                                 "achieved / frac count the dense 4*B*T*T*D flops (25.77 GFLOP); ") + "achieved_executed the flops of the key tiles the kernel "
                                "multiplies (%.2f GFLOP: tiles wholly above the diagonal are skipped), achieved_causal_useful the scores on and below "
                                "the diagonal (%.2f GFLOP)" % (executed_flops / 1e9, useful_flops / 1e9)}
                if cpu:
                    nb = 2
                    cv = (lambda t: O.Arr(f32_to_bf16_bits(np.asarray(t, np.float32)), O.BFLOAT16)) if dt == BFLOAT16 else (lambda t: O.Arr(np.ascontiguousarray(t)))
                    oq, ok_, ov = cv(q[:nb]), cv(k[:nb]), cv(v[:nb])
                    oo = cv(np.zeros((nb, 1024, 64), np.float16 if dt == HALF else np.float32))
                    q32, k32, v32 = (np.asarray(t[:nb], np.float32) for t in (q, k, v))

                    def fast():
                        lg = np.einsum("bid,bjd->bij", q32, k32) * 0.125
                        lg = np.where(np.tril(np.ones((1024, 1024), bool)), lg, -1e9)
                        ee = np.exp(lg - lg.max(-1, keepdims=True))
                        return (ee / ee.sum(-1, keepdims=True)) @ v32
                    line["cpu_baseline"] = cpu_entry(4.0 * nb * 1024 * 1024 * 64, 1e12, "TFLOP/s", lambda: O.attention_v2(oq, ov, ok_, oo, scale=0.125, causal=True), fast,
                                                     "first %d of 96 batch entries (dense flop count)" % nb, "numpy einsum / exp / matmul in fp32", fast_cores=os.cpu_count())
                ops.append(line)
                del Q, K_, V, O_
        result["ops"] = ops
    if not args.skip_decode:
        print("[bench] decode leg", file=sys.stderr, flush=True)
        ops = result.setdefault("ops", [])
        # config 5: GPT-2-small-shaped greedy decode, bf16, prefill 512 then 128 steps with a key/value cache
        from deeplearning4j_amd.decoder import Decoder, DecoderConfig, init_weights
        cfg = DecoderConfig.gpt2_small()
        weights = init_weights(cfg, 5005)
        n_param_bytes = 2 * (cfg.n_layer * (cfg.d_model * 3 * cfg.d_model + cfg.d_model * cfg.d_model + 2 * cfg.d_model * cfg.d_ff) + cfg.vocab * cfg.d_model)
        prefill, n_new = 512, 128
        for batch in [int(b) for b in args.decode_batches.split(",") if b.strip()]:
            print("[bench] decode batch %d" % batch, file=sys.stderr, flush=True)
            ids = np.random.default_rng(5005).integers(0, cfg.vocab, (batch, prefill))
            dec = Decoder(cfg, weights, BFLOAT16, batch=batch, executioner=ex)
            dec.generate(ids[:, :prefill], 4)      # builds and warms the prefill program and the first decode programs
            for _ in range(1 if args.replay_kernels else 2):   # second pass replays fully built programs
                dec.reset()
                L.streamSynchronize(None)
                t0 = time.perf_counter()
                dec.forward(ids)
                L.streamSynchronize(None)
                t1 = time.perf_counter()
                for _ in range(n_new - 1):
                    dec.forward(None)
                L.streamSynchronize(None)
                t2 = time.perf_counter()
            eager_ms = (t2 - t1) * 1e3 / (n_new - 1)
            prefill_s = t1 - t0
            # the same steps replayed as captured HIP graphs (one per cache length): the first pass records them, the timed
            # passes replay; every kernel of the step still runs, only the per-op launch path on the host is gone
            # Two ways to replay a recorded step (nd4jhipSetGraphReplayMode): the instantiated graph, and the merged sequence
            # launched kernel by kernel from inside the library.  Both are timed, alternating; the line reports the faster.
            dec.use_graphs = not args.no_graphs
            replay_ms = {}
            for rep in range(3 if dec.use_graphs else 0):
                for mode, name in ((0, "graph"), (1, "kernels")):
                    if args.replay_kernels and mode == 0:
                        continue
                    L.nd4jhipSetGraphReplayMode(mode)
                    dec.reset()
                    dec.forward(ids)
                    L.streamSynchronize(None)
                    t1 = time.perf_counter()
                    for _ in range(n_new - 1):
                        dec.forward(None)
                    L.streamSynchronize(None)
                    t2 = time.perf_counter()
                    if rep > 0 or args.replay_kernels:   # the first pass records
                        replay_ms[name] = min(replay_ms.get(name, 1e9), (t2 - t1) * 1e3 / (n_new - 1))
            L.nd4jhipSetGraphReplayMode(0)
            best = min(replay_ms, key=replay_ms.get) if replay_ms else None
            step_ms = replay_ms[best] if best else eager_ms   # the op-by-op figure when graphs are off
            dec.close()
            kv_bytes = cfg.n_layer * 2 * (prefill + n_new / 2) * cfg.d_model * 2 * batch
            how = {"graph": "recorded steps replayed as HIP graphs", "kernels": "recorded, merged steps launched kernel by kernel by the library",
                   None: "op by op"}[best]
            ops.append({"op": "gpt2-small decode bf16 batch %d (prefill %d, %d greedy steps, KV cache, %s)" % (batch, prefill, n_new, how),
                        "ms": round(step_ms, 4), "wall_ms": round(step_ms, 4), "tokens_per_s": round(batch * 1e3 / step_ms, 1),
                        "replay_ms": {k: round(v, 4) for k, v in replay_ms.items()},
                        "op_by_op_ms": round(eager_ms, 4), "op_by_op_tokens_per_s": round(batch * 1e3 / eager_ms, 1),
                        "prefill_ms": round(prefill_s * 1e3, 3), "prefill_tokens_per_s": round(batch * prefill / prefill_s, 1),
                        "roofline": hbm_entry(n_param_bytes + kv_bytes, step_ms)})
            del dec
        if not args.skip_cpu:
            # CPU side of config 5 (part of the cpu-baseline leg): the oracle's composition of the same ops, fp32, on a bounded
            # sample per batch size (a short prompt, a few greedy steps); at batch 1 its ids are also compared with the HIP fp32 run
            from oracle import oracle as O
            from oracle.decoder_oracle import OracleDecoder
            decode_lines = {int(l["op"].split("batch ")[1].split(" ")[0]): l for l in ops if l["op"].startswith("gpt2-small decode")}
            for batch, n_steps, n_prompt in ((1, 7, 32), (32, 3, 8)):
                if batch not in decode_lines:
                    continue
                ids = np.random.default_rng(5005).integers(0, cfg.vocab, (batch, n_prompt))
                cpu = OracleDecoder(cfg, weights, O.FLOAT32, batch=batch)
                nxt = cpu.forward(ids)
                cpu_ids = [nxt]
                t0 = time.perf_counter()
                for _ in range(n_steps):
                    nxt = cpu.forward(nxt.reshape(batch, 1))
                    cpu_ids.append(nxt)
                cpu_step = (time.perf_counter() - t0) / n_steps
                line = decode_lines[batch]
                line["cpu_baseline"] = {"value": round(batch / cpu_step, 2), "unit": "tokens/s", "cores": O.get_threads(), "kind": "port",
                                        "sample": "oracle decoder (the same op composition on the CPU restatement), fp32, batch %d, %d greedy steps after a %d-token prompt, %.1f s"
                                                  % (batch, n_steps, n_prompt, cpu_step * n_steps)}
                if batch == 1:
                    dec = Decoder(cfg, weights, FLOAT32, batch=1, executioner=ex)
                    gpu_ids = dec.generate(ids, n_steps + 1)
                    line["fp32_ids_match_cpu"] = bool((gpu_ids == np.stack(cpu_ids, 1)).all())
                    del dec
                del cpu
        result["ops"] = ops
    print(json.dumps(result))
    sys.stdout.flush()
    # One compact row per line of the record, last on stderr, so that a reader who only keeps the tail of the output still
    # has every figure: time per call, fraction of the roofline cold (and warm / of the same-size copy where measured), CPU
    # port and CPU fast in the roofline's unit (tokens/s for the decode).
    def row(name, ms, rf, cb):
        f = lambda v: "-" if v is None else ("%.3f" % v)
        port = cb.get("value") if cb else None
        fast = cb.get("fast", {}).get("value") if cb else None
        g = lambda v: "-" if v is None else ("%.4g" % v)
        return "%-34.34s|%8.4f|%5s|%5s|%5s|%8s|%8s" % (name, ms, f(rf.get("frac")), f(rf.get("frac_warm")), f(rf.get("frac_of_copy")), g(port), g(fast))
    print("%-34s|%8s|%5s|%5s|%5s|%8s|%8s" % ("op", "ms", "frac", "warm", "/copy", "cpu port", "cpu fast"), file=sys.stderr)
    print(row("mmul bf16 4096^3 (headline)", result["ms_per_step"], result["roofline"], result.get("cpu_baseline")), file=sys.stderr)
    for l in result.get("ops", []):
        short = l["op"].replace("dot_product_attention_v2", "attention").replace(" (transform_same Copy; calibrates HBM counters)", "").replace("[8192,4096]", "").replace("[16,1024,768]", "")
        short = short.replace("gpt2-small decode bf16", "decode").replace("[16,12,1024,1024]", "").replace("  ", " ")
        print(row(short, l["ms"], l["roofline"], l.get("cpu_baseline")), file=sys.stderr)
    sys.stderr.flush()


if __name__ == "__main__":
    main()
