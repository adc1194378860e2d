#!/usr/bin/env python3
"""Benchmark of the op path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Prints ONE JSON line.  The headline workload is BASELINE.json's config 2 at its largest size: mmul bf16,
M = N = K = 4096, entries ~ N(0, 1/sqrt(K)) from seed 2002, output bf16, fp32 accumulation; one "step" is one
execCustomOp2(matmul) call through the C ABI with the operands already resident in HBM.
`value` = 2*M*N*K*steps / wall time of the timed region.  The `roofline` object prices the dominant kernel
against the dense bf16 MFMA peak; `cpu_baseline` times the CPU oracle (a restatement of the reference's
nd4j-native path) on a bounded sample of the same product on the host cores.  The `ops` list carries the other
BASELINE configs (legacy chain, row ops, attention) measured the same way, each with its own roofline entry.
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
    "mmul bf16 4096": 235.2, "mmul f16 4096": 235.2, "mmul f32 4096^3": 859.1, "mmul f32 4096^3 transposeB": 866.0,
    "mmul f32 1024": 29.5, "mmul f16 1024": 14.8, "mmul bf16 1024": 14.8,
    "copy fp32": 268.4, "pairwise_add fp32": 402.6, "transform_tanh fp32": 268.4, "reduce_sum": 134.5, "argmax dim1": 134.5,
    "layer_norm fp32": 100.8, "gelu fp32": 100.7, "softmax fp32": 1610.6, "layer_norm bf16": 50.4, "gelu bf16": 50.4,
    "softmax bf16": 805.3, "dot_product_attention_v2": 53.5,
}


def traffic_of(label):
    best = None
    for k, v in TRAFFIC_MB.items():
        if label.startswith(k) and (best is None or len(k) > len(best[0])):
            best = (k, v)
    return None if best is None else int(best[1] * 1e6)


def timed(ex, L, fn, steps, warmup):
    """Run fn() warmup + steps times; returns (wall ms per step, event ms per step on the execution stream)."""
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


def hbm_entry(bytes_per_launch, ev_ms, label=""):
    ach = bytes_per_launch / (ev_ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
            "traffic": traffic_of(label)}


def mfma_entry(flops, ev_ms, dtype, label=""):
    ach = flops / (ev_ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(ach, 2), "peak": MFMA_PEAK[dtype], "unit": "TFLOP/s", "frac": round(ach / MFMA_PEAK[dtype], 4),
            "traffic": traffic_of(label)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--skip-ops", action="store_true", help="leave out the per-op lines of BASELINE configs 1-4")
    ap.add_argument("--skip-cpu", action="store_true", help="leave out the cpu_baseline leg")
    ap.add_argument("--skip-decode", action="store_true", help="leave out the GPT-2-shaped decode (tens of thousands of launches)")
    ap.add_argument("--no-graphs", action="store_true",
                    help="time the decode op by op only (for runs under rocprofv3: its kernel tracing aborts the queue on graph replays)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend is built and measured on one GPU; --gpus %d is not supported (no collectives are part of the op path)" % args.gpus)

    from deeplearning4j_amd.executioner import Executioner, IndexReduce, Pairwise, ReduceSame, TransformSame, TransformStrict
    from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32, HALF, NDArray, f32_to_bf16_bits

    ex = Executioner()
    L = ex.L
    L.nd4jhipSetSyncAfterCustomOp(0)     # the timed loop synchronises once at its end
    steps, warmup = args.steps, args.warmup

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
    wall_ms, ev_ms = timed(ex, L, ex.bind_custom("matmul", [A, B], [Z]), steps, warmup)
    value = flops / (wall_ms * 1e-3) / 1e12
    result = {
        "metric": "mmul TFLOP/s (bf16, M=N=K=4096, fp32 accumulate)", "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "mmul bf16 A[4096,4096] x B[4096,4096] (BASELINE config 2), N(0,1/sqrt(K)) seed 2002, via execCustomOp2(matmul)"},
        "roofline": mfma_entry(flops, ev_ms, "bf16", "mmul bf16 4096"),
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
    if not args.skip_ops:
        print("[bench] per-op leg", file=sys.stderr, flush=True)
        del A, B, Z
        # config 1: legacy chain, fp32 [8192, 4096]
        rng = np.random.default_rng(1001)
        shp = (8192, 4096)
        ne = shp[0] * shp[1]
        X = NDArray.from_numpy(rng.uniform(-1, 1, shp).astype(np.float32))
        Y = NDArray.from_numpy(rng.uniform(-1, 1, shp).astype(np.float32))
        S, T = NDArray.empty(shp, FLOAT32), NDArray.empty(shp, FLOAT32)
        R = NDArray.empty((shp[0],), FLOAT32)
        from deeplearning4j_amd.ndarray import INT64
        AM = NDArray.empty((shp[0],), INT64)
        X.sync_to_device(); Y.sync_to_device()
        ex.exec_pairwise(Pairwise.Add, X, Y, S)
        ex.exec_transform_strict(TransformStrict.Tanh, S, T)
        for name, fn, nbytes in [
            ("copy fp32 [8192,4096] (transform_same Copy; calibrates HBM counters)", lambda: ex.exec_transform_same(TransformSame.Copy, X, S), 2 * 4 * ne),
            ("pairwise_add fp32 [8192,4096]", lambda: ex.exec_pairwise(Pairwise.Add, X, Y, S), 3 * 4 * ne),
            ("transform_tanh fp32 [8192,4096]", lambda: ex.exec_transform_strict(TransformStrict.Tanh, S, T), 2 * 4 * ne),
            ("reduce_sum dim1 fp32 [8192,4096]", lambda: ex.exec_reduce_same(ReduceSame.Sum, T, [1], z=R), 4 * ne + 4 * shp[0]),
            ("argmax dim1 fp32 [8192,4096]", lambda: ex.exec_index_reduce(IndexReduce.IndexMax, T, [1], z=AM), 4 * ne + 8 * shp[0]),
        ]:
            w, e = timed(ex, L, fn, steps, warmup)
            ops.append({"op": name, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(nbytes, e, name)})
        del X, Y, S, T, R, AM
        # config 3: row ops on [16, 1024, 768] and softmax on [16, 12, 1024, 1024]
        rng = np.random.default_rng(3003)
        for dt, dtn, es in [(FLOAT32, "fp32", 4), (BFLOAT16, "bf16", 2)]:
            xs = (16, 1024, 768)
            nx = 16 * 1024 * 768
            Xr = NDArray.from_numpy(rng.normal(0, 1, xs).astype(np.float32), dt)
            G = NDArray.from_numpy(rng.normal(1, 0.02, 768).astype(np.float32), dt)
            Bv = NDArray.from_numpy(rng.normal(0, 0.02, 768).astype(np.float32), dt)
            Zr, Zg = NDArray.empty(xs, dt), NDArray.empty(xs, dt)
            for arr in (Xr, G, Bv):
                arr.sync_to_device()
            w, e = timed(ex, L, ex.bind_custom("layer_norm", [Xr, G, Bv], [Zr], i_args=[2], b_args=[False]), steps, warmup)
            ops.append({"op": "layer_norm %s [16,1024,768]" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(2 * es * nx + 2 * es * 768, e, "layer_norm %s" % dtn)})
            w, e = timed(ex, L, lambda: ex.exec_transform_strict(TransformStrict.GELU, Zr, Zg), steps, warmup)
            ops.append({"op": "gelu %s [16,1024,768]" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(2 * es * nx, e, "gelu %s" % dtn)})
            del Xr, Zr, Zg
            ls = (16, 12, 1024, 1024)
            nl = 16 * 12 * 1024 * 1024
            # logits are generated in the permuted storage layout [16, 1024, 12, 1024]; the dense case uses the same numbers
            raw = rng.normal(0, 2, (16, 1024, 12, 1024)).astype(np.float32)
            Lg = NDArray.from_numpy(raw, dt)
            del raw
            Lg.sync_to_device()
            Zs = NDArray.empty(ls, dt)
            dense = Lg.reshape(16, 12, 1024, 1024)
            w, e = timed(ex, L, ex.bind_custom("softmax", [dense], [Zs], i_args=[3]), steps, warmup)
            ops.append({"op": "softmax %s [16,12,1024,1024]" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(2 * es * nl, e, "softmax %s" % dtn)})
            view = Lg.permute(0, 2, 1, 3)
            w, e = timed(ex, L, ex.bind_custom("softmax", [view], [Zs], i_args=[3]), steps, warmup)
            ops.append({"op": "softmax %s permuted[0,2,1,3] view" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4), "roofline": hbm_entry(2 * es * nl, e, "softmax %s" % dtn)})
            del Lg, Zs, dense, view
        # config 2, the remaining sizes/dtypes
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
                    ops.append({"op": "mmul %s %d^3%s" % (dtn, m, " transposeB" if transb else ""), "ms": round(e, 4), "wall_ms": round(w, 4),
                                "roofline": mfma_entry(2.0 * m * m * m, e, peak, "mmul %s %d^3%s" % (dtn, m, " transposeB" if transb else ""))})
                    del Am, Bm, Zm
        # config 4: attention prefill, causal
        for dt, dtn in [(HALF, "f16"), (BFLOAT16, "bf16")]:
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
            ops.append({"op": "dot_product_attention_v2 %s causal [96,1024,64] (output only)" % dtn, "ms": round(e, 4), "wall_ms": round(w, 4),
                        "roofline": mfma_entry(4.0 * 96 * 1024 * 1024 * 64, e, dtn, "dot_product_attention_v2"),
                        "note": "achieved counts the dense 4*B*T*T*D flops; the causal mask makes about half of them useful"})
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
        for batch in (1, 32):
            print("[bench] decode batch %d" % batch, file=sys.stderr, flush=True)
            ids = np.random.default_rng(5005).integers(0, cfg.vocab, (batch, prefill))
            dec = Decoder(cfg, weights, BFLOAT16, batch=batch, executioner=ex)
            dec.generate(ids[:, :prefill], 4)      # builds and warms the prefill program and the first decode programs
            for _ in range(2):                     # second pass replays fully built programs
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
            dec.use_graphs = not args.no_graphs
            for _ in range(3 if dec.use_graphs else 0):
                dec.reset()
                dec.forward(ids)
                L.streamSynchronize(None)
                t1 = time.perf_counter()
                for _ in range(n_new - 1):
                    dec.forward(None)
                L.streamSynchronize(None)
                t2 = time.perf_counter()
            step_ms = (t2 - t1) * 1e3 / (n_new - 1)   # the op-by-op figure when graphs are off
            dec.close()
            kv_bytes = cfg.n_layer * 2 * (prefill + n_new / 2) * cfg.d_model * 2 * batch
            how = "steps replayed as HIP graphs" if dec.use_graphs else "op by op"
            ops.append({"op": "gpt2-small decode bf16 batch %d (prefill %d, %d greedy steps, KV cache, %s)" % (batch, prefill, n_new, how),
                        "ms": round(step_ms, 4), "wall_ms": round(step_ms, 4), "tokens_per_s": round(batch * 1e3 / step_ms, 1),
                        "op_by_op_ms": round(eager_ms, 4), "op_by_op_tokens_per_s": round(batch * 1e3 / eager_ms, 1),
                        "prefill_ms": round(prefill_s * 1e3, 3), "prefill_tokens_per_s": round(batch * prefill / prefill_s, 1),
                        "roofline": hbm_entry(n_param_bytes + kv_bytes, step_ms)})
            del dec
        if not args.skip_cpu:
            # CPU side of config 5 (part of the cpu-baseline leg): the oracle's composition of the same ops, fp32, batch 1,
            # on a bounded sample (prompt of 32 tokens, 8 greedy steps); its ids are also compared with the HIP fp32 run
            from oracle import oracle as O
            from oracle.decoder_oracle import OracleDecoder
            ids = np.random.default_rng(5005).integers(0, cfg.vocab, (1, 32))
            cpu = OracleDecoder(cfg, weights, O.FLOAT32, batch=1)
            nxt = cpu.forward(ids)
            cpu_ids = [nxt]
            t0 = time.perf_counter()
            for _ in range(7):
                nxt = cpu.forward(nxt.reshape(1, 1))
                cpu_ids.append(nxt)
            cpu_step = (time.perf_counter() - t0) / 7
            dec = Decoder(cfg, weights, FLOAT32, batch=1, executioner=ex)
            gpu_ids = dec.generate(ids, 8)
            ops[-2]["cpu_tokens_per_s"] = round(1.0 / cpu_step, 2)
            ops[-2]["cpu_sample"] = "oracle decoder fp32, batch 1, 7 decode steps after a 32-token prompt, %d threads" % O.get_threads()
            ops[-2]["fp32_ids_match_cpu"] = bool((gpu_ids == np.stack(cpu_ids, 1)).all())
            del dec, cpu
        result["ops"] = ops
    print(json.dumps(result))


if __name__ == "__main__":
    main()
