#!/usr/bin/env python3
"""Benchmark of the SpTMM hot path on one MI355X: the headline GEMV and every other configured shape.

Headline (the `value` of the JSON line): SpTMM split-K=32 GEMV at M=1, K=6912, N=2560, S=4096.  A step is one
launch of the C ABI's sptmm_gemv_i8_batched: 32 independent GEMVs of that shape, each on its own device copy
of the u16-list stream.  The copies together (671 MB) exceed the 256 MB last-level cache, so every GEMV
streams its 21 MB of row indices from HBM ("cold"), as a decoder walking through gigabytes of layer weights
does, and the dispatch latency is paid once per step instead of once per GEMV.  The same GEMV launched one
per launch (what the reference's loop does, main.cu:994-1459) is reported beside it at the top level.

Legs (all on by default): the other two encodings at the headline shape; config 1 (M=4); config 2 (gap
stream, fp16 rows); config 3 (the decoder layer's four shapes at M=1 and M=4, per shape and summed); config 4
(K=13824 N=5120 at M=1, 8, 16, lists against i2s).  Every timed object is first checked bit-exact against the
other encodings of the same matrix, and the CPU leg checks one GPU result per configuration against the oracle.

Prints ONE JSON line on stdout: the headline with its roofline and CPU baseline and one figure per configuration
(final_line(), a few KB).  The per-row tables of every leg go to a side file (--detail, default
gpurun_out/bench_detail.json) and, one JSON object per leg, to stderr.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "µs/GEMV and achieved HBM GB/s (% roofline) at M=1 K=6912 N=2560 S=4096"
K, N, S, M, SPLIT = 6912, 2560, 4096, 1, 32
BATCH = 32  # GEMVs per launch = device copies of the stream: 32 x 21 MB = 671 MB > 256 MB Infinity Cache
PEAK_GBPS = 8000.0
TRAFFIC_SIDECAR = os.path.join(ROOT, "profiles", "traffic_lists_kernel_batched_i8_u16_cfg0.json")

# config 3: BitNet-b1.58-2B decoder layer (name, K, N, S, how many of them a layer holds)
LAYER = [("q/o", 2560, 2560, 1536, 2), ("k/v", 2560, 640, 1536, 2), ("gate/up", 2560, 6912, 1536, 2),
         ("down", 6912, 2560, 4160, 1)]
LARGE = ("large", 13824, 5120, 8320)  # config 4
# nonzeros per column of the headline shape for the density leg: 3.7 % (the reference's default flags, -K 3072 -S 256,
# are 8.3 %), 7.4, 12.5 (u16 lists as many bytes as i2s), 18.5, 25 % (8-bit gaps as many bytes as i2s)
DENSITY_S = (256, 512, 864, 1280, 1728)


def algorithmic_bytes(stream_bytes, m, k, n, act_bytes=1):
    # weight stream (indices counted once, whatever M) + activations + output
    return stream_bytes + m * k * act_bytes + 4 * m * n


def pct(nbytes, us):
    return round(100.0 * nbytes / us / 1e3 / PEAK_GBPS, 2)


def cpu_baseline(sp_lists, gpu_headline, checks, dense_w=None, budget_s=12.0):
    """The oracle's gather-sum (a port of main.cu:577-593) on the host cores, bounded sample; and the
    oracle as checker of what the GPU legs computed."""
    import numpy as np

    import oracle

    pos, neg = sp_lists
    have = len(os.sched_getaffinity(0))
    cores = min(have, 16)
    X = oracle.make_x_i8(0xC0FFEE ^ M, M, K)
    out = np.empty((M, N), np.int32)
    want = oracle.sptmm_i8(X, pos, neg)
    headline_ok = bool((gpu_headline == want).all())
    res = {}
    for threads in (1, cores):
        oracle.sptmm_i8_mt(X, pos, neg, threads, out)  # warm-up
        assert (out == want).all()
        reps, t0 = 0, time.perf_counter()
        while True:
            oracle.sptmm_i8_mt(X, pos, neg, threads, out)
            reps += 1
            el = time.perf_counter() - t0
            if el > budget_s / 2 or reps >= 4000:
                break
        res[threads] = (el / reps * 1e6, reps)
    us, reps = res[cores]
    # for context: the dense int8 product of the same matrix (single thread), and that it gives the same numbers
    dense_us = None
    if dense_w is not None:
        t = []
        for _ in range(3):
            t0 = time.perf_counter()
            dense = oracle.dense_i8(X, dense_w)
            t.append(time.perf_counter() - t0)
        assert (dense == want).all()
        dense_us = round(sorted(t)[1] * 1e6, 1)
    bad = []
    for label, Xc, p, n, got, s_nz in checks:
        if Xc.dtype == np.int8:
            ok = bool((got == oracle.sptmm_i8_mt(Xc, p, n, cores)).all())
        else:  # fp16 rows, fp32 sums: within 1e-3 of the float64 gather-sum, relative to max(|ref|, sqrt(S))
            ref = oracle.sptmm_f64(Xc, p, n)
            ok = bool((np.abs(got - ref) / np.maximum(np.abs(ref), math.sqrt(s_nz))).max() <= 1e-3)
        if not ok:
            bad.append(label)
    return {
        "value": round(us, 2), "unit": "us/GEMV", "cores": cores, "cores_available": have, "kind": "port",
        "sample": "%d full GEMVs of the same W and X (oracle gather-sum over u16 lists, %d pthreads of the %d cores "
                  "this process may use); single thread: %.1f us/GEMV over %d GEMVs" % (reps, cores, have, res[1][0], res[1][1]),
        "value_1core": round(res[1][0], 2), "dense_int8_1core_us": dense_us,
        "gbps": round(algorithmic_bytes(2 * S * N, M, K, N) / us / 1e3, 2),
        "gpu_headline_equals_oracle": headline_ok,
        "gpu_results_checked_against_oracle": len(checks) + 1,
        "gpu_results_that_differ": bad + ([] if headline_ok else ["headline"]),
    }


# config 3 as a sequence.  (name, K, N, S, stage): the steps of a stage read the same input and do not depend on each other.
LAYER_SEVEN = [("q", 2560, 2560, 1536, 0), ("k", 2560, 640, 1536, 0), ("v", 2560, 640, 1536, 0), ("o", 2560, 2560, 1536, 1),
               ("gate", 2560, 6912, 1536, 2), ("up", 2560, 6912, 1536, 2), ("down", 6912, 2560, 4160, 3)]
# the fused shapes the reference instantiates (main.cu:1107-1120: N=13824; main.cu:1916-1917: N=3840)
LAYER_FOUR = [("qkv", 2560, 3840, 1536, 0), ("o", 2560, 2560, 1536, 1), ("gate_up", 2560, 13824, 1536, 2), ("down", 6912, 2560, 4160, 3)]


def layer_sequence(sp, st, checks, reps):
    """The decoder layer of config 3 timed as what it is, a sequence of launches on one stream (the loop of main.cu:767-782
    around a whole layer instead of one kernel): 7 launches; 5 (k, v and gate, up as batched pairs); 4 with the fused shapes;
    each also as a HIP graph, the 7 with independent projections on parallel branches.  One pass walks `layers` layers with
    their own device copies of every matrix (more bytes than the last-level cache holds), microseconds per layer.  Outputs
    of the first and last layer of every variant are compared across encodings, one per shape against the oracle."""
    import numpy as np

    rows, gens, seen = [], {}, {}
    for m in (1, 4):
        xs = {stage: sp.make_x_i8(0xC0FFEE ^ (m + 16 * stage), m, k) for stage, k in enumerate((2560, 2560, 2560, 6912))}
        xbuf = {stage: sp.DeviceBuffer.from_numpy(x) for stage, x in xs.items()}
        for enc in ("u16", "delta", "i2s"):
            for label, shapes in (("seven", LAYER_SEVEN), ("four_fused", LAYER_FOUR)):
                base, nbytes = {}, 0
                for name, k_rows, n_cols, s_nz, stage in shapes:
                    key = (k_rows, n_cols, s_nz)
                    if key not in gens:
                        gens[key] = sp.generate_ternary(k_rows, n_cols, s_nz, dense=True)
                    Wm, p, n = gens[key]
                    if key not in base:
                        base[key] = (sp.Weights.upload_u16(p, n, k_rows, 0) if enc == "u16" else
                                     sp.Weights.upload_delta(p, n, k_rows, 0, rows=m) if enc == "delta" else sp.Weights.upload_i2s(Wm))
                    nbytes += algorithmic_bytes(base[key].info["stream_bytes"], m, k_rows, n_cols)
                layers = max(4, min(32, int(math.ceil(512e6 / nbytes))))
                owned, steps, outs = list(base.values()), [], []
                for l in range(layers):
                    for name, k_rows, n_cols, s_nz, stage in shapes:
                        w = base[(k_rows, n_cols, s_nz)].clone()
                        c = sp.DeviceBuffer(4 * m * n_cols)
                        owned += [w, c]
                        steps.append((w, xbuf[stage], c, m, 0, 4 * l + stage))
                        outs.append((l, name, (k_rows, n_cols, s_nz), stage, c))
                r = {"M": m, "enc": enc, "layer": label, "launches_per_layer": len(shapes), "layers_per_pass": layers, "bytes_per_layer": nbytes,
                     "floor_us_at_8TBps": round(nbytes / PEAK_GBPS / 1e3, 2)}
                for mode_name, mode in sp.SEQ_MODES.items():
                    if label == "four_fused" and mode_name in ("graph_branches", "streams", "batched_pairs"):
                        continue  # a chain: nothing to put side by side
                    for c in (o[-1] for o in outs):
                        c.fill(0xFF)
                    sp.measure_sequence(steps, max(2, reps // 10), mode, st)
                    us = min(sp.measure_sequence(steps, reps, mode, st) for _ in range(2)) / layers
                    r[mode_name + "_us"] = round(us, 2)
                    # every projection of the first and the last layer: the same numbers in every encoding and variant
                    for l, name, key, stage, c in outs:
                        if l not in (0, layers - 1):
                            continue
                        got = c.to_numpy(np.int32, (m, key[1]))
                        ref = seen.setdefault((m, key, stage), got)
                        if ref is got:
                            checks.append(("layer %s M=%d" % (name, m), xs[stage], gens[key][1], gens[key][2], got, key[2]))
                        assert (got == ref).all(), ("layer sequence", enc, label, mode_name, name, l)
                best = min(v for k, v in r.items() if k.endswith("_us") and k != "floor_us_at_8TBps")
                r["best_us"] = best
                r["best_pct_roofline"] = pct(nbytes, best)
                rows.append(r)
                for o in owned:
                    o.free()
        for b in xbuf.values():
            b.free()
    summary = {"columns": ["seven_launches_us", "five_launches_batched_pairs_us", "seven_graph_branches_us", "four_fused_launches_us", "four_fused_graph_us",
                           "floor_us_of_seven_at_8TBps"]}
    for m in (1, 4):
        for enc in ("u16", "delta", "i2s"):
            a7 = _row(rows, M=m, enc=enc, layer="seven")
            a4 = _row(rows, M=m, enc=enc, layer="four_fused")
            summary["M%d_%s" % (m, enc)] = [a7["launches_us"], a7["batched_pairs_us"], a7["graph_branches_us"], a4["launches_us"], a4["graph_chain_us"],
                                            a7["floor_us_at_8TBps"]]
    return {"rows": rows, "summary": summary,
            "protocol": "one pass = `layers_per_pass` layers, each with its own device copy of every matrix (> 512 MB per pass: HBM-cold); "
                        "us per layer between two HIP events around `reps` passes (sptmm_measure_sequence)"}


def quantising_leg(sp, st, k_rows, n_cols, s_nz, calls=600):
    """The calls around the int8 GEMV that BitNet inference makes (not in the reference, which has the GEMV only): one
    call per launch sequence, HBM-cold (rotating over device copies of the stream), microseconds per call by the host's
    clock around `calls` calls and a stream synchronise: the int8 GEMV, the same with its sums scaled on the way out
    (rows quantised by the caller), the fused quantising launch on fp16 rows, and its workspace variant (beyond four
    rows: the rows quantised once in a launch of their own)."""
    import numpy as np

    _, p, n = sp.generate_ternary(k_rows, n_cols, s_nz)
    rows = []
    for enc in ("u16", "delta"):
        for m in (1, 4, 8, 16):
            w = sp.Weights.upload_u16(p, n, k_rows, 0) if enc == "u16" else sp.Weights.upload_delta(p, n, k_rows, 0, rows=m if m <= 8 else 0)
            ncp = max(4, min(64, int(math.ceil(600e6 / w.nbytes))))
            cps = [w] + [w.clone() for _ in range(ncp - 1)]
            xh = sp.DeviceBuffer.from_numpy(sp.make_x_normal(0xC0FFEE ^ m, m, k_rows))
            xq = sp.DeviceBuffer.from_numpy(sp.make_x_i8(0xC0FFEE ^ m, m, k_rows))
            inv = sp.DeviceBuffer.from_numpy(np.full(m, 1.0 / 127.0, np.float32))
            yb = sp.DeviceBuffer(4 * m * n_cols)
            need = w.q8_workspace_bytes(m)
            ws = sp.DeviceBuffer(need)
            variants = (("int8_us", lambda c: c.gemv_i8(xq, m, yb, st)),
                        ("int8_scaled_us", lambda c: c.gemv_i8_scaled(xq, inv, m, 1.0, yb, st)),
                        ("quantising_fused_us", lambda c: c.gemv_q8(xh, 1, m, 1.0, yb, st)),
                        ("quantising_workspace_us", lambda c: c.gemv_q8_ws(xh, 1, m, 1.0, yb, ws, need, st)))
            r = {"K": k_rows, "N": n_cols, "S": s_nz, "enc": enc, "M": m}
            for name, call in variants:
                for c in cps:
                    call(c)
                st.sync()
                best = None
                for _ in range(3):
                    t0 = time.perf_counter()
                    done = 0
                    while done < calls:
                        for c in cps:
                            call(c)
                        done += ncp
                    st.sync()
                    us = (time.perf_counter() - t0) / done * 1e6
                    best = us if best is None else min(best, us)
                r[name] = round(best, 2)
            rows.append(r)
            for o in cps + [xh, xq, inv, yb, ws]:
                o.free()
    return {"rows": rows, "protocol": "host clock around %d calls + stream synchronise, best of three; one call = one or two launches on one stream, "
                                      "rotating over device copies of the stream (HBM-cold)" % calls}


def plans_leg(sp, n_shapes=12):
    """The launch-shape model against a bounded on-device search (sptmm_weights_tune), over seeded random shapes the model
    was never fitted on: K and N multiples of 256, 8-60 % nonzeros, both list encodings, a lone GEMV, a batched launch of 16
    GEMVs, and one of 16 four-row products.  Microseconds per GEMV, HBM-cold, with the model's shape and with the best plan found."""
    import numpy as np

    rng = np.random.default_rng(20250)
    rows = []
    for i in range(n_shapes):
        k_rows = int(rng.integers(4, 55)) * 256
        n_cols = int(rng.integers(1, 33)) * 256
        s_nz = max(32, int(k_rows * rng.uniform(0.08, 0.6)) // 32 * 32)
        Wm, p, n = sp.generate_ternary(k_rows, n_cols, s_nz)
        for enc in ("u16", "delta"):
            for m, batch in ((1, 0), (1, 16), (4, 16)):
                w = sp.Weights.upload_u16(p, n, k_rows, 0) if enc == "u16" else sp.Weights.upload_delta(p, n, k_rows, 0, rows=m if m <= 8 else 0)
                us_model, us_best, plan = w.tune(m, batch)
                rows.append({"K": k_rows, "N": n_cols, "S": s_nz, "enc": enc, "M": m, "gemvs_per_launch": batch or 1, "split_k": w.info["split_k"],
                             "model_us": round(us_model, 3), "best_plan_us": round(us_best, 3), "model_over_best": round(us_model / us_best, 3),
                             "plan": {k: v for k, v in plan.items() if v}})
                w.free()
    worst = max(rows, key=lambda r: r["model_over_best"])
    over = [r for r in rows if r["model_over_best"] > 1.10]
    return {"rows": rows, "summary": {"cases": len(rows), "model_more_than_10pct_behind_best_plan": len(over),
                                      "worst_model_over_best": worst["model_over_best"],
                                      "worst_case": {k: worst[k] for k in ("K", "N", "S", "enc", "M", "gemvs_per_launch")},
                                      "median_model_over_best": round(float(np.median([r["model_over_best"] for r in rows])), 3)}}


def run(argv=None):
    """-> the full result: the contract keys plus every leg's table."""
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256, help="timed steps; one step = one launch of BATCH GEMVs")
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--reps", type=int, default=0,
                    help="launches per timed loop of the legs (0: 1500, the headline shape's other encodings 4096); counter "
                         "runs under a profiler, where every launch is serialised, use a few dozen")
    ap.add_argument("--legs", default="single,others,ceiling,cfg1,cfg2,cfg3,layer,cfg4,density,plans,q8",
                    help="extra legs besides the headline loop: single (one GEMV per launch: cold, warm, sync-each-call, four streams), "
                         "others (delta and i2s encodings at the headline shape), cfg1 (the same matrix at M=4), cfg2 (gap "
                         "stream with fp16 rows), cfg3 (decoder-layer shapes, M=1 and 4), cfg4 (K=13824 N=5120, M=1/8/16), "
                         "layer (config 3 as a sequence: the decoder layer's 7 projections, or 4 with q+k+v and gate+up fused, "
                         "issued in order / as a HIP graph, rotating over enough layers to stay HBM-cold), "
                         "density (the headline shape at 3.7-25 % nonzeros against i2s), "
                         "plans (the launch-shape model against sptmm_weights_tune over random shapes), "
                         "q8 (the headline shape through the int8, scaled-int8 and quantising calls, one call at a time), "
                         "copy (4 launches of a 1 GiB copy kernel, for counter calibration), ceiling (a pure streaming "
                         "read of as many bytes as one step moves); profiling runs use --legs none or one leg")
    ap.add_argument("--detail", default=os.path.join(ROOT, "gpurun_out", "bench_detail.json"),
                    help="side file for the full result (every leg's per-row table); '' writes none")
    a = ap.parse_args(argv)
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus %d is not supported "
                 "(columns shard across GPUs with no collective, but nothing here runs a second GPU)" % a.gpus)

    import numpy as np

    import sptmm_amd as sp

    info = sp.device_init(0)
    Wd, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    X = sp.make_x_i8(0xC0FFEE ^ M, M, K)
    xb = sp.DeviceBuffer.from_numpy(X)
    cb = sp.DeviceBuffer(4 * M * N * BATCH)
    st = sp.Stream()
    legs = set(a.legs.replace("m4", "cfg1").split(","))
    checks = []  # (label, X, pos, neg, GPU result, S) for the CPU leg's oracle comparison

    def timed(weights, launches, warmup, mode):
        """-> (us per GEMV from two HIP events on the launch stream, host wall-clock ms per launch)."""
        per = len(weights) if mode == 3 else 1
        if warmup > 0:
            sp.measure_gemv(weights, 0, xb, M, cb, warmup * per, mode, st)
        sp.device_sync()
        t0 = time.perf_counter()
        us = sp.measure_gemv(weights, 0, xb, M, cb, launches * per, mode, st)
        sp.device_sync()
        return us, (time.perf_counter() - t0) * 1e3 / launches

    def time_encoding(w, act, Xh, m, n_cols, k_rows, reps=1500):
        reps = a.reps or reps
        """One weights object at one activation shape: one GEMV per launch on the same stream every launch
        (cache-warm) and rotating over enough device copies to exceed the last-level cache (HBM-cold), and
        32 (or as many as there are copies) per launch, HBM-cold.  Best of two, microseconds per GEMV."""
        xd = sp.DeviceBuffer.from_numpy(Xh)
        ncp = max(2, min(160, int(math.ceil(600e6 / w.nbytes))))
        cps = [w] + [w.clone() for _ in range(ncp - 1)]
        cd = sp.DeviceBuffer(4 * m * n_cols * min(ncp, BATCH))
        nb = algorithmic_bytes(w.info["stream_bytes"], m, k_rows, n_cols, Xh.itemsize)
        sp.measure_gemv(cps[:1], act, xd, m, cd, min(200, reps), 0, st)
        warm = min(sp.measure_gemv(cps[:1], act, xd, m, cd, reps, 0, st) for _ in range(2))
        sp.measure_gemv(cps, act, xd, m, cd, 2 * ncp, 0, st)
        cold = min(sp.measure_gemv(cps, act, xd, m, cd, reps, 0, st) for _ in range(2))
        groups = [cps[i:i + BATCH] for i in range(0, ncp, BATCH) if len(cps[i:i + BATCH]) == min(ncp, BATCH)]
        for g in groups:
            sp.measure_gemv(g, act, xd, m, cd, 2 * len(g), 3, st)
        per_group = max(8, min(96, reps) // len(groups))
        bat = min(sum(sp.measure_gemv(g, act, xd, m, cd, per_group * len(g), 3, st) for g in groups) / len(groups) for _ in range(2))
        for o in cps[1:] + [xd, cd]:
            o.free()
        return {"bytes": nb, "alone_warm_us": round(warm, 3), "alone_cold_us": round(cold, 3),
                "alone_cold_gbps": round(nb / cold / 1e3, 1), "alone_cold_pct_roofline": pct(nb, cold),
                "batched_us": round(bat, 3), "batched_gbps": round(nb / bat / 1e3, 1), "batched_pct_roofline": pct(nb, bat),
                "gemvs_per_batched_launch": len(groups[0])}

    def run_matrix(label, k_rows, n_cols, s_nz, ms, lists=None, split=0, from_dense=False):
        """The three encodings of one seeded matrix at the given row counts -> list of rows.  split = 0: the split
        the library picks for the shape (sptmm_choose_split_k); the row's `split_k` says which.  from_dense: the gap
        stream is built from the dense matrix (the builder for any ternary matrix), which walks gaps of more than 127
        rows over zero slots of the tile instead of widening every gap to 16 bits."""
        Wm, p, n = lists if lists is not None else sp.generate_ternary(k_rows, n_cols, s_nz, dense=True)
        rows = []
        # streams are built for the number of activation rows they will meet (the _rows upload calls): the gap stream for
        # GEMVs at M = 1, wide streams -- the lists read once for up to 16 rows -- beyond 8 rows
        makers = (("u16", lambda m: sp.Weights.upload_u16(p, n, k_rows, split if m <= 8 or split <= 64 else 0, rows=m)),
                  ("delta", (lambda m: sp.Weights.upload_dense(Wm, sp.KIND_DELTA, split, rows=m)) if from_dense else
                            (lambda m: sp.Weights.upload_delta(p, n, k_rows, split, rows=m))),
                  ("i2s", lambda m: sp.Weights.upload_i2s(Wm)))
        built_for = lambda enc, m: 0 if enc == "i2s" else 16 if m > 8 else 1 if (m == 1 and enc == "delta") else 4
        refs = {}
        for enc, mk in makers:
            w, have = None, None
            for m in ms:
                if w is None or built_for(enc, m) != have:
                    if w is not None:
                        w.free()
                    w, have = mk(m), built_for(enc, m)
                Xm = sp.make_x_i8(0xC0FFEE ^ m, m, k_rows)
                got = w.matmul(Xm)
                if m not in refs:
                    refs[m] = got
                    checks.append(("%s M=%d" % (label, m), Xm, p, n, got, s_nz))
                r = {"shape": label, "K": k_rows, "N": n_cols, "S": s_nz, "M": m, "enc": enc, "split_k": w.info["split_k"],
                     "row_bytes": w.info["row_bytes"], "delta_bits": w.info["delta_bits"], "zero_slot_detours": w.info["stones"],
                     "k_tile": w.info["k_tile"], "bit_exact_across_encodings": bool((got == refs[m]).all())}
                r.update(time_encoding(w, 0, Xm, m, n_cols, k_rows))
                rows.append(r)
            w.free()
        return rows

    w = sp.Weights.upload_u16(pos, neg, K, SPLIT)
    copies = [w] + [w.clone() for _ in range(BATCH - 1)]
    nbytes = algorithmic_bytes(w.nbytes, M, K, N)

    # correctness of what is about to be timed: every copy, through the batched entry point
    ref = w.matmul(X)
    outs = [sp.DeviceBuffer(4 * M * N) for _ in copies]
    sp.gemv_i8_batched(copies, [xb] * BATCH, outs, M, st)
    st.sync()
    for o in outs:
        assert (o.to_numpy(np.int32, (M, N)) == ref).all()
        o.free()

    # headline: EXACTLY --steps launches, each BATCH independent config-0 GEMVs over BATCH distinct
    # device copies of the stream (671 MB per launch: nothing survives in the 256 MB last-level cache)
    us_gemv, ms_step = timed(copies, a.steps, a.warmup, 3)
    launch_us = us_gemv * BATCH

    single = {}
    if "single" in legs:
        n1 = a.reps or 4096  # launches per timed loop
        single = {
            "cold_us": round(timed(copies, n1, 256, 0)[0], 3),   # one GEMV per launch, rotating over the copies
            "warm_us": round(timed(copies[:1], n1, 256, 0)[0], 3),  # same stream every launch (reference protocol)
            "sync_each_call_us": round(timed(copies[:1], min(n1, 2000), 50, 1)[0], 3),  # + host sync per launch (main.cu:1456)
            # still one GEMV per launch, launch i on stream i % 4: independent GEMVs overlap each other's ramp and tail
            # (best of three: here the host has to issue a launch every 0.8 us, and anything else running on it shows)
            "cold_four_streams_us": round(min(timed(copies, n1, 256, 4)[0] for _ in range(3)), 3),
        }
        # the same matrix at split-K 64 (one column per wavefront, ten wavefronts per CU instead of five): shorter wavefronts
        # leave less gathering to do once the last bytes have arrived -- the library's faster shape for a lone launch
        # (not BASELINE's configuration, which names split-K 32; slower than it in batched launches)
        w64 = sp.Weights.upload_u16(pos, neg, K, 64)
        assert (w64.matmul(X) == ref).all()
        c64 = [w64] + [w64.clone() for _ in range(BATCH - 1)]
        single["split64_cold_us"] = round(timed(c64, n1, 256, 0)[0], 3)
        single["split64_warm_us"] = round(timed(c64[:1], n1, 256, 0)[0], 3)
        single["split64_cold_pct_roofline"] = pct(nbytes, single["split64_cold_us"])
        for c in c64:
            c.free()
        single["cold_gbps"] = round(nbytes / single["cold_us"] / 1e3, 1)
        single["warm_gbps"] = round(nbytes / single["warm_us"] / 1e3, 1)
        single["cold_pct_roofline"] = pct(nbytes, single["cold_us"])
        single["cold_four_streams_pct_roofline"] = pct(nbytes, single["cold_four_streams_us"])
    for c in copies[1:]:
        c.free()

    if "copy" in legs:
        # plain copy kernel of known size: the yardstick the traffic counters are scaled by
        nb = 1 << 30
        src, dst = sp.DeviceBuffer(nb), sp.DeviceBuffer(nb)
        src.fill(1)
        for _ in range(4):
            sp.copy_kernel(dst, src, nb, st)
        st.sync()
        src.free()
        dst.free()

    ceiling = None
    if "ceiling" in legs:
        # the same bytes as one headline step, read with the kernels' own load instruction and thrown away
        nb = nbytes * BATCH // 16 * 16
        buf = sp.DeviceBuffer(nb)
        buf.fill(1)
        best = min(sp.read_kernel(buf, nb, st, 20, wgs) for wgs in (256, 512, 4096) for _ in range(2))
        ceiling = {"bytes": nb, "us": round(best, 2), "gbps": round(nb / best / 1e3, 1)}
        # and launched the way one GEMV per launch is: one stream's worth of bytes per launch, rotating over
        # BATCH regions (HBM-cold) or staying on one (cache-warm) -- the floor under `single_launch`
        one = nbytes // 16 * 16
        cold1 = min(sp.read_kernel(buf, one, st, 2048, wgs, BATCH, one) for wgs in (256, 512, 1024))
        warm1 = min(sp.read_kernel(buf, one, st, 2048, wgs) for wgs in (256, 512, 1024))
        buf.free()
        ceiling["per_launch_read"] = {"bytes": one, "cold_us": round(cold1, 3), "warm_us": round(warm1, 3)}

    others = {}
    if "others" in legs:
        for name, mk in (("delta8_split32", lambda: sp.Weights.upload_delta(pos, neg, K, SPLIT, rows=M)),
                         ("i2s", lambda: sp.Weights.upload_i2s(Wd))):
            ww = mk()
            assert (ww.matmul(X) == ref).all(), name
            others[name] = time_encoding(ww, 0, X, M, N, K, 4096)
            ww.free()

    configs = {}
    if "cfg1" in legs:
        # config 1: the same matrix at four activation rows (indices still read once per GEMV)
        configs["cfg1_m4"] = run_matrix("headline", K, N, S, (4,), (Wd, pos, neg), SPLIT)
    if "cfg2" in legs:
        # config 2: gap stream, fp16 rows ~N(0,1), fp32 sums
        rows = []
        ww = sp.Weights.upload_delta(pos, neg, K, SPLIT)
        for m in (1, 4):
            Xh = sp.make_x_normal(0xC0FFEE ^ m, m, K)  # seeded Box-Muller over the activations' own PRNG, as rcr -act f16
            got = ww.matmul(Xh)
            checks.append(("cfg2 fp16 M=%d" % m, Xh, pos, neg, got, S))
            r = {"shape": "headline", "K": K, "N": N, "S": S, "M": m, "enc": "delta", "split_k": SPLIT, "act": "fp16", "delta_bits": ww.info["delta_bits"]}
            r.update(time_encoding(ww, 1, Xh, m, N, K))
            rows.append(r)
        ww.free()
        configs["cfg2_delta_fp16"] = rows
    if "cfg3" in legs:
        rows = []
        for name, k_rows, n_cols, s_nz, _ in LAYER:
            rows += run_matrix(name, k_rows, n_cols, s_nz, (1, 4), (Wd, pos, neg) if (k_rows, n_cols, s_nz) == (K, N, S) else None)
        sums = []
        for m in (1, 4):
            for enc in ("u16", "delta", "i2s"):
                tot = {"M": m, "enc": enc, "gemvs": sum(mult for *_, mult in LAYER)}
                for key in ("alone_warm_us", "alone_cold_us", "batched_us", "bytes"):
                    tot[key] = round(sum(mult * next(r[key] for r in rows if (r["shape"], r["M"], r["enc"]) == (name, m, enc))
                                         for name, *_, mult in LAYER), 3)
                tot["batched_pct_roofline"] = pct(tot["bytes"], tot["batched_us"])
                sums.append(tot)
        configs["cfg3_layer"] = {"shapes": rows, "summed_layer": sums}
    if "cfg4" in legs:
        rows = run_matrix(*LARGE, (1, 8, 16))
        # M = 16 above ran on wide streams (K-tiled, 16-row tiles: the lists read once), which is what an upload that declares
        # 16 rows builds.  For comparison the ordinary streams at M = 16: two passes of eight rows, because a 16-row tile of
        # K = 13824 does not fit the LDS.
        name, k_rows, n_cols, s_nz = LARGE
        Wl, pl, nl = sp.generate_ternary(k_rows, n_cols, s_nz, dense=True)
        X16 = sp.make_x_i8(0xC0FFEE ^ 16, 16, k_rows)
        ref16 = next(g for lab, xx, _, _, g, _ in checks if lab == "large M=16")
        for enc, mk in (("u16, ordinary stream in two passes", lambda: sp.Weights.upload_u16(pl, nl, k_rows, 0)),
                        ("delta, ordinary stream in two passes", lambda: sp.Weights.upload_delta(pl, nl, k_rows, 0))):
            ww = mk()
            r = {"shape": name, "K": k_rows, "N": n_cols, "S": s_nz, "M": 16, "enc": enc, "split_k": ww.info["split_k"], "k_tile": ww.info["k_tile"],
                 "bit_exact_across_encodings": bool((ww.matmul(X16) == ref16).all())}
            r.update(time_encoding(ww, 0, X16, 16, n_cols, k_rows))
            rows.append(r)
            ww.free()
        configs["cfg4_large"] = rows

    layer_seq = None
    if "layer" in legs:
        layer_seq = layer_sequence(sp, st, checks, a.reps or 300)

    density = None
    if "density" in legs:
        # Where index lists overtake the 2-bit baseline: the same shape at fewer nonzeros per column.  i2s stores
        # every weight (K*N/4 bytes whatever S), the lists 2 bytes per nonzero, gap streams 1 byte per nonzero plus one
        # per zero slot visited on the way over a gap of more than 127 rows.
        rows = []
        for s_nz in DENSITY_S:
            rows += run_matrix("density %.1f %%" % (100.0 * s_nz / K), K, N, s_nz, (1,), from_dense=True)
        cross = []
        for s_nz in DENSITY_S:
            mine = [r for r in rows if r["S"] == s_nz]
            i2s_us = next(r["batched_us"] for r in mine if r["enc"] == "i2s")
            best = min((r for r in mine if r["enc"] != "i2s"), key=lambda r: r["batched_us"])
            cross.append({"S": s_nz, "density_pct": round(100.0 * s_nz / K, 1), "best_lists_enc": best["enc"],
                          "lists_batched_us": best["batched_us"], "i2s_batched_us": i2s_us,
                          "lists_over_i2s": round(best["batched_us"] / i2s_us, 3)})
        wins = [c["density_pct"] for c in cross if c["lists_over_i2s"] < 1.0]
        density = {"shapes": rows, "against_i2s": cross, "lists_beat_i2s_up_to_density_pct": max(wins) if wins else None}

    plans = plans_leg(sp) if "plans" in legs else None
    quantising = quantising_leg(sp, st, K, N, S, calls=min(a.reps or 600, 600)) if "q8" in legs else None

    gbps = nbytes / us_gemv / 1e3
    traffic, traffic_src = None, None
    if os.path.exists(TRAFFIC_SIDECAR):
        # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, scaled by what the same counters read for
        # a 1 GiB copy kernel: measured under the profiler at the commit the file names, not re-measured by this run
        traffic_src = json.load(open(TRAFFIC_SIDECAR))
        traffic = traffic_src.get("traffic_bytes_per_launch")
    i2s_m1 = others.get("i2s", {})
    out = {
        "metric": METRIC, "value": round(us_gemv, 3), "unit": "us/GEMV", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_step, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "int32", "data": "synthetic",
        "config": {"workload": "config 0: SpTMM u16 index lists, split-K=32, GEMV M=1 K=6912 N=2560 S=4096 "
                               "(2048 +1 / 2048 -1 rows per column, seed 0xCAFEBABE^col), int8 activations "
                               "uniform [-127,127] seeded, int32 accumulate; one step = one "
                               "sptmm_gemv_i8_batched launch of %d independent GEMVs of this shape, each on its "
                               "own device copy of the stream (HBM-cold)" % BATCH,
                   "M": M, "K": K, "N": N, "S": S, "split_k": SPLIT, "gemvs_per_step": BATCH,
                   "protocol": "launches back to back on one stream between two HIP events; value = event time "
                               "/ (steps * gemvs_per_step)"},
        "hbm_gbps": round(gbps, 1), "pct_roofline": round(100 * gbps / PEAK_GBPS, 2),
        # the same GEMV issued the way the reference's loop issues it: one per launch, HBM-cold
        "single_launch_cold_us": single.get("cold_us"), "single_launch_cold_pct_roofline": single.get("cold_pct_roofline"),
        "targets": {
            "hbm_70pct_in_batched_launches": bool(gbps / PEAK_GBPS >= 0.70),
            "hbm_70pct_one_gemv_per_launch": (single["cold_pct_roofline"] >= 70.0) if single else None,
            "hbm_70pct_one_gemv_per_launch_over_four_streams": (single["cold_four_streams_pct_roofline"] >= 70.0) if single else None,
            "beats_i2s_at_m1_batched": (us_gemv < i2s_m1["batched_us"]) if i2s_m1 else None,
            "beats_i2s_at_m1_one_per_launch": (single["cold_us"] < i2s_m1["alone_cold_us"]) if i2s_m1 and single else None,
            # at BASELINE's 59 % nonzeros the lists hold 4.7x (gap stream 2.4x) the bytes of i2s; they win where they are smaller
            "beats_i2s_batched_up_to_density_pct": density["lists_beat_i2s_up_to_density_pct"] if density else None,
        },
        "single_launch": single, "other_encodings": others, "configs": configs, "layer_sequence": layer_seq, "density_sweep": density, "launch_plans": plans,
        "quantising_calls": quantising,
        "device": {"arch": info["arch"], "compute_units": info["compute_units"]},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_src,
                     "kernel": "lists_kernel_batched<int8, MT=1, u16>", "launch_us": round(launch_us, 2),
                     "algorithmic_bytes_per_launch": nbytes * BATCH},
    }
    if ceiling:
        # not the roofline's peak (that stays the published 8 TB/s): what a pure read of the same size reaches here
        out["roofline"]["streaming_read_ceiling"] = ceiling
        out["roofline"]["frac_of_streaming_read"] = round(gbps / ceiling["gbps"], 4)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline((pos, neg), ref, checks, Wd)
    w.free()
    out["detail_file"] = os.path.relpath(a.detail, ROOT) if a.detail else None
    return out


def _row(rows, **want):
    for r in rows or ():
        if all(r.get(k) == v for k, v in want.items()):
            return r
    return None


def _pick(d, *keys):
    return {k: d[k] for k in keys if d and k in d}


def final_line(full):
    """The one stdout line: the contract keys, `roofline`, `cpu_baseline`, the single-launch figures, `targets`, and per
    configuration one compact row (us per GEMV in a batched HBM-cold launch and its % of 8 TB/s, plus the lone-launch
    HBM-cold us) -- a few KB whatever legs ran.  Everything else stays in the detail file."""
    out = {k: full[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                                 "vs_baseline", "dtype", "data", "config", "hbm_gbps", "pct_roofline", "single_launch_cold_us",
                                 "single_launch_cold_pct_roofline", "targets", "device") if k in full}
    rf = dict(full["roofline"])
    src = rf.pop("traffic_source", None)
    if src:
        rf["traffic_measured_at_commit"] = src.get("measured_at_commit")
        rf["traffic_file"] = os.path.relpath(TRAFFIC_SIDECAR, ROOT)
    ceil = rf.pop("streaming_read_ceiling", None)
    if ceil:
        rf["streaming_read_gbps"] = ceil["gbps"]
        rf["read_only_launch_us"] = _pick(ceil.get("per_launch_read"), "cold_us", "warm_us")
    out["roofline"] = rf
    if "cpu_baseline" in full:
        out["cpu_baseline"] = full["cpu_baseline"]
    if full.get("single_launch"):
        out["single_launch"] = full["single_launch"]

    def brief(r):  # [us per GEMV batched, % of 8 TB/s batched, us alone HBM-cold]
        return [r["batched_us"], r["batched_pct_roofline"], r["alone_cold_us"]] if r else None

    summary = {"columns": ["batched_us_per_gemv", "batched_pct_of_8TBps", "one_per_launch_cold_us"]}
    oth = full.get("other_encodings") or {}
    if oth:
        summary["cfg0_other_encodings"] = {k: brief(v) for k, v in oth.items()}
    cf = full.get("configs") or {}
    if "cfg1_m4" in cf:
        summary["cfg1_m4"] = {e: brief(_row(cf["cfg1_m4"], enc=e)) for e in ("u16", "delta", "i2s")}
    if "cfg2_delta_fp16" in cf:
        summary["cfg2_delta_fp16"] = {"M%d" % r["M"]: brief(r) for r in cf["cfg2_delta_fp16"]}
    if "cfg3_layer" in cf:
        summary["cfg3_layer_summed"] = {"M%d_%s" % (t["M"], t["enc"]): [t["batched_us"], t["batched_pct_roofline"], t["alone_cold_us"]]
                                        for t in cf["cfg3_layer"]["summed_layer"]}
    if "cfg4_large" in cf:
        summary["cfg4_large"] = {"M%d_%s" % (r["M"], r["enc"].split(",")[0] + ("_two_passes" if "," in r["enc"] else "")): brief(r) for r in cf["cfg4_large"]}
    if full.get("layer_sequence"):
        summary["layer_sequence"] = full["layer_sequence"]["summary"]
    dn = full.get("density_sweep")
    if dn:
        summary["density_lists_over_i2s"] = {str(c["density_pct"]): c["lists_over_i2s"] for c in dn["against_i2s"]}
    if full.get("launch_plans"):
        summary["launch_plans_model_vs_tuned"] = full["launch_plans"]["summary"]
    if full.get("quantising_calls"):
        summary["quantising_calls_us"] = {"columns": ["int8", "int8_scaled", "quantising_fused", "quantising_workspace"]}
        for r in full["quantising_calls"]["rows"]:
            summary["quantising_calls_us"]["M%d_%s" % (r["M"], r["enc"])] = [r["int8_us"], r["int8_scaled_us"], r["quantising_fused_us"], r["quantising_workspace_us"]]
    out["summary"] = summary
    out["detail_file"] = full.get("detail_file")
    return json.dumps(out, ensure_ascii=False, separators=(",", ":"))


def main():
    full = run()
    path = full.get("detail_file")
    if path:
        path = os.path.join(ROOT, path)
        try:
            os.makedirs(os.path.dirname(path), exist_ok=True)
            with open(path, "w") as f:
                json.dump(full, f, ensure_ascii=False, indent=1)
        except OSError as e:  # a read-only tree: the tables still go to stderr
            print("bench.py: cannot write %s: %s" % (path, e), file=sys.stderr)
    for leg in ("single_launch", "other_encodings", "configs", "layer_sequence", "density_sweep", "launch_plans", "quantising_calls"):
        if full.get(leg):
            print(json.dumps({leg: full[leg]}, ensure_ascii=False), file=sys.stderr)
    print(final_line(full), flush=True)


if __name__ == "__main__":
    main()
