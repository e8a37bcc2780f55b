#!/usr/bin/env python3
"""Headline benchmark: SpTMM split-K=32 GEMV at M=1, K=6912, N=2560, S=4096 on one MI355X.

A step is one launch of the C ABI's sptmm_gemv_i8_batched: 32 independent
GEMVs of the headline shape, each on its own device copy of the u16-list stream.
The copies together (671 MB) exceed the 256 MB last-level cache, so every GEMV
streams its 21 MB of row indices from HBM ("cold"), as a decoder walking
through gigabytes of layer weights does, and the dispatch latency is paid once
per step instead of once per GEMV.  Reported beside it: one GEMV per launch
(cold; warm = the reference's protocol, main.cu:994-1459; and with its per-call
host sync) and the other two encodings.

Prints ONE JSON line (see the keys at the bottom).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "µs/GEMV and achieved HBM GB/s (% roofline) at M=1 K=6912 N=2560 S=4096"
K, N, S, M, SPLIT = 6912, 2560, 4096, 1, 32
BATCH = 32  # GEMVs per launch = device copies of the stream: 32 x 21 MB = 671 MB > 256 MB Infinity Cache
PEAK_GBPS = 8000.0


def algorithmic_bytes(stream_bytes, m=M):
    # weight stream (indices counted once, whatever M) + activations + output
    return stream_bytes + m * K + 4 * m * N


def cpu_baseline(sp_lists, budget_s=12.0):
    """The oracle's gather-sum (a port of main.cu:577-593) on the host cores; bounded sample."""
    import numpy as np

    import oracle

    pos, neg = sp_lists
    cores = min(len(os.sched_getaffinity(0)), 16)
    X = oracle.make_x_i8(0xC0FFEE ^ M, M, K)
    out = np.empty((M, N), np.int32)
    want = oracle.sptmm_i8(X, pos, neg)
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
    return {
        "value": round(us, 2), "unit": "us/GEMV", "cores": cores, "kind": "port",
        "sample": "%d full GEMVs of the same W and X (oracle gather-sum over u16 lists, %d pthreads); "
                  "single thread: %.1f us/GEMV over %d GEMVs" % (reps, cores, res[1][0], res[1][1]),
        "value_1core": round(res[1][0], 2),
        "gbps": round(algorithmic_bytes(2 * S * N) / us / 1e3, 2),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256, help="timed steps; one step = one launch of BATCH GEMVs")
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--legs", default="single,others,ceiling,m4",
                    help="extra legs besides the headline loop: single (one GEMV per launch: cold, warm, "
                         "sync-each-call), others (delta and i2s encodings), m4 (config 1: the same matrix at M=4, all three "
                         "encodings), copy (4 launches of a 1 GiB copy kernel, for counter "
                         "calibration), ceiling (a pure streaming read of as many bytes as one step moves: the practical HBM read "
                         "ceiling on this box); profiling runs use --legs none or --legs copy")
    a = ap.parse_args()
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
    legs = set(a.legs.split(","))

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

    w = sp.Weights.upload_u16(pos, neg, K, SPLIT)
    copies = [w] + [w.clone() for _ in range(BATCH - 1)]
    nbytes = algorithmic_bytes(w.nbytes)

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
        n1 = 4096
        single = {
            "cold_us": round(timed(copies, n1, 256, 0)[0], 3),   # one GEMV per launch, rotating over the copies
            "warm_us": round(timed(copies[:1], n1, 256, 0)[0], 3),  # same stream every launch (reference protocol)
            "sync_each_call_us": round(timed(copies[:1], 2000, 50, 1)[0], 3),  # + host sync per launch (main.cu:1456)
        }
        single["cold_gbps"] = round(nbytes / single["cold_us"] / 1e3, 1)
        single["warm_gbps"] = round(nbytes / single["warm_us"] / 1e3, 1)
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
        for name, mk in (("delta8_split32", lambda: sp.Weights.upload_delta(pos, neg, K, SPLIT)),
                         ("i2s", lambda: sp.Weights.upload_i2s(Wd))):
            ww = mk()
            assert (ww.matmul(X) == ref).all(), name
            cps = [ww] + [ww.clone() for _ in range(BATCH * (4 if name == "i2s" else 2) - 1)]
            b = algorithmic_bytes(ww.nbytes)
            r = {"bytes": b, "single_cold_us": round(timed(cps, 4096, 256, 0)[0], 3),
                 "single_warm_us": round(timed(cps[:1], 4096, 256, 0)[0], 3)}
            # 32 per launch; the small i2s streams rotate over four such groups to stay out of the last-level cache
            groups = [cps[i:i + BATCH] for i in range(0, len(cps), BATCH)]
            for g in groups:
                sp.measure_gemv(g, 0, xb, M, cb, BATCH * max(a.warmup // len(groups), 1), 3, st)
            t = [sp.measure_gemv(g, 0, xb, M, cb, BATCH * max(a.steps // len(groups), 1), 3, st) for g in groups]
            r["batched_cold_us"] = round(sum(t) / len(t), 3)
            r["batched_cold_gbps"] = round(b / r["batched_cold_us"] / 1e3, 1)
            others[name] = r
            for c in cps:
                c.free()

    m4 = {}
    if "m4" in legs:
        # config 1: the same matrix at four activation rows (indices still read once per GEMV)
        M4 = 4
        X4 = sp.make_x_i8(0xC0FFEE ^ M4, M4, K)
        x4 = sp.DeviceBuffer.from_numpy(X4)
        c4 = sp.DeviceBuffer(4 * M4 * N * BATCH)
        ref4 = None
        for name, mk, ncp in (("u16_split32", lambda: sp.Weights.upload_u16(pos, neg, K, SPLIT), BATCH),
                              ("delta8_split16", lambda: sp.Weights.upload_delta(pos, neg, K, 16), 2 * BATCH),
                              ("i2s", lambda: sp.Weights.upload_i2s(Wd), 4 * BATCH)):
            ww = mk()
            got = ww.matmul(X4)
            ref4 = got if ref4 is None else ref4
            assert (got == ref4).all(), name
            cps = [ww] + [ww.clone() for _ in range(ncp - 1)]
            b = algorithmic_bytes(ww.nbytes, M4)
            sp.measure_gemv(cps, 0, x4, M4, c4, 256, 0, st)
            r = {"bytes": b, "single_cold_us": round(sp.measure_gemv(cps, 0, x4, M4, c4, 4096, 0, st), 3)}
            sp.measure_gemv(cps[:1], 0, x4, M4, c4, 256, 0, st)
            r["single_warm_us"] = round(sp.measure_gemv(cps[:1], 0, x4, M4, c4, 4096, 0, st), 3)
            groups = [cps[i:i + BATCH] for i in range(0, len(cps), BATCH)]
            for g in groups:
                sp.measure_gemv(g, 0, x4, M4, c4, BATCH * max(a.warmup // len(groups), 1), 3, st)
            t = [sp.measure_gemv(g, 0, x4, M4, c4, BATCH * max(a.steps // len(groups), 1), 3, st) for g in groups]
            r["batched_cold_us"] = round(sum(t) / len(t), 3)
            r["batched_cold_gbps"] = round(b / r["batched_cold_us"] / 1e3, 1)
            r["batched_pct_roofline"] = round(100 * r["batched_cold_gbps"] / PEAK_GBPS, 2)
            m4[name] = r
            for c in cps:
                c.free()
        x4.free()
        c4.free()

    gbps = nbytes / us_gemv / 1e3
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
        "single_launch": single, "other_encodings": others, "config1_m4": m4,
        "device": {"arch": info["arch"], "compute_units": info["compute_units"]},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / PEAK_GBPS, 4),
                     # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE (x2.0) + WRITE_SIZE (x1.0), scale factors
                     # from the 1 GiB copy kernel; measured once and recorded in profiles/, not re-measured here
                     "traffic": 671.8e6,
                     "kernel": "lists_kernel_batched<int8, MT=1, u16>", "launch_us": round(launch_us, 2),
                     "algorithmic_bytes_per_launch": nbytes * BATCH},
    }
    if ceiling:
        # not the roofline's peak (that stays the published 8 TB/s): what a pure read of the same size reaches here
        out["roofline"]["streaming_read_ceiling"] = ceiling
        out["roofline"]["frac_of_streaming_read"] = round(gbps / ceiling["gbps"], 4)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline((pos, neg))
    w.free()
    print(json.dumps(out, ensure_ascii=False))


if __name__ == "__main__":
    main()
