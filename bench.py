#!/usr/bin/env python3
"""Headline benchmark: SpTMM split-K=32 GEMV at M=1, K=6912, N=2560, S=4096 on one MI355X.

A step is one GEMV launch through the C ABI (sptmm_gemv_i8 on the u16-list
stream).  Launch i reads device copy i % COPIES of the same matrix; the copies
together exceed the 256 MB last-level cache, so every step streams its 21 MB of
row indices from HBM ("cold"), as a decoder that walks through gigabytes of
layer weights does.  The same loop over a single copy ("warm", the reference's
protocol, main.cu:994-1459) and the other two encodings are reported beside it.

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
COPIES = 32  # 32 x 21 MB = 671 MB of index streams > 256 MB Infinity Cache
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
    ap.add_argument("--steps", type=int, default=4096)
    ap.add_argument("--warmup", type=int, default=256)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus %d is not supported "
                 "(columns shard across GPUs with no collective, but nothing here runs a second GPU)" % a.gpus)

    import numpy as np

    import sptmm_amd as sp

    info = sp.device_init(0)
    _, pos, neg = sp.generate_ternary(K, N, S)
    Wd, _, _ = sp.generate_ternary(K, N, S, dense=True)
    X = sp.make_x_i8(0xC0FFEE ^ M, M, K)
    xb = sp.DeviceBuffer.from_numpy(X)
    cb = sp.DeviceBuffer(4 * M * N)
    st = sp.Stream()

    def timed(weights, steps, warmup, mode=0):
        """-> (us per launch from HIP events on the launch stream, host wall-clock ms per step)."""
        if warmup > 0:
            sp.measure_gemv(weights, 0, xb, M, cb, warmup, mode, st)
        sp.device_sync()
        t0 = time.perf_counter()
        us = sp.measure_gemv(weights, 0, xb, M, cb, steps, mode, st)
        sp.device_sync()
        return us, (time.perf_counter() - t0) * 1e3 / steps

    w = sp.Weights.upload_u16(pos, neg, K, SPLIT)
    copies = [w] + [w.clone() for _ in range(COPIES - 1)]
    nbytes = algorithmic_bytes(w.nbytes)

    # correctness of what is about to be timed (every copy), against the other two encodings
    ref = w.matmul(X)
    for c in copies[1:]:
        c.gemv_i8(xb, M, cb, st)
        st.sync()
        assert (cb.to_numpy(np.int32, (M, N)) == ref).all()

    cold_us, cold_ms_step = timed(copies, a.steps, a.warmup)
    warm_us, _ = timed(copies[:1], a.steps, a.warmup)
    sync_us, _ = timed(copies[:1], min(a.steps, 2000), 50, mode=1)
    for c in copies[1:]:
        c.free()

    others = {}
    for name, ww in (("delta8_split32", sp.Weights.upload_delta(pos, neg, K, SPLIT)), ("i2s", sp.Weights.upload_i2s(Wd))):
        assert (ww.matmul(X) == ref).all(), name
        cps = [ww] + [ww.clone() for _ in range(COPIES * (4 if name == "i2s" else 2) - 1)]
        c_us, _ = timed(cps, a.steps, a.warmup)
        w_us, _ = timed(cps[:1], a.steps, a.warmup)
        b = algorithmic_bytes(ww.nbytes)
        others[name] = {"cold_us": round(c_us, 3), "warm_us": round(w_us, 3), "bytes": b,
                        "cold_gbps": round(b / c_us / 1e3, 1), "warm_gbps": round(b / w_us / 1e3, 1)}
        for c in cps:
            c.free()

    out = {
        "metric": METRIC, "value": round(cold_us, 3), "unit": "us/GEMV", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(cold_ms_step, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "int32", "data": "synthetic",
        "config": {"workload": "config 0: SpTMM u16 index lists, split-K=32, single GEMV M=1 K=6912 N=2560 "
                               "S=4096 (2048 +1 / 2048 -1 rows per column, seed 0xCAFEBABE^col), int8 "
                               "activations uniform [-127,127] seeded, int32 accumulate",
                   "M": M, "K": K, "N": N, "S": S, "split_k": SPLIT, "weight_copies_rotated": COPIES,
                   "protocol": "back-to-back launches on one stream between two HIP events, no sync inside"},
        "hbm_gbps": round(nbytes / cold_us / 1e3, 1), "pct_roofline": round(100 * nbytes / cold_us / 1e3 / PEAK_GBPS, 2),
        "warm_us": round(warm_us, 3), "warm_gbps": round(nbytes / warm_us / 1e3, 1),
        "sync_each_call_us": round(sync_us, 3),
        "other_encodings": others,
        "device": {"arch": info["arch"], "compute_units": info["compute_units"]},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / cold_us / 1e3, 1), "peak": PEAK_GBPS, "unit": "GB/s",
                     "frac": round(nbytes / cold_us / 1e3 / PEAK_GBPS, 4), "traffic": None,
                     "kernel": "lists_kernel<int8,1,u16>", "algorithmic_bytes_per_launch": nbytes,
                     "avg_launch_us": round(cold_us, 3)},
    }
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline((pos, neg))
    w.free()
    print(json.dumps(out, ensure_ascii=False))


if __name__ == "__main__":
    main()
