"""Timing sweeps over the benchmark's other shapes, all three encodings of the same seeded matrix.

    python -m sptmm_amd.sweep layer     # BitNet-b1.58-2B decoder layer: q/o, k/v, gate/up (K=2560), down (K=6912)
    python -m sptmm_amd.sweep large     # K=13824 N=5120 S=8320, M in {1, 8, 16}
    python -m sptmm_amd.sweep headline  # K=6912 N=2560 S=4096, M in {1, 4}
    python -m sptmm_amd.sweep fused     # the layer with q+k+v (N=3840) and gate+up (N=13824) as single launches,
                                        # the fusions the reference benchmarks (main.cu:1107-1190): 4 launches per layer
    python -m sptmm_amd.sweep density   # K=6912 N=2560 M=1 at S = 256 ... 4096: where the index lists move fewer bytes than 2 bits per weight
    python -m sptmm_amd.sweep float     # fp16 / fp32 activations (the gap stream with fp16 rows is the benchmark's third configuration)
    python -m sptmm_amd.sweep q8        # sptmm_gemv_q8 (fp16 rows quantised in the kernel, float output) against sptmm_gemv_i8
    python -m sptmm_amd.sweep ragged    # the same four launches on matrices with independent entries (30 % +1, 30 % -1):
                                        # columns differ in nonzeros, streams carry per-task counts

Per shape and encoding: microseconds per GEMV launched alone (cache-warm = the same stream every launch;
HBM-cold = rotating over enough device copies to exceed the 256 MB last-level cache) and, for the list
encodings, per GEMV inside one batched launch.  Every timed object is first checked against the other
encodings (bit-exact int32).  Prints a table and one JSON line.
"""
from __future__ import annotations

import json
import sys

import numpy as np

from . import _capi as sp

PEAK_GBPS = 8000.0
LAYER = [("q/o", 2560, 2560, 1536, 2), ("k/v", 2560, 640, 1536, 2), ("gate/up", 2560, 6912, 1536, 2),
         ("down", 6912, 2560, 4160, 1)]
FUSED = [("qkv", 2560, 3840, 1536, 1), ("o", 2560, 2560, 1536, 1), ("gate+up", 2560, 13824, 1536, 1),
         ("down", 6912, 2560, 4160, 1)]


def copies_for(nbytes: int) -> int:
    return max(2, min(64, int(np.ceil(640e6 / nbytes))))


def time_weights(w, X, M, N, st, batched: bool):
    xb = sp.DeviceBuffer.from_numpy(X)
    n = copies_for(w.nbytes)
    cps = [w] + [w.clone() for _ in range(n - 1)]
    cb = sp.DeviceBuffer(4 * M * N * min(n, 32))
    sp.measure_gemv(cps[:1], 0, xb, M, cb, 200, 0, st)
    warm = min(sp.measure_gemv(cps[:1], 0, xb, M, cb, 2000, 0, st) for _ in range(3))
    sp.measure_gemv(cps, 0, xb, M, cb, 2 * n, 0, st)
    cold = min(sp.measure_gemv(cps, 0, xb, M, cb, 2000, 0, st) for _ in range(3))
    bat = None
    if batched:
        nb = min(n, 32)
        sp.measure_gemv(cps[:nb], 0, xb, M, cb, 4 * nb, 3, st)
        bat = min(sp.measure_gemv(cps[:nb], 0, xb, M, cb, 64 * nb, 3, st) for _ in range(3))
    for c in cps[1:]:
        c.free()
    xb.free()
    cb.free()
    return warm, cold, bat


def run_shape(name, K, N, S, Ms, splits, st, rows, iid=None):
    if iid is None:
        W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    else:
        W = sp.generate_ternary_iid(K, N, 0x5EED ^ N, *iid)
    for M in Ms:
        X = sp.make_x_i8(0xC0FFEE ^ M, M, K)
        ref = None
        if iid is None:
            cands = [("u16/%d" % s, lambda s=s: sp.Weights.upload_u16(pos, neg, K, s)) for s in splits if (S // 2) % s == 0]
            cands += [("delta/%d" % s, lambda s=s: sp.Weights.upload_delta(pos, neg, K, s)) for s in splits
                      if s <= 64 and (S // 2) % s == 0]
        else:
            cands = [("u16/%d" % s, lambda s=s: sp.Weights.upload_dense(W, sp.KIND_U16, s)) for s in splits]
            cands += [("delta/%d" % s, lambda s=s: sp.Weights.upload_dense(W, sp.KIND_DELTA, s)) for s in splits if s <= 64]
        cands += [("i2s", lambda: sp.Weights.upload_i2s(W))]
        for enc, mk in cands:
            w = mk()
            got = w.matmul(X)
            if ref is None:
                ref = got
            ok = bool((got == ref).all())
            nbytes = w.info["stream_bytes"] + M * K + 4 * M * N  # what one GEMV reads and writes
            warm, cold, bat = time_weights(w, X, M, N, st, True)
            w.free()
            rows.append({"shape": name, "K": K, "N": N, "S": S, "M": M, "enc": enc, "bytes": nbytes, "ok": ok,
                         "warm_us": round(warm, 3), "cold_us": round(cold, 3),
                         "batched_us": None if bat is None else round(bat, 3)})
            r = rows[-1]
            print("%-8s K=%-5d N=%-5d S=%-5d M=%-2d %-9s %s  warm %7.2f us  cold %7.2f us (%5.0f GB/s)  batched %s"
                  % (name, K, N, S, M, enc, "ok " if ok else "BAD", warm, cold, nbytes / cold / 1e3,
                     "   -   " if bat is None else "%7.2f us (%5.0f GB/s, %4.1f%%)" % (bat, nbytes / bat / 1e3,
                                                                                     nbytes / bat / 1e3 / PEAK_GBPS * 100)),
                  flush=True)


def layer_sequence(shapes, M, st, rows, iid=None):
    """The layer's launches one after the other on one stream, each with its best split: plain launches and
    one HIP graph per layer; cache-warm (one set of streams) and HBM-cold (rotating over 8 sets)."""
    Kmax, Nmax = max(k for _, k, *_ in shapes), max(n for _, _, n, *_ in shapes)
    xb = sp.DeviceBuffer.from_numpy(sp.make_x_i8(0xC0FFEE ^ M, M, Kmax))
    cb = sp.DeviceBuffer(4 * M * Nmax)
    for kind in ("u16", "delta", "i2s"):
        layer, nbytes = [], 0
        for name, K, N, S, mult in shapes:
            best = min((r for r in rows if r["shape"] == name and r["M"] == M and r["enc"].startswith(kind)), key=lambda r: r["warm_us"])
            split = int(best["enc"].split("/")[1]) if "/" in best["enc"] else 0
            if iid is None:
                W, pos, neg = sp.generate_ternary(K, N, S, dense=kind == "i2s")
                w = (sp.Weights.upload_i2s(W) if kind == "i2s" else sp.Weights.upload_u16(pos, neg, K, split) if kind == "u16"
                     else sp.Weights.upload_delta(pos, neg, K, split))
            else:
                W = sp.generate_ternary_iid(K, N, 0x5EED ^ N, *iid)
                w = sp.Weights.upload_dense(W, {"u16": sp.KIND_U16, "delta": sp.KIND_DELTA, "i2s": sp.KIND_I2S}[kind], split or 32)
            layer += [w] * mult
            nbytes += mult * (w.info["stream_bytes"] + M * K + 4 * M * N)
        sets = [layer] + [[w.clone() for w in layer] for _ in range(7)]
        flat = [w for s_ in sets for w in s_]
        out = {"shape": "layer_sequence", "M": M, "enc": kind, "launches": len(layer), "bytes": nbytes}
        for label, ws in (("warm", layer), ("cold", flat)):
            for mode, mname in ((0, "launches"), (2, "graph")):
                sp.measure_gemv(ws, 0, xb, M, cb, 2 * len(ws), mode, st)
                t = min(sp.measure_gemv(ws, 0, xb, M, cb, 40 * len(ws), mode, st) for _ in range(3)) * len(layer)
                out["%s_%s_us" % (label, mname)] = round(t, 2)
        print("layer in %d launches M=%d %-5s: warm %.1f us (graph %.1f)  cold %.1f us (graph %.1f; %.0f GB/s)"
              % (len(layer), M, kind, out["warm_launches_us"], out["warm_graph_us"], out["cold_launches_us"], out["cold_graph_us"],
                 nbytes / out["cold_graph_us"] / 1e3), flush=True)
        rows.append(out)
        for s_ in sets[1:]:
            for w in s_:
                w.free()
        for w in set(layer):
            w.free()
    xb.free()
    cb.free()


def q8_rows(st, rows):
    """The fused quantise -> GEMV -> rescale launch against the plain int8 GEMV, same streams."""
    for name, K, N, S, split in (("headline", 6912, 2560, 4096, 32), ("qkv", 2560, 3840, 1536, 32), ("gate+up", 2560, 13824, 1536, 16),
                                 ("down", 6912, 2560, 4160, 32)):
        _, pos, neg = sp.generate_ternary(K, N, S)
        for M in (1, 4):
            rng = np.random.default_rng(M)
            xh = sp.DeviceBuffer.from_numpy(rng.standard_normal((M, K)).astype(np.float16))
            xi = sp.DeviceBuffer.from_numpy(sp.make_x_i8(M, M, K))
            cb = sp.DeviceBuffer(4 * M * N)
            for enc in ("u16", "delta"):
                w = sp.Weights.upload_u16(pos, neg, K, split) if enc == "u16" else sp.Weights.upload_delta(pos, neg, K, split)
                n = copies_for(w.nbytes)
                cps = [w] + [w.clone() for _ in range(n - 1)]
                out = {"shape": name, "K": K, "N": N, "M": M, "enc": "%s/%d" % (enc, split)}
                for act, xb, tag in ((0, xi, "i8"), (3, xh, "q8")):
                    sp.measure_gemv(cps[:1], act, xb, M, cb, 200, 0, st)
                    out[tag + "_warm_us"] = round(min(sp.measure_gemv(cps[:1], act, xb, M, cb, 2000, 0, st) for _ in range(3)), 3)
                    sp.measure_gemv(cps, act, xb, M, cb, 2 * n, 0, st)
                    out[tag + "_cold_us"] = round(min(sp.measure_gemv(cps, act, xb, M, cb, 2000, 0, st) for _ in range(3)), 3)
                print("%-8s M=%d %-8s int8 GEMV warm %6.2f cold %6.2f us | fused q8 warm %6.2f cold %6.2f us"
                      % (name, M, out["enc"], out["i8_warm_us"], out["i8_cold_us"], out["q8_warm_us"], out["q8_cold_us"]), flush=True)
                rows.append(out)
                for c in cps:
                    c.free()
            for b in (xh, xi, cb):
                b.free()


def float_rows(st, rows):
    """fp16 / fp32 activations (fp32 sums) against int8 on the headline matrix, one GEMV per launch."""
    K, N, S = 6912, 2560, 4096
    _, pos, neg = sp.generate_ternary(K, N, S)
    rng = np.random.default_rng(0)
    for M in (1, 4):
        xs = ((0, "i8", sp.make_x_i8(1, M, K)), (1, "f16", rng.standard_normal((M, K)).astype(np.float16)),
              (2, "f32", rng.standard_normal((M, K)).astype(np.float32)))
        cb = sp.DeviceBuffer(4 * M * N)
        cbb = sp.DeviceBuffer(4 * M * N * 32)
        for enc, split in (("delta", 32), ("u16", 32)):
            w = sp.Weights.upload_delta(pos, neg, K, split) if enc == "delta" else sp.Weights.upload_u16(pos, neg, K, split)
            n = copies_for(w.nbytes)
            cps = [w] + [w.clone() for _ in range(n - 1)]
            for act, name, X in xs:
                xb = sp.DeviceBuffer.from_numpy(X)
                sp.measure_gemv(cps[:1], act, xb, M, cb, 200, 0, st)
                warm = min(sp.measure_gemv(cps[:1], act, xb, M, cb, 2000, 0, st) for _ in range(3))
                sp.measure_gemv(cps, act, xb, M, cb, 2 * n, 0, st)
                cold = min(sp.measure_gemv(cps, act, xb, M, cb, 2000, 0, st) for _ in range(3))
                nb = min(n, 32)
                sp.measure_gemv(cps[:nb], act, xb, M, cbb, 4 * nb, 3, st)
                bat = min(sp.measure_gemv(cps[:nb], act, xb, M, cbb, 64 * nb, 3, st) for _ in range(3))
                nbytes = w.info["stream_bytes"] + M * K * X.itemsize + 4 * M * N
                xb.free()
                print("headline M=%d %s/%d %-3s activations: warm %6.2f us  cold %6.2f us  %d per launch %6.2f us (%.1f%% of HBM peak)"
                      % (M, enc, split, name, warm, cold, nb, bat, nbytes / bat / 1e3 / PEAK_GBPS * 100), flush=True)
                rows.append({"shape": "headline", "M": M, "enc": "%s/%d" % (enc, split), "act": name, "bytes": nbytes,
                             "warm_us": round(warm, 3), "cold_us": round(cold, 3), "batched_us": round(bat, 3)})
            for c in cps:
                c.free()
        cb.free()
        cbb.free()


def main(argv):
    which = argv[1] if len(argv) > 1 else "layer"
    info = sp.device_init(0)
    st = sp.Stream()
    rows = []
    if which in ("layer", "fused", "ragged"):
        shapes = LAYER if which == "layer" else FUSED
        for name, K, N, S, _ in shapes:
            run_shape(name, K, N, S, (1, 4), (8, 16, 32, 64) if which == "layer" else (16, 32, 64), st, rows,
                      iid=(0.3, 0.3) if which == "ragged" else None)
        for M in (1, 4):
            for kind in ("u16", "delta", "i2s"):
                tot_w = tot_c = 0.0
                for name, K, N, S, mult in shapes:
                    best = [r for r in rows if r["shape"] == name and r["M"] == M and r["enc"].startswith(kind)]
                    tot_w += mult * min(r["warm_us"] for r in best)
                    tot_c += mult * min(r["cold_us"] for r in best)
                print("layer sum (%d launches, best split per shape) M=%d %-5s: warm %.1f us  cold %.1f us"
                      % (sum(m for *_, m in shapes), M, kind, tot_w, tot_c))
                rows.append({"shape": "layer_sum", "M": M, "enc": kind, "warm_us": round(tot_w, 2), "cold_us": round(tot_c, 2)})
        if which != "layer":
            for M in (1, 4):
                layer_sequence(shapes, M, st, rows, iid=(0.3, 0.3) if which == "ragged" else None)
    elif which == "density":
        for S in (256, 512, 1024, 2048, 4096):
            run_shape("S=%d" % S, 6912, 2560, S, (1,), (32,), st, rows)
    elif which == "float":
        float_rows(st, rows)
    elif which == "q8":
        q8_rows(st, rows)
    elif which == "large":
        run_shape("large", 13824, 5120, 8320, (1, 8, 16), (32, 64), st, rows)
    elif which == "headline":
        run_shape("headline", 6912, 2560, 4096, (1, 4), (16, 32, 64), st, rows)
    else:
        sys.exit("usage: python -m sptmm_amd.sweep layer|large|headline|fused|ragged|density|float|q8")
    assert all(r.get("ok", True) for r in rows), "encodings disagree"
    print(json.dumps({"device": info["arch"], "rows": rows}))


if __name__ == "__main__":
    main(sys.argv)
