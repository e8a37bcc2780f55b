"""Seeded random shapes through every list encoding, against the oracle's dense int8 product.

Covers what the fixed-shape tests leave open: per-task counts that straddle the straight-line /
ring kernel choice, tails of every length, empty tasks, every split, M around the 1/4/8 tile sizes.
"""
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def device():
    return sp.device_init(0)


def cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        K = 16 * int(rng.integers(1, 400))
        N = 16 * int(rng.integers(1, 24))
        dens = float(rng.choice([0.0, 0.02, 0.1, 0.3, 0.6, 0.9, 1.0]))
        bal = float(rng.uniform(0.2, 0.8))
        M = int(rng.integers(1, 10))
        out.append((K, N, dens * bal, dens * (1 - bal), M, int(rng.integers(0, 2**31))))
    return out


@pytest.mark.parametrize("kind,splits", [(sp.KIND_U16, (8, 16, 32, 64, 128, 256)), (sp.KIND_DELTA, (8, 16, 32, 64))])
def test_ragged_random_shapes(kind, splits):
    detours = 0  # gap streams that walk long gaps over zero slots of the tile
    for i, (K, N, pp, pn, M, seed) in enumerate(cases(20240 + kind, 40)):
        W = sp.generate_ternary_iid(K, N, seed, pp, pn)
        X = oracle.make_x_i8(seed ^ 0x55, M, K)
        want = oracle.dense_i8(X, W)
        split = splits[i % len(splits)]
        print("random ragged", kind, "K", K, "N", N, "p", round(pp, 3), round(pn, 3), "M", M, "split", split, flush=True)
        sys.stdout.flush()
        w = sp.Weights.upload_dense(W, kind, split, rows=1 if kind == sp.KIND_DELTA and i % 3 == 0 else 0)
        detours += w.info["stones"]
        got = w.matmul(X)
        w.free()
        assert (got == want).all(), (K, N, pp, pn, M, split)
    assert kind == sp.KIND_U16 or detours >= 3, detours


def test_balanced_random_shapes():
    rng = np.random.default_rng(7)
    for i in range(40):
        split = int(rng.choice([8, 16, 32, 64, 128, 256]))
        n_lane = int(rng.integers(1, 40))
        half = split * n_lane
        K = 16 * ((2 * half) // 16 + int(rng.integers(1, 60)))
        if K >= 65536:
            continue
        N = 16 * int(rng.integers(1, 16))
        M = int(rng.integers(1, 10))
        _, pos, neg = sp.generate_ternary(K, N, 2 * half)
        X = oracle.make_x_i8(i + 1, M, K)
        want = oracle.sptmm_i8(X, pos, neg)
        print("random balanced K", K, "N", N, "S", 2 * half, "split", split, "n_lane", n_lane, "M", M, flush=True)
        sys.stdout.flush()
        w = sp.Weights.upload_u16(pos, neg, K, split)
        assert (w.matmul(X) == want).all(), ("u16", K, N, half, split, M)
        w.free()
        if split <= 64:
            w = sp.Weights.upload_delta(pos, neg, K, split)
            assert (w.matmul(X) == want).all(), ("delta", K, N, half, split, M, w.info["delta_bits"])
            w.free()


def test_batched_random_shapes():
    """One launch of 1-40 GEMVs of one random shape, every stream kind and row count: each output equals the oracle's.
    Batched launches regroup their tasks (up to 16 per wavefront, workgroups of up to 16 wavefronts); the shapes here
    make task counts that do not divide evenly."""
    rng = np.random.default_rng(99)
    kinds = ("u16", "gap", "gap1", "dense gap", "dense gap1", "wide u16", "wide gap", "i2s")
    for i in range(48):
        kind = kinds[i % len(kinds)]
        K = 16 * int(rng.integers(4, 500))
        N = 16 * int(rng.integers(1, 60))
        split = int(rng.choice([8, 16, 32, 64]))
        M = int(rng.choice([1, 1, 2, 4, 5, 8, 9, 16]))
        count = int(rng.choice([1, 2, 4, 5, 7, 8, 13, 32, 33, 40]))
        dens = float(rng.choice([0.03, 0.1, 0.3, 0.6]))
        if kind in ("u16", "gap", "gap1"):
            n_lane = max(1, int(dens * K / 2 / split))
            S = 2 * split * n_lane
            if S >= K:
                S = 2 * split * max(1, (K - 16) // (2 * split))
            W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
            w = (sp.Weights.upload_u16(pos, neg, K, split) if kind == "u16" else
                 sp.Weights.upload_delta(pos, neg, K, split, rows=1 if kind == "gap1" else 0))
        else:
            W = sp.generate_ternary_iid(K, N, int(rng.integers(0, 2**31)), dens * 0.6, dens * 0.4)
            w = (sp.Weights.upload_dense(W, sp.KIND_DELTA, split, rows=1 if kind == "dense gap1" else 0) if kind.startswith("dense") else
                 sp.Weights.upload_wide(W, sp.KIND_U16 if kind == "wide u16" else sp.KIND_DELTA, split) if kind.startswith("wide") else
                 sp.Weights.upload_i2s(W))
        print("random batched", kind, "K", K, "N", N, "split", split, "M", M, "count", count, "dens", dens, flush=True)
        sys.stdout.flush()
        ws = [w] + [w.clone() for _ in range(min(count, 3) - 1)]
        ws = [ws[j % len(ws)] for j in range(count)]
        Xs = [oracle.make_x_i8(1000 * i + j, M, K) for j in range(min(count, 4))]
        xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
        cb = [sp.DeviceBuffer(4 * M * N) for _ in range(count)]
        for c in cb:
            c.fill(0xEE)
        st = sp.Stream()
        sp.gemv_i8_batched(ws, [xb[j % len(xb)] for j in range(count)], cb, M, st)
        st.sync()
        want = [oracle.dense_i8(x, W) for x in Xs]
        for j in range(count):
            assert (cb[j].to_numpy(np.int32, (M, N)) == want[j % len(want)]).all(), (kind, K, N, split, M, count, j)
        for o in xb + cb:
            o.free()
        for o in set(ws):
            o.free()
