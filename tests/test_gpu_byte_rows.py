"""GPU parity of the gap streams scheduled for single activation rows (sptmm_*_rows with rows = 1).

Such a stream holds the same runs per lane in another visiting order, and an int8 GEMV at M = 1 gathers
from a tile of one byte per row (the running row is the LDS address).  Every other call (M > 1, fp16/fp32
rows, the quantising GEMV) is served from the ordinary tiles.  Oracle: the CPU gather-sum (balanced
matrices) or the dense int8 product (ragged ones); int32 results bit-exact, float rows within
    |got - ref| <= 1e-3 * max(|ref|, sqrt(S))
of the float64 gather-sum.
"""
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu
DELTA = sp.KIND_DELTA


@pytest.fixture(scope="module", autouse=True)
def device():
    return sp.device_init(0)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("K,N,S,splits", [
    (6912, 2560, 4096, (8, 16, 32, 64)),   # headline: straight-line bodies of 16, 8, 4, 2 rounds
    (6912, 64, 4160, (8, 16, 32)),         # 260 / 130 / 65 gaps per lane: ring, tails of 1, 2, 4 bytes
    (2560, 640, 1536, (8, 16, 32, 64)),    # 96 .. 12 gaps per lane
    (13824, 5120, 8320, (64,)),            # config 4
    (512, 48, 256, (8, 16, 32, 64)),       # no full round at the larger splits
    (64, 16, 32, (8, 16)),                 # one or two entries per lane
])
def test_balanced_matrix_bit_exact_at_every_m(K, N, S, splits):
    _, pos, neg = sp.generate_ternary(K, N, S)
    for split in splits:
        w = sp.Weights.upload_delta(pos, neg, K, split, rows=1)
        i = w.info
        assert i["delta_bits"] == 8 and i["row_bytes"] == 1 and i["stream_bytes"] == sp.Weights.upload_delta(pos, neg, K, split).info["stream_bytes"]
        for M in (1, 2, 5, 9):
            say("byte rows", K, N, S, "split", split, "M", M)
            X = oracle.make_x_i8(S + 31 * M, M, K)
            assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), (split, M)
        for X in (np.full((1, K), 127, np.int8), np.full((1, K), -128, np.int8), np.eye(1, K, K - 1, dtype=np.int8)):
            assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all()
        Xh = oracle.make_x_normal(split, 2, K, np.float16)
        got = w.matmul(Xh)
        ref = oracle.sptmm_f64(Xh, pos, neg)
        assert (np.abs(got - ref) / np.maximum(np.abs(ref), np.sqrt(S))).max() <= 1e-3
        w.free()


def test_sparse_matrix_keeps_16_bit_gaps():
    K, N, S = 6912, 32, 64
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_delta(pos, neg, K, 8, rows=1)
    assert w.info["delta_bits"] == 16 and w.info["row_bytes"] == 0  # sorted order: nothing to schedule
    X = oracle.make_x_i8(5, 1, K)
    assert (w.matmul(X) == oracle.sptmm_i8(X, pos, neg)).all()
    w.free()


@pytest.mark.parametrize("count", [1, 3, 32, 40])
def test_batched_launch_equals_single_launches(count):
    K, N, S, split = 6912, 2560, 4096, 32
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_delta(pos, neg, K, split, rows=1)
    ws = [w] + [w.clone() for _ in range(min(count, 4) - 1)]
    ws = [ws[i % len(ws)] for i in range(count)]
    st = sp.Stream()
    Xs = [oracle.make_x_i8(100 + i, 1, K) for i in range(count)]
    xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
    cb = [sp.DeviceBuffer(4 * N) for _ in range(count)]
    say("byte rows batched", count)
    sp.gemv_i8_batched(ws, xb, cb, 1, st)
    st.sync()
    for i in range(count):
        assert (cb[i].to_numpy(np.int32, (1, N)) == oracle.sptmm_i8_mt(Xs[i], pos, neg, 8)).all(), i
    # a plain stream of the same shape does not mix with it in one launch
    if count >= 2:
        plain = sp.Weights.upload_delta(pos, neg, K, split)
        with pytest.raises(sp.SptmmError):
            sp.gemv_i8_batched([w, plain], xb[:2], cb[:2], 1, st)
    for o in xb + cb:
        o.free()


def special_matrix(K, N):
    """Columns that stress the padding rules: empty, one sign only, single entries at both ends, full."""
    rng = np.random.default_rng(3)
    W = rng.choice(np.array([-1, 0, 1], np.int8), size=(N, K), p=[0.3, 0.4, 0.3])
    W[0] = 0
    W[1] = 0
    W[1, 0] = 1
    W[2] = 0
    W[2, K - 1] = -1
    W[3] = 1
    W[4] = -1
    W[5] = 0
    W[5, ::2] = 1
    return np.ascontiguousarray(W)


@pytest.mark.parametrize("split", [8, 16, 32, 64])
def test_ragged_matrices(split):
    for K, N, W in ((2560, 640, sp.generate_ternary_iid(2560, 640, 0xABCD, 0.3, 0.3)), (6912, 256, sp.generate_ternary_iid(6912, 256, 7, 0.4, 0.2)),
                    (512, 64, special_matrix(512, 64))):
        w = sp.Weights.upload_dense(W, DELTA, split, rows=1)
        bits = w.info["delta_bits"]
        assert w.info["row_bytes"] == (1 if bits == 8 else 0) and w.info["ragged"] == 1
        for M in (1, 4):
            say("byte rows ragged", K, N, "split", split, "bits", bits, "M", M)
            X = oracle.make_x_i8(17 + M, M, K)
            assert (w.matmul(X) == oracle.dense_i8(X, W)).all()
        w.free()


def test_weight_file_keeps_the_schedule(tmp_path):
    K, N, S, split = 2560, 640, 1536, 16
    _, pos, neg = sp.generate_ternary(K, N, S)
    X = oracle.make_x_i8(9, 1, K)
    want = oracle.sptmm_i8(X, pos, neg)
    for rows in (0, 1):
        w = sp.Weights.upload_delta(pos, neg, K, split, rows=rows)
        path = str(tmp_path / ("rows%d.sptmm" % rows))
        w.save(path)
        w2 = sp.Weights.load(path)
        assert w2.info == w.info and w2.info["row_bytes"] == (1 if rows == 1 else 4)
        assert (w2.matmul(X) == want).all()
        w.free()
        w2.free()


def test_quantising_gemv_takes_the_stream_too():
    K, N, S, split = 2560, 640, 1536, 32
    _, pos, neg = sp.generate_ternary(K, N, S)
    rng = np.random.default_rng(4)
    X = rng.standard_normal((1, K)).astype(np.float16)
    a = sp.Weights.upload_delta(pos, neg, K, split, rows=1)
    b = sp.Weights.upload_delta(pos, neg, K, split)
    ya, yb = a.matmul_q8(X, w_scale=0.05), b.matmul_q8(X, w_scale=0.05)
    assert ya.dtype == np.float32 and (ya == yb).all()
    a.free()
    b.free()
