"""GPU parity of the wide streams (K-tiled, 16 int8 / 8 fp16 rows per tile) through the C ABI.

int8: bit-exact against the oracle's dense int8 product.  fp16: max |got - ref| <= 1e-3 * max(|ref|, sqrt(nnz per
column)) against a float64 product of the same matrix."""
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu
REL_TOL = 1e-3


@pytest.fixture(scope="module", autouse=True)
def device():
    return sp.device_init(0)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def check_fp(got, X, W):
    ref = X.astype(np.float64) @ W.astype(np.float64).T
    scale = np.maximum(np.abs(ref), np.sqrt(np.maximum((W != 0).sum(axis=1), 1))[None, :])
    err = np.abs(got.astype(np.float64) - ref) / scale
    assert err.max() <= REL_TOL, "max rel err %.3e" % err.max()


@pytest.mark.parametrize("kind", [sp.KIND_U16, sp.KIND_DELTA])
@pytest.mark.parametrize("split", [8, 16, 32, 64])
def test_small_matrix_every_split_and_row_count(kind, split):
    K, N = 2560, 640
    W = sp.generate_ternary_iid(K, N, 11, 0.3, 0.3)
    w = sp.Weights.upload_wide(W, kind, split)
    assert w.info["k_tile"] == 2560 and w.info["ragged"] == 1
    for M in (1, 3, 8, 9, 16, 17, 33):
        say("wide", kind, "split", split, "M", M)
        X = oracle.make_x_i8(600 + M, M, K)
        assert (w.matmul(X) == oracle.dense_i8(X, W)).all(), M
    for M in (1, 5, 8, 9):
        say("wide fp16", kind, "split", split, "M", M)
        Xh = oracle.make_x_normal(700 + M, M, K, np.float16)
        check_fp(w.matmul(Xh), Xh, W)
    w.free()


@pytest.mark.parametrize("kind", [sp.KIND_U16, sp.KIND_DELTA])
def test_config4_shape_two_k_tiles(kind):
    """K = 13824: a 16-row tile of the whole K does not fit the LDS; the stream comes in two K-tiles of 6912 rows."""
    K, N, S = 13824, 5120, 8320
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    w = sp.Weights.upload_wide(W, kind, 32)
    assert w.info["k_tile"] == 6912
    if kind == sp.KIND_DELTA:
        assert w.info["delta_bits"] == 8
    say("wide cfg4", kind, "stream bytes", w.info["stream_bytes"], "of", w.nbytes)
    assert w.info["stream_bytes"] <= 1.06 * (2 if kind == sp.KIND_U16 else 1) * S * N + 2 * 256 * (N // 2 if kind == sp.KIND_DELTA else 0) + 65536
    for M in (16, 8, 1, 20):
        say("wide cfg4", kind, "M", M)
        X = oracle.make_x_i8(4000 + M, M, K)
        assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), M
    Xh = oracle.make_x_normal(3, 8, K, np.float16)
    say("wide cfg4 fp16")
    check_fp(w.matmul(Xh), Xh, W)
    w.free()


@pytest.mark.parametrize("K,N,pp,pn,split", [(64, 16, 0.3, 0.3, 8), (512, 48, 0.5, 0.5, 16), (4096, 32, 0.012, 0.012, 16), (2560, 64, 0.0, 0.0, 32),
                                             (20480, 32, 0.3, 0.2, 64), (40960, 16, 0.1, 0.1, 32)])
def test_odd_shapes_sparse_and_many_k_tiles(K, N, pp, pn, split):
    W = sp.generate_ternary_iid(K, N, K + N, pp, pn)
    for kind in (sp.KIND_U16, sp.KIND_DELTA):
        w = sp.Weights.upload_wide(W, kind, split)
        say("wide odd", K, N, kind, "k_tile", w.info["k_tile"], "bits", w.info["delta_bits"])
        for M in (1, 16, 11):
            X = oracle.make_x_i8(K + M, M, K)
            assert (w.matmul(X) == oracle.dense_i8(X, W)).all(), (kind, M)
        Xh = oracle.make_x_normal(K, 8, K, np.float16)
        check_fp(w.matmul(Xh), Xh, W)
        w.free()


@pytest.mark.parametrize("kind", [sp.KIND_U16, sp.KIND_DELTA])
def test_batched_launch_equals_single_launches(kind):
    K, N = 2560, 640
    W = sp.generate_ternary_iid(K, N, 3, 0.3, 0.3)
    base = sp.Weights.upload_wide(W, kind, 32)
    for M, count, dtype, act in ((16, 5, np.int8, 0), (9, 40, np.int8, 0), (8, 3, np.float16, 1)):
        ws = [base] + [base.clone() for _ in range(count - 1)]
        Xs = [oracle.make_x_i8(50 + i, M, K) if dtype == np.int8 else oracle.make_x_normal(50 + i, M, K, np.float16) for i in range(count)]
        xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
        cb = [sp.DeviceBuffer(4 * M * N) for _ in range(count)]
        for c in cb:
            c.fill(0xFF)
        say("wide batched", kind, "M", M, "count", count, dtype.__name__)
        sp.gemv_batched(ws, xb, cb, M, act)
        sp.device_sync()
        for i in range(count):
            if dtype == np.int8:
                assert (cb[i].to_numpy(np.int32, (M, N)) == oracle.dense_i8(Xs[i], W)).all(), i
            else:
                got = cb[i].to_numpy(np.float32, (M, N))
                check_fp(got, Xs[i], W)
                assert (got == base.matmul(Xs[i])).all()
        for o in ws[1:] + xb + cb:
            o.free()
    base.free()


@pytest.mark.parametrize("bad", [np.inf, np.nan])
def test_non_finite_fp16_row_stays_in_its_row_and_columns(bad):
    K, N = 2560, 640
    W = sp.generate_ternary_iid(K, N, 21, 0.3, 0.3)
    for kind in (sp.KIND_U16, sp.KIND_DELTA):
        w = sp.Weights.upload_wide(W, kind, 16)
        for k in (0, 1337, K - 1):
            say("wide non-finite", kind, k, bad)
            X = oracle.make_x_normal(k, 8, K, np.float16)
            X[2, k] = bad
            clean = X.copy()
            clean[2, k] = 0
            got = w.matmul(X)
            away = W[:, k] == 0
            assert 0 < away.sum() < N
            rows = [0, 1, 3, 4, 5, 6, 7]
            assert np.isfinite(got[rows]).all() and np.isfinite(got[2, away]).all()
            check_fp(got[rows], clean[rows], W)
            check_fp(got[2:3, away], clean[2:3], W[away])
            assert (~np.isfinite(got[2, ~away])).all()
        w.free()


@pytest.mark.parametrize("bad", [np.inf, np.nan])
def test_non_finite_value_in_one_k_tile_only(bad):
    """Two K-tiles (K = 13824 -> 2 x 6912) whose finiteness differs: the tile with the Inf / NaN is summed on the vector
    unit, the other on the matrix unit, and the two write the same outputs from different lanes of the wavefront.  The
    second tile's sums are added to what the first stored, whichever path each took."""
    K, N = 13824, 320
    W = sp.generate_ternary_iid(K, N, 33, 0.3, 0.3)
    for kind in (sp.KIND_U16, sp.KIND_DELTA):
        w = sp.Weights.upload_wide(W, kind, 32)
        assert w.info["k_tile"] == 6912
        for k in (5, 6911, 6912, 13823):  # first tile only, then second tile only
            say("wide non-finite, one K-tile", kind, k, bad)
            X = oracle.make_x_normal(k, 8, K, np.float16)
            X[5, k] = bad
            clean = X.copy()
            clean[5, k] = 0
            got = w.matmul(X)
            away = W[:, k] == 0
            assert 0 < away.sum() < N
            rows = [0, 1, 2, 3, 4, 6, 7]
            assert np.isfinite(got[rows]).all() and np.isfinite(got[5, away]).all()
            check_fp(got[rows], clean[rows], W)
            check_fp(got[5:6, away], clean[5:6], W[away])
            assert (~np.isfinite(got[5, ~away])).all()
        w.free()


def test_uploads_that_declare_more_than_eight_rows_build_wide_streams():
    """The _rows upload calls build the stream for the rows a call will bring: beyond eight, a wide stream (the lists read
    once for up to 16 rows); up to eight, the ordinary one.  Whichever it is, the sums are the oracle's at any M."""
    K, N, S = 2560, 640, 1536
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    made = {
        "u16 rows=16": sp.Weights.upload_u16(pos, neg, K, 0, rows=16),
        "u16 rows=9, split 32": sp.Weights.upload_u16(pos, neg, K, 32, rows=9),
        "delta rows=16": sp.Weights.upload_delta(pos, neg, K, 0, rows=16),
        "dense u16 rows=12": sp.Weights.upload_dense(W, sp.KIND_U16, 0, rows=12),
        "dense delta rows=16": sp.Weights.upload_dense(W, sp.KIND_DELTA, 16, rows=16),
        "u16 rows=8": sp.Weights.upload_u16(pos, neg, K, 0, rows=8),
        "delta rows=8": sp.Weights.upload_delta(pos, neg, K, 0, rows=8),
        "u16 rows=16, split 128": sp.Weights.upload_u16(pos, neg, K, 128, rows=16),  # wide streams stop at 64 lanes per column
    }
    for name, w in made.items():
        wide = "rows=8" not in name and "split 128" not in name
        say("declared rows:", name, "k_tile", w.info["k_tile"])
        assert (w.info["k_tile"] != 0) == wide, name
        if wide and "dense" not in name:
            assert w.info["S"] == S
        for M in (1, 9, 16):
            X = oracle.make_x_i8(M, M, K)
            assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), (name, M)
        w.free()


def test_refusals():
    K, N = 512, 48
    W = sp.generate_ternary_iid(K, N, 1, 0.3, 0.3)
    w = sp.Weights.upload_wide(W, sp.KIND_U16, 32)
    xb = sp.DeviceBuffer(4 * K)
    cb = sp.DeviceBuffer(4 * N)
    with pytest.raises(sp.SptmmError) as e:
        w.gemv_f32(xb, 1, cb)
    assert e.value.code == -2
    with pytest.raises(sp.SptmmError) as e:
        w.gemv_q8(xb, 1, 1, 1.0, cb)
    assert e.value.code == -2
    with pytest.raises(sp.SptmmError):
        sp.Weights.upload_wide(W, sp.KIND_I2S, 32)
    with pytest.raises(sp.SptmmError) as e:
        sp.Weights.upload_wide(W, sp.KIND_U16, 128)  # wide streams take split_k up to 64; an explicit larger one is refused, not clamped
    assert e.value.code == -1
    for o in (w, xb, cb):
        o.free()
