"""GPU parity of 8-bit gap streams of sparse matrices: gaps of more than 127 rows walked over zero slots of the tile.

The reference's default flags (-K 3072 -S 256: 8 % nonzeros, main.cu:38-49) are such a matrix; its delta kernel narrows
every gap to a byte without a check (main.cu:376-394).  Here the activation tile keeps 16 zero slots behind every 96
rows, the stream holds tile positions, and a long gap becomes several entries of which all but the last add nothing.
Oracle: the dense int8 product (bit-exact); float rows within
    |got - ref| <= 1e-3 * max(|ref|, sqrt(nonzeros of the column))
of the float64 product.
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


def sparse_matrix(K, N, seed, p):
    W = sp.generate_ternary_iid(K, N, seed, p, p)
    W[0] = 0              # an empty column
    W[1] = 0
    W[1, K - 1] = 1       # one entry at the far end of the tile
    W[2] = 0
    W[2, 0] = -1          # one at the near end
    W[3] = 0
    W[3, 95::96] = 1      # the last row in front of every block of zero slots
    return np.ascontiguousarray(W)


@pytest.mark.parametrize("K,N,p,splits", [
    (6912, 256, 0.03, (8, 16, 32)),    # headline K
    (3072, 768, 0.0417, (8, 16)),      # the reference's default shape and density
    (13824, 64, 0.02, (16, 64)),       # 144 blocks; eight-row tile of 129 KB
    (2560, 48, 0.03, (8, 64)),         # a partial last block; 64 lanes per column: two or three entries per lane, as many zero slots
    (256, 16, 0.02, (8,)),             # three blocks, the last one partial
])
def test_sparse_matrix_bit_exact_at_every_m(K, N, p, splits):
    W = sparse_matrix(K, N, 0x5EED, p)
    for split in splits:
        for rows in (0, 1):
            w = sp.Weights.upload_dense(W, DELTA, split, rows=rows)
            i = w.info
            assert i["delta_bits"] == 8 and i["stones"] == 1, "this matrix was picked to need the zero slots"
            assert i["row_bytes"] == (1 if rows == 1 else 4) and i["nnz"] == int((W != 0).sum())
            for M in (1, 3, 4, 8, 9):
                say("sparse", K, N, p, "split", split, "rows", rows, "M", M)
                X = oracle.make_x_i8(7 + M, M, K)
                assert (w.matmul(X) == oracle.dense_i8(X, W)).all(), (split, rows, M)
            for X in (np.full((1, K), 127, np.int8), np.full((2, K), -128, np.int8)):
                assert (w.matmul(X) == oracle.dense_i8(X, W)).all()
            w.free()


def test_forced_byte_gaps_where_16_bits_would_be_chosen():
    K, N = 6912, 32
    W = sparse_matrix(K, N, 5, 0.01)
    auto = sp.Weights.upload_dense(W, DELTA, 32)
    assert auto.info["delta_bits"] == 16 and auto.info["stones"] == 0
    X = oracle.make_x_i8(3, 2, K)
    want = oracle.dense_i8(X, W)
    assert (auto.matmul(X) == want).all()
    auto.free()
    packed, inf = sp.pack_ragged(W, DELTA, 32, bits=8)
    assert inf["bits"] == 8 and (sp.unpack_ragged(packed, K, N, DELTA, 32, 8) == W).all()


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_float_rows(dtype):
    K, N = 6912, 128
    W = sparse_matrix(K, N, 0x51, 0.04)
    w = sp.Weights.upload_dense(W, DELTA, 16)
    assert w.info["stones"] == 1
    for M in (1, 4, 6):
        say("sparse float", dtype.__name__, "M", M)
        X = oracle.make_x_normal(1000 + M, M, K, dtype)
        ref = X.astype(np.float64) @ W.T.astype(np.float64)
        got = w.matmul(X)
        scale = np.maximum(np.abs(ref), np.sqrt(np.maximum((W != 0).sum(1), 1))[None, :])
        assert (np.abs(got - ref) / scale).max() <= 1e-3
    # a row holding Inf / NaN: the zero slots stay zero, and only columns that gather the row see it
    X = oracle.make_x_normal(5, 4, K, np.float16) if dtype == np.float16 else None
    if X is not None:
        X[2, 17] = np.inf
        got = w.matmul(X)
        with np.errstate(invalid="ignore"):
            ref = X.astype(np.float64) @ W.T.astype(np.float64)
        hit = W[:, 17] != 0
        assert np.isinf(got[2, hit]).all() and np.isfinite(got[2, ~hit]).all() and np.isfinite(got[[0, 1, 3]]).all()
        assert np.isfinite(ref[[0, 1, 3]]).all()
    w.free()


def test_quantising_gemv_batched_launch_and_weight_file(tmp_path):
    K, N = 6912, 256
    W = sparse_matrix(K, N, 0x77, 0.04)
    a = sp.Weights.upload_dense(W, DELTA, 16, rows=1)
    b = sp.Weights.upload_dense(W, sp.KIND_U16, 16)
    assert a.info["stones"] == 1 and a.info["stream_bytes"] < 0.65 * b.info["stream_bytes"]
    rng = np.random.default_rng(4)
    Xh = rng.standard_normal((3, K)).astype(np.float16)
    say("sparse q8")
    assert (a.matmul_q8(Xh, w_scale=0.05) == b.matmul_q8(Xh, w_scale=0.05)).all()
    # batched launch = single launches; a plain stream of the same shape does not mix with it
    count = 5
    ws = [a, a.clone(), a.clone(), a, a.clone()]
    Xs = [oracle.make_x_i8(100 + i, 1, K) for i in range(count)]
    xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
    cb = [sp.DeviceBuffer(4 * N) for _ in range(count)]
    st = sp.Stream()
    say("sparse batched")
    sp.gemv_i8_batched(ws, xb, cb, 1, st)
    st.sync()
    for i in range(count):
        assert (cb[i].to_numpy(np.int32, (1, N)) == oracle.dense_i8(Xs[i], W)).all(), i
    dense = sp.Weights.upload_dense(sp.generate_ternary_iid(K, N, 1, 0.3, 0.3), DELTA, 16, rows=1)
    assert dense.info["stones"] == 0
    with pytest.raises(sp.SptmmError):
        sp.gemv_i8_batched([a, dense], xb[:2], cb[:2], 1, st)
    # weight file: the stream says itself that it holds positions
    path = str(tmp_path / "sparse.sptmm")
    a.save(path)
    c = sp.Weights.load(path)
    assert c.info == a.info
    X = oracle.make_x_i8(9, 4, K)
    say("sparse weight file")
    assert (c.matmul(X) == oracle.dense_i8(X, W)).all()
    for o in xb + cb:
        o.free()
