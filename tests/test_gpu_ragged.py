"""GPU parity of the ragged streams (columns that differ in nonzeros), through the C ABI.

Oracle: the dense int8 matmul of the CPU oracle on the same matrix (int32, bit-exact);
float activations against a float64 product with tolerance
    |got - ref| <= 1e-3 * max(|ref|, sqrt(nnz per column)).
"""
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu
U16, DELTA, I2S = sp.KIND_U16, sp.KIND_DELTA, sp.KIND_I2S


@pytest.fixture(scope="module", autouse=True)
def device():
    return sp.device_init(0)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def special_matrix(K, N):
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
    W[6, : K // 2] = 0
    W[7, K // 2:] = 0
    return np.ascontiguousarray(W)


@pytest.mark.parametrize("kind,splits", [(U16, (8, 16, 32, 64, 128, 256)), (DELTA, (8, 16, 32, 64))])
@pytest.mark.parametrize("K,N,pp,pn", [(2560, 640, 0.3, 0.3), (6912, 256, 0.35, 0.25), (256, 16, 0.3, 0.3)])
def test_iid_matrix_bit_exact(kind, splits, K, N, pp, pn):
    W = sp.generate_ternary_iid(K, N, 0xABCD, pp, pn)
    for M in (1, 4, 8):
        X = oracle.make_x_i8(17 + M, M, K)
        want = oracle.dense_i8(X, W)
        for split in splits:
            say("ragged iid", kind, K, N, "split", split, "M", M)
            w = sp.Weights.upload_dense(W, kind, split)
            i = w.info
            assert i["ragged"] == 1 and i["nnz"] == int((W != 0).sum()) and i["stream_bytes"] <= w.nbytes
            got = w.matmul(X)
            w.free()
            assert got.dtype == np.int32 and (got == want).all()


@pytest.mark.parametrize("kind,split", [(U16, 8), (U16, 32), (U16, 64), (U16, 256), (DELTA, 16), (DELTA, 32), (DELTA, 64)])
def test_special_columns_bit_exact(kind, split):
    K, N = 1024, 32
    W = special_matrix(K, N)
    say("ragged special", kind, split)
    w = sp.Weights.upload_dense(W, kind, split)
    for M in (1, 3):
        X = oracle.make_x_i8(5 + M, M, K)
        assert (w.matmul(X) == oracle.dense_i8(X, W)).all()
    ones = np.ones((1, K), np.int8)
    got = w.matmul(ones)[0]
    assert (got == W.astype(np.int32).sum(1)).all()  # +1 count minus -1 count per column
    w.free()


def test_all_zero_and_sparse_16_bit():
    K, N = 6912, 32
    Z = np.zeros((N, K), np.int8)
    X = oracle.make_x_i8(3, 2, K)
    for kind in (U16, DELTA):
        say("ragged zero matrix", kind)
        w = sp.Weights.upload_dense(Z, kind, 32)
        assert (w.matmul(X) == 0).all()
        w.free()
    S = sp.generate_ternary_iid(K, N, 5, 0.01, 0.01)
    say("ragged sparse 16-bit gaps")
    w = sp.Weights.upload_dense(S, DELTA, 32)
    assert w.info["delta_bits"] == 16
    assert (w.matmul(X) == oracle.dense_i8(X, S)).all()
    w.free()


def test_balanced_matrix_agrees_with_the_balanced_streams():
    """A matrix with exactly S/2 per sign and column gives the same output through either builder."""
    K, N, S = 2560, 640, 1536
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    X = oracle.make_x_i8(99, 4, K)
    say("ragged vs balanced")
    a = sp.Weights.upload_u16(pos, neg, K, 32)
    want = a.matmul(X)
    a.free()
    for kind in (U16, DELTA, I2S):
        b = sp.Weights.upload_dense(W, kind, 32)
        assert (b.matmul(X) == want).all()
        b.free()


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("kind", [U16, DELTA])
def test_float_activations(dtype, kind):
    K, N = 2560, 640
    W = sp.generate_ternary_iid(K, N, 0x51, 0.3, 0.3)
    for M in (1, 4):
        X = oracle.make_x_normal(1000 + M, M, K, dtype)
        ref = X.astype(np.float64) @ W.T.astype(np.float64)
        say("ragged float", dtype.__name__, kind, "M", M)
        w = sp.Weights.upload_dense(W, kind, 32)
        got = w.matmul(X)
        w.free()
        scale = np.maximum(np.abs(ref), np.sqrt((W != 0).sum(1))[None, :])
        assert (np.abs(got - ref) / scale).max() <= 1e-3


def test_full_size_iid_layer_and_batched_launch():
    """BitNet-sized down projection with iid entries; linearity at full size; batched = single launches."""
    K, N = 6912, 2560
    W = sp.generate_ternary_iid(K, N, 0x2B, 0.3, 0.3)
    X = oracle.make_x_i8(41, 1, K)
    want = oracle.dense_i8(X, W)
    for kind in (U16, DELTA):
        say("ragged full size", kind)
        w = sp.Weights.upload_dense(W, kind, 32)
        got = w.matmul(X)
        assert (got == want).all()
        assert (w.matmul((2 * (X // 2)).astype(np.int8)) == 2 * w.matmul((X // 2).astype(np.int8))).all()
        ws = [w, w.clone(), w.clone()]
        xs = [sp.DeviceBuffer.from_numpy(oracle.make_x_i8(50 + i, 1, K)) for i in range(3)]
        cs = [sp.DeviceBuffer(4 * N) for _ in range(3)]
        sp.gemv_i8_batched(ws, xs, cs, 1)
        sp.device_sync()
        for i in range(3):
            assert (cs[i].to_numpy(np.int32, (1, N)) == oracle.dense_i8(oracle.make_x_i8(50 + i, 1, K), W)).all()
        for b in xs + cs:
            b.free()
        for v in ws:
            v.free()


def test_outputs_match_golden_fixture(golden_dir):
    """The committed vectors come from a numpy restatement of generator and product that shares no code
    with the library or the oracle (tests/golden/make_golden.py)."""
    import hashlib
    import json
    import os

    for e in json.load(open(os.path.join(golden_dir, "generator_kats.json")))["iid_matrices"]:
        W = sp.generate_ternary_iid(e["K"], e["N"], e["seed"], e["p_pos"], e["p_neg"])
        X = sp.make_x_i8(e["x_seed"], e["M"], e["K"])
        for kind in (U16, DELTA):
            say("ragged golden", e["K"], e["N"], kind)
            w = sp.Weights.upload_dense(W, kind, 32)
            got = w.matmul(X)
            w.free()
            assert got[0, :8].tolist() == e["C_head"]
            assert hashlib.sha256(got.tobytes()).hexdigest() == e["sha256_C"]


@pytest.mark.parametrize("K,N,S,split", [(6912, 2560, 1728, 16), (2560, 640, 1536, 32), (2560, 640, 1536, 8)])
def test_ragged_stream_with_tasks_of_one_length(K, N, S, split):
    """A balanced matrix packed from its dense form is a ragged stream whose tasks all have one length; behind its count
    table it is laid out like the stream of balanced lists, and the launch takes the kernels for tasks of one length.
    Same results as the balanced stream and the oracle: u16 lists, gap streams for four-byte and one-byte rows, one
    row, a four-row and an eight-row tile, alone and in a batched launch."""
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    for M in (1, 4, 8):
        X = oracle.make_x_i8(30 + M, M, K)
        ref = oracle.sptmm_i8_mt(X, pos, neg, 8)
        for kind, rows in ((sp.KIND_U16, 0), (sp.KIND_DELTA, 0), (sp.KIND_DELTA, 1)):
            say("uniform ragged", K, N, S, split, "M", M, "kind", kind, "rows", rows)
            w = sp.Weights.upload_dense(W, kind, split, rows=rows)
            assert w.info["ragged"] == 1 and w.info["stones"] == 0
            assert np.array_equal(w.matmul(X), ref)
            xb = [sp.DeviceBuffer.from_numpy(X) for _ in range(8)]
            cb = [sp.DeviceBuffer(4 * M * N) for _ in range(8)]
            sp.gemv_batched([w] * 8, xb, cb, M, 0)
            sp.device_sync()
            for c in cb:
                assert np.array_equal(c.to_numpy(np.int32, (M, N)), ref)
            for o in [w] + xb + cb:
                o.free()
    Xh = oracle.make_x_normal(77, 4, K, np.float16)
    w = sp.Weights.upload_dense(W, sp.KIND_DELTA, split)
    got = w.matmul(Xh)
    w.free()
    ref = oracle.sptmm_f64(Xh, pos, neg)
    assert np.abs(got - ref).max() <= 1e-3 * max(1.0, np.abs(ref).max())
