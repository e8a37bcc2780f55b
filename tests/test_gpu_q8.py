"""GPU parity of the fused quantise -> GEMV -> rescale entry point (sptmm_gemv_q8).

Reference arithmetic, restated in numpy float32 (oracle.quantise_rows / oracle.rescale) exactly as
include/sptmm.h states it:
    a_m = max(max_k |x[m][k]|, 1e-5);  s_m = 127 / a_m;  q = clip(rint(x * s_m), -127, 127)   (round-half-even)
    C = q . W  (exact int32: the CPU oracle's sums);  y = float(C) * (a_m / 127) * w_scale
Every step is a single correctly rounded float32 operation, so the result must match bit for bit; the
test also pins q itself through sptmm_gemv_i8 on the same q.
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


bf16_bits, quantise_ref, y_ref = oracle.bf16_bits, oracle.quantise_rows, oracle.rescale


def rows(seed, M, K, dtype):
    x = oracle.make_x_normal(seed, M, K, np.float32)
    x[:, ::7] *= 3.0  # a few outliers, as activations have
    if dtype == "bf16":
        bits = bf16_bits(x)
        return bits, (bits.astype(np.uint32) << 16).view(np.float32)
    h = x.astype(np.float16)
    return h, h.astype(np.float32)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("enc,split", [("u16", 32), ("u16", 8), ("u16", 128), ("delta", 32), ("delta", 16)])
def test_q8_balanced_matrix_bit_exact(enc, split, dtype):
    K, N, S = 2560, 640, 1536
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, split) if enc == "u16" else sp.Weights.upload_delta(pos, neg, K, split)
    for M in (1, 3, 4, 8):
        print("q8", enc, split, dtype, "M", M, flush=True)
        sys.stdout.flush()
        X, xf = rows(100 + M, M, K, dtype)
        q, a = quantise_ref(xf)
        C = oracle.sptmm_i8(q, pos, neg)
        assert (w.matmul(q) == C).all()
        got = w.matmul_q8(X, w_scale=0.0371, bf16=dtype == "bf16")
        want = y_ref(C, a, 0.0371)
        assert got.dtype == np.float32 and (got == want).all(), np.abs(got - want).max()
    w.free()


@pytest.mark.parametrize("kind", [sp.KIND_U16, sp.KIND_DELTA])
def test_q8_ragged_headline_sized(kind):
    K, N = 6912, 2560
    W = sp.generate_ternary_iid(K, N, 0x77, 0.3, 0.3)
    w = sp.Weights.upload_dense(W, kind, 32)
    for M in (1, 4):
        print("q8 ragged", kind, "M", M, flush=True)
        sys.stdout.flush()
        X, xf = rows(7 + M, M, K, "f16")
        q, a = quantise_ref(xf)
        C = oracle.dense_i8(q, W)
        got = w.matmul_q8(X, w_scale=1.0)
        assert (got == y_ref(C, a, 1.0)).all()
    w.free()


def test_q8_large_k_multi_pass_staging_and_edge_rows():
    """K = 13824: a thread stages several items; rows of zeros (scale clamps at 1e-5), a row whose
    maximum sits in the last element, exact .5 cases (round-half-even)."""
    K, N, S = 13824, 64, 8320
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, 64)
    x = np.zeros((4, K), np.float32)
    x[1, :] = 0.25
    x[1, K - 1] = -127.0          # s = 1 exactly: q = rint(x): 0.25 -> 0
    x[2, :] = np.tile(np.array([0.5, 1.5, 2.5, -0.5, -1.5, 127.0], np.float32), K // 6)  # ties go to even
    x[3, :] = oracle.make_x_normal(3, 1, K, np.float32)[0] * 1e-3
    X = x.astype(np.float16)
    xf = X.astype(np.float32)
    q, a = quantise_ref(xf)
    assert (q[0] == 0).all() and q[1, K - 1] == -127 and set(np.unique(q[2])) <= {0, 2, -2, 127}
    C = oracle.sptmm_i8(q, pos, neg)
    got = w.matmul_q8(X, w_scale=2.0)
    assert (got == y_ref(C, a, 2.0)).all()
    assert (got[0] == 0).all()
    w.free()


def test_q8_argument_errors():
    K, N, S = 256, 16, 64
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    w = sp.Weights.upload_u16(pos, neg, K, 8)
    xb = sp.DeviceBuffer(2 * K)
    yb = sp.DeviceBuffer(4 * N)
    with pytest.raises(sp.SptmmError):
        w.gemv_q8(xb, 0, 1, 1.0, yb)
    with pytest.raises(sp.SptmmError):
        w.gemv_q8(xb, 1, 0, 1.0, yb)
    i = sp.Weights.upload_i2s(W)
    with pytest.raises(sp.SptmmError):
        i.gemv_q8(xb, 1, 1, 1.0, yb)
    for o in (w, i):
        o.free()
    xb.free()
    yb.free()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_q8_with_a_workspace_is_the_same_arithmetic(dtype):
    """sptmm_gemv_q8_ws: beyond four rows the rows are quantised once by a launch of their own and the int8 GEMV scales its
    sums on the way out; up to four rows it is the fused launch.  Either way the floats are the fused call's, bit for bit,
    and the float32 arithmetic's around the oracle's integer sums -- balanced and ragged streams, every lanes-per-column
    case of the eight-row tiles, row counts that leave the last tile partly filled."""
    K, N, S = 2560, 640, 1536
    Wd, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    ragged = sp.generate_ternary_iid(K, N, 0x99, 0.25, 0.35)
    streams = [("u16 %d" % sk, sp.Weights.upload_u16(pos, neg, K, sk), None) for sk in (8, 16, 32, 64, 128)]
    streams += [("gap %d" % sk, sp.Weights.upload_delta(pos, neg, K, sk), None) for sk in (8, 32, 64)]
    streams += [("gap for one row", sp.Weights.upload_delta(pos, neg, K, 32, rows=1), None)]
    streams += [("ragged u16", sp.Weights.upload_dense(ragged, sp.KIND_U16, 32), ragged), ("ragged gap", sp.Weights.upload_dense(ragged, sp.KIND_DELTA, 16), ragged)]
    try:
        for name, w, dense in streams:
            for M in (1, 4, 5, 8, 9, 13, 16, 20):
                print("q8 workspace", name, dtype, "M", M, flush=True)
                sys.stdout.flush()
                X, xf = rows(300 + M, M, K, dtype)
                if M >= 9:
                    xf[M - 1] = 0  # a row of zeros: its scale clamps at 1e-5
                    X[M - 1] = 0
                q, a = quantise_ref(xf)
                C = oracle.sptmm_i8_mt(q, pos, neg, 8) if dense is None else oracle.dense_i8(q, dense)
                want = y_ref(C, a, 0.25)
                got = w.matmul_q8(X, w_scale=0.25, bf16=dtype == "bf16", workspace=True)
                assert (got == want).all(), (name, M, np.abs(got - want).max())
                assert (got == w.matmul_q8(X, w_scale=0.25, bf16=dtype == "bf16")).all(), (name, M)
    finally:
        for _, w, _ in streams:
            w.free()


def test_q8_workspace_is_checked_and_reusable():
    K, N, S = 6912, 2560, 4096
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, 32)
    i2 = sp.Weights.upload_i2s(sp.generate_ternary(256, 32, 64, dense=True)[0])
    M = 8
    need = w.q8_workspace_bytes(M)
    assert need >= M * K + 4 * M and need % 256 == 0 and w.q8_workspace_bytes(16) > need
    ws = sp.DeviceBuffer(need)
    yb = sp.DeviceBuffer(4 * M * N)
    st = sp.Stream()
    try:
        for seed in (1, 2, 3):  # one workspace, call after call on one stream
            X, xf = rows(seed, M, K, "f16")
            xb = sp.DeviceBuffer.from_numpy(X)
            w.gemv_q8_ws(xb, 1, M, 1.0, yb, ws, need, st)
            st.sync()
            q, a = quantise_ref(xf)
            assert (yb.to_numpy(np.float32, (M, N)) == y_ref(oracle.sptmm_i8_mt(q, pos, neg, 8), a, 1.0)).all()
            xb.free()
        X, _ = rows(9, M, K, "f16")
        xb = sp.DeviceBuffer.from_numpy(X)
        for bad in (lambda: w.gemv_q8_ws(xb, 1, M, 1.0, yb, ws, need - 1, st), lambda: w.gemv_q8_ws(xb, 1, M, 1.0, yb, None, need, st),
                    lambda: w.gemv_q8_ws(xb, 3, M, 1.0, yb, ws, need, st), lambda: i2.gemv_q8_ws(xb, 1, M, 1.0, yb, ws, need, st)):
            with pytest.raises(sp.SptmmError):
                bad()
        w.gemv_q8_ws(xb, 1, 4, 1.0, yb, None, 0, st)  # up to four rows: the fused launch, no workspace needed
        st.sync()
        xb.free()
    finally:
        for o in (ws, yb, w, i2):
            o.free()


def test_q8_workspace_with_few_rows_of_a_long_k():
    """Two to four rows of more than 32 K values go the two-launch way as well (four-row int8 tiles scaling their sums on
    the way out); one row never does."""
    K, N, S = 13824, 1280, 8320
    _, pos, neg = sp.generate_ternary(K, N, S)
    for name, w in (("u16", sp.Weights.upload_u16(pos, neg, K, 0)), ("gap", sp.Weights.upload_delta(pos, neg, K, 0)), ("u16 64", sp.Weights.upload_u16(pos, neg, K, 64))):
        for M in (1, 2, 3, 4):
            print("q8 workspace, long K", name, "M", M, flush=True)
            sys.stdout.flush()
            X, xf = rows(500 + M, M, K, "f16")
            q, a = quantise_ref(xf)
            want = y_ref(oracle.sptmm_i8_mt(q, pos, neg, 8), a, 2.0)
            assert (w.matmul_q8(X, w_scale=2.0, workspace=True) == want).all(), (name, M)
            assert (w.matmul_q8(X, w_scale=2.0) == want).all(), (name, M)
        w.free()


def test_int8_rows_with_their_scales_go_through_one_launch():
    """sptmm_gemv_i8_scaled: activations quantised by the caller (int8 rows and a / 127 per row) -> the floats of the
    quantising call, from the int8 GEMV's own launch: every row count class (the lone one-row kernels with two wavefronts
    per task and on the byte tile included), balanced, ragged and sparse streams, columns that span wavefronts."""
    K, N, S = 2560, 640, 1536
    Wd, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    ragged = sp.generate_ternary_iid(K, N, 0x42, 0.2, 0.3)
    sparse = sp.generate_ternary_iid(K, N, 0x43, 0.02, 0.03)
    streams = [("u16 %d" % sk, sp.Weights.upload_u16(pos, neg, K, sk), None) for sk in (8, 16, 32, 64, 128, 256)]
    streams += [("gap %d" % sk, sp.Weights.upload_delta(pos, neg, K, sk), None) for sk in (16, 64)]
    streams += [("gap for one row", sp.Weights.upload_delta(pos, neg, K, 32, rows=1), None)]
    streams += [("ragged u16", sp.Weights.upload_dense(ragged, sp.KIND_U16, 32), ragged), ("ragged gap", sp.Weights.upload_dense(ragged, sp.KIND_DELTA, 16), ragged),
                ("sparse gap", sp.Weights.upload_dense(sparse, sp.KIND_DELTA, 8), sparse), ("sparse gap for one row", sp.Weights.upload_dense(sparse, sp.KIND_DELTA, 8, rows=1), sparse)]
    try:
        for name, w, dense in streams:
            for M in (1, 2, 4, 5, 8, 11):
                print("i8 scaled", name, "M", M, flush=True)
                sys.stdout.flush()
                _, xf = rows(700 + M, M, K, "f16")
                q, a = quantise_ref(xf)
                inv = (a / np.float32(127.0)).astype(np.float32)
                C = oracle.sptmm_i8_mt(q, pos, neg, 8) if dense is None else oracle.dense_i8(q, dense)
                got = w.matmul_i8_scaled(q, inv, 0.3)
                assert got.dtype == np.float32 and (got == y_ref(C, a, 0.3)).all(), (name, M)
        big = sp.Weights.upload_u16(*sp.generate_ternary(6912, 2560, 4096)[1:], 6912, 32)  # the headline: two wavefronts per task at M = 1
        _, xf = rows(9, 1, 6912, "f16")
        q, a = quantise_ref(xf)
        _, bp, bn = sp.generate_ternary(6912, 2560, 4096)
        assert (big.matmul_i8_scaled(q, (a / np.float32(127.0)).astype(np.float32), 2.0) == y_ref(oracle.sptmm_i8_mt(q, bp, bn, 8), a, 2.0)).all()
        big.free()
        i2 = sp.Weights.upload_i2s(Wd)
        with pytest.raises(sp.SptmmError):
            i2.matmul_i8_scaled(q[:, :K] if q.shape[1] >= K else np.zeros((1, K), np.int8), np.ones(1, np.float32))
        i2.free()
    finally:
        for _, w, _ in streams:
            w.free()
