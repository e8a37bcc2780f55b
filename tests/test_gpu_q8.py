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
