"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle.

Integer paths must be bit-exact.  Floating-point activation variants (fp16 /
fp32 inputs, fp32 sums) must satisfy
    max |got - ref| <= 1e-3 * max(|ref|, sqrt(S))          per element,
with ref the float64 gather-sum (sqrt(S) is the scale of a sum of S unit-variance
terms; it keeps the relative bound meaningful where the sum cancels to ~0).
"""
import hashlib
import json
import os
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
_CACHE = {}


@pytest.fixture(scope="module", autouse=True)
def device():
    info = sp.device_init(0)
    print("device:", info, flush=True)
    return info


def matrix(K, N, S, dense=False):
    key = (K, N, S)
    if key not in _CACHE or (dense and _CACHE[key][0] is None):
        _CACHE.clear()  # keep host memory bounded
        W, pos, neg = sp.generate_ternary(K, N, S, dense=dense)
        Wo, po, no = oracle.generate(K, N, S, dense=False)
        assert (pos == po).all() and (neg == no).all()
        _CACHE[key] = (W, pos, neg)
    return _CACHE[key]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def x_i8(seed, M, K):
    return oracle.make_x_i8(seed, M, K)


def check_fp(got, ref, S):
    if got.size == 0:
        return
    scale = np.maximum(np.abs(ref), np.sqrt(S))
    err = np.abs(got.astype(np.float64) - ref) / scale
    assert err.max() <= REL_TOL, "max rel err %.3e" % err.max()


# ------------------------------------------------------------------ u16 lists
@pytest.mark.parametrize("split", [8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("M", [1, 4])
def test_u16_headline_shape_bit_exact(split, M, golden_dir):
    K, N, S = 6912, 2560, 4096
    say("u16 cfg0/1", K, N, S, "split", split, "M", M)
    _, pos, neg = matrix(K, N, S)
    X = x_i8(0xC0FFEE ^ M, M, K)
    want = oracle.sptmm_i8_mt(X, pos, neg, 8)
    w = sp.Weights.upload_u16(pos, neg, K, split)
    assert w.nbytes == 2 * S * N
    got = w.matmul(X)
    w.free()
    assert got.dtype == np.int32 and (got == want).all()
    kats = json.load(open(os.path.join(golden_dir, "generator_kats.json")))
    e = [m for m in kats["matrices"] if (m["K"], m["N"], m["S"]) == (K, N, S)][0]
    o = [o for o in e["outputs"] if o["M"] == M][0]
    assert hashlib.sha256(got.tobytes()).hexdigest() == o["sha256_C"]


@pytest.mark.parametrize("M", [2, 3, 5, 7, 8, 9, 16, 33, 64])
def test_u16_row_counts(M):
    K, N, S = 6912, 256, 4096
    say("u16 rows", M)
    _, pos, neg = matrix(K, N, S)
    X = x_i8(100 + M, M, K)
    want = oracle.sptmm_i8_mt(X, pos, neg, 8)
    for split in (32, 128):
        w = sp.Weights.upload_u16(pos, neg, K, split)
        got = w.matmul(X)
        w.free()
        assert (got == want).all(), split


@pytest.mark.parametrize("split", [8, 16, 32, 64, 128, 256])
def test_multi_row_tiles_every_split(split):
    """Four- and eight-row tiles (sums on the matrix unit): every lanes-per-column layout of the result tiles."""
    K, N, S = 2560, 640, 1536
    say("multi-row tiles, split", split)
    _, pos, neg = matrix(K, N, S)
    ws = [sp.Weights.upload_u16(pos, neg, K, split)]
    if split <= 64:
        ws.append(sp.Weights.upload_delta(pos, neg, K, split))
    for M in (4, 8):
        X = x_i8(300 + M, M, K)
        want = oracle.sptmm_i8_mt(X, pos, neg, 8)
        for w in ws:
            assert (w.matmul(X) == want).all(), (M, w.info["kind"])
    Xh = oracle.make_x_normal(77, 4, K, np.float16)
    ref = oracle.sptmm_f64(Xh, pos, neg)
    for w in ws:
        check_fp(w.matmul(Xh), ref, S)
    for w in ws:
        w.free()


@pytest.mark.parametrize("K,N,S,splits", [
    (64, 16, 32, (8, 16)),               # one or two entries per lane: tails only
    (512, 48, 256, (8, 16, 32, 64, 128)),
    (6912, 64, 4160, (8, 16, 32)),       # S/2 = 2080 = 32*65: ragged tail rounds
    (2560, 640, 1536, (8, 16, 32, 64, 256)),
    (4096, 32, 3584, (256,)),            # n_lane = 7: 8+4+2-byte tail rounds
])
def test_u16_ragged_and_small_shapes(K, N, S, splits):
    _, pos, neg = matrix(K, N, S)
    for M in (1, 4, 6):
        X = x_i8(K + M, M, K)
        want = oracle.sptmm_i8_mt(X, pos, neg, 4)
        for split in splits:
            say("u16 ragged", K, N, S, "split", split, "M", M)
            w = sp.Weights.upload_u16(pos, neg, K, split)
            got = w.matmul(X)
            w.free()
            assert (got == want).all(), (split, M)


def test_u16_special_inputs():
    K, N, S = 2560, 640, 1536
    W, pos, neg = matrix(K, N, S, dense=True)
    w = sp.Weights.upload_u16(pos, neg, K, 32)
    say("u16 ones")
    assert (w.matmul(np.ones((1, K), np.int8)) == 0).all()            # balanced signs
    assert (w.matmul(np.full((2, K), -127, np.int8)) == 0).all()
    for k in (0, 1, 1279, K - 1):
        e = np.zeros((1, K), np.int8)
        e[0, k] = 1
        say("u16 unit", k)
        assert (w.matmul(e)[0] == W[:, k]).all()                      # unit vector picks row k of W
    X = np.full((1, K), 127, np.int8)
    X[0, ::2] = -127
    assert (w.matmul(X) == oracle.sptmm_i8(X, pos, neg)).all()        # extreme magnitudes
    w.free()


@pytest.mark.parametrize("K,N,S", [(6912, 2560, 4096), (2560, 640, 1536), (6912, 128, 4096), (13824, 256, 8320)])
def test_automatic_split_k(K, N, S, device):
    """split_k = 0: the library picks (sptmm_choose_split_k for this device); the result is the same as with any split."""
    W, pos, neg = matrix(K, N, S, dense=True)
    cus = device["compute_units"]
    ws = [sp.Weights.upload_u16(pos, neg, K, 0), sp.Weights.upload_delta(pos, neg, K, 0), sp.Weights.upload_dense(W, sp.KIND_U16, 0),
          sp.Weights.upload_dense(W, sp.KIND_DELTA, 0), sp.Weights.upload_wide(W, sp.KIND_U16, 0), sp.Weights.upload_wide(W, sp.KIND_DELTA, 0)]
    assert ws[0].info["split_k"] == sp.choose_split_k(sp.KIND_U16, N, S, cus)
    assert ws[1].info["split_k"] == sp.choose_split_k(sp.KIND_DELTA, N, S, cus)
    for M in (1, 4, 9):
        X = x_i8(50 + M, M, K)
        want = oracle.sptmm_i8_mt(X, pos, neg, 8)
        for w in ws:
            say("auto split", K, N, S, "kind", w.info["kind"], "ragged", w.info["ragged"], "k_tile", w.info["k_tile"], "split", w.info["split_k"], "M", M)
            assert w.info["split_k"] in (8, 16, 32, 64, 128, 256)
            assert (w.matmul(X) == want).all()
    for w in ws:
        w.free()


def test_linearity_and_split_invariance_full_size():
    K, N, S = 6912, 2560, 4096
    _, pos, neg = matrix(K, N, S)
    rng = np.random.default_rng(11)
    X1 = rng.integers(-60, 61, (4, K), dtype=np.int8)
    X2 = rng.integers(-60, 61, (4, K), dtype=np.int8)
    outs = []
    for split in (8, 32, 64, 256):
        say("linearity split", split)
        w = sp.Weights.upload_u16(pos, neg, K, split)
        a, b, ab = w.matmul(X1), w.matmul(X2), w.matmul((X1 + X2).astype(np.int8))
        w.free()
        assert (a + b == ab).all()
        outs.append(ab)
    for o in outs[1:]:
        assert (o == outs[0]).all()


# ---------------------------------------------------------------- gap streams
@pytest.mark.parametrize("split", [8, 16, 32, 64])
def test_delta_headline_shape_int8_bit_exact(split):
    K, N, S = 6912, 2560, 4096
    say("delta i8 split", split)
    _, pos, neg = matrix(K, N, S)
    w = sp.Weights.upload_delta(pos, neg, K, split)
    assert w.info["delta_bits"] == 8 and w.info["ragged"] == 0
    for M in (1, 4):
        X = x_i8(0xC0FFEE ^ M, M, K)
        assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), M
    w.free()


@pytest.mark.parametrize("K,N,S,split", [(6912, 2560, 4096, 32), (6912, 2560, 4096, 64), (2560, 640, 1536, 32),
                                         (6912, 64, 4160, 32), (512, 48, 256, 64), (6912, 32, 64, 32)])
def test_delta_all_activation_types(K, N, S, split):
    _, pos, neg = matrix(K, N, S)
    w = sp.Weights.upload_delta(pos, neg, K, split)
    for M in (1, 3, 4, 8):
        say("delta", K, N, S, "split", split, "M", M, "bits", w.info["delta_bits"])
        X = x_i8(31 * M + 1, M, K)
        assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), M
    Xh = oracle.make_x_normal(1, 2, K, np.float16)
    check_fp(w.matmul(Xh), oracle.sptmm_f64(Xh, pos, neg), S)
    Xf = oracle.make_x_normal(1, 1, K, np.float32)
    check_fp(w.matmul(Xf), oracle.sptmm_f64(Xf, pos, neg), S)
    w.free()


def test_delta_matches_reference_layout_walk():
    # the oracle's walk of the reference's own div256 byte layout (main.cu:644-675)
    K, N, S = 6912, 64, 4096
    _, pos, neg = matrix(K, N, S)
    dp, wp = oracle.delta8(pos)
    dn, wn = oracle.delta8(neg)
    assert wp == 0 and wn == 0
    X = x_i8(77, 2, K)
    want = oracle.sptmm_delta_i8(X, oracle.delta_div256(dp), oracle.delta_div256(dn), N, S // 2)
    say("delta vs div256 walk")
    w = sp.Weights.upload_delta(pos, neg, K, 32)
    got = w.matmul(X)
    w.free()
    assert (got == want).all()


def test_delta_fp16_config2():
    K, N, S = 6912, 2560, 4096
    _, pos, neg = matrix(K, N, S)
    X = oracle.make_x_normal(2, 1, K, np.float16)
    ref = oracle.sptmm_f64(X, pos, neg)
    say("delta fp16 cfg2")
    w = sp.Weights.upload_delta(pos, neg, K, 32)
    got = w.matmul(X)
    assert got.dtype == np.float32
    check_fp(got, ref, S)
    X4 = oracle.make_x_normal(3, 4, K, np.float16)
    check_fp(w.matmul(X4), oracle.sptmm_f64(X4, pos, neg), S)
    w.free()


@pytest.mark.parametrize("K,N,S,splits", [
    (6912, 32, 64, (8, 16, 32)),         # sparse: gaps above 255 -> 16-bit stream
    (6912, 16, 256, (8, 64)),
    (6912, 64, 4160, (8, 16, 32)),       # ragged: 65 / 130 / 260 gaps per lane
    (2560, 640, 1536, (8, 16, 32, 64)),
    (512, 48, 256, (8, 16, 32, 64)),
    (64, 16, 32, (8, 16)),
])
def test_delta_ragged_sparse_and_16bit(K, N, S, splits):
    _, pos, neg = matrix(K, N, S)
    for split in splits:
        w = sp.Weights.upload_delta(pos, neg, K, split)
        bits = w.info["delta_bits"]
        # byte gaps where every gap of the sorted lists fits; else 16-bit gaps, or byte gaps again with the long ones
        # walked over zero slots of the tile, whichever stream is smaller
        assert bits == sp.delta_bits(pos, neg, split) or (bits == 8 and w.info["stones"] == 1)
        for M in (1, 4, 5):
            say("delta", K, N, S, "split", split, "bits", bits, "stones", w.info["stones"], "M", M)
            X = x_i8(S + M, M, K)
            assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 4)).all(), (split, M)
        Xh = oracle.make_x_normal(split, 2, K, np.float16)
        check_fp(w.matmul(Xh), oracle.sptmm_f64(Xh, pos, neg), S)
        w.free()


# ----------------------------------------------------- floating-point variants
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("M", [1, 3, 4])
def test_u16_float_activations(dtype, M):
    K, N, S = 6912, 2560, 4096
    _, pos, neg = matrix(K, N, S)
    X = oracle.make_x_normal(40 + M, M, K, dtype)
    ref = oracle.sptmm_f64(X, pos, neg)
    for split in (32, 128):
        say("u16 float", dtype.__name__, "M", M, "split", split)
        w = sp.Weights.upload_u16(pos, neg, K, split)
        got = w.matmul(X)
        w.free()
        check_fp(got, ref, S)


@pytest.mark.parametrize("K,N,S", [(6912, 2560, 4096), (2560, 640, 1536)])
@pytest.mark.parametrize("M", [5, 8, 9, 16])
def test_fp16_eight_row_tiles(K, N, S, M):
    """Five to eight fp16 rows share one tile of 16-byte slots (all eight rows of an index) and are summed on the matrix
    unit; every lanes-per-column case of its result layout (8, 16, 32, 64 lanes, and columns that span wavefronts), on
    u16 lists and on gap streams, against the fp64 oracle to the usual 1e-3."""
    _, pos, neg = matrix(K, N, S)
    X = oracle.make_x_normal(70 + M, M, K, np.float16)
    ref = oracle.sptmm_f64(X, pos, neg)
    for kind, splits in (("u16", (8, 16, 32, 64, 128)), ("delta", (8, 16, 32, 64))):
        for split in splits:
            say("fp16 eight rows", K, N, S, "M", M, kind, split)
            w = sp.Weights.upload_u16(pos, neg, K, split) if kind == "u16" else sp.Weights.upload_delta(pos, neg, K, split)
            got = w.matmul(X)
            w.free()
            check_fp(got, ref, S)


def finite_columns(pos, neg, k):
    """Columns whose lists do not hold row k."""
    return ~((pos == k).any(axis=1) | (neg == k).any(axis=1))


@pytest.mark.parametrize("kind,split", [("u16", 8), ("u16", 16), ("u16", 32), ("u16", 128), ("delta", 16), ("delta", 32)])
@pytest.mark.parametrize("bad", [np.inf, -np.inf, np.nan])
def test_non_finite_activation_stays_in_its_row_and_columns(kind, split, bad):
    """One Inf / NaN at X[0][k]: only the outputs C[0][n] of columns n that gather row k may be non-finite.
    Rows 1.. (other sequences of the batch) and the columns that do not gather k equal the fp64 oracle to the
    usual 1e-3 -- in particular on the four-row fp16 tiles, whose sums run on the matrix unit when all is finite."""
    K, N, S = 2560, 640, 1536
    _, pos, neg = matrix(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, split) if kind == "u16" else sp.Weights.upload_delta(pos, neg, K, split)
    for M, dtype in ((4, np.float16), (3, np.float16), (1, np.float16), (4, np.float32), (8, np.float16), (6, np.float16)):
        for k in (0, 1337, K - 1):
            say("non-finite", kind, split, dtype.__name__, "M", M, "k", k, bad)
            X = oracle.make_x_normal(500 + M + k, M, K, dtype)
            X[0, k] = bad
            clean = X.copy()
            clean[0, k] = 0
            ref = oracle.sptmm_f64(clean, pos, neg)
            got = w.matmul(X)
            away = finite_columns(pos, neg, k)
            assert 0 < away.sum() < N
            assert np.isfinite(got[1:]).all() and np.isfinite(got[0, away]).all()
            check_fp(got[1:], ref[1:], S)
            check_fp(got[0:1, away], ref[0:1, away], S)
            assert (~np.isfinite(got[0, ~away])).all()  # Inf or NaN where the row is gathered, as IEEE sums give
    w.free()


def test_non_finite_activation_batched_launch_only_touches_its_own_gemv():
    K, N, S = 2560, 640, 1536
    _, pos, neg = matrix(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, 32)
    Xs = [oracle.make_x_normal(900 + i, 4, K, np.float16) for i in range(3)]
    Xs[1][2, 77] = np.inf
    xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
    cb = [sp.DeviceBuffer(4 * 4 * N) for _ in Xs]
    say("non-finite batched")
    sp.gemv_batched([w, w, w], xb, cb, 4, 1)
    sp.device_sync()
    for i in (0, 2):
        check_fp(cb[i].to_numpy(np.float32, (4, N)), oracle.sptmm_f64(Xs[i], pos, neg), S)
    got = cb[1].to_numpy(np.float32, (4, N))
    clean = Xs[1].copy()
    clean[2, 77] = 0
    ref = oracle.sptmm_f64(clean, pos, neg)
    away = finite_columns(pos, neg, 77)
    check_fp(got[[0, 1, 3]], ref[[0, 1, 3]], S)
    check_fp(got[2:3, away], ref[2:3, away], S)
    assert (~np.isfinite(got[2, ~away])).all()
    for o in [w] + xb + cb:
        o.free()


# ------------------------------------------------------------------------ i2s
@pytest.mark.parametrize("K,N,S", [(6912, 2560, 4096), (2560, 2560, 1536), (2560, 640, 1536),
                                   (2560, 6912, 1536), (304, 32, 100), (512, 48, 256), (64, 16, 32)])
def test_i2s_bit_exact(K, N, S):
    W, pos, neg = matrix(K, N, S, dense=True)
    w = sp.Weights.upload_i2s(W)
    assert w.nbytes == N * ((K + 255) // 256 * 256) // 4
    for M in (1, 2, 4, 5, 8, 11):
        say("i2s", K, N, S, "M", M)
        X = x_i8(K ^ M, M, K)
        assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), M
    w.free()


def test_i2s_matches_oracle_i2s_and_dense():
    K, N, S = 512, 48, 256
    W, pos, neg = matrix(K, N, S, dense=True)
    X = x_i8(9, 3, K)
    w = sp.Weights.upload_i2s(W)
    got = w.matmul(X)
    w.free()
    assert (got == oracle.i2s_gemv(X, oracle.i2s_pack(W))).all()
    assert (got == oracle.dense_i8(X, W)).all()


# --------------------------------------------------------- benchmark configs 3, 4
LAYER = [("q/o", 2560, 2560, 1536), ("k/v", 2560, 640, 1536), ("gate/up", 2560, 6912, 1536),
         ("down", 6912, 2560, 4160)]


@pytest.mark.parametrize("name,K,N,S", LAYER)
def test_decoder_layer_shapes_all_formats(name, K, N, S):
    W, pos, neg = matrix(K, N, S, dense=True)
    ws = [sp.Weights.upload_u16(pos, neg, K, 32), sp.Weights.upload_delta(pos, neg, K, 32), sp.Weights.upload_i2s(W)]
    for M in (1, 4):
        X = x_i8(1000 + M, M, K)
        want = oracle.sptmm_i8_mt(X, pos, neg, 8)
        for w in ws:
            say("layer", name, "kind", w.info["kind"], "M", M)
            assert (w.matmul(X) == want).all(), (name, w.info, M)
    for w in ws:
        w.free()


# The fused projections the reference times (main.cu:1107-1120 for the lists at N = 13824, main.cu:1916-1917 for
# i2s at N = 3840): q+k+v as one K=2560 -> N=3840 matrix, gate+up as one K=2560 -> N=13824 matrix.  N = 13824 at
# split 32 is 6,912 tasks: several workgroups per compute unit and more than one task per wavefront in one launch.
FUSED = [("q+k+v", 2560, 3840, 1536), ("gate+up", 2560, 13824, 1536)]


@pytest.mark.parametrize("name,K,N,S", FUSED)
def test_fused_projection_shapes_single_and_batched(name, K, N, S):
    W, pos, neg = matrix(K, N, S, dense=True)
    encodings = [("u16", s, lambda s=s: sp.Weights.upload_u16(pos, neg, K, s)) for s in (16, 32, 64)]
    encodings += [("delta", s, lambda s=s: sp.Weights.upload_delta(pos, neg, K, s)) for s in (16, 32)]
    encodings += [("i2s", 0, lambda: sp.Weights.upload_i2s(W))]
    Xs = {M: [x_i8(7000 + 10 * M + i, M, K) for i in range(3)] for M in (1, 4, 8)}
    want = {M: [oracle.sptmm_i8_mt(x, pos, neg, 8) for x in Xs[M]] for M in Xs}
    st = sp.Stream()
    for kind, split, make in encodings:
        w = make()
        ws = [w, w.clone(), w.clone()]
        for M in (1, 4, 8):
            say("fused", name, kind, "split", split, "M", M, "single")
            assert (w.matmul(Xs[M][0]) == want[M][0]).all(), (kind, split, M)
            say("fused", name, kind, "split", split, "M", M, "batched x3")
            xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs[M]]
            cb = [sp.DeviceBuffer(4 * M * N) for _ in ws]
            for c in cb:
                c.fill(0xFF)
            sp.gemv_i8_batched(ws, xb, cb, M, st)
            st.sync()
            for i in range(3):
                assert (cb[i].to_numpy(np.int32, (M, N)) == want[M][i]).all(), (kind, split, M, i)
            for o in xb + cb:
                o.free()
        for o in ws:
            o.free()
    st.destroy()


def test_large_layer_config4_three_encodings():
    K, N, S = 13824, 5120, 8320
    W, pos, neg = matrix(K, N, S, dense=True)
    ws = [sp.Weights.upload_u16(pos, neg, K, 32), sp.Weights.upload_u16(pos, neg, K, 64),
          sp.Weights.upload_delta(pos, neg, K, 32), sp.Weights.upload_i2s(W)]
    assert ws[0].nbytes == 2 * S * N and ws[3].nbytes == K * N // 4
    for M in (1, 8, 16):
        X = x_i8(4000 + M, M, K)
        want = oracle.sptmm_i8_mt(X, pos, neg, 8)
        for w in ws:
            say("cfg4 kind", w.info["kind"], "split", w.info["split_k"], "M", M)
            assert (w.matmul(X) == want).all(), (w.info, M)
    for w in ws:
        w.free()


# ------------------------------------------------------------- boundary behaviour
def test_argument_errors_are_status_codes():
    K, N, S = 512, 48, 256
    _, pos, neg = matrix(K, N, S)
    with pytest.raises(sp.SptmmError) as e:
        sp.Weights.upload_u16(pos, neg, K, 12)
    assert e.value.code == -1 and "split" in str(e.value).lower()
    with pytest.raises(sp.SptmmError):
        sp.Weights.upload_delta(pos, neg, K, 128)
    w = sp.Weights.upload_delta(pos, neg, K, 32)
    xb = sp.DeviceBuffer(K)
    cb = sp.DeviceBuffer(4 * N)
    with pytest.raises(sp.SptmmError):
        w.gemv_i8(xb, 0, cb)
    W = np.zeros((N, K), np.int8)
    wi = sp.Weights.upload_i2s(W)
    with pytest.raises(sp.SptmmError) as e:
        wi.gemv_f16(xb, 1, cb)
    assert e.value.code == -2
    for o in (w, wi, xb, cb):
        o.free()


def test_tile_limit_and_largest_k():
    """One activation row takes 4 bytes of LDS per row of K: K = 40,880 is the last that fits 160 KB."""
    for K, fits in ((40880, True), (40896 + 64, False)):
        N, S = 32, 512
        _, pos, neg = sp.generate_ternary(K, N, S)
        X = x_i8(K, 1, K)
        say("tile limit K", K)
        for w in (sp.Weights.upload_u16(pos, neg, K, 32), sp.Weights.upload_delta(pos, neg, K, 32)):
            if fits:
                assert (w.matmul(X) == oracle.sptmm_i8(X, pos, neg)).all()
            else:
                with pytest.raises(sp.SptmmError) as e:
                    w.matmul(X)
                assert e.value.code == -2 and "LDS" in str(e.value)
            w.free()


def test_eight_row_tiles_up_to_the_last_k_that_fits():
    """Eight-row int8 tiles take 8 bytes of LDS per row of K plus what the workgroup keeps behind the tile; where
    that no longer fits, the launch falls back to four-row tiles instead of failing (K around 20,400)."""
    N, S = 32, 512
    for K in (20352, 20368, 20384, 20400, 20416):
        _, pos, neg = sp.generate_ternary(K, N, S)
        X = x_i8(K, 8, K)
        want = oracle.sptmm_i8(X, pos, neg)
        for w in (sp.Weights.upload_u16(pos, neg, K, 32), sp.Weights.upload_u16(pos, neg, K, 256), sp.Weights.upload_delta(pos, neg, K, 32)):
            say("eight-row limit K", K, w.info["kind"], w.info["split_k"])
            assert (w.matmul(X) == want).all()
            Xh = oracle.make_x_normal(K, 8, K, np.float32).astype(np.float16)
            q, a = oracle.quantise_rows(Xh.astype(np.float32))
            got = w.matmul_q8(Xh, w_scale=0.5)
            assert (got == oracle.rescale(oracle.sptmm_i8(q, pos, neg), a, 0.5)).all()
            w.free()


def test_streams_and_clone():
    K, N, S = 2560, 640, 1536
    _, pos, neg = matrix(K, N, S)
    X = x_i8(5, 1, K)
    want = oracle.sptmm_i8(X, pos, neg)
    w = sp.Weights.upload_u16(pos, neg, K, 32)
    w2 = w.clone()
    st = sp.Stream()
    xb = sp.DeviceBuffer.from_numpy(X)
    cb = sp.DeviceBuffer(4 * N)
    ev0, ev1 = sp.Event(), sp.Event()
    ev0.record(st)
    for _ in range(10):
        w2.gemv_i8(xb, 1, cb, st)
    ev1.record(st)
    ev1.sync()
    assert ev0.elapsed_us(ev1) > 0
    assert (cb.to_numpy(np.int32, (1, N)) == want).all()
    for o in (w, w2, xb, cb):
        o.free()
    st.destroy()


# ------------------------------------------------------------------ batched launch
@pytest.mark.parametrize("kind", ["u16", "delta", "i2s"])
@pytest.mark.parametrize("M,count", [(1, 3), (4, 5), (1, 40), (8, 9), (16, 2)])
def test_batched_launch_equals_single_launches(kind, M, count):
    K, N, S = 2560, 640, 1536
    W, pos, neg = matrix(K, N, S, dense=True)
    base = (sp.Weights.upload_i2s(W) if kind == "i2s" else sp.Weights.upload_u16(pos, neg, K, 32) if kind == "u16"
            else sp.Weights.upload_delta(pos, neg, K, 32))
    ws = [base] + [base.clone() for _ in range(count - 1)]
    Xs = [x_i8(9000 + i, M, K) for i in range(count)]
    xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
    cb = [sp.DeviceBuffer(4 * M * N) for _ in range(count)]
    for c in cb:
        c.fill(0xFF)
    say("batched", kind, "M", M, "count", count)
    st = sp.Stream()
    sp.gemv_i8_batched(ws, xb, cb, M, st)
    st.sync()
    for i in range(count):
        want = oracle.sptmm_i8_mt(Xs[i], pos, neg, 4)
        assert (cb[i].to_numpy(np.int32, (M, N)) == want).all(), i
    for o in ws + xb + cb:
        o.free()
    st.destroy()


@pytest.mark.parametrize("M,count", [(9, 4), (16, 5), (20, 4), (3, 6)])
def test_i2s_batched_launch_column_tiles_past_the_last_group(M, count):
    """From four GEMVs per launch the matrix-unit kernel gives a wavefront 4 column tiles (8 from nine rows on);
    43 groups of 16 columns leave the last workgroup with tiles past the end, and 20 rows take two row tiles."""
    K, N, S = 2560, 688, 1536
    W, pos, neg = matrix(K, N, S, dense=True)
    base = sp.Weights.upload_i2s(W)
    ws = [base] + [base.clone() for _ in range(count - 1)]
    Xs = [x_i8(9500 + i, M, K) for i in range(count)]
    xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
    cb = [sp.DeviceBuffer(4 * M * N) for _ in range(count)]
    for c in cb:
        c.fill(0xFF)
    say("i2s batched", "M", M, "count", count)
    st = sp.Stream()
    sp.gemv_i8_batched(ws, xb, cb, M, st)
    st.sync()
    for i in range(count):
        assert (cb[i].to_numpy(np.int32, (M, N)) == oracle.sptmm_i8_mt(Xs[i], pos, neg, 4)).all(), i
    for o in ws + xb + cb:
        o.free()
    st.destroy()


@pytest.mark.parametrize("kind", ["u16", "delta"])
@pytest.mark.parametrize("dtype,act", [(np.float16, 1), (np.float32, 2)])
def test_batched_launch_float_activations(kind, dtype, act):
    K, N, S = 2560, 640, 1536
    _, pos, neg = matrix(K, N, S)
    base = sp.Weights.upload_u16(pos, neg, K, 32) if kind == "u16" else sp.Weights.upload_delta(pos, neg, K, 32)
    for M, count in ((1, 4), (4, 3)):
        ws = [base] + [base.clone() for _ in range(count - 1)]
        Xs = [oracle.make_x_normal(70 + i, M, K, dtype) for i in range(count)]
        xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
        cb = [sp.DeviceBuffer(4 * M * N) for _ in range(count)]
        say("batched float", kind, dtype.__name__, "M", M, "count", count)
        sp.gemv_batched(ws, xb, cb, M, act)
        sp.device_sync()
        for i in range(count):
            got = cb[i].to_numpy(np.float32, (M, N))
            check_fp(got, oracle.sptmm_f64(Xs[i], pos, neg), S)
            assert (got == base.matmul(Xs[i])).all()  # and bit-identical to the single launch
        for o in ws[1:] + xb + cb:
            o.free()
    base.free()


def test_batched_launch_rejects_mixed_shapes():
    _, pos, neg = matrix(512, 48, 256)
    a = sp.Weights.upload_u16(pos, neg, 512, 32)
    b = sp.Weights.upload_u16(pos, neg, 512, 16)
    xb = sp.DeviceBuffer(512)
    cb = sp.DeviceBuffer(4 * 48)
    with pytest.raises(sp.SptmmError) as e:
        sp.gemv_i8_batched([a, b], [xb, xb], [cb, cb], 1)
    assert e.value.code == -1
    for o in (a, b, xb, cb):
        o.free()


def test_threads_share_one_weights_object():
    """Four host threads, each with its own stream and buffers, launch on the same weights objects at once."""
    import threading

    K, N, S = 2560, 640, 1536
    W, pos, neg = matrix(K, N, S, dense=True)
    ws = [sp.Weights.upload_u16(pos, neg, K, 32), sp.Weights.upload_delta(pos, neg, K, 16), sp.Weights.upload_i2s(W)]
    errors = []

    def worker(tid):
        try:
            st = sp.Stream()
            for rep in range(12):
                M = (1, 4, 8)[(tid + rep) % 3]
                X = x_i8(4000 + 31 * tid + rep, M, K)
                want = oracle.sptmm_i8(X, pos, neg)
                xb = sp.DeviceBuffer.from_numpy(X)
                cbs = [sp.DeviceBuffer(4 * M * N) for _ in ws]
                for w, cb in zip(ws, cbs):
                    w.gemv_i8(xb, M, cb, st)
                st.sync()
                for w, cb in zip(ws, cbs):
                    if not (cb.to_numpy(np.int32, (M, N)) == want).all():
                        errors.append((tid, rep, w.info["kind"]))
                for o in [xb] + cbs:
                    o.free()
            st.destroy()
        except Exception as e:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append((tid, repr(e)))

    say("threads: 4 x 12 rounds on shared weights")
    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for w in ws:
        w.free()
    assert not errors, errors


@pytest.mark.parametrize("mode,outputs", [(0, 1), (1, 1), (2, 1), (3, 3), (4, 4)])
def test_timing_entry_point_leaves_the_results_of_its_launches(mode, outputs):
    """sptmm_measure_gemv issues the product's own launches: whatever the protocol (one stream, a host sync per launch,
    a graph, batched, four streams), the output buffer afterwards holds the GEMV of the rows it was given."""
    sp.device_init(0)
    K, N, S, M = 2560, 640, 1536, 1
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, 32)
    ws = [w, w.clone(), w.clone()]
    X = oracle.make_x_i8(41 + mode, M, K)
    xb = sp.DeviceBuffer.from_numpy(X)
    cb = sp.DeviceBuffer(4 * M * N * 4)
    cb.fill(0xEE)
    st = sp.Stream()
    say("timing entry point, mode", mode)
    us = sp.measure_gemv(ws, 0, xb, M, cb, 12, mode, st)
    st.sync()
    assert 0.0 < us < 1e5
    got = cb.to_numpy(np.int32, (4, M * N))
    want = oracle.sptmm_i8(X, pos, neg).reshape(-1)
    for i in range(outputs):
        assert (got[i] == want).all(), (mode, i)
    with pytest.raises(sp.SptmmError):
        sp.measure_gemv(ws, 0, xb, M, cb, 4, 5, st)
    for o in (xb, cb):
        o.free()
    for o in ws:
        o.free()


@pytest.mark.parametrize("K,N,S,split,count,M", [
    (6912, 2560, 4096, 32, 32, 4),    # ten tasks per wavefront: the next task's rounds are requested while one is walked
    (6912, 2560, 4096, 32, 5, 3),
    (6912, 2560, 4096, 16, 7, 4),     # eight rounds per task
    (2560, 6912, 1536, 16, 32, 4),    # three rounds
    (6912, 2560, 4160, 32, 9, 2),     # four rounds and a one-entry tail
])
def test_gap_stream_four_rows_batched_with_many_tasks_per_wavefront(K, N, S, split, count, M):
    sp.device_init(0)
    _, pos, neg = matrix(K, N, S)
    w = sp.Weights.upload_delta(pos, neg, K, split)
    ws = [w] + [w.clone() for _ in range(min(count, 3) - 1)]
    ws = [ws[i % len(ws)] for i in range(count)]
    Xs = [x_i8(300 + i, M, K) for i in range(count)]
    xb = [sp.DeviceBuffer.from_numpy(x) for x in Xs]
    cb = [sp.DeviceBuffer(4 * M * N) for _ in range(count)]
    for c in cb:
        c.fill(0xEE)
    st = sp.Stream()
    say("gap stream, four rows, batched", K, N, S, split, count, M)
    sp.gemv_i8_batched(ws, xb, cb, M, st)
    st.sync()
    for i in range(count):
        assert (cb[i].to_numpy(np.int32, (M, N)) == oracle.sptmm_i8_mt(Xs[i], pos, neg, 8)).all(), i
    for o in xb + cb:
        o.free()


@pytest.mark.parametrize("K,N,S,split,count,M", [
    (6912, 2560, 4096, 32, 32, 8),    # one result tile (columns of 32 lanes), ten tasks per wavefront, rounds requested a task ahead
    (13824, 5120, 8320, 64, 14, 8),   # columns of 64 lanes, nine tasks per wavefront, a one-entry tail
    (6912, 2560, 4160, 32, 9, 6),
    (2560, 640, 1536, 32, 5, 7),      # fewer tasks than wavefronts in the last workgroups
    (2560, 6912, 1536, 16, 32, 8),    # columns of 16 lanes: two result tiles, no requests ahead
    (6912, 2560, 4096, 8, 6, 5),      # columns of 8 lanes
])
def test_gap_stream_eight_rows_batched_with_many_tasks_per_wavefront(K, N, S, split, count, M):
    test_gap_stream_four_rows_batched_with_many_tasks_per_wavefront(K, N, S, split, count, M)


def test_gap_stream_eight_rows_single_launch_with_several_tasks_per_wavefront():
    sp.device_init(0)
    K, N, S = 2560, 13824, 1536
    _, pos, neg = matrix(K, N, S)
    for split in (16, 32, 64):
        w = sp.Weights.upload_delta(pos, neg, K, split)
        for M in (8, 5):
            say("gap stream, eight rows, many tasks", split, M)
            X = x_i8(177 + M, M, K)
            assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), (split, M)
        w.free()


def test_gap_stream_four_rows_single_launch_with_several_tasks_per_wavefront():
    """A lone launch walks more than one task per wavefront when the tasks outnumber the wavefronts the chip holds."""
    sp.device_init(0)
    K, N, S = 2560, 13824, 1536
    _, pos, neg = matrix(K, N, S)
    for split in (16, 32, 64):
        w = sp.Weights.upload_delta(pos, neg, K, split)
        for M in (4, 2):
            say("gap stream, four rows, many tasks", split, M)
            X = x_i8(77 + M, M, K)
            assert (w.matmul(X) == oracle.sptmm_i8_mt(X, pos, neg, 8)).all(), (split, M)
        w.free()


@pytest.mark.parametrize("M", [5, 8, 9, 13])
def test_fp32_rows_beyond_one_four_row_tile(M):
    """fp32 rows are summed in tiles of four (a 16-byte slot per index): M above four takes several tiles in one launch
    (the grid's second dimension), the last one partly empty.  u16 lists, both gap widths, a ragged matrix, alone and
    batched, against the float64 gather-sum within 1e-3 of max(|ref|, sqrt(S))."""
    K, N, S = 2560, 640, 1536
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    X = oracle.make_x_normal(50 + M, M, K, np.float32)
    ref = oracle.sptmm_f64(X, pos, neg)
    for name, w in (("u16", sp.Weights.upload_u16(pos, neg, K, 32)), ("u16 split 128", sp.Weights.upload_u16(pos, neg, K, 128)),
                    ("gaps", sp.Weights.upload_delta(pos, neg, K, 16)), ("ragged u16", sp.Weights.upload_dense(W, sp.KIND_U16, 32)),
                    ("ragged gaps", sp.Weights.upload_dense(W, sp.KIND_DELTA, 8))):
        say("fp32 rows", name, "M", M)
        check_fp(w.matmul(X), ref, S)
        xb = [sp.DeviceBuffer.from_numpy(X) for _ in range(3)]
        cb = [sp.DeviceBuffer(4 * M * N) for _ in range(3)]
        cl = [w, w.clone(), w.clone()]
        sp.gemv_batched(cl, xb, cb, M, 2)
        sp.device_sync()
        for c in cb:
            check_fp(c.to_numpy(np.float32, (M, N)), ref, S)
        for o in xb + cb + cl:
            o.free()
    # a matrix too sparse for plain byte gaps (balanced lists: the stream walks long gaps over zero slots, or takes 16-bit gaps)
    Ks, Ns, Ss = 6912, 64, 256
    _, ps, ns = sp.generate_ternary(Ks, Ns, Ss)
    Xs = oracle.make_x_normal(9, M, Ks, np.float32)
    w = sp.Weights.upload_delta(ps, ns, Ks, 8)
    check_fp(w.matmul(Xs), oracle.sptmm_f64(Xs, ps, ns), Ss)
    w.free()
