"""GPU: a mixed sequence of GEMV launches captured through the C ABI into one HIP graph.

Every replay is checked against the same calls issued eagerly and against the CPU
oracle, with new activations in the captured buffers and eager work and
synchronisations between the replays (a graph that only holds up on its first
replay would pass a single check).
"""
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def test_graph_replays_match_eager_and_oracle():
    sp.device_init(0)
    K, N, S, M = 2560, 640, 1536, 4
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    Wr = sp.generate_ternary_iid(K, N, 77, 0.3, 0.3)
    w_u16 = sp.Weights.upload_u16(pos, neg, K, 32)
    w_gap = sp.Weights.upload_delta(pos, neg, K, 32)
    w_i2s = sp.Weights.upload_i2s(W)
    w_rag = sp.Weights.upload_dense(Wr, sp.KIND_U16, 32)
    w_b = [w_gap, w_gap.clone(), w_gap.clone()]
    st = sp.Stream()

    xi = sp.DeviceBuffer(M * K)              # int8 rows
    xh = sp.DeviceBuffer(2 * M * K)          # fp16 rows
    xb = [sp.DeviceBuffer(K) for _ in w_b]   # one int8 row per batched GEMV
    names = ["u16 i8", "gap f16", "i2s i8", "ragged q8"] + ["batched %d" % i for i in range(len(w_b))]
    outs = {n: sp.DeviceBuffer(4 * M * N) for n in names}
    eager = {n: sp.DeviceBuffer(4 * M * N) for n in names}

    def issue(dst):
        w_u16.gemv_i8(xi, M, dst["u16 i8"], st)
        w_gap.gemv_f16(xh, M, dst["gap f16"], st)
        w_i2s.gemv_i8(xi, M, dst["i2s i8"], st)
        w_rag.gemv_q8(xh, 1, M, 0.5, dst["ragged q8"], st)
        sp.gemv_i8_batched(w_b, xb, [dst["batched %d" % i] for i in range(len(w_b))], 1, st)

    def load_inputs(seed):
        Xi = oracle.make_x_i8(seed, M, K)
        Xh = oracle.make_x_normal(seed + 1, M, K, np.float16)
        Xb = [oracle.make_x_i8(seed + 10 + i, 1, K) for i in range(len(w_b))]
        xi.upload(Xi)
        xh.upload(Xh)
        for b, x in zip(xb, Xb):
            b.upload(x)
        return Xi, Xh, Xb

    load_inputs(1)
    say("graph: capture")
    with sp.Graph(st) as g:
        issue(outs)
    st.sync()

    for rep in range(4):
        Xi, Xh, Xb = load_inputs(100 + 17 * rep)
        for b in list(outs.values()) + list(eager.values()):
            b.fill(0xFF)
        say("graph: replay", rep)
        g.launch(st)
        st.sync()
        got = {n: outs[n].to_numpy(np.int32, (M, N)) for n in names}
        issue(eager)  # the program's own eager work between replays
        st.sync()
        for n in names:
            assert (got[n] == eager[n].to_numpy(np.int32, (M, N))).all(), (rep, n)
        assert (got["u16 i8"] == oracle.sptmm_i8(Xi, pos, neg)).all(), rep
        assert (got["i2s i8"] == oracle.dense_i8(Xi, W)).all(), rep
        for i, x in enumerate(Xb):
            assert (got["batched %d" % i][:1] == oracle.sptmm_i8(x, pos, neg)).all(), (rep, i)
        ref = oracle.sptmm_f64(Xh, pos, neg)
        gf = got["gap f16"].view(np.float32)
        assert (np.abs(gf - ref) / np.maximum(np.abs(ref), np.sqrt(S))).max() <= 1e-3
        q, a = oracle.quantise_rows(Xh.astype(np.float32))
        want = oracle.rescale(oracle.dense_i8(q, Wr), a, 0.5)
        assert np.allclose(got["ragged q8"].view(np.float32), want, rtol=1e-6, atol=0), rep

    g.destroy()
    for o in [w_u16, w_i2s, w_rag] + w_b + [xi, xh] + xb + list(outs.values()) + list(eager.values()):
        o.free()
    st.destroy()


def test_capture_reports_a_failed_call_and_leaves_the_stream_usable():
    sp.device_init(0)
    K, N, S = 512, 48, 256
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, 32)
    st = sp.Stream()
    X = oracle.make_x_i8(3, 1, K)
    xb, cb = sp.DeviceBuffer.from_numpy(X), sp.DeviceBuffer(4 * N)
    with pytest.raises(sp.SptmmError):
        with sp.Graph(st):
            w.gemv_i8(xb, 0, cb, st)  # M = 0 is rejected before anything is launched
    w.gemv_i8(xb, 1, cb, st)          # the capture was closed: the stream runs eagerly again
    st.sync()
    assert (cb.to_numpy(np.int32, (1, N)) == oracle.sptmm_i8(X, pos, neg)).all()
    for o in (w, xb, cb):
        o.free()
    st.destroy()
