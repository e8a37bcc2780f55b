"""GPU: the decoder layer of BASELINE's config 3 as a sequence, at its real shapes.

The layer's seven projections (q, k, v of one input, then o, then gate and up of one input,
then down) and the same layer with the fused shapes the reference instantiates (q+k+v as one
K=2560 -> N=3840 product, gate+up as N=13824: main.cu:1107-1120, 1916-1917) are captured
through the C ABI into HIP graphs -- the seven with the independent projections of a stage on
parallel branches (a side stream joins the capture with sptmm_stream_wait_event and leaves it
again) -- and replayed with new activations between the program's own eager launches.  Every
output of every replay is compared with the CPU oracle, for all three encodings, at M = 1 and 4.
sptmm_measure_sequence, the native timing loop over such a sequence, is run in each of its
modes and has to leave the oracle's numbers behind as well.
"""
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu

# (name, K, N, S, stage): the steps of a stage share their input and do not depend on each other
SEVEN = [("q", 2560, 2560, 1536, 0), ("k", 2560, 640, 1536, 0), ("v", 2560, 640, 1536, 0), ("o", 2560, 2560, 1536, 1),
         ("gate", 2560, 6912, 1536, 2), ("up", 2560, 6912, 1536, 2), ("down", 6912, 2560, 4160, 3)]
FOUR = [("qkv", 2560, 3840, 1536, 0), ("o", 2560, 2560, 1536, 1), ("gate_up", 2560, 13824, 1536, 2), ("down", 6912, 2560, 4160, 3)]
STAGE_K = (2560, 2560, 2560, 6912)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def matrices():
    sp.device_init(0)
    return {(k, n, s): sp.generate_ternary(k, n, s, dense=True) for _, k, n, s, _ in SEVEN + FOUR}


def upload(enc, mats, key, m):
    W, pos, neg = mats[key]
    if enc == "u16":
        return sp.Weights.upload_u16(pos, neg, key[0], 0)
    if enc == "delta":
        return sp.Weights.upload_delta(pos, neg, key[0], 0, rows=m)
    return sp.Weights.upload_i2s(W)


def capture_layer(shapes, ws, xb, cb, m, st, side, branches):
    """One layer into a graph; with `branches`, the steps of a stage behind the first go to side streams."""
    fork, joins = sp.Event(), [sp.Event() for _ in side]
    with sp.Graph(st) as g:
        i = 0
        while i < len(shapes):
            j = i + 1
            while j < len(shapes) and shapes[j][4] == shapes[i][4]:
                j += 1
            if branches and j - i > 1:
                fork.record(st)
                for b in range(1, j - i):
                    side[b - 1].wait(fork)
                for b in range(j - i):
                    ws[i + b].gemv_i8(xb[shapes[i][4]], m, cb[i + b], side[b - 1] if b else st)
                for b in range(1, j - i):
                    joins[b - 1].record(side[b - 1])
                    st.wait(joins[b - 1])
            else:
                for b in range(i, j):
                    ws[b].gemv_i8(xb[shapes[b][4]], m, cb[b], st)
            i = j
    return g, [fork] + joins


@pytest.mark.parametrize("enc", ["u16", "delta", "i2s"])
@pytest.mark.parametrize("m", [1, 4])
def test_layer_graphs_replay_to_the_oracle(matrices, enc, m):
    st, side = sp.Stream(), [sp.Stream(), sp.Stream()]
    xb = [sp.DeviceBuffer(m * k) for k in STAGE_K]
    for label, shapes, branches in (("seven, parallel branches", SEVEN, True), ("four fused, chain", FOUR, False)):
        say("layer graph:", enc, "M=%d" % m, label)
        ws = [upload(enc, matrices, (k, n, s), m) for _, k, n, s, _ in shapes]
        cb = [sp.DeviceBuffer(4 * m * n) for _, _, n, _, _ in shapes]
        eager = [sp.DeviceBuffer(4 * m * n) for _, _, n, _, _ in shapes]
        for b, k in zip(xb, STAGE_K):
            b.upload(oracle.make_x_i8(1, m, k))
        g, events = capture_layer(shapes, ws, xb, cb, m, st, side, branches)
        st.sync()
        for rep in range(3):
            xs = [oracle.make_x_i8(1000 * rep + 31 * stage + m, m, k) for stage, k in enumerate(STAGE_K)]
            for b, x in zip(xb, xs):
                b.upload(x)
            for c in cb + eager:
                c.fill(0xFF)
            g.launch(st)
            st.sync()
            for i, (name, k, n, s, stage) in enumerate(shapes):  # the program's own eager launches between replays
                ws[i].gemv_i8(xb[stage], m, eager[i], st)
            st.sync()
            for i, (name, k, n, s, stage) in enumerate(shapes):
                _, pos, neg = matrices[(k, n, s)]
                want = oracle.sptmm_i8_mt(xs[stage], pos, neg, 8)
                assert (cb[i].to_numpy(np.int32, (m, n)) == want).all(), (label, rep, name, "graph")
                assert (eager[i].to_numpy(np.int32, (m, n)) == want).all(), (label, rep, name, "eager")
        g.destroy()
        for o in ws + cb + eager + events:
            (o.free if hasattr(o, "free") else o.destroy)()
    for o in xb:
        o.free()
    for s_ in [st] + side:
        s_.destroy()


@pytest.mark.parametrize("mode", sorted(sp.SEQ_MODES.values()))
def test_measure_sequence_leaves_the_oracles_numbers(matrices, mode):
    """Two layers of the seven projections (gap streams, M = 4) through every mode of the native timing loop."""
    m, layers = 4, 2
    st = sp.Stream()
    xs = [oracle.make_x_i8(7 + stage, m, k) for stage, k in enumerate(STAGE_K)]
    xb = [sp.DeviceBuffer.from_numpy(x) for x in xs]
    steps, outs, owned = [], [], []
    for layer in range(layers):
        for name, k, n, s, stage in SEVEN:
            w = upload("delta" if layer else "u16", matrices, (k, n, s), m)
            c = sp.DeviceBuffer(4 * m * n)
            c.fill(0xFF)
            owned += [w, c]
            steps.append((w, xb[stage], c, m, 0, 4 * layer + stage))
            outs.append((name, (k, n, s), stage, c))
    say("measure_sequence mode", mode)
    us = sp.measure_sequence(steps, 5, mode, st)
    assert 5.0 < us < 5000.0
    for name, key, stage, c in outs:
        _, pos, neg = matrices[key]
        assert (c.to_numpy(np.int32, (m, key[1])) == oracle.sptmm_i8_mt(xs[stage], pos, neg, 8)).all(), (mode, name)
    for o in owned + xb:
        o.free()
    st.destroy()


def test_measure_sequence_refuses_bad_sequences(matrices):
    st = sp.Stream()
    w = upload("u16", matrices, (2560, 640, 1536), 1)
    x, c = sp.DeviceBuffer(2560), sp.DeviceBuffer(4 * 640)
    with pytest.raises(sp.SptmmError):
        sp.measure_sequence([(w, x, c, 1, 0, 1), (w, x, c, 1, 0, 0)], 1, 0, st)   # stages decrease
    with pytest.raises(sp.SptmmError):
        sp.measure_sequence([(w, x, c, 1, 0, 0)], 1, 9, st)                       # no such mode
    with pytest.raises(sp.SptmmError):
        sp.measure_sequence([(w, x, c, 0, 0, 0)], 1, 2, st)                       # M = 0, inside what would be a capture
    w.gemv_i8(x, 1, c, st)  # the stream is still usable
    st.sync()
    for o in (w, x, c):
        o.free()
    st.destroy()
