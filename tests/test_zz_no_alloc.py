"""GPU: sptmm_gemv_q8_static, the quantising GEMV for callers that cannot allocate: the workspace of sptmm_gemv_q8_ws
lives in a static array of the library's device image.  Through the C ABI, its floats equal sptmm_gemv_q8_ws's bit for
bit -- on two calls in a row, the second with a smaller input (fewer rows, a smaller matrix), so that what the first
call left in the array is still there -- and a call whose workspace would not fit the array is refused."""
import sys

import numpy as np
import pytest

import sptmm_amd as sp

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def both(w, X, M, N, w_scale, st):
    xb = sp.DeviceBuffer.from_numpy(X)
    need = w.q8_workspace_bytes(M)
    ws = sp.DeviceBuffer(need)
    y_ws, y_st = sp.DeviceBuffer(4 * M * N), sp.DeviceBuffer(4 * M * N)
    try:
        y_ws.fill(0xFF)
        y_st.fill(0xEE)
        w.gemv_q8_ws(xb, 1, M, w_scale, y_ws, ws, need, st)
        w.gemv_q8_static(xb, 1, M, w_scale, y_st, st)
        st.sync()
        return y_ws.to_numpy(np.float32, (M, N)), y_st.to_numpy(np.float32, (M, N))
    finally:
        for o in (xb, ws, y_ws, y_st):
            o.free()


def test_static_scratch_gives_the_workspace_calls_floats_twice_in_a_row():
    sp.device_init(0)
    st = sp.Stream()
    # first call: 16 rows of K = 6912 (110,592 int8 values in the array); second: 5 rows of K = 2560, another matrix
    cases = [((6912, 2560, 4096), "u16", 16), ((2560, 640, 1536), "gap", 5), ((13824, 1280, 8320), "gap", 3), ((6912, 2560, 4096), "u16", 4)]
    for (K, N, S), kind, M in cases:
        _, pos, neg = sp.generate_ternary(K, N, S)
        w = sp.Weights.upload_u16(pos, neg, K, 0) if kind == "u16" else sp.Weights.upload_delta(pos, neg, K, 0)
        X = sp.make_x_normal(0x5EED ^ M, M, K)
        say("no-alloc q8:", (K, N, S), kind, "rows", M)
        a, b = both(w, X, M, N, 0.5, st)
        assert np.isfinite(a).all() and (a != 0).any()
        assert (a.view(np.uint32) == b.view(np.uint32)).all(), ((K, N, S), kind, M)
        w.free()


def test_static_scratch_refuses_what_does_not_fit():
    sp.device_init(0)
    K, N, S = 13824, 256, 8320
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_u16(pos, neg, K, 0)
    M = 40  # 552,960 int8 values: more than the array's 524,288
    assert w.q8_workspace_bytes(M) > 528384 >= w.q8_workspace_bytes(38) and w.q8_workspace_bytes(39) > 528384
    X = sp.make_x_normal(1, M, K)
    xb, yb = sp.DeviceBuffer.from_numpy(X), sp.DeviceBuffer(4 * M * N)
    try:
        with pytest.raises(sp.SptmmError) as e:
            w.gemv_q8_static(xb, 1, M, 1.0, yb)
        assert "static array holds" in str(e.value)
        w.gemv_q8_static(xb, 1, 38, 1.0, yb)  # the largest that fits
        sp.device_sync()
    finally:
        for o in (xb, yb, w):
            o.free()


def test_static_scratch_call_under_graph_capture():
    """The caller this entry point is for: a captured stream, where nothing may be allocated.  Three replays with new
    activations in the captured buffer, eager work between them, each against the workspace call's floats."""
    sp.device_init(0)
    K, N, S, M = 6912, 2560, 4096, 8
    _, pos, neg = sp.generate_ternary(K, N, S)
    w = sp.Weights.upload_delta(pos, neg, K, 0)
    st = sp.Stream()
    xb = sp.DeviceBuffer(2 * M * K)
    need = w.q8_workspace_bytes(M)
    ws, y_graph, y_eager = sp.DeviceBuffer(need), sp.DeviceBuffer(4 * M * N), sp.DeviceBuffer(4 * M * N)
    try:
        xb.upload(sp.make_x_normal(1, M, K))
        with sp.Graph(st) as g:
            w.gemv_q8_static(xb, 1, M, 0.125, y_graph, st)
        st.sync()
        for rep in range(3):
            say("no-alloc q8 under capture: replay", rep)
            xb.upload(sp.make_x_normal(100 + rep, M, K))
            y_graph.fill(0xFF)
            y_eager.fill(0xEE)
            g.launch(st)
            st.sync()
            w.gemv_q8_ws(xb, 1, M, 0.125, y_eager, ws, need, st)  # eager work between the replays
            st.sync()
            a, b = y_graph.to_numpy(np.uint32, (M, N)), y_eager.to_numpy(np.uint32, (M, N))
            assert (a == b).all() and (a != 0xFFFFFFFF).all(), rep
        g.destroy()
    finally:
        for o in (xb, ws, y_graph, y_eager, w):
            o.free()
