"""GPU: launch plans.  A stream may carry its own launch shape per kind of call (sptmm_weights_set_plan), found by a
bounded search on the device (sptmm_weights_tune) or set by hand.  No plan changes a result: every plan of the swept
space -- including values the kernels cannot take, which are ignored -- gives the oracle's sums, for every encoding,
lone and batched, at M = 1, 4, 8, 16.  Plans survive save / load and clone."""
import itertools
import os
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


K, N, S = 2560, 640, 1536


@pytest.fixture(scope="module")
def streams():
    sp.device_init(0)
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    return W, pos, neg, {
        "u16": lambda: sp.Weights.upload_u16(pos, neg, K, 16),
        "u16 split 128": lambda: sp.Weights.upload_u16(pos, neg, K, 128),
        "delta": lambda: sp.Weights.upload_delta(pos, neg, K, 32),
        "delta rows=1": lambda: sp.Weights.upload_delta(pos, neg, K, 32, rows=1),
        "ragged u16": lambda: sp.Weights.upload_dense(sp.generate_ternary_iid(K, N, 9, 0.3, 0.3), sp.KIND_U16, 32),
        "wide delta": lambda: sp.Weights.upload_wide(W, sp.KIND_DELTA, 32),
        "i2s": lambda: sp.Weights.upload_i2s(W),
    }


def plans_for(name, batched):
    if name == "i2s":
        return [dict(i2s_ct=c, waves_per_wg=w) for c in (0, 1, 2, 4, 8, 3) for w in (0, 1, 4, 8, 9)]
    if name.startswith("wide"):
        return [dict(waves_per_wg=w) for w in (0, 1, 4, 7, 12, 16, 17)]
    if batched:
        return [dict(waves_per_wg=w, tasks_per_wave=t) for w in (0, 2, 5, 8, 16, 64) for t in (0, 1, 3, 16, 1000)]
    return [dict(waves_per_wg=w, wgs_per_cu=g, share_log=s) for w in (0, 2, 5, 8, 16) for g in (0, 1, 3) for s in (0, -1, 1, 2)]


def test_no_plan_changes_a_result(streams):
    W, pos, neg, makers = streams
    for name, mk in makers.items():
        w = mk()
        copies = [w, w.clone(), w.clone()]
        for M in (1, 4, 8, 16):
            X = oracle.make_x_i8(31 * M, M, K)
            if name == "ragged u16":
                want = oracle.dense_i8(X, sp.generate_ternary_iid(K, N, 9, 0.3, 0.3))
            else:
                want = oracle.sptmm_i8_mt(X, pos, neg, 8)
            xb = sp.DeviceBuffer.from_numpy(X)
            cbs = [sp.DeviceBuffer(4 * M * N) for _ in copies]
            for batched in (False, True):
                say("plans:", name, "M", M, "batched" if batched else "lone", len(plans_for(name, batched)), "plans")
                for plan in plans_for(name, batched):
                    for c in copies:
                        c.set_plan(M, batched, **plan)
                    assert w.get_plan(M, batched) == {**{k: 0 for k in sp.PlanStruct.NAMES}, **plan}
                    for cb in cbs:
                        cb.fill(0xFF)
                    if batched:
                        sp.gemv_i8_batched(copies, [xb] * len(copies), cbs, M)
                    else:
                        w.gemv_i8(xb, M, cbs[0])
                    sp.device_sync()
                    for cb in (cbs if batched else cbs[:1]):
                        assert (cb.to_numpy(np.int32, (M, N)) == want).all(), (name, M, batched, plan)
            for o in [xb] + cbs:
                o.free()
        for c in copies:
            c.free()


def test_tune_keeps_results_and_never_slows_a_stream_down(streams, tmp_path):
    W, pos, neg, makers = streams
    X = oracle.make_x_i8(3, 4, K)
    want = oracle.sptmm_i8_mt(X, pos, neg, 8)
    for name in ("u16", "delta", "wide delta", "i2s"):
        w = makers[name]()
        for M, batch in ((1, 0), (4, 0), (4, 8)):
            us_model, us_tuned, plan = w.tune(M, batch)
            say("tune:", name, "M", M, "batch", batch, "model %.3f us -> %.3f us" % (us_model, us_tuned), plan)
            assert 0 < us_tuned <= us_model
            if any(plan.values()):
                assert us_tuned < 0.98 * us_model
        assert (w.matmul(X) == want).all() and (w.matmul(X[:1]) == want[:1]).all()
        # plans travel with the file and with a clone
        path = str(tmp_path / "tuned.sptmm")
        w.save(path)
        back, twin = sp.Weights.load(path), w.clone()
        for M, batched in ((1, False), (4, False), (4, True), (16, True)):
            assert back.get_plan(M, batched) == w.get_plan(M, batched) == twin.get_plan(M, batched)
        assert (back.matmul(X) == want).all()
        for o in (w, back, twin):
            o.free()


def test_fp16_rows_tune_and_refusals(streams):
    W, pos, neg, makers = streams
    w = makers["delta"]()
    us_model, us_tuned, plan = w.tune(4, 0, act=1)
    assert 0 < us_tuned <= us_model
    Xh = oracle.make_x_normal(5, 4, K, np.float16)
    ref = oracle.sptmm_f64(Xh, pos, neg)
    assert (np.abs(w.matmul(Xh) - ref) / np.maximum(np.abs(ref), np.sqrt(S))).max() <= 1e-3
    # the quantising GEMV (fp16 rows -> int8 in the kernel) tunes as a lone call; its results stay the float32 arithmetic's
    us_model, us_tuned, plan = w.tune(4, 0, act=3)
    say("tune, quantising call:", "model %.3f us -> %.3f us" % (us_model, us_tuned), plan)
    assert 0 < us_tuned <= us_model
    q, a = oracle.quantise_rows(Xh.astype(np.float32))
    assert (w.matmul_q8(Xh, 0.5) == oracle.rescale(oracle.sptmm_i8_mt(q, pos, neg, 8), a, 0.5)).all()
    i2 = makers["i2s"]()
    for bad in (lambda: i2.tune(1, 0, act=1), lambda: w.tune(0, 0), lambda: w.tune(1, -1), lambda: w.tune(1, 0, act=7), lambda: w.set_plan(0, False),
                lambda: w.tune(4, 8, act=3), lambda: i2.tune(1, 0, act=3)):
        with pytest.raises(sp.SptmmError):
            bad()
    w.free()
    i2.free()
