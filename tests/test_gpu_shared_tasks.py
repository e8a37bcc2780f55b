"""GPU: a lone GEMV of one int8 row on u16 lists may give every task two (or four) wavefronts, each taking every
second (fourth) round and the sums meeting in LDS.  Whatever the number of wavefronts per task -- none shared, the
library's own choice, two, four -- the int32 result is the oracle's, for tasks of 2 to 8 rounds with and without a
tail, for 8 to 64 lanes per column, and for launches with fewer and with more tasks than the chip holds at once."""
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


@pytest.fixture
def knobs():
    saved = {k: os.environ.get(k) for k in ("SPTMM_SHARE_LOG", "SPTMM_WAVES_PER_WG")}
    yield
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v
    sp.device_init(0)  # the launch-shape overrides are read here


# (K, N, S, split_k): rounds per task = S / 2 / split_k / 8
SHAPES = [
    (6912, 2560, 4096, 32),   # the headline: 8 rounds
    (6912, 2560, 4160, 32),   # 8 rounds and a tail of one entry
    (2560, 2560, 1536, 16),   # 6 rounds
    (2560, 640, 1536, 32),    # 3 rounds: not shared by two, not by four
    (6912, 2560, 1024, 16),   # 4 rounds
    (4608, 48, 4096, 64),     # 4 rounds, one column per wavefront
    (1024, 64, 288, 8),       # 2 rounds and a tail of 2
    (2048, 16, 1024, 8),      # 8 rounds, two tasks in all
    (2560, 13824, 1536, 16),  # more tasks than the chip holds at ten wavefronts per compute unit
    (16400, 64, 2048, 32),    # row indices stored unscaled (4 K does not fit 16 bits)
]


def test_every_number_of_wavefronts_per_task_gives_the_oracles_sums(knobs):
    for K, N, S, split in SHAPES:
        _, pos, neg = sp.generate_ternary(K, N, S)
        X = oracle.make_x_i8(K + N, 1, K)
        want = oracle.sptmm_i8_mt(X, pos, neg, 8)
        w = sp.Weights.upload_u16(pos, neg, K, split)
        for share_log, waves in ((-1, 0), (0, 0), (1, 0), (1, 2), (1, 16), (2, 4), (2, 16)):
            os.environ["SPTMM_SHARE_LOG"] = str(share_log)
            os.environ["SPTMM_WAVES_PER_WG"] = str(waves)
            sp.device_init(0)
            say("shared tasks:", (K, N, S, split), "share_log", share_log, "waves per workgroup", waves)
            got = w.matmul(X)
            assert (got == want).all(), ((K, N, S, split), share_log, waves)
        w.free()
