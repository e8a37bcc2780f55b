"""Host-side checks of the ragged streams (matrices whose columns differ in nonzeros).

The reference has no such path (its generator fixes S/2 entries per sign and
column, main.cu:90, 276), so the pins are: an independent numpy restatement of
the seeded iid generator, exact pack -> unpack round trips, the closed-form size
of the streams, and the bank statistics the u16 scheduler promises.
"""
import numpy as np
import pytest

import sptmm_amd as sp
from sptmm_amd import _capi as capi

U16, DELTA = sp.KIND_U16, sp.KIND_DELTA


def iid_numpy(K, N, seed, p_pos, p_neg):
    """xorshift32 per column, vectorised over columns; top 24 bits against two thresholds."""
    st = (np.uint32(seed) ^ (np.uint32(0x9E3779B9) * np.arange(1, N + 1, dtype=np.uint32))).astype(np.uint32)
    st[st == 0] = 1
    t_pos = np.uint32(int(p_pos * 16777216.0))
    t_neg = np.uint32(int((p_pos + p_neg) * 16777216.0))
    W = np.zeros((N, K), np.int8)
    for r in range(K):
        st ^= st << np.uint32(13)
        st ^= st >> np.uint32(17)
        st ^= st << np.uint32(5)
        u = st >> np.uint32(8)
        W[:, r] = np.where(u < t_pos, 1, np.where(u < t_neg, -1, 0))
    return W


def slot_offset(n_lane, esz, sign, lane, j):
    """Byte offset of entry j of a lane inside a task's rounds (16-byte rounds, then 8/4/2/1-byte tails)."""
    e16 = 16 // esz
    full = n_lane // e16
    if j < full * e16:
        return (j // e16) * 2048 + sign * 1024 + lane * 16 + (j % e16) * esz
    base, rem, first = full * 2048, n_lane - full * e16, full * e16
    w = 8
    while w >= esz:
        cnt = w // esz
        if rem & cnt:
            if j < first + cnt:
                return base + sign * 64 * w + lane * w + (j - first) * esz
            first += cnt
            base += 128 * w
        w //= 2
    raise AssertionError


@pytest.mark.parametrize("K,N,seed,pp,pn", [(64, 16, 1, 0.3, 0.3), (2560, 48, 0xBEEF, 0.35, 0.25), (256, 32, 0, 0.0, 1.0),
                                            (128, 16, 5, 0.0, 0.0)])
def test_iid_generator_matches_numpy(K, N, seed, pp, pn):
    W = sp.generate_ternary_iid(K, N, seed, pp, pn)
    assert W.shape == (N, K) and (W == iid_numpy(K, N, seed, pp, pn)).all()
    if pp == 0.0 and pn == 1.0:
        assert (W == -1).all()
    if pp == 0.0 and pn == 0.0:
        assert (W == 0).all()


def test_iid_generator_density():
    W = sp.generate_ternary_iid(2560, 640, 7, 0.3, 0.3)
    assert abs((W == 1).mean() - 0.3) < 2e-3 and abs((W == -1).mean() - 0.3) < 2e-3
    nnz = (W != 0).sum(1)
    assert nnz.min() < nnz.max()  # columns really differ


def special_matrix(K, N):
    """Columns that stress the padding rules: empty, one sign only, single entries at both ends, full."""
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
@pytest.mark.parametrize("K,N", [(256, 16), (2560, 64), (6912, 32)])
def test_round_trip_iid_and_special(kind, splits, K, N):
    for W in (sp.generate_ternary_iid(K, N, 11, 0.3, 0.3), sp.generate_ternary_iid(K, N, 12, 0.45, 0.15), special_matrix(K, N)):
        for split in splits:
            packed, inf = sp.pack_ragged(W, kind, split)
            assert inf["nnz"] == int((W != 0).sum())
            back = sp.unpack_ragged(packed, K, N, kind, split, inf["bits"])
            assert (back == W).all(), (kind, split)


@pytest.mark.parametrize("split", [8, 16, 32, 64])
def test_sizes_and_counts_closed_form(split):
    K, N = 2560, 128
    W = sp.generate_ternary_iid(K, N, 21, 0.3, 0.3)
    L, G = min(split, 64), 64 // min(split, 64)
    cnt = np.stack([(W == 1).sum(1), (W == -1).sum(1)], 1)  # [N][2]
    # gap streams (and u16 below 64 lanes): a task's count is its longest list over its lanes, rounded up
    n_task = np.maximum(1, -(-cnt.reshape(N // G, G * 2).max(1) // L))
    tasks = N // G
    table = -(-(16 + 2 * tasks) // 256) * 256  # preamble + u16 counts, zero filled to 256 bytes
    for kind, hdr, esz in ((DELTA, 256, 1), (U16, 0, 2)):
        if kind == U16 and split == 64:
            continue  # 64 lanes per column: u16 lists deal a column over two half-wavefronts instead
        packed, inf = sp.pack_ragged(W, kind, split)
        assert inf["bits"] == (8 if kind == DELTA else 0) and (inf["n_min"], inf["n_max"]) == (n_task.min(), n_task.max())
        assert len(packed) == table + tasks * (hdr + 128 * esz * n_task.max())
        assert inf["read_bytes"] == 16 + 2 * tasks + int((hdr + 128 * esz * n_task).sum())
        pre = packed[:16].view(np.uint32)
        assert pre[0] == int.from_bytes(b"SPTR", "little") and tuple(pre[1:]) == (tasks, n_task.max(), n_task.min())
        assert (packed[16:16 + 2 * tasks].view(np.uint16) == n_task).all() and not packed[16 + 2 * tasks:table].any()


def test_gap_stream_lanes_visit_their_run_then_the_zero_row():
    """Lane v holds entries [v*n, (v+1)*n) of the sorted list, visited in a scheduled order with signed
    8-bit steps; past the end of the list it steps to row K and stays."""
    K, N, split = 512, 16, 16
    W = sp.generate_ternary_iid(K, N, 33, 0.3, 0.2)
    packed, inf = sp.pack_ragged(W, DELTA, split)
    assert inf["bits"] == 8
    G, L = 64 // split, split
    stride, table = 256 + 128 * inf["n_max"], 256
    for c in (0, 5, 15):
        task = packed[table + (c // G) * stride:table + (c // G + 1) * stride]
        n = int(packed[16 + 2 * (c // G):][:2].view(np.uint16)[0])
        for sign, val in ((0, 1), (1, -1)):
            rows = np.flatnonzero(W[c] == val)
            for v in range(L):
                lane = (c % G) * L + v
                want = list(rows[v * n:(v + 1) * n]) + [K] * (n - len(rows[v * n:(v + 1) * n]))
                first = int(task[sign * 128 + 2 * lane: sign * 128 + 2 * lane + 2].view(np.uint16)[0])
                gaps = task[[256 + slot_offset(n, 1, sign, lane, j) for j in range(n)]].view(np.int8).astype(int)
                walk = first + np.cumsum(gaps)
                assert gaps[0] == 0 and sorted(walk) == want


@pytest.mark.parametrize("split", [8, 16, 32, 64])
def test_gap_stream_for_single_rows_holds_the_same_matrix_on_other_banks(split):
    """rows = 1: the same runs per lane, visited in an order that spreads a half-wavefront over the banks
    (row / 4) mod 32 of a tile with one byte per row; size, counts and what unpacks are unchanged."""
    K, N = 2560, 32
    for W in (sp.generate_ternary_iid(K, N, 17, 0.3, 0.3), special_matrix(K, N)):
        plain, inf0 = sp.pack_ragged(W, DELTA, split)
        packed, inf = sp.pack_ragged(W, DELTA, split, rows=1)
        assert inf == inf0 and len(packed) == len(plain)  # (the special matrix takes 16-bit gaps: sorted order either way)
        assert (sp.unpack_ragged(packed, K, N, DELTA, split, inf["bits"]) == W).all()
        assert (sp.pack_ragged(W, DELTA, split, rows=4)[0] == plain).all()
    # a matrix with independent entries: count the LDS passes of the walks on both bank functions
    W = sp.generate_ternary_iid(K, N, 17, 0.3, 0.3)
    tasks, table = N // (64 // split), -(-(16 + 2 * (N // (64 // split))) // 256) * 256
    res = {}
    for rows in (0, 1):
        packed, inf = sp.pack_ragged(W, DELTA, split, rows=rows)
        stride = 256 + 128 * inf["n_max"]
        for shift in (0, 2):
            passes = slots = 0
            for t in range(tasks):
                task = packed[table + t * stride:table + (t + 1) * stride]
                n = int(packed[16 + 2 * t:][:2].view(np.uint16)[0])
                for sign in (0, 1):
                    walks = np.empty((64, n), int)
                    for lane in range(64):
                        first = int(task[sign * 128 + 2 * lane: sign * 128 + 2 * lane + 2].view(np.uint16)[0])
                        gaps = task[[256 + slot_offset(n, 1, sign, lane, j) for j in range(n)]].view(np.int8).astype(int)
                        walks[lane] = first + np.cumsum(gaps)
                    for h in range(2):
                        for j in range(n):
                            real = walks[32 * h:32 * h + 32, j]
                            real = real[real < K]  # the zero row is one address for every lane: no conflict
                            if shift:
                                real = np.unique(real >> 2) << 2  # lanes on one dword of the byte tile are served together
                            passes += max(1, np.bincount((real >> shift) & 31, minlength=32).max()) if len(real) else 1
                            slots += 1
            res[rows, shift] = passes / slots
    assert res[1, 2] <= 1.6 and res[0, 0] <= 1.6, res      # each stream on the banks it was scheduled for
    assert res[1, 0] > res[1, 2] + 0.5 and res[0, 2] > res[0, 0] + 0.5, res  # and clearly worse on the other tile


def stone_pos(r):
    """Position of row r in a tile that keeps 16 zero slots behind every 96 rows."""
    return r + 16 * (r // 96)


def walks_of(packed, n_max, table, task, sign):
    """-> [64][n] positions the lanes of one sign of a gap-stream task visit, and n."""
    stride = 256 + 128 * n_max
    t = packed[table + task * stride:table + (task + 1) * stride]
    n = int(packed[16 + 2 * task:][:2].view(np.uint16)[0])
    out = np.empty((64, n), int)
    for lane in range(64):
        first = int(t[sign * 128 + 2 * lane: sign * 128 + 2 * lane + 2].view(np.uint16)[0])
        gaps = t[[256 + slot_offset(n, 1, sign, lane, j) for j in range(n)]].view(np.int8).astype(int)
        assert gaps[0] == 0
        out[lane] = first + np.cumsum(gaps)
    return out, n


@pytest.mark.parametrize("K,N,split,p", [(6912, 32, 32, 0.01), (6912, 32, 16, 0.04), (2560, 64, 8, 0.02), (3072, 48, 16, 0.04), (2560, 16, 64, 0.02)])
def test_sparse_matrix_walks_long_gaps_over_zero_slots(K, N, split, p):
    """Gaps of more than 127 rows: an 8-bit stream of tile positions (16 zero slots behind every 96 rows) whose lanes
    step over zero slots.  Every lane visits exactly the positions of its share of the sorted list, plus zero slots
    only; every step fits a signed byte; what unpacks is the matrix."""
    W = sp.generate_ternary_iid(K, N, 5, p, p)
    W[0] = 0          # an empty column
    W[1] = 0
    W[1, K - 1] = 1   # one entry at the far end
    packed, inf = sp.pack_ragged(W, DELTA, split, bits=8)
    assert inf["bits"] == 8 and packed[:4].tobytes() == b"SPTS"
    assert (sp.unpack_ragged(packed, K, N, DELTA, split, 8) == W).all()
    G, L = 64 // split, split
    tasks = N // G
    table = -(-(16 + 2 * tasks) // 256) * 256
    tile = 112 * -(-K // 96)
    grew = 0
    for task in range(tasks):
        n0 = max(1, max(-(-int((W[task * G + c] == v).sum()) // L) for c in range(G) for v in (1, -1)))
        for sign, val in ((0, 1), (1, -1)):
            walks, n = walks_of(packed, inf["n_max"], table, task, sign)
            grew += n - n0
            assert n >= n0 and walks.min() >= 0 and walks.max() < tile
            assert np.abs(np.diff(walks, axis=1)).max(initial=0) <= 128 and np.diff(walks, axis=1).max(initial=0) <= 127
            for lane in range(64):
                rows = np.flatnonzero(W[task * G + lane // L] == val)
                mine = [stone_pos(int(r)) for r in rows[(lane % L) * n0:(lane % L + 1) * n0]]
                seen = walks[lane]
                real = sorted(int(x) for x in seen if x % 112 < 96)
                assert real == mine, (task, sign, lane)   # every other visit is a zero slot
    assert grew > 0  # some task did need a detour
    # the same stream for tiles of one byte per row: same size, same matrix
    p1, i1 = sp.pack_ragged(W, DELTA, split, bits=8, rows=1)
    assert i1 == inf and len(p1) == len(packed) and (sp.unpack_ragged(p1, K, N, DELTA, split, 8) == W).all()


def test_gap_width_is_chosen_by_size():
    """bits = 0: byte gaps where every gap fits; else the smaller of the stream with zero-slot detours and 16-bit gaps."""
    K, N = 6912, 32
    dense = sp.generate_ternary_iid(K, N, 5, 0.3, 0.3)
    packed, inf = sp.pack_ragged(dense, DELTA, 32)
    assert inf["bits"] == 8 and packed[:4].tobytes() == b"SPTR"
    p16, i16 = sp.pack_ragged(dense, DELTA, 32, bits=16)  # the wide form may always be asked for
    assert i16["bits"] == 16 and (sp.unpack_ragged(p16, K, N, DELTA, 32, 16) == dense).all()
    for p in (0.002, 0.01, 0.03, 0.06):
        W = sp.generate_ternary_iid(K, N, 7, p, p)
        auto, ia = sp.pack_ragged(W, DELTA, 16)
        p8, i8 = sp.pack_ragged(W, DELTA, 16, bits=8)
        p16, i16 = sp.pack_ragged(W, DELTA, 16, bits=16)
        assert i8["bits"] == 8 and i16["bits"] == 16 and p16[:4].tobytes() == b"SPTR"
        assert len(auto) == min(len(p8), len(p16)) or (len(p8) == len(p16) and ia["bits"] == 16)
        assert ia["bits"] == (8 if len(p8) < len(p16) else 16)
        assert (sp.unpack_ragged(auto, K, N, DELTA, 16, ia["bits"]) == W).all()
    # the densest of them is the case the detours are for: nearly all gaps fit, a few do not
    assert ia["bits"] == 8 and auto[:4].tobytes() == b"SPTS" and len(auto) < 0.6 * len(p16)


def lds_passes(tasks_bytes, K, N, split, n_task, n_max, shift):
    """Mean number of LDS passes per half-wavefront gather: the fullest bank among its 32 rows
    (equal rows broadcast and count once)."""
    G, W_ = max(1, 64 // split), max(1, split // 64)
    tasks = N // G * W_
    stride = 256 * n_max
    tot = cnt = 0
    for t in range(0, tasks, max(1, tasks // 24)):
        task = tasks_bytes[t * stride:(t + 1) * stride]
        n = int(n_task[t])
        for sign in range(2):
            for j in range(n):
                rows = np.array([int(task[slot_offset(n, 2, sign, lane, j):][:2].view(np.uint16)[0]) >> shift for lane in range(64)])
                for h in range(2):
                    u = np.unique(rows[32 * h:32 * h + 32])
                    tot += np.bincount(u & 31, minlength=32).max()
                    cnt += 1
    return tot / cnt


@pytest.mark.parametrize("split", [16, 32, 64])
def test_u16_ragged_keeps_lds_banks_apart(split):
    K, N = 2560, 256
    W = sp.generate_ternary_iid(K, N, 77, 0.3, 0.3)
    packed, inf = sp.pack_ragged(W, U16, split)
    tasks = N // max(1, 64 // split) * max(1, split // 64)
    table = -(-(16 + 2 * tasks) // 256) * 256
    n_task = packed[16:16 + 2 * tasks].view(np.uint16)
    p = lds_passes(packed[table:], K, N, split, n_task, inf["n_max"], 2)
    assert p <= 1.4, p
    # every padding field points at a zero row behind the tile
    assert (packed[table:].view(np.uint16) >> 2).max() < K + 64


def test_dense_from_reference_word_order():
    K, N = 64, 16
    W = sp.generate_ternary_iid(K, N, 9, 0.3, 0.3)
    words = np.array([[capi.i2s_pack_word(W[c, 16 * g:16 * g + 16]) for g in range(K // 16)] for c in range(N)], np.uint32)
    assert (sp.dense_from_i2s_words(words, K) == W).all()
    # hand-made word: element e sits at bit 8*(e%4) + 2*(e/4), code = w + 2
    w16 = np.zeros(16, np.int8)
    w16[0], w16[5] = 1, -1
    word = 0
    for e in range(16):
        word |= (int(w16[e]) + 2) << (8 * (e % 4) + 2 * (e // 4))
    assert (sp.dense_from_i2s_words(np.full((1, 1), word, np.uint32), 16)[0] == w16).all()
    with pytest.raises(sp.SptmmError):
        sp.dense_from_i2s_words(np.zeros((1, 1), np.uint32), 16)  # code 0 is no ternary weight


def test_argument_errors():
    W = np.zeros((16, 64), np.int8)
    for bad in (lambda: sp.pack_ragged(W, sp.KIND_I2S, 32), lambda: sp.pack_ragged(W, U16, 7), lambda: sp.pack_ragged(W, DELTA, 128),
                lambda: sp.pack_ragged(np.full((16, 64), 2, np.int8), U16, 32), lambda: sp.pack_ragged(np.zeros((16, 72), np.int8), U16, 32),
                lambda: sp.pack_ragged(np.zeros((16, 65520), np.int8), U16, 32), lambda: sp.generate_ternary_iid(64, 16, 1, 0.7, 0.7)):
        with pytest.raises(sp.SptmmError):
            bad()
    packed, inf = sp.pack_ragged(W, U16, 32)  # an all-zero matrix is fine: one padded entry per lane
    assert inf["nnz"] == 0 and inf["n_max"] == 1 and (sp.unpack_ragged(packed, 64, 16, U16, 32) == 0).all()
    with pytest.raises(sp.SptmmError):
        sp.unpack_ragged(np.zeros(4096, np.uint8), 64, 16, U16, 32)  # no preamble


def test_iid_generator_matches_golden_fixture(golden_dir):
    import hashlib
    import json
    import os

    kats = json.load(open(os.path.join(golden_dir, "generator_kats.json")))["iid_matrices"]
    assert len(kats) >= 3
    for e in kats:
        W = sp.generate_ternary_iid(e["K"], e["N"], e["seed"], e["p_pos"], e["p_neg"])
        assert hashlib.sha256(W.tobytes()).hexdigest() == e["sha256_W_colmajor"] and int((W != 0).sum()) == e["nnz"]
