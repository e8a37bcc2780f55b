"""Host logic of the library (generator, stream builders) -- no GPU needed.

The library's own generator is compared with the oracle's restatement of
main.cu:246-276; the three device streams are checked as bijections of the row
lists / dense matrix, against closed-form offset formulas, and through
pack -> unpack round trips.
"""
import numpy as np
import pytest

import oracle
import sptmm_amd as sp

SHAPES = [(64, 16, 32), (512, 32, 256), (2560, 64, 1536), (6912, 32, 4096), (6912, 16, 4160)]


@pytest.mark.parametrize("K,N,S", SHAPES)
def test_generator_equals_oracle(K, N, S):
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    Wo, po, no = oracle.generate(K, N, S)
    assert (W == Wo).all() and (pos == po).all() and (neg == no).all()
    p2, n2 = sp.lists_from_dense(W, S)
    assert (p2 == pos).all() and (n2 == neg).all()


def test_make_x_equals_oracle():
    for seed, M, K in ((0xC0FFEE ^ 1, 1, 6912), (0xC0FFEE ^ 4, 4, 512), (7, 3, 64)):
        assert (sp.make_x_i8(seed, M, K) == oracle.make_x_i8(seed, M, K)).all()


@pytest.mark.parametrize("bad", [
    dict(K=100, N=16, S=32), dict(K=64, N=20, S=32), dict(K=65536, N=16, S=32),
    dict(K=64, N=16, S=31), dict(K=64, N=16, S=64), dict(K=0, N=16, S=0),
])
def test_shape_rules_of_init_ctx(bad):
    # main.cu:85-91
    with pytest.raises(sp.SptmmError) as e:
        sp.generate_ternary(bad["K"], bad["N"], bad["S"])
    assert e.value.code == -1


def u16_shift(K):
    return 2 if 4 * K <= 65535 else 0


@pytest.mark.parametrize("split", [8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("K,N,S", [(2560, 64, 1536), (6912, 32, 4096), (6912, 16, 4160), (4096, 16, 3584),
                                   (16400, 16, 4096)])
def test_u16_stream_is_a_permutation_and_round_trips(K, N, S, split):
    _, pos, neg = sp.generate_ternary(K, N, S)
    if (S // 2) % split:
        with pytest.raises(sp.SptmmError):
            sp.pack_u16(pos, neg, K, split)
        return
    pk = sp.pack_u16(pos, neg, K, split)
    assert pk.nbytes == 2 * S * N  # exactly the algorithmic bytes: no padding
    p2, n2 = sp.unpack_u16(pk, K, N, S, split)
    assert (p2 == pos).all() and (n2 == neg).all()
    allidx = np.sort(np.concatenate([pos.ravel(), neg.ravel()]).astype(np.uint32) << u16_shift(K))
    assert (np.sort(pk.view(np.uint16)) == allidx).all()


def u16_cell(n_lane, sign, lane, slot):
    """u16 index (in units of 2 bytes) of a cell inside its task: full 16-byte rounds, then 8/4/2-byte tails."""
    full = n_lane // 8
    if slot < full * 8:
        return (slot // 8) * 1024 + sign * 512 + lane * 8 + slot % 8
    base, first, rem = full * 1024, full * 8, n_lane - full * 8
    for cnt in (4, 2, 1):
        if rem & cnt:
            if slot < first + cnt:
                return base + sign * 64 * cnt + lane * cnt + (slot - first)
            first += cnt
            base += 128 * cnt
    raise AssertionError


@pytest.mark.parametrize("K,N,S,split", [(6912, 16, 4160, 32), (6912, 16, 4160, 8), (4096, 16, 3584, 256),
                                         (2560, 32, 1536, 64), (2560, 32, 1536, 16)])
def test_u16_stream_geometry_closed_form(K, N, S, split):
    """Column c owns lanes (c % G)*L .. +L of task c/G (or all 64 lanes of tasks c*W .. c*W+W-1)."""
    _, pos, neg = sp.generate_ternary(K, N, S)
    pk = sp.pack_u16(pos, neg, K, split).view(np.uint16)
    half = S // 2
    n_lane = half // split
    L, W = min(split, 64), max(1, split // 64)
    G = 64 // L
    task_words = 128 * n_lane
    for c in (0, 1, N // 2, N - 1):
        for sign, lst in ((0, pos), (1, neg)):
            got = []
            for part in range(W):
                task = c * W + part if W > 1 else c // G
                l0 = 0 if L == 64 else (c % G) * L
                for lane in range(l0, l0 + L):
                    for slot in range(n_lane):
                        got.append(pk[task * task_words + u16_cell(n_lane, sign, lane, slot)])
            got = np.sort(np.array(got, np.uint32) >> u16_shift(K))
            assert (got == lst[c]).all()


def lds_passes(pk, K, n_lane):
    """LDS passes per (task, slot, sign): max multiplicity of (row mod 32) over each 32-lane half."""
    sh = u16_shift(K)
    tasks = pk.size // (128 * n_lane)
    assert n_lane % 8 == 0
    a = (pk.reshape(tasks, n_lane // 8, 2, 64, 8) >> sh) & 31        # [task][round][sign][lane][e]
    a = a.reshape(tasks, n_lane // 8, 2, 2, 32, 8)                   # split lanes in halves
    total = 0
    for b in range(32):
        pass
    mult = np.zeros(a.shape[:4] + (8,), np.int64)
    for b in range(32):
        mult = np.maximum(mult, (a == b).sum(axis=4))
    return int(mult.sum()), mult.size


@pytest.mark.parametrize("split", [8, 16, 32, 64, 128])
def test_u16_schedule_keeps_half_waves_on_distinct_banks(split):
    K, N, S = 6912, 64, 4096
    _, pos, neg = sp.generate_ternary(K, N, S)
    n_lane = (S // 2) // split
    pk = sp.pack_u16(pos, neg, K, split).view(np.uint16)
    passes, slots = lds_passes(pk, K, n_lane)
    # a random assignment needs ~3.5 passes per slot; the scheduler must stay below 1.4
    assert passes <= 1.4 * slots, (passes, slots)


@pytest.mark.parametrize("split", [8, 16, 32, 64])
@pytest.mark.parametrize("K,N,S", [(2560, 64, 1536), (6912, 32, 4096), (6912, 16, 4160), (6912, 16, 64)])
def test_delta_stream_round_trips(K, N, S, split):
    _, pos, neg = sp.generate_ternary(K, N, S)
    if (S // 2) % split:
        return
    bits = sp.delta_bits(pos, neg, split)
    n_lane = (S // 2) // split
    gaps_fit = True
    for lst in (pos, neg):
        runs = lst.reshape(N, split, n_lane).astype(int)
        gaps_fit &= bool((np.diff(runs, axis=2) <= 127).all())  # 8-bit gaps are signed
    assert bits == (8 if gaps_fit else 16)
    pk, b = sp.pack_delta(pos, neg, K, split)
    assert b == bits and pk.nbytes == N // (64 // split) * (256 + 128 * n_lane * bits // 8)
    p2, n2 = sp.unpack_delta(pk, K, N, S, split, bits)
    assert (p2 == pos).all() and (n2 == neg).all()
    if bits == 8:  # the wider form must carry the same lists
        pk16, _ = sp.pack_delta(pos, neg, K, split, bits=16)
        p3, n3 = sp.unpack_delta(pk16, K, N, S, split, 16)
        assert (p3 == pos).all() and (n3 == neg).all()


def test_delta_8bit_refuses_wide_gaps():
    K, N, S = 6912, 16, 64  # mean gap ~200: some gaps exceed a byte
    _, pos, neg = sp.generate_ternary(K, N, S)
    assert sp.delta_bits(pos, neg, 8) == 16
    with pytest.raises(sp.SptmmError):
        sp.pack_delta(pos, neg, K, 8, bits=8)
    # a gap of 128 no longer fits the signed byte, 127 does
    for gap, want in ((127, 8), (128, 16)):
        pos = np.tile(np.arange(8, dtype=np.uint16), (16, 1))
        pos[:, 1:] += gap - 1
        neg = pos + 300
        assert sp.delta_bits(pos, neg, 8) == 8  # one entry per lane: no in-run gap at all
        assert sp.delta_bits(np.ascontiguousarray(np.repeat(pos, 2, 1)[:, :16] + np.arange(16, dtype=np.uint16) % 2 * gap),
                             np.ascontiguousarray(np.repeat(neg, 2, 1)[:, :16] + np.arange(16, dtype=np.uint16) % 2 * gap), 8) == want


def lane_walk(task, n_lane, esz, sign, lane):
    """Rows one lane visits, in order: first row from the header, then the (signed 8-bit / unsigned 16-bit) gaps."""
    first = int(task[sign * 128 + 2 * lane: sign * 128 + 2 * lane + 2].view(np.uint16)[0])
    off = [256 + slot_offset(n_lane, esz, sign, lane, j) for j in range(n_lane)]
    if esz == 1:
        gaps = task[off].view(np.int8).astype(int)
    else:
        gaps = np.array([int(task[o:o + 2].view(np.uint16)[0]) for o in off])
    assert gaps[0] == 0
    return first + np.cumsum(gaps)


def slot_offset(n_lane, esz, sign, lane, j):
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


@pytest.mark.parametrize("rows", [0, 1, 4])
@pytest.mark.parametrize("K,N,S,split", [(2560, 16, 1536, 32), (6912, 16, 4096, 64), (6912, 16, 4160, 16), (2560, 16, 1536, 8)])
def test_delta_8bit_lanes_walk_their_own_run_in_a_bank_friendly_order(K, N, S, split, rows):
    """Each lane visits exactly the contiguous run of the sorted list the reference's gaps describe
    (main.cu:376-394: gap i = row i - row i-1), in an order whose steps fit a signed byte, and the 32
    lanes of a half-wavefront mostly sit on 32 different banks: row mod 32 for tiles of four bytes per
    row, (row / 4) mod 32 for the one-byte-per-row tile of streams packed with rows = 1."""
    _, pos, neg = sp.generate_ternary(K, N, S)
    d_ref, wrapped = oracle.delta8(pos)
    assert wrapped == 0
    pk, bits = sp.pack_delta(pos, neg, K, split, rows=rows)
    assert bits == 8
    if rows != 1:  # any hint but 1 is the plain stream
        assert (pk == sp.pack_delta(pos, neg, K, split)[0]).all()
    p2, n2 = sp.unpack_delta(pk, K, N, S, split, 8)  # the visiting order does not change what the stream holds
    assert (p2 == pos).all() and (n2 == neg).all()
    bank_shift = 2 if rows == 1 else 0
    L, G = min(split, 64), 64 // min(split, 64)
    n_lane = (S // 2) // split
    task_bytes = 256 + 128 * n_lane
    passes = slots = 0
    for t in range(N // G):
        task = pk[t * task_bytes:(t + 1) * task_bytes]
        for sign, lst in ((0, pos), (1, neg)):
            walks = []
            for lane in range(64):
                c, v = t * G + lane // L, lane % L
                w = lane_walk(task, n_lane, 1, sign, lane)
                run = lst[c, v * n_lane:(v + 1) * n_lane].astype(int)
                assert sorted(w) == list(run)
                assert np.abs(np.diff(w)).max(initial=0) <= 128
                if sign == 0 and n_lane > 1:  # the sorted run's gaps are the reference's delta bytes
                    assert (np.diff(run) == d_ref[c, v * n_lane + 1:(v + 1) * n_lane]).all()
                walks.append(w)
            walks = np.array(walks)
            for h in range(2):
                for j in range(n_lane):
                    passes += np.bincount((walks[32 * h:32 * h + 32, j] >> bank_shift) & 31, minlength=32).max()
                    slots += 1
    # sorted order needs ~3.5 passes per step; the schedule must stay well below 2
    assert passes <= 1.45 * slots, (passes / slots)


def test_delta_16bit_follows_sorted_order():
    K, N, S, split = 6912, 16, 256, 8
    _, pos, neg = sp.generate_ternary(K, N, S)
    pk, bits = sp.pack_delta(pos, neg, K, split)
    assert bits == 16
    n_lane = (S // 2) // split
    task_bytes = 256 + 256 * n_lane
    for c in (0, 9):
        task = pk[(c // 8) * task_bytes:(c // 8 + 1) * task_bytes]
        for v in (0, 7):
            w = lane_walk(task, n_lane, 2, 1, (c % 8) * 8 + v)
            assert (w == neg[c, v * n_lane:(v + 1) * n_lane]).all()


def test_i2s_word_and_stream():
    w = np.zeros(16, np.int8)
    w[0], w[2] = 1, -1
    assert sp.i2s_pack_word(w) == 0xAAA9AAAB == oracle.i2s_pack_word(w)
    rng = np.random.default_rng(0)
    for _ in range(50):
        w = rng.integers(-1, 2, 16).astype(np.int8)
        word = sp.i2s_pack_word(w)
        assert word == oracle.i2s_pack_word(w)
        assert (sp.i2s_decode_word(word) == w).all() and (oracle.i2s_decode_word(word) == w).all()
    for K, N, S in ((512, 32, 300), (2560, 16, 1536), (6912, 16, 4096), (304, 16, 100)):
        W, _, _ = sp.generate_ternary(K, N, S, dense=True)
        pk = sp.pack_i2s(W)
        Kp = (K + 255) // 256 * 256
        assert pk.nbytes == N * Kp // 4
        assert (sp.unpack_i2s(pk, K, N) == W).all()
        # same multiset of words as the oracle's plain order (plus all-zero-weight pad words)
        words = np.sort(pk.view(np.uint32))
        ref = np.sort(np.concatenate([oracle.i2s_pack(W).ravel(),
                                      np.full(N * (Kp - K) // 16, 0xAAAAAAAA, np.uint32)]))
        assert (words == ref).all()


def test_i2s_rejects_non_ternary():
    W = np.zeros((16, 64), np.int8)
    W[3, 5] = 2
    with pytest.raises(sp.SptmmError):
        sp.pack_i2s(W)


def test_random_shapes_round_trip_or_are_refused():
    """300 seeded shapes, valid and invalid alike: every packer either refuses with a status code or
    round-trips exactly (the same loop runs clean under AddressSanitizer / UBSan on a host-only build)."""
    rng = np.random.default_rng(7)
    packed = refused = 0
    for it in range(300):
        K = 16 * int(rng.integers(1, 40))
        N = int(rng.choice([16, 17, 32, 48])) if rng.random() < 0.3 else 16 * int(rng.integers(1, 5))
        S = int(rng.integers(0, K + 4))
        if rng.random() < 0.8:
            S -= S % 2
        split = int(rng.choice([4, 8, 16, 32, 64, 128, 256, 512, 24]))
        try:
            _, pos, neg = sp.generate_ternary(K, N, S)
        except sp.SptmmError as e:
            assert e.code == -1
            refused += 1
            continue
        try:
            buf = sp.pack_u16(pos, neg, K, split)
            p2, n2 = sp.unpack_u16(buf, K, N, S, split)
            assert (np.sort(p2, 1) == pos).all() and (np.sort(n2, 1) == neg).all()
            packed += 1
        except sp.SptmmError as e:
            assert e.code == -1
            refused += 1
        try:
            buf, bits = sp.pack_delta(pos, neg, K, split)
            p2, n2 = sp.unpack_delta(buf, K, N, S, split, bits)
            assert (p2 == pos).all() and (n2 == neg).all()
            packed += 1
        except sp.SptmmError as e:
            assert e.code == -1
            refused += 1
        W = sp.generate_ternary_iid(K, N, it, float(rng.random() * 0.6), float(rng.random() * 0.4))
        for kind in (sp.KIND_U16, sp.KIND_DELTA):
            try:
                buf, meta = sp.pack_ragged(W, kind, split)
                assert (sp.unpack_ragged(buf, K, N, kind, split, meta["bits"]) == W).all()
                packed += 1
            except sp.SptmmError as e:
                assert e.code == -1
                refused += 1
    assert packed > 200 and refused > 200, (packed, refused)


def test_non_positive_shapes_are_refused_before_anything_is_read():
    """Negative or zero K, N, S reach every packer with buffers sized for a small valid shape: each call must
    return a status code without touching memory beyond them (the same loop runs under AddressSanitizer)."""
    L = sp.lib()
    pos = np.zeros((16, 16), np.uint16)
    neg = np.ones((16, 16), np.uint16)
    W = np.zeros((16, 64), np.int8)
    out = np.zeros(1 << 16, np.uint8)
    P = lambda a: a.ctypes.data
    import ctypes as C

    for K, N, S in [(64, -16, 32), (64, 16, -32), (-64, 16, 32), (0, 16, 32), (64, 0, 32), (64, 16, 0), (64, -16, -32),
                    (-64, -16, -32), (64, 16, -2), (64, -1, 32)]:
        for split in (8, 16, 64):
            assert L.sptmm_pack_u16(C.c_void_p(P(pos)), C.c_void_p(P(neg)), K, N, S, split, C.c_void_p(P(out))) == -1
            assert L.sptmm_unpack_u16(C.c_void_p(P(out)), K, N, S, split, C.c_void_p(P(pos)), C.c_void_p(P(neg))) == -1
            for bits in (8, 16):
                assert L.sptmm_pack_delta(C.c_void_p(P(pos)), C.c_void_p(P(neg)), K, N, S, split, bits, C.c_void_p(P(out))) == -1
                assert L.sptmm_unpack_delta(C.c_void_p(P(out)), K, N, S, split, bits, C.c_void_p(P(pos)), C.c_void_p(P(neg))) == -1
                assert N > 0 and S > 0 or L.sptmm_pack_delta_bytes(N, S, split, bits) == 0  # (takes no K)
            if N <= 0 or S <= 0:
                assert L.sptmm_delta_bits(C.c_void_p(P(pos)), C.c_void_p(P(neg)), N, S, split) == -1
                assert L.sptmm_pack_u16_bytes(N, S, split) == 0
            assert L.sptmm_generate_ternary(K, N, S, None, C.c_void_p(P(pos)), C.c_void_p(P(neg))) == -1
            assert L.sptmm_lists_from_dense(C.c_void_p(P(W)), K, N, S, C.c_void_p(P(pos)), C.c_void_p(P(neg))) == -1
    for K, N in [(-64, 16), (64, -16), (0, 16), (64, 0), (-16, -16)]:
        for kind in (sp.KIND_U16, sp.KIND_DELTA):
            assert L.sptmm_pack_ragged_bytes(C.c_void_p(P(W)), K, N, kind, 32, None, None, None, None, None) == 0
            assert L.sptmm_pack_ragged(C.c_void_p(P(W)), K, N, kind, 32, 8, C.c_void_p(P(out))) == -1
        assert L.sptmm_pack_i2s_bytes(K, N) == 0
        assert L.sptmm_pack_i2s(C.c_void_p(P(W)), K, N, C.c_void_p(P(out))) == -1


def test_automatic_split_k_is_valid_and_follows_the_measured_rule():
    """split_k = 0 in the upload calls: 30-70 entries per lane where the matrix is wide enough for two tasks per
    compute unit, shorter lanes (down to 24 entries) where it is not; always a split the packers accept."""
    want = {(sp.KIND_U16, 2560, 4096): 32, (sp.KIND_DELTA, 2560, 4096): 32, (sp.KIND_U16, 640, 1536): 32, (sp.KIND_U16, 2560, 1536): 16,
            (sp.KIND_U16, 6912, 1536): 16, (sp.KIND_U16, 5120, 8320): 64, (sp.KIND_DELTA, 5120, 8320): 64, (sp.KIND_U16, 128, 4096): 64,
            (sp.KIND_DELTA, 128, 4096): 64, (sp.KIND_U16, 2560, 4160): 32, (sp.KIND_U16, 640, 4096): 64, (sp.KIND_U16, 768, 256): 8,
            (sp.KIND_DELTA, 768, 512): 8}
    for (kind, N, S), split in want.items():
        assert sp.choose_split_k(kind, N, S, 256) == split, (kind, N, S)
    rng = np.random.default_rng(3)
    for _ in range(300):
        N = 16 * int(rng.integers(1, 900))
        S = 2 * int(rng.integers(1, 5000))
        for kind in (sp.KIND_U16, sp.KIND_DELTA):
            try:
                s = sp.choose_split_k(kind, N, S, int(rng.choice([0, 64, 256, 304])))
            except sp.SptmmError as e:
                assert e.code == -1 and all((S // 2) % x for x in (8, 16, 32, 64, 128, 256)[: 6 if kind == sp.KIND_U16 else 4])
                continue
            assert s in (8, 16, 32, 64, 128, 256)[: 6 if kind == sp.KIND_U16 else 4] and (S // 2) % s == 0 and N % max(1, 64 // s) == 0
            n = sp.lib().sptmm_pack_u16_bytes(N, S, s) if kind == sp.KIND_U16 else sp.lib().sptmm_pack_delta_bytes(N, S, s, 8)
            assert n > 0
    for bad in ((sp.KIND_I2S, 64, 64), (sp.KIND_U16, 0, 64), (sp.KIND_U16, 64, 0), (sp.KIND_U16, 64, 31), (sp.KIND_U16, -16, 64)):
        with pytest.raises(sp.SptmmError):
            sp.choose_split_k(*bad)


def test_seeded_normal_activations_are_box_muller_over_xorshift32():
    """sptmm_make_x_normal against the same recipe in numpy / Python: pairs (u1, u2) from consecutive xorshift32 draws,
    r = sqrt(-2 ln u1), values r cos(2 pi u2), r sin(2 pi u2); the fp16 output is the fp32 one rounded to nearest even."""
    import math

    def xs(s):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        return s

    seed, n = 0xC0FFEE ^ 3, 41
    st, want = seed, []
    while len(want) < n:
        st = xs(st)
        u1 = (st + 1.0) / 4294967297.0
        st = xs(st)
        u2 = st / 4294967296.0
        r = math.sqrt(-2.0 * math.log(u1))
        want += [r * math.cos(6.283185307179586 * u2), r * math.sin(6.283185307179586 * u2)]
    want = np.array(want[:n], np.float64)
    x32 = sp.make_x_normal(seed, 1, n, np.float32)[0]
    x16 = sp.make_x_normal(seed, 1, n, np.float16)[0]
    assert np.allclose(x32, want, rtol=1e-6, atol=1e-7)
    assert (x16 == x32.astype(np.float16)).all()
    big = sp.make_x_normal(7, 64, 4096, np.float32)
    assert abs(big.mean()) < 0.01 and abs(big.std() - 1.0) < 0.01
