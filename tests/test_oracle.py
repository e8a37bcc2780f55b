"""Pins the CPU oracle (oracle/sptmm_oracle.c) from outside.

The reference keeps no golden vectors and never reads a result back, so each
oracle function is pinned by something it does not share code with:
published RNG values, an independent numpy generator (tests/golden), closed
forms, and brute-force int64 matmuls.
"""
import hashlib
import json
import os

import numpy as np
import pytest

import oracle


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.fixture(scope="module")
def kats(golden_dir):
    with open(os.path.join(golden_dir, "generator_kats.json")) as f:
        return json.load(f)


def test_xorshift32_published_sequence(kats):
    # seed 1 -> 270369, 67634689, ... is the sequence printed in Marsaglia-style
    # xorshift32 (13,17,5) references.
    for seed, want in kats["xorshift32"].items():
        assert oracle.xorshift32_seq(int(seed), 4) == want


def test_first_swaps_column0(kats):
    seq = oracle.xorshift32_seq(0xCAFEBABE ^ 0, 2)
    got = [[6911, seq[0] % 6912], [6910, seq[1] % 6911]]
    assert got == kats["first_swaps_col0_K6912"]


def test_generator_matches_independent_numpy(kats):
    for e in kats["matrices"]:
        W, pos, neg = oracle.generate(e["K"], e["N"], e["S"])
        assert sha(W) == e["sha256_W_colmajor"], (e["K"], e["N"], e["S"])
        assert sha(pos) == e["sha256_pos"] and sha(neg) == e["sha256_neg"]
        assert pos[0, :8].tolist() == e["pos_col0_head"]
        assert neg[0, :8].tolist() == e["neg_col0_head"]


@pytest.mark.parametrize("K,N,S", [(64, 16, 32), (512, 48, 256), (2560, 64, 1536)])
def test_generator_invariants(K, N, S):
    W, pos, neg = oracle.generate(K, N, S)
    half = S // 2
    assert ((W == 1).sum(axis=1) == half).all() and ((W == -1).sum(axis=1) == half).all()
    assert (np.diff(pos.astype(int), axis=1) > 0).all() and (np.diff(neg.astype(int), axis=1) > 0).all()
    assert pos.max() < K and neg.max() < K
    # scatter(lists) == dense
    R = np.zeros_like(W)
    for c in range(N):
        R[c, pos[c]] += 1
        R[c, neg[c]] -= 1
    assert (R == W).all()
    # columns differ (different seeds)
    assert len({sha(W[c]) for c in range(N)}) == N


@pytest.mark.parametrize("P", [8, 16, 32])
def test_split_layout_is_the_stated_permutation(P):
    K, N, S = 512, 32, 256
    _, pos, _ = oracle.generate(K, N, S, dense=False)
    half = S // 2
    out = oracle.split_layout(pos, P)
    want = pos.reshape(N, half // P, P).transpose(1, 0, 2).reshape(-1)  # [chunk][col][lane]
    assert (out == want).all()


def test_delta_cumsum_and_wrap_count():
    K, N, S = 2560, 32, 1536
    _, pos, neg = oracle.generate(K, N, S, dense=False)
    for lst in (pos, neg):
        d, wrapped = oracle.delta8(lst)
        assert wrapped == 0
        assert (np.cumsum(d.astype(np.int64), axis=1) == lst).all()
        d16 = oracle.delta16(lst)
        assert (np.cumsum(d16.astype(np.int64), axis=1) == lst).all()
    # a sparse column forces gaps above 255: the byte format must report them
    _, pos, _ = oracle.generate(6912, 16, 32, dense=False)
    d, wrapped = oracle.delta8(pos)
    big = (np.diff(np.concatenate([np.zeros((16, 1), int), pos.astype(int)], axis=1), axis=1) > 255).sum()
    assert wrapped == big and big > 0


def test_delta_div256_layout():
    N, half = 16, 640  # 2.5 chunks -> ragged tail
    rng = np.random.default_rng(1)
    d = rng.integers(0, 256, (N, half), dtype=np.uint8)
    out = oracle.delta_div256(d).reshape(3, N, 256)
    for ch in range(3):
        n = min(256, half - ch * 256)
        assert (out[ch, :, :n] == d[:, ch * 256: ch * 256 + n]).all()
        assert (out[ch, :, n:] == 0).all()


SHAPES = [(64, 16, 32, 1), (512, 32, 256, 3), (2560, 64, 1536, 4), (6912, 32, 4096, 2)]


@pytest.mark.parametrize("K,N,S,M", SHAPES)
def test_sptmm_equals_bruteforce_int64(K, N, S, M):
    W, pos, neg = oracle.generate(K, N, S)
    X = np.random.default_rng(K + M).integers(-127, 128, (M, K), dtype=np.int8)
    want = (X.astype(np.int64) @ W.T.astype(np.int64)).astype(np.int32)
    assert (oracle.sptmm_i8(X, pos, neg) == want).all()
    assert (oracle.sptmm_i8_mt(X, pos, neg, 3) == want).all()
    assert (oracle.dense_i8(X, W) == want).all()


@pytest.mark.parametrize("split", [8, 16, 32])
def test_split_kernel_walk_equals_bruteforce(split):
    K, N, S, M = 512, 32, 256, 2
    W, pos, neg = oracle.generate(K, N, S)
    X = np.random.default_rng(split).integers(-127, 128, (M, K), dtype=np.int8)
    want = (X.astype(np.int64) @ W.T.astype(np.int64)).astype(np.int32)
    got = oracle.sptmm_split_i8(X, oracle.split_layout(pos, split), oracle.split_layout(neg, split),
                                N, S // 2, split)
    assert (got == want).all()


@pytest.mark.parametrize("K,N,S", [(2560, 32, 1536), (2560, 16, 1600), (6912, 16, 4096)])
def test_delta_kernel_walk_equals_bruteforce(K, N, S):
    W, pos, neg = oracle.generate(K, N, S)
    X = np.random.default_rng(S).integers(-127, 128, (2, K), dtype=np.int8)
    want = (X.astype(np.int64) @ W.T.astype(np.int64)).astype(np.int32)
    dp, wp = oracle.delta8(pos)
    dn, wn = oracle.delta8(neg)
    assert wp == 0 and wn == 0
    got = oracle.sptmm_delta_i8(X, oracle.delta_div256(dp), oracle.delta_div256(dn), N, S // 2)
    assert (got == want).all()


def test_special_inputs():
    K, N, S = 512, 32, 256
    W, pos, neg = oracle.generate(K, N, S)
    ones = np.ones((1, K), np.int8)
    assert (oracle.sptmm_i8(ones, pos, neg) == 0).all()  # balanced signs
    for k in (0, 17, K - 1):
        e = np.zeros((1, K), np.int8)
        e[0, k] = 1
        assert (oracle.sptmm_i8(e, pos, neg)[0] == W[:, k]).all()  # unit vector picks a row of W


def test_i2s_word_hand_kat():
    # weights (+1, 0, -1, 0, 0, ... 0): codes 3,2,1,2 then 2s.  Byte b holds elements
    # b, b+4, b+8, b+12 at bit pairs 0,2,4,6:  byte0 = 3|2<<2|2<<4|2<<6 = 0xAB,
    # byte1 = 0xAA, byte2 = 1|0xA8 = 0xA9, byte3 = 0xAA.
    w = np.zeros(16, np.int8)
    w[0], w[2] = 1, -1
    assert oracle.i2s_pack_word(w) == 0xAAA9AAAB
    assert (oracle.i2s_decode_word(0xAAA9AAAB) == w).all()
    # element 5 alone: byte 1, bit pair 1 -> code 3 there, code 2 elsewhere
    w = np.zeros(16, np.int8)
    w[5] = 1
    assert oracle.i2s_pack_word(w) == (0xAAAAAAAA | (1 << 10))


def test_i2s_roundtrip_and_gemv():
    K, N, S, M = 512, 32, 300, 3
    W, _, _ = oracle.generate(K, N, S)
    packed = oracle.i2s_pack(W)
    back = np.stack([np.concatenate([oracle.i2s_decode_word(int(x)) for x in packed[c]]) for c in range(N)])
    assert (back == W).all()
    X = np.random.default_rng(5).integers(-127, 128, (M, K), dtype=np.int8)
    want = (X.astype(np.int64) @ W.T.astype(np.int64)).astype(np.int32)
    assert (oracle.i2s_gemv(X, packed) == want).all()


def test_make_x_and_golden_outputs(kats):
    for e in kats["matrices"]:
        W, pos, neg = oracle.generate(e["K"], e["N"], e["S"], dense=False)
        for o in e["outputs"]:
            X = oracle.make_x_i8(o["x_seed"], o["M"], e["K"])
            assert X.min() >= -127 and sha(X) == o["sha256_X"]
            Cm = oracle.sptmm_i8_mt(X, pos, neg, 4)
            assert sha(Cm) == o["sha256_C"] and Cm[0, :8].tolist() == o["C_head"]


def test_f64_reference_matches_dense():
    K, N, S = 512, 16, 256
    W, pos, neg = oracle.generate(K, N, S)
    X = oracle.make_x_normal(3, 2, K, np.float16)
    want = X.astype(np.float64) @ W.T.astype(np.float64)
    assert np.allclose(oracle.sptmm_f64(X, pos, neg), want, rtol=0, atol=1e-9)


def test_quantise_and_rescale_known_answers():
    # s = 1 exactly when the row maximum is 127: q = rint(x), ties to even
    x = np.array([[0.5, 1.5, 2.5, -0.5, -1.5, 3.49, -3.51, 127.0]], np.float32)
    q, a = oracle.quantise_rows(x)
    assert a.tolist() == [127.0] and q.tolist() == [[0, 2, 2, 0, -2, 3, -4, 127]]
    # a row of zeros: the scale clamps at 1e-5, every q is 0
    q, a = oracle.quantise_rows(np.zeros((1, 4), np.float32))
    assert q.tolist() == [[0, 0, 0, 0]] and a[0] == np.float32(1e-5)
    # maximum 2: s = 63.5, 1.0 -> 63.5 -> 64 (tie to even), -2 -> -127
    q, a = oracle.quantise_rows(np.array([[1.0, -2.0, 0.0078125]], np.float32))
    assert q.tolist() == [[64, -127, 0]]
    y = oracle.rescale(np.array([[254, -127]]), np.array([127.0], np.float32), 0.5)
    assert y.tolist() == [[127.0, -63.5]]
    # bf16: 1 + 2^-8 is a tie between 1.0 and 1 + 2^-7 -> even (0x3f80); 1 + 3*2^-8 rounds up to 1 + 2^-6
    bits = oracle.bf16_bits(np.array([1.0, 1.00390625, 1.01171875, -2.5], np.float32))
    assert [hex(b) for b in bits] == ["0x3f80", "0x3f80", "0x3f82", "0xc020"]
