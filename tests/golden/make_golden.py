"""Writes tests/golden/generator_kats.json.

An independent numpy restatement of the reference's weight generator
(main.cu:246-276 with the RNG of macro.cuh:69-76), vectorised over columns,
and of the output C = X.W as a dense int64 matmul.  It shares no code with
oracle/sptmm_oracle.c, so agreement between the two pins the exact matrix.
Run from the repo root:  python tests/golden/make_golden.py
"""
import hashlib
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def xorshift32_vec(state):
    state ^= (state << np.uint32(13))
    state ^= (state >> np.uint32(17))
    state ^= (state << np.uint32(5))
    return state


def generate(K, N, S):
    """Dense W as [N][K] int8 (column c of the K x N matrix is row c here)."""
    half = S // 2
    W = np.zeros((N, K), np.int8)
    W[:, :half] = -1
    W[:, half:S] = 1
    cols = np.arange(N)
    state = (np.uint32(0xCAFEBABE) ^ cols.astype(np.uint32)).astype(np.uint32)
    for i in range(K - 1, 0, -1):
        state = xorshift32_vec(state)
        j = (state % np.uint32(i + 1)).astype(np.int64)
        a = W[:, i].copy()
        W[:, i] = W[cols, j]
        W[cols, j] = a
    return W


def lists(W, S):
    N, K = W.shape
    half = S // 2
    pos = np.empty((N, half), np.uint16)
    neg = np.empty((N, half), np.uint16)
    for c in range(N):
        pos[c] = np.nonzero(W[c] == 1)[0]
        neg[c] = np.nonzero(W[c] == -1)[0]
    return pos, neg


def make_x(seed, M, K):
    """Seeded uniform int8 on [-127,127]: xorshift32 stream, r % 255 - 127."""
    out = np.empty(M * K, np.int8)
    s = seed
    for i in range(M * K):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        out[i] = (s % 255) - 127
    return out.reshape(M, K)


def generate_iid(K, N, seed, p_pos, p_neg):
    """Independent entries: per column a xorshift32 stream seeded seed ^ 0x9E3779B9*(col+1) (0 -> 1);
    entry = top 24 bits of the next state: below p_pos*2^24 -> +1, below (p_pos+p_neg)*2^24 -> -1."""
    state = (np.uint32(seed) ^ (np.uint32(0x9E3779B9) * np.arange(1, N + 1, dtype=np.uint32))).astype(np.uint32)
    state[state == 0] = 1
    t_pos, t_neg = np.uint32(int(p_pos * 16777216.0)), np.uint32(int((p_pos + p_neg) * 16777216.0))
    W = np.zeros((N, K), np.int8)
    for r in range(K):
        state = xorshift32_vec(state)
        u = state >> np.uint32(8)
        W[:, r] = np.where(u < t_pos, 1, np.where(u < t_neg, -1, 0))
    return W


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    shapes = [(64, 16, 32), (256, 32, 128), (2560, 640, 1536), (6912, 2560, 4096)]
    out = {
        "xorshift32": {
            "1": [270369, 67634689, 2647435461, 307599695],
            "3405691582": [2827483434, 2750467483, 4064143354, 2526188539],
            "3405691583": [2827213067, 2818100122, 1878085439, 2227636916],
        },
        "first_swaps_col0_K6912": [[6911, 5418], [6910, 59]],
        "matrices": [],
    }
    for K, N, S in shapes:
        W = generate(K, N, S)
        pos, neg = lists(W, S)
        entry = {
            "K": K, "N": N, "S": S,
            "sha256_W_colmajor": sha(W),
            "sha256_pos": sha(pos), "sha256_neg": sha(neg),
            "pos_col0_head": pos[0, :8].tolist(), "neg_col0_head": neg[0, :8].tolist(),
            "outputs": [],
        }
        for M in (1, 4):
            seed = 0xC0FFEE ^ M
            X = make_x(seed, M, K)
            Cm = X.astype(np.int64) @ W.T.astype(np.int64)
            assert np.abs(Cm).max() < 2**31
            Cm = Cm.astype(np.int32)
            entry["outputs"].append({"M": M, "x_seed": seed, "sha256_X": sha(X),
                                     "sha256_C": sha(Cm), "C_head": Cm[0, :8].tolist()})
        out["matrices"].append(entry)
        print(K, N, S, entry["sha256_W_colmajor"][:16])
    out["iid_matrices"] = []
    for K, N, seed, pp, pn in ((256, 16, 1, 0.3, 0.3), (2560, 640, 0xABCD, 0.35, 0.25), (6912, 2560, 0x2B, 0.3, 0.3)):
        W = generate_iid(K, N, seed, pp, pn)
        X = make_x(0xC0FFEE ^ 4, 4, K)
        Cm = (X.astype(np.int64) @ W.T.astype(np.int64)).astype(np.int32)
        out["iid_matrices"].append({"K": K, "N": N, "seed": seed, "p_pos": pp, "p_neg": pn, "sha256_W_colmajor": sha(W),
                                    "nnz": int((W != 0).sum()), "x_seed": 0xC0FFEE ^ 4, "M": 4, "sha256_C": sha(Cm),
                                    "C_head": Cm[0, :8].tolist()})
        print("iid", K, N, out["iid_matrices"][-1]["sha256_W_colmajor"][:16])
    with open(os.path.join(HERE, "generator_kats.json"), "w") as f:
        json.dump(out, f, indent=1)


if __name__ == "__main__":
    main()
