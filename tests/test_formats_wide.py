"""Wide streams (K-tiled, 16-byte slots): the host-side format, pinned without a GPU.

pack -> unpack must give back the matrix for every kind, split, K-tile and gap width; the stream's own
header and count tables must agree with the closed forms; what the documented walk of a task visits must
be the column's nonzeros (that walk is what sptmm_unpack_wide does, lane by lane as the kernel would)."""
import numpy as np
import pytest

import sptmm_amd as sp


def pos_of(r):
    return r ^ ((r >> 4) & 15)


@pytest.mark.parametrize("kind", [sp.KIND_U16, sp.KIND_DELTA])
@pytest.mark.parametrize("split", [8, 16, 32, 64])
@pytest.mark.parametrize("K,N,k_tile", [(64, 16, 64), (512, 48, 512), (512, 48, 128), (1024, 32, 400 // 16 * 16), (2560, 64, 1280)])
def test_round_trip_iid_matrices(kind, split, K, N, k_tile):
    for seed, (pp, pn) in enumerate([(0.3, 0.3), (0.02, 0.01), (0.0, 0.0), (0.5, 0.5), (0.9, 0.0)]):
        W = sp.generate_ternary_iid(K, N, 17 * seed + split, pp, pn)
        buf, meta = sp.pack_wide(W, kind, split, k_tile)
        assert meta["nnz"] == int((W != 0).sum())
        assert (sp.unpack_wide(buf, K, N) == W).all(), (seed, meta)
        hdr = buf[:256].view(np.uint32)
        P = -(-K // k_tile)
        assert hdr[0] == 0x57545053 and hdr[1] == P and hdr[2] == k_tile and hdr[3] == K and hdr[4] == N
        assert hdr[5] == kind and hdr[6] == meta["bits"] and hdr[7] == split
        assert meta["read_bytes"] <= len(buf)
        esz = 2 if kind == sp.KIND_U16 else meta["bits"] // 8
        tasks = N // (64 // split)
        for p in range(P):
            off, stride, n_min, n_max = (int(x) for x in hdr[8 + 4 * p: 12 + 4 * p])
            assert off % 256 == 0 and stride == (256 if kind == sp.KIND_DELTA else 0) + 128 * esz * n_max
            pre = buf[off:off + 16].view(np.uint32)
            counts = buf[off + 16: off + 16 + 2 * tasks].view(np.uint16)
            assert pre[0] == 0x52545053 and pre[1] == tasks and pre[2] == n_max and pre[3] == n_min
            assert counts.min() == n_min and counts.max() == n_max


def test_balanced_benchmark_matrix_two_k_tiles_and_padding_overhead():
    """The seeded benchmark generator at a config-4-like density, cut into two K-tiles: padding (lists that do not
    split evenly over lanes and tiles) stays within a few percent of 2 bytes per nonzero."""
    K, N, S = 1728, 64, 1040
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    for kind, per_entry in ((sp.KIND_U16, 2.0), (sp.KIND_DELTA, 1.0)):
        buf, meta = sp.pack_wide(W, kind, 32, 864)
        assert (sp.unpack_wide(buf, K, N) == W).all()
        assert meta["bits"] == (0 if kind == sp.KIND_U16 else 8)
        assert meta["read_bytes"] <= 1.12 * per_entry * S * N + 512 + 2 * (256 + 2 * N) + (2 * 256 * (N // 2) if kind == sp.KIND_DELTA else 0)


def test_u16_fields_are_positions_and_banks_are_spread():
    """u16 wide stream: every field is position << 2; per LDS pass (the 16 lanes a 16-byte read serves together:
    {0-3, 12-15, 20-23, 24-27}, {4-11, 16-19, 28-31} and both + 32) and slot the positions fall on distinct bank groups
    (position mod 16) nearly always: at most 1.35 cycles per pass on a random matrix."""
    K, N, split = 2048, 32, 32
    W = sp.generate_ternary_iid(K, N, 5, 0.3, 0.3)
    buf, meta = sp.pack_wide(W, sp.KIND_U16, split, K)
    hdr = buf[:256].view(np.uint32)
    off, stride, n_min, n_max = (int(x) for x in hdr[8:12])
    tasks = N // 2
    counts = buf[off + 16: off + 16 + 2 * tasks].view(np.uint16)
    base = off + (16 + 2 * tasks + 255) // 256 * 256
    passes = slots = 0
    for t in range(tasks):
        n = int(counts[t])
        task = buf[base + t * stride: base + t * stride + 256 * n].view(np.uint16)
        assert (task & 3 == 0).all() and (task >> 2).max() < K + 64
        full = n // 8
        rounds = task[: full * 1024].reshape(full, 2, 64, 8)  # [round][sign][lane][entry]
        for d in range(4):
            lanes = [x + 32 * (d >> 1) for x in ((0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27) if d % 2 == 0 else
                                                  (4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31))]
            grp = (rounds[:, :, lanes, :] >> 2) & 15  # bank group per lane of one LDS pass
            for r in range(full):
                for s in range(2):
                    for e in range(8):
                        passes += np.bincount(grp[r, s, :, e], minlength=16).max()
                        slots += 1
    assert passes / slots <= 1.35, passes / slots


def test_gap_stream_walk_and_16_bit_fallback():
    K, N = 4096, 16
    dense = sp.generate_ternary_iid(K, N, 9, 0.3, 0.3)
    buf, meta = sp.pack_wide(dense, sp.KIND_DELTA, 16, 2048)
    assert meta["bits"] == 8 and (sp.unpack_wide(buf, K, N) == dense).all()
    sparse = sp.generate_ternary_iid(K, N, 9, 0.012, 0.012)
    buf, meta = sp.pack_wide(sparse, sp.KIND_DELTA, 16, 2048)
    assert meta["bits"] == 16 and (sp.unpack_wide(buf, K, N) == sparse).all()
    with pytest.raises(sp.SptmmError) as e:
        sp.pack_wide(sparse, sp.KIND_DELTA, 16, 2048, bits=8)
    assert "8 bits" in str(e.value)
    buf16, meta16 = sp.pack_wide(dense, sp.KIND_DELTA, 16, 2048, bits=16)
    assert meta16["bits"] == 16 and (sp.unpack_wide(buf16, K, N) == dense).all()


def test_k_tile_choice_and_refusals():
    assert sp.wide_k_tile(13824, 160 * 1024) == 6912        # two tiles of (6912 + 64) * 16 = 111,616 bytes
    assert sp.wide_k_tile(6912, 160 * 1024) == 6912         # one tile
    assert sp.wide_k_tile(2560, 64 * 1024) == 2560
    assert sp.wide_k_tile(40960, 160 * 1024) % 16 == 0 and -(-40960 // sp.wide_k_tile(40960, 160 * 1024)) == 5
    W = np.zeros((16, 64), np.int8)
    for bad in (dict(kind=sp.KIND_I2S), dict(split=128), dict(split=12), dict(k_tile=24), dict(k_tile=0), dict(k_tile=-16)):
        a = dict(kind=sp.KIND_U16, split=8, k_tile=64)
        a.update(bad)
        with pytest.raises(sp.SptmmError):
            sp.pack_wide(W, a["kind"], a["split"], a["k_tile"])
    W[0, 0] = 2
    with pytest.raises(sp.SptmmError):
        sp.pack_wide(W, sp.KIND_U16, 8, 64)
    with pytest.raises(sp.SptmmError):
        sp.pack_wide(np.zeros((16, 16 * 17), np.int8), sp.KIND_U16, 8, 16)   # seventeen K-tiles
    good, _ = sp.pack_wide(np.zeros((16, 64), np.int8), sp.KIND_U16, 8, 64)
    corrupt = good.copy()
    corrupt[0] ^= 1
    with pytest.raises(sp.SptmmError):
        sp.unpack_wide(corrupt, 64, 16)
    with pytest.raises(sp.SptmmError):
        sp.unpack_wide(good, 128, 16)


def test_positions_stay_inside_their_block_of_16_rows():
    r = np.arange(1 << 16)
    p = pos_of(r)
    assert (p >> 4 == r >> 4).all() and (pos_of(p) == r).all()
    # 16 consecutive blocks written row by row touch 16 different bank groups at every step
    for c in range(16):
        assert len({int(pos_of(16 * item + c)) & 15 for item in range(16)}) == 16
