"""Weight files (sptmm_weights_save / _load): round trips on the GPU, refusals without one."""
import os
import sys

import numpy as np
import pytest

import oracle
import sptmm_amd as sp

HEADER = 120          # the fixed header
PLANS = 8 * 8 * 4     # version 3: the stream's launch plans (8 kinds of call x 8 int32) between header and stream
DATA = HEADER + PLANS


def test_load_refuses_what_is_not_a_weight_file(tmp_path):
    # these are rejected from the header alone, before any device call
    p = tmp_path / "x.sptmm"
    with pytest.raises(sp.SptmmError):
        sp.Weights.load(str(p))  # missing
    p.write_bytes(b"")
    with pytest.raises(sp.SptmmError):
        sp.Weights.load(str(p))
    p.write_bytes(b"NOTSPTMM" + bytes(200))
    with pytest.raises(sp.SptmmError):
        sp.Weights.load(str(p))
    hdr = bytearray(b"SPTMMW1\0" + (120).to_bytes(4, "little") + (1).to_bytes(4, "little") + bytes(104))
    p.write_bytes(bytes(hdr))  # right magic, kind 0
    with pytest.raises(sp.SptmmError) as e:
        sp.Weights.load(str(p))
    assert "kind" in str(e.value)


@pytest.mark.gpu
def test_save_load_round_trip_every_encoding(tmp_path):
    sp.device_init(0)
    K, N, S = 2560, 640, 1536
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    Wi = sp.generate_ternary_iid(K, N, 3, 0.3, 0.3)
    Ws = sp.generate_ternary_iid(K, N, 4, 0.03, 0.03)
    X = oracle.make_x_i8(7, 4, K)
    makers = {
        "u16": lambda: sp.Weights.upload_u16(pos, neg, K, 32),
        "u16_256": lambda: sp.Weights.upload_u16(pos, neg, K, 256),
        "delta8": lambda: sp.Weights.upload_delta(pos, neg, K, 32),
        "i2s": lambda: sp.Weights.upload_i2s(W),
        "ragged_u16": lambda: sp.Weights.upload_dense(Wi, sp.KIND_U16, 32),
        "ragged_delta": lambda: sp.Weights.upload_dense(Wi, sp.KIND_DELTA, 16),
        "ragged_sparse_delta": lambda: sp.Weights.upload_dense(Ws, sp.KIND_DELTA, 16, rows=1),   # 8-bit gaps over zero slots
        "ragged_wide_u16": lambda: sp.Weights.upload_wide(Wi, sp.KIND_U16, 32),
        "ragged_wide_delta": lambda: sp.Weights.upload_wide(Wi, sp.KIND_DELTA, 16),
    }
    for name, mk in makers.items():
        print("weight file", name, flush=True)
        sys.stdout.flush()
        w = mk()
        want = w.matmul(X)
        path = str(tmp_path / (name + ".sptmm"))
        w.save(path)
        assert os.path.getsize(path) == DATA + w.nbytes
        v = sp.Weights.load(path)
        assert v.info == w.info and v.nbytes == w.nbytes
        assert (v.matmul(X) == want).all()
        assert (want == oracle.dense_i8(X, Ws if "sparse" in name else Wi if name.startswith("ragged") else W)).all()
        w.free()
        v.free()
        # one flipped stream byte, a truncated file and trailing bytes are all refused
        raw = bytearray(open(path, "rb").read())
        raw[DATA + len(raw) // 3] ^= 0x40
        open(path, "wb").write(bytes(raw))
        with pytest.raises(sp.SptmmError) as e:
            sp.Weights.load(path)
        assert "checksum" in str(e.value) or "corrupt" in str(e.value)
        raw[DATA + len(raw) // 3] ^= 0x40
        raw[HEADER + 5] ^= 1  # ... and so is a flipped byte of the plans
        open(path, "wb").write(bytes(raw))
        with pytest.raises(sp.SptmmError) as e:
            sp.Weights.load(path)
        assert "checksum" in str(e.value)
        raw[HEADER + 5] ^= 1
        open(path, "wb").write(bytes(raw[:-5]))
        with pytest.raises(sp.SptmmError):
            sp.Weights.load(path)
        open(path, "wb").write(bytes(raw) + b"\0")
        with pytest.raises(sp.SptmmError):
            sp.Weights.load(path)
        # a header that disagrees with the stream size
        bad = bytearray(raw)
        bad[20:24] = (K + 16).to_bytes(4, "little")  # K
        open(path, "wb").write(bytes(bad))
        with pytest.raises(sp.SptmmError):
            sp.Weights.load(path)


def _fnv1a(data: bytes) -> int:
    h = 1469598103934665603
    for b in data:
        h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


@pytest.mark.gpu
def test_version_1_i2s_file_is_retiled_on_load(tmp_path):
    """Files of format version 1 kept the 16-byte unit of (column c, quarter q) at position 4c + q of its 1 KiB
    tile; the stream now keeps it at 16q + c.  A version-1 file is rebuilt here from a fresh one and must load
    to the same matrix."""
    sp.device_init(0)
    K, N, S = 512, 48, 256
    W, pos, neg = sp.generate_ternary(K, N, S, dense=True)
    X = oracle.make_x_i8(3, 5, K)
    w = sp.Weights.upload_i2s(W)
    path = str(tmp_path / "new.sptmm")
    w.save(path)
    w.free()
    raw = bytearray(open(path, "rb").read())
    assert int.from_bytes(raw[12:16], "little") == 3
    stream = np.frombuffer(bytes(raw[DATA:]), np.uint8).reshape(-1, 4, 16, 16)     # [tile][q][c][16 bytes]
    old = np.ascontiguousarray(stream.transpose(0, 2, 1, 3)).tobytes()             # [tile][c][q][16 bytes]
    hdr = bytearray(raw[:120])
    hdr[12:16] = (1).to_bytes(4, "little")
    hdr[112:120] = bytes(8)
    hdr[112:120] = _fnv1a(bytes(hdr) + old).to_bytes(8, "little")
    p1 = str(tmp_path / "v1.sptmm")
    open(p1, "wb").write(bytes(hdr) + old)  # versions 1 and 2 have no plans behind the header
    v = sp.Weights.load(p1)
    assert (v.matmul(X) == oracle.dense_i8(X, W)).all()
    v.free()
    # version 2: the current tile order, still without plans
    hdr[12:16] = (2).to_bytes(4, "little")
    hdr[112:120] = bytes(8)
    hdr[112:120] = _fnv1a(bytes(hdr) + bytes(raw[DATA:])).to_bytes(8, "little")
    p2 = str(tmp_path / "v2.sptmm")
    open(p2, "wb").write(bytes(hdr) + bytes(raw[DATA:]))
    v = sp.Weights.load(p2)
    assert (v.matmul(X) == oracle.dense_i8(X, W)).all() and not any(v.get_plan(1, False).values())
    v.free()


@pytest.mark.gpu
def test_wide_file_with_a_bad_table_is_refused_although_its_checksum_holds(tmp_path):
    """The K-tiles' offsets, strides and per-task counts are what the kernel follows: a file whose checksum was
    recomputed over a damaged table must still not load."""
    sp.device_init(0)
    K, N = 2560, 64
    W = sp.generate_ternary_iid(K, N, 5, 0.3, 0.3)
    w = sp.Weights.upload_wide(W, sp.KIND_DELTA, 32)
    path = str(tmp_path / "wide.sptmm")
    w.save(path)
    X = oracle.make_x_i8(3, 16, K)
    v = sp.Weights.load(path)
    assert v.info == w.info and v.info["k_tile"] > 0 and (v.matmul(X) == oracle.dense_i8(X, W)).all()
    v.free()
    w.free()
    raw = bytearray(open(path, "rb").read())
    hdr = np.frombuffer(bytes(raw[DATA:DATA + 512]), np.uint32)
    off = int(hdr[8])
    damages = {
        "count above n_max": (DATA + off + 16, (65535).to_bytes(2, "little")),
        "offset past the stream": (DATA + 4 * 8, (len(raw)).to_bytes(4, "little")),
        "stride": (DATA + 4 * 9, (int(hdr[9]) + 128).to_bytes(4, "little")),
        "k_tile": (DATA + 4 * 2, (16320).to_bytes(4, "little")),
        "phases": (DATA + 4 * 1, (3).to_bytes(4, "little")),
    }
    for what, (at, val) in damages.items():
        bad = bytearray(raw)
        bad[at:at + len(val)] = val
        bad[112:120] = bytes(8)                      # the checksum covers the header with this field zero, the plans, then the stream
        bad[112:120] = _fnv1a(bytes(bad)).to_bytes(8, "little")
        open(path, "wb").write(bytes(bad))
        with pytest.raises(sp.SptmmError) as e:
            sp.Weights.load(path)
        assert "checksum" not in str(e.value), (what, str(e.value))
