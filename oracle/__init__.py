"""CPU oracle for the SpTMM hot path -- TEST INFRASTRUCTURE ONLY.

ctypes front end of ``sptmm_oracle.c`` (a plain-C restatement of the reference
benchmark's arithmetic; each C function cites the reference lines it follows)
plus a few numpy helpers for the floating-point activation variants, which the
reference does not have.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package, and only as the checker.  The shipped
library (``sptmm_amd``) never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile sptmm_oracle.c with the committed Makefile."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _SO


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        L.orc_xorshift32.restype = C.c_uint32
        L.orc_i2s_pack_word.restype = C.c_uint32
        for name in ("orc_generate", "orc_delta8", "orc_lists_from_column"):
            getattr(L, name).restype = C.c_int
        _lib = L
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def xorshift32_seq(seed: int, n: int) -> list[int]:
    st = C.c_uint32(seed)
    return [int(lib().orc_xorshift32(C.byref(st))) for _ in range(n)]


def gen_column(K: int, S: int, col: int) -> np.ndarray:
    w = np.empty(K, np.int8)
    lib().orc_gen_column(K, S, C.c_uint32(col), _p(w))
    return w


def generate(K: int, N: int, S: int, dense: bool = True):
    """-> (W dense [N][K] int8, i.e. column-major K x N, or None; pos [N][S/2]; neg [N][S/2])."""
    half = S // 2
    W = np.empty((N, K), np.int8) if dense else None
    pos = np.empty((N, half), np.uint16)
    neg = np.empty((N, half), np.uint16)
    bad = lib().orc_generate(K, N, S, _p(W) if dense else None, _p(pos), _p(neg))
    assert bad == 0, "W matrix corrupt"
    return W, pos, neg


def split_layout(lst: np.ndarray, P: int) -> np.ndarray:
    N, half = lst.shape
    out = np.empty(N * half, np.uint16)
    lib().orc_split_layout(_p(lst), N, half, P, _p(out))
    return out


def delta8(lst: np.ndarray):
    """-> (u8 gaps [N][half], number of gaps that did not fit a byte)."""
    N, half = lst.shape
    d = np.empty((N, half), np.uint8)
    wrapped = lib().orc_delta8(_p(lst), N, half, _p(d))
    return d, int(wrapped)


def delta16(lst: np.ndarray) -> np.ndarray:
    N, half = lst.shape
    d = np.empty((N, half), np.uint16)
    lib().orc_delta16(_p(lst), N, half, _p(d))
    return d


def delta_div256(d: np.ndarray) -> np.ndarray:
    N, half = d.shape
    chunks = (half + 255) // 256
    out = np.zeros(chunks * N * 256, np.uint8)
    lib().orc_delta_div256(_p(d), N, half, _p(out))
    return out


def sptmm_i8(X: np.ndarray, pos: np.ndarray, neg: np.ndarray) -> np.ndarray:
    M, K = X.shape
    N, half = pos.shape
    out = np.empty((M, N), np.int32)
    lib().orc_sptmm_i8(_p(X), M, K, _p(pos), _p(neg), N, half, _p(out))
    return out


def sptmm_i8_mt(X: np.ndarray, pos: np.ndarray, neg: np.ndarray, threads: int, out=None) -> np.ndarray:
    M, K = X.shape
    N, half = pos.shape
    if out is None:
        out = np.empty((M, N), np.int32)
    lib().orc_sptmm_i8_mt(_p(X), M, K, _p(pos), _p(neg), N, half, _p(out), threads)
    return out


def sptmm_split_i8(X, pos_div, neg_div, N, half, split) -> np.ndarray:
    M, K = X.shape
    out = np.empty((M, N), np.int32)
    lib().orc_sptmm_split_i8(_p(X), M, K, _p(pos_div), _p(neg_div), N, half, split, _p(out))
    return out


def sptmm_delta_i8(X, dpos256, dneg256, N, half) -> np.ndarray:
    M, K = X.shape
    out = np.empty((M, N), np.int32)
    lib().orc_sptmm_delta_i8(_p(X), M, K, _p(dpos256), _p(dneg256), N, half, _p(out))
    return out


def i2s_pack_word(w16) -> int:
    a = np.ascontiguousarray(w16, np.int8)
    assert a.size == 16
    return int(lib().orc_i2s_pack_word(_p(a)))


def i2s_decode_word(word: int) -> np.ndarray:
    out = np.empty(16, np.int8)
    lib().orc_i2s_decode_word(C.c_uint32(word), _p(out))
    return out


def i2s_pack(W: np.ndarray) -> np.ndarray:
    N, K = W.shape
    out = np.empty((N, K // 16), np.uint32)
    lib().orc_i2s_pack(_p(W), K, N, _p(out))
    return out


def i2s_gemv(X: np.ndarray, packed: np.ndarray) -> np.ndarray:
    M, K = X.shape
    N = packed.shape[0]
    out = np.empty((M, N), np.int32)
    lib().orc_i2s_gemv(_p(X), M, K, _p(packed), N, _p(out))
    return out


def dense_i8(X: np.ndarray, W: np.ndarray) -> np.ndarray:
    M, K = X.shape
    N = W.shape[0]
    out = np.empty((M, N), np.int32)
    lib().orc_dense_i8(_p(X), M, K, _p(W), N, _p(out))
    return out


def make_x_i8(seed: int, M: int, K: int) -> np.ndarray:
    X = np.empty((M, K), np.int8)
    lib().orc_make_x_i8(C.c_uint32(seed), C.c_size_t(M * K), _p(X))
    return X


# ---- floating-point activation variants (not in the reference; the benchmark
# definition adds them).  Reference value = gather-sum carried in float64 over
# the exactly-representable fp16/fp32 inputs (main.cu:577-593 semantics).
def sptmm_f64(X: np.ndarray, pos: np.ndarray, neg: np.ndarray) -> np.ndarray:
    X64 = X.astype(np.float64)
    out = np.empty((X.shape[0], pos.shape[0]), np.float64)
    for m in range(X.shape[0]):
        out[m] = X64[m][pos].sum(axis=1) - X64[m][neg].sum(axis=1)
    return out


def make_x_normal(seed: int, M: int, K: int, dtype=np.float16) -> np.ndarray:
    """~N(0,1) activations, seeded, rounded to `dtype`."""
    rng = np.random.default_rng(seed)
    return rng.standard_normal((M, K)).astype(dtype)


# ---- the wrapper BitNet inference puts around the integer GEMV (no reference code: the reference
# ---- only passes an unused scale, main.cu:1862).  Every step is one correctly rounded float32
# ---- operation, so an implementation that follows the same order matches bit for bit.
def bf16_bits(x32: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns (round to nearest even), as uint16."""
    b = np.ascontiguousarray(x32, np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def quantise_rows(xf: np.ndarray):
    """Per row: a = max(max|x|, 1e-5), s = 127 / a, q = clip(rint(x * s), -127, 127) (round-half-even).
    -> (q int8 [M][K], a float32 [M])."""
    xf = xf.astype(np.float32)
    a = np.maximum(np.abs(xf).max(axis=1), np.float32(1e-5)).astype(np.float32)
    s = (np.float32(127.0) / a).astype(np.float32)
    q = np.clip(np.rint(xf * s[:, None]), -127, 127).astype(np.int8)
    return q, a


def rescale(C: np.ndarray, a: np.ndarray, w_scale: float) -> np.ndarray:
    """y = float32(C) * (a / 127) * w_scale, evaluated in this order in float32."""
    inv = (a / np.float32(127.0)).astype(np.float32)
    return ((C.astype(np.float32) * inv[:, None]).astype(np.float32) * np.float32(w_scale)).astype(np.float32)

