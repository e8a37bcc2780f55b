"""ctypes binding of include/sptmm.h (libsptmm.so, built in-tree by sptmm_amd.build)."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

__all__ = [
    "SptmmError", "lib", "lib_path", "device_init", "generate_ternary", "lists_from_dense", "make_x_i8", "make_x_normal",
    "pack_u16", "unpack_u16", "delta_bits", "pack_delta", "unpack_delta", "pack_i2s", "unpack_i2s", "pack_ragged", "unpack_ragged",
    "generate_ternary_iid", "dense_from_i2s_words", "choose_split_k", "wide_k_tile", "pack_wide", "unpack_wide",
    "i2s_pack_word", "i2s_decode_word", "Weights", "DeviceBuffer", "Stream", "Event", "copy_kernel", "read_kernel",
    "device_sync", "Graph", "measure_gemv", "measure_sequence", "Step", "SEQ_MODES", "PlanStruct", "gemv_i8_batched", "gemv_batched", "KIND_U16", "KIND_DELTA", "KIND_I2S", "EXPORTS",
]

KIND_U16, KIND_DELTA, KIND_I2S = 1, 2, 3
# modes of sptmm_measure_sequence
SEQ_MODES = {"launches": 0, "graph_chain": 1, "graph_branches": 2, "streams": 3, "batched_pairs": 4}
_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB = None

# every symbol include/sptmm.h declares
EXPORTS = [
    "sptmm_last_error", "sptmm_version", "sptmm_generate_ternary", "sptmm_lists_from_dense", "sptmm_make_x_i8", "sptmm_make_x_normal",
    "sptmm_pack_u16_bytes", "sptmm_pack_u16", "sptmm_unpack_u16", "sptmm_delta_bits", "sptmm_pack_delta_bytes",
    "sptmm_pack_delta", "sptmm_unpack_delta", "sptmm_i2s_pack_word", "sptmm_i2s_decode_word",
    "sptmm_pack_i2s_bytes", "sptmm_pack_i2s", "sptmm_unpack_i2s", "sptmm_pack_ragged_bytes", "sptmm_pack_ragged",
    "sptmm_unpack_ragged", "sptmm_generate_ternary_iid", "sptmm_dense_from_i2s_words", "sptmm_weights_upload_dense",
    "sptmm_choose_split_k", "sptmm_wide_k_tile", "sptmm_pack_wide_bytes", "sptmm_pack_wide", "sptmm_unpack_wide", "sptmm_weights_upload_wide",
    "sptmm_device_init",
    "sptmm_weights_upload_u16", "sptmm_weights_upload_u16_rows", "sptmm_weights_upload_delta", "sptmm_weights_upload_delta_rows", "sptmm_weights_upload_dense_rows",
    "sptmm_pack_delta_rows", "sptmm_pack_ragged_rows",
    "sptmm_weights_upload_i2s", "sptmm_weights_clone", "sptmm_weights_save", "sptmm_weights_load",
    "sptmm_weights_free", "sptmm_weights_info", "sptmm_weights_bytes", "sptmm_gemv_i8", "sptmm_gemv_f16",
    "sptmm_gemv_f32", "sptmm_gemv_q8", "sptmm_gemv_q8_ws", "sptmm_gemv_q8_workspace_bytes", "sptmm_gemv_q8_static", "sptmm_gemv_i8_scaled", "sptmm_gemv_i8_batched", "sptmm_gemv_batched", "sptmm_malloc", "sptmm_free", "sptmm_memcpy_h2d", "sptmm_memcpy_d2h", "sptmm_memset",
    "sptmm_stream_create", "sptmm_stream_destroy", "sptmm_stream_sync", "sptmm_device_sync",
    "sptmm_event_create", "sptmm_event_destroy", "sptmm_event_record", "sptmm_event_sync",
    "sptmm_event_elapsed_us", "sptmm_measure_gemv", "sptmm_copy_kernel", "sptmm_read_kernel",
    "sptmm_graph_begin", "sptmm_graph_end", "sptmm_graph_launch", "sptmm_graph_destroy",
    "sptmm_stream_wait_event", "sptmm_measure_sequence", "sptmm_weights_set_plan", "sptmm_weights_get_plan", "sptmm_weights_tune",
]


class SptmmError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("sptmm error %d: %s" % (code, msg))
        self.code = code


class DevInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_int),
                ("wave_size", C.c_int), ("lds_bytes_per_workgroup", C.c_int), ("l2_bytes", C.c_int),
                ("hbm_bytes", C.c_uint64), ("peak_hbm_gbps", C.c_double)]


class WInfo(C.Structure):
    _fields_ = [("kind", C.c_int), ("K", C.c_int), ("N", C.c_int), ("S", C.c_int), ("split_k", C.c_int),
                ("delta_bits", C.c_int), ("stream_bytes", C.c_uint64),
                ("ragged", C.c_int), ("nnz", C.c_uint64), ("k_tile", C.c_int), ("row_bytes", C.c_int), ("stones", C.c_int)]


class PlanStruct(C.Structure):
    """sptmm_plan: the launch shape of one kind of call on one stream (0 = the library's model)."""
    _fields_ = [("waves_per_wg", C.c_int), ("wgs_per_cu", C.c_int), ("tasks_per_wave", C.c_int), ("share_log", C.c_int), ("i2s_ct", C.c_int),
                ("reserved", C.c_int * 3)]
    NAMES = ("waves_per_wg", "wgs_per_cu", "tasks_per_wave", "share_log", "i2s_ct")


class Step(C.Structure):
    """sptmm_step: one GEMV of a sequence (see sptmm_measure_sequence)."""
    _fields_ = [("w", C.c_void_p), ("X_dev", C.c_void_p), ("C_dev", C.c_void_p), ("M", C.c_int), ("act", C.c_int), ("stage", C.c_int)]


def lib_path() -> str:
    return os.path.join(_PKG, "libsptmm.so")


def lib() -> C.CDLL:
    """The HIP library.  Raises if it has not been built: there is no fallback path."""
    global _LIB
    if _LIB is None:
        p = lib_path()
        if not os.path.exists(p):
            raise RuntimeError("%s is missing: build it with `python -m sptmm_amd.build` "
                               "(hipcc --offload-arch=gfx950); there is no CPU fallback" % p)
        L = C.CDLL(p)
        L.sptmm_last_error.restype = C.c_char_p
        L.sptmm_version.restype = C.c_char_p
        for n in ("sptmm_pack_u16_bytes", "sptmm_pack_delta_bytes", "sptmm_pack_i2s_bytes", "sptmm_weights_bytes",
                  "sptmm_pack_ragged_bytes", "sptmm_pack_wide_bytes"):
            getattr(L, n).restype = C.c_size_t
        L.sptmm_i2s_pack_word.restype = C.c_uint32
        L.sptmm_i2s_decode_word.restype = None
        L.sptmm_weights_free.restype = None
        L.sptmm_weights_free.argtypes = [C.c_void_p]
        L.sptmm_weights_bytes.argtypes = [C.c_void_p]
        L.sptmm_weights_info.argtypes = [C.c_void_p, C.POINTER(WInfo)]
        L.sptmm_weights_clone.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.sptmm_weights_save.argtypes = [C.c_void_p, C.c_char_p]
        L.sptmm_weights_load.argtypes = [C.c_char_p, C.POINTER(C.c_void_p)]
        for n in ("sptmm_gemv_i8", "sptmm_gemv_f16", "sptmm_gemv_f32"):
            getattr(L, n).argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        L.sptmm_gemv_q8.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p]
        L.sptmm_gemv_q8_ws.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.sptmm_gemv_q8_workspace_bytes.argtypes = [C.c_void_p, C.c_int]
        L.sptmm_gemv_q8_static.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p]
        L.sptmm_gemv_i8_scaled.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_void_p, C.c_void_p]
        L.sptmm_gemv_q8_workspace_bytes.restype = C.c_size_t
        L.sptmm_gemv_batched.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.sptmm_gemv_i8_batched.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        L.sptmm_malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        L.sptmm_free.argtypes = [C.c_void_p]
        L.sptmm_memcpy_h2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.sptmm_memcpy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.sptmm_memset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        L.sptmm_measure_gemv.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                         C.c_int, C.c_void_p, C.POINTER(C.c_double)]
        L.sptmm_copy_kernel.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.sptmm_read_kernel.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                        C.POINTER(C.c_double)]
        L.sptmm_make_x_i8.argtypes = [C.c_uint32, C.c_size_t, C.c_void_p]
        L.sptmm_make_x_normal.argtypes = [C.c_uint32, C.c_size_t, C.c_void_p, C.c_void_p]
        L.sptmm_generate_ternary_iid.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_double, C.c_double, C.c_void_p]
        for n in ("sptmm_stream_create", "sptmm_event_create"):
            getattr(L, n).argtypes = [C.POINTER(C.c_void_p)]
        for n in ("sptmm_stream_destroy", "sptmm_stream_sync", "sptmm_event_destroy", "sptmm_event_sync"):
            getattr(L, n).argtypes = [C.c_void_p]
        L.sptmm_event_record.argtypes = [C.c_void_p, C.c_void_p]
        L.sptmm_graph_begin.argtypes = [C.c_void_p]
        L.sptmm_graph_end.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.sptmm_graph_launch.argtypes = [C.c_void_p, C.c_void_p]
        L.sptmm_graph_destroy.argtypes = [C.c_void_p]
        L.sptmm_event_elapsed_us.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_double)]
        L.sptmm_weights_set_plan.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(PlanStruct)]
        L.sptmm_weights_get_plan.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(PlanStruct)]
        L.sptmm_weights_tune.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
        L.sptmm_stream_wait_event.argtypes = [C.c_void_p, C.c_void_p]
        L.sptmm_measure_sequence.argtypes = [C.POINTER(Step), C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_double)]
        _LIB = L
    return _LIB


def _ck(rc: int) -> int:
    if rc < 0:
        raise SptmmError(rc, lib().sptmm_last_error().decode())
    return rc


def _p(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "need a C-contiguous numpy array"
    return a.ctypes.data_as(C.c_void_p)


# ------------------------------------------------------------------ host side
def device_init(device: int = 0) -> dict:
    info = DevInfo()
    _ck(lib().sptmm_device_init(device, C.byref(info)))
    return {f: (getattr(info, f).decode() if isinstance(getattr(info, f), bytes) else getattr(info, f))
            for f, _ in DevInfo._fields_}


def generate_ternary(K: int, N: int, S: int, dense: bool = False):
    """-> (W [N][K] int8 = column-major K x N, or None; pos [N][S/2] u16; neg [N][S/2] u16)."""
    half = max(S // 2, 0)
    W = np.empty((N, K), np.int8) if dense and K > 0 and N > 0 else None
    pos = np.empty((max(N, 0), half), np.uint16)
    neg = np.empty((max(N, 0), half), np.uint16)
    _ck(lib().sptmm_generate_ternary(K, N, S, _p(W), _p(pos), _p(neg)))
    return W, pos, neg


def lists_from_dense(W: np.ndarray, S: int):
    N, K = W.shape
    pos = np.empty((N, S // 2), np.uint16)
    neg = np.empty((N, S // 2), np.uint16)
    _ck(lib().sptmm_lists_from_dense(_p(W), K, N, S, _p(pos), _p(neg)))
    return pos, neg


def make_x_i8(seed: int, M: int, K: int) -> np.ndarray:
    X = np.empty((M, K), np.int8)
    _ck(lib().sptmm_make_x_i8(seed, M * K, _p(X)))
    return X


def make_x_normal(seed: int, M: int, K: int, dtype=np.float16) -> np.ndarray:
    """Seeded ~N(0,1) activations (Box-Muller over xorshift32), float16 or float32."""
    if dtype == np.float32:
        X = np.empty((M, K), np.float32)
        _ck(lib().sptmm_make_x_normal(seed, M * K, _p(X), None))
        return X
    assert dtype == np.float16
    X = np.empty((M, K), np.uint16)
    _ck(lib().sptmm_make_x_normal(seed, M * K, None, _p(X)))
    return X.view(np.float16)


def pack_u16(pos, neg, K, split_k) -> np.ndarray:
    N, half = pos.shape
    n = lib().sptmm_pack_u16_bytes(N, 2 * half, split_k)
    out = np.zeros(max(n, 1), np.uint8)
    _ck(lib().sptmm_pack_u16(_p(pos), _p(neg), K, N, 2 * half, split_k, _p(out)))
    return out[:n]


def unpack_u16(packed, K, N, S, split_k):
    pos = np.empty((N, S // 2), np.uint16)
    neg = np.empty((N, S // 2), np.uint16)
    _ck(lib().sptmm_unpack_u16(_p(packed), K, N, S, split_k, _p(pos), _p(neg)))
    return pos, neg


def delta_bits(pos, neg, split_k) -> int:
    N, half = pos.shape
    return _ck(lib().sptmm_delta_bits(_p(pos), _p(neg), N, 2 * half, split_k))


def pack_delta(pos, neg, K, split_k, bits=None, rows=0) -> tuple[np.ndarray, int]:
    """rows = 1: 8-bit gaps visited in the order scheduled for a tile of one byte per row (GEMV, int8, M = 1)."""
    N, half = pos.shape
    if bits is None:
        bits = delta_bits(pos, neg, split_k)
    n = lib().sptmm_pack_delta_bytes(N, 2 * half, split_k, bits)
    out = np.zeros(max(n, 1), np.uint8)
    _ck(lib().sptmm_pack_delta_rows(_p(pos), _p(neg), K, N, 2 * half, split_k, bits, rows, _p(out)))
    return out[:n], bits


def unpack_delta(packed, K, N, S, split_k, bits):
    pos = np.empty((N, S // 2), np.uint16)
    neg = np.empty((N, S // 2), np.uint16)
    _ck(lib().sptmm_unpack_delta(_p(packed), K, N, S, split_k, bits, _p(pos), _p(neg)))
    return pos, neg


def i2s_pack_word(w16) -> int:
    a = np.ascontiguousarray(w16, np.int8)
    assert a.size == 16
    return int(lib().sptmm_i2s_pack_word(_p(a)))


def i2s_decode_word(word: int) -> np.ndarray:
    out = np.empty(16, np.int8)
    lib().sptmm_i2s_decode_word(C.c_uint32(word), _p(out))
    return out


def pack_i2s(W: np.ndarray) -> np.ndarray:
    N, K = W.shape
    n = lib().sptmm_pack_i2s_bytes(K, N)
    out = np.zeros(max(n, 1), np.uint8)
    _ck(lib().sptmm_pack_i2s(_p(W), K, N, _p(out)))
    return out[:n]


def unpack_i2s(packed, K, N) -> np.ndarray:
    W = np.empty((N, K), np.int8)
    _ck(lib().sptmm_unpack_i2s(_p(packed), K, N, _p(W)))
    return W


def generate_ternary_iid(K: int, N: int, seed: int, p_pos: float, p_neg: float) -> np.ndarray:
    """-> W [N][K] int8 (column-major K x N) with independent entries."""
    W = np.empty((max(N, 0), max(K, 0)), np.int8)
    _ck(lib().sptmm_generate_ternary_iid(K, N, seed & 0xFFFFFFFF, p_pos, p_neg, _p(W)))
    return W


def dense_from_i2s_words(words: np.ndarray, K: int) -> np.ndarray:
    """words [N][K/16] u32 in the reference's order -> W [N][K] int8."""
    N = words.shape[0]
    W = np.empty((N, K), np.int8)
    _ck(lib().sptmm_dense_from_i2s_words(_p(np.ascontiguousarray(words, np.uint32)), K, N, _p(W)))
    return W


def pack_ragged(W: np.ndarray, kind: int, split_k: int, bits: int = 0, rows: int = 0):
    """Any ternary matrix W [N][K] -> (stream bytes, dict(bits, read_bytes, n_min, n_max, nnz))."""
    N, K = W.shape
    b, rb, lo, hi, nnz = C.c_int(bits), C.c_size_t(), C.c_int(), C.c_int(), C.c_uint64()
    n = lib().sptmm_pack_ragged_bytes(_p(W), K, N, kind, split_k, C.byref(b), C.byref(rb), C.byref(lo), C.byref(hi), C.byref(nnz))
    if not n:
        raise SptmmError(-1, lib().sptmm_last_error().decode())
    out = np.zeros(n, np.uint8)
    _ck(lib().sptmm_pack_ragged_rows(_p(W), K, N, kind, split_k, b.value, rows, _p(out)))
    return out, {"bits": b.value, "read_bytes": rb.value, "n_min": lo.value, "n_max": hi.value, "nnz": nnz.value}


def unpack_ragged(packed: np.ndarray, K: int, N: int, kind: int, split_k: int, bits: int = 0) -> np.ndarray:
    W = np.empty((N, K), np.int8)
    _ck(lib().sptmm_unpack_ragged(_p(packed), K, N, kind, split_k, bits, _p(W)))
    return W


def choose_split_k(kind: int, N: int, S: int, compute_units: int = 0) -> int:
    """The split_k the upload calls pick when handed 0."""
    return _ck(lib().sptmm_choose_split_k(kind, N, S, compute_units))


def wide_k_tile(K: int, lds_bytes: int = 160 * 1024) -> int:
    return _ck(lib().sptmm_wide_k_tile(K, lds_bytes))


def pack_wide(W: np.ndarray, kind: int, split_k: int, k_tile: int, bits: int = 0):
    """Any ternary matrix W [N][K] -> (wide stream bytes, dict(bits, read_bytes, nnz))."""
    N, K = W.shape
    b, rb, nnz = C.c_int(bits), C.c_size_t(), C.c_uint64()
    n = lib().sptmm_pack_wide_bytes(_p(W), K, N, kind, split_k, k_tile, C.byref(b), C.byref(rb), C.byref(nnz))
    if not n:
        raise SptmmError(-1, lib().sptmm_last_error().decode())
    out = np.zeros(n, np.uint8)
    _ck(lib().sptmm_pack_wide(_p(W), K, N, kind, split_k, k_tile, b.value, _p(out)))
    return out, {"bits": b.value, "read_bytes": rb.value, "nnz": nnz.value}


def unpack_wide(packed: np.ndarray, K: int, N: int) -> np.ndarray:
    W = np.empty((N, K), np.int8)
    _ck(lib().sptmm_unpack_wide(_p(packed), K, N, _p(W)))
    return W


# ---------------------------------------------------------------- device side
class DeviceBuffer:
    """A device allocation owned through the C ABI."""

    def __init__(self, nbytes: int):
        self.ptr = C.c_void_p()
        self.nbytes = int(nbytes)
        _ck(lib().sptmm_malloc(C.byref(self.ptr), self.nbytes))

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        if a.nbytes:
            _ck(lib().sptmm_memcpy_h2d(b.ptr, _p(a), a.nbytes))
        return b

    def upload(self, a: np.ndarray):
        """Overwrite the start of the buffer with `a` (synchronous copy)."""
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        if a.nbytes:
            _ck(lib().sptmm_memcpy_h2d(self.ptr, _p(a), a.nbytes))

    def to_numpy(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            _ck(lib().sptmm_memcpy_d2h(_p(out), self.ptr, out.nbytes))
        return out

    def fill(self, byte: int = 0):
        _ck(lib().sptmm_memset(self.ptr, byte, self.nbytes))

    def free(self):
        if self.ptr:
            lib().sptmm_free(self.ptr)
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        self.handle = C.c_void_p()
        _ck(lib().sptmm_stream_create(C.byref(self.handle)))

    def sync(self):
        _ck(lib().sptmm_stream_sync(self.handle))

    def wait(self, event: "Event"):
        """Later work on this stream waits for what `event` recorded (inside a capture: joins / leaves the capture)."""
        _ck(lib().sptmm_stream_wait_event(self.handle, event.handle))

    def destroy(self):
        if self.handle:
            lib().sptmm_stream_destroy(self.handle)
            self.handle = C.c_void_p()


class Graph:
    """The launches issued on `stream` inside the `with` block, as one executable HIP graph.

        with sp.Graph(st) as g:
            w0.gemv_i8(x0, 1, c0, st); w1.gemv_i8(x1, 1, c1, st)
        g.launch(st)
    """

    def __init__(self, stream: Stream):
        self.stream = stream
        self.handle = C.c_void_p()

    def __enter__(self):
        _ck(lib().sptmm_graph_begin(self.stream.handle))
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = lib().sptmm_graph_end(self.stream.handle, C.byref(self.handle))
        if exc_type is None:
            _ck(rc)
        elif rc == 0:
            self.destroy()  # the block failed: the capture is closed and its graph dropped
        return False

    def launch(self, stream: Stream | None = None):
        _ck(lib().sptmm_graph_launch(self.handle, (stream or self.stream).handle))

    def destroy(self):
        if self.handle:
            lib().sptmm_graph_destroy(self.handle)
            self.handle = C.c_void_p()


class Event:
    def __init__(self):
        self.handle = C.c_void_p()
        _ck(lib().sptmm_event_create(C.byref(self.handle)))

    def record(self, stream: Stream | None = None):
        _ck(lib().sptmm_event_record(self.handle, stream.handle if stream else None))

    def sync(self):
        _ck(lib().sptmm_event_sync(self.handle))

    def elapsed_us(self, later: "Event") -> float:
        us = C.c_double()
        _ck(lib().sptmm_event_elapsed_us(self.handle, later.handle, C.byref(us)))
        return us.value

    def destroy(self):
        if self.handle:
            lib().sptmm_event_destroy(self.handle)
            self.handle = C.c_void_p()


def measure_gemv(weights, act: int, X: "DeviceBuffer", M: int, Cout: "DeviceBuffer", iters: int, mode: int = 0,
                 stream: "Stream | None" = None) -> float:
    """Mean microseconds per launch over `iters` launches rotating over `weights` (see sptmm_measure_gemv)."""
    arr = (C.c_void_p * len(weights))(*[w.handle for w in weights])
    us = C.c_double()
    own = stream is None
    if own:
        stream = Stream()
    try:
        _ck(lib().sptmm_measure_gemv(arr, len(weights), act, X.ptr, M, Cout.ptr, iters, mode, stream.handle, C.byref(us)))
    finally:
        if own:
            stream.destroy()
    return us.value


def _steps(steps):
    return (Step * len(steps))(*[Step(w.handle, x.ptr, c.ptr, m, act, stage) for w, x, c, m, act, stage in steps])


def measure_sequence(steps, reps: int, mode: int, stream: "Stream") -> float:
    """Mean microseconds per pass over `steps` = [(weights, X buffer, C buffer, M, act, stage), ...] (see sptmm_measure_sequence)."""
    us = C.c_double()
    _ck(lib().sptmm_measure_sequence(_steps(steps), len(steps), reps, mode, stream.handle, C.byref(us)))
    return us.value


def gemv_batched(weights, Xs, Cs, M: int, act: int = 0, stream: "Stream | None" = None):
    """One launch for len(weights) GEMVs of one shape: Cs[i] = Xs[i] . weights[i] (device buffers).
    act: 0 int8 -> int32, 1 fp16 -> fp32, 2 fp32 -> fp32."""
    n = len(weights)
    assert len(Xs) == n and len(Cs) == n
    wa = (C.c_void_p * n)(*[w.handle for w in weights])
    xa = (C.c_void_p * n)(*[x.ptr for x in Xs])
    ca = (C.c_void_p * n)(*[c.ptr for c in Cs])
    _ck(lib().sptmm_gemv_batched(wa, xa, ca, n, M, act, stream.handle if stream else None))


def gemv_i8_batched(weights, Xs, Cs, M: int, stream: "Stream | None" = None):
    gemv_batched(weights, Xs, Cs, M, 0, stream)


def device_sync():
    _ck(lib().sptmm_device_sync())


def read_kernel(src: DeviceBuffer, nbytes: int, stream: Stream, launches: int = 20, workgroups: int = 0,
                regions: int = 1, stride: int = 0) -> float:
    """Mean microseconds per launch of a pure streaming read of `nbytes`; launch i reads region i % regions of `src`."""
    sink = DeviceBuffer(16)
    us = C.c_double()
    try:
        _ck(lib().sptmm_read_kernel(src.ptr, nbytes, stride, regions, sink.ptr, workgroups, launches, stream.handle, C.byref(us)))
    finally:
        sink.free()
    return us.value


def copy_kernel(dst: DeviceBuffer, src: DeviceBuffer, nbytes: int, stream: Stream | None = None):
    _ck(lib().sptmm_copy_kernel(dst.ptr, src.ptr, nbytes, stream.handle if stream else None))


class Weights:
    """One ternary K x N matrix resident on the device in one of the three encodings."""

    def __init__(self, handle):
        self.handle = handle

    @classmethod
    def upload_u16(cls, pos, neg, K, split_k, rows=0) -> "Weights":
        """rows: activation rows per call the stream is built for (more than 8: a wide stream; 0: no preference)."""
        N, half = pos.shape
        h = C.c_void_p()
        _ck(lib().sptmm_weights_upload_u16_rows(_p(pos), _p(neg), K, N, 2 * half, split_k, rows, C.byref(h)))
        return cls(h)

    @classmethod
    def upload_delta(cls, pos, neg, K, split_k, rows=0) -> "Weights":
        """rows: activation rows per call the gap stream is scheduled for (1: the GEMV stream, int8 M = 1; 0: no preference)."""
        N, half = pos.shape
        h = C.c_void_p()
        _ck(lib().sptmm_weights_upload_delta_rows(_p(pos), _p(neg), K, N, 2 * half, split_k, rows, C.byref(h)))
        return cls(h)

    @classmethod
    def upload_i2s(cls, W: np.ndarray) -> "Weights":
        N, K = W.shape
        h = C.c_void_p()
        _ck(lib().sptmm_weights_upload_i2s(_p(W), K, N, C.byref(h)))
        return cls(h)

    @classmethod
    def upload_dense(cls, W: np.ndarray, kind: int, split_k: int = 32, rows: int = 0) -> "Weights":
        """Any ternary matrix W [N][K] (columns free to differ in nonzeros) in the given encoding; rows as in upload_delta."""
        N, K = W.shape
        h = C.c_void_p()
        _ck(lib().sptmm_weights_upload_dense_rows(_p(W), K, N, kind, split_k, rows, C.byref(h)))
        return cls(h)

    @classmethod
    def upload_wide(cls, W: np.ndarray, kind: int, split_k: int = 32) -> "Weights":
        """Any ternary matrix W [N][K] as a wide stream (K-tiled, 16 int8 / 8 fp16 rows per tile): for M > 8."""
        N, K = W.shape
        h = C.c_void_p()
        _ck(lib().sptmm_weights_upload_wide(_p(W), K, N, kind, split_k, C.byref(h)))
        return cls(h)

    def save(self, path: str):
        _ck(lib().sptmm_weights_save(self.handle, os.fsencode(path)))

    @classmethod
    def load(cls, path: str) -> "Weights":
        h = C.c_void_p()
        _ck(lib().sptmm_weights_load(os.fsencode(path), C.byref(h)))
        return cls(h)

    def clone(self) -> "Weights":
        h = C.c_void_p()
        _ck(lib().sptmm_weights_clone(self.handle, C.byref(h)))
        return Weights(h)

    @property
    def info(self) -> dict:
        wi = WInfo()
        _ck(lib().sptmm_weights_info(self.handle, C.byref(wi)))
        return {f: getattr(wi, f) for f, _ in WInfo._fields_}

    @property
    def nbytes(self) -> int:
        return int(lib().sptmm_weights_bytes(self.handle))

    # launch plans (see sptmm_plan): the stream's own launch shape per kind of call, zeros = the library's model
    def set_plan(self, M: int, batched: bool, **fields):
        p = PlanStruct()
        for k, v in fields.items():
            assert k in PlanStruct.NAMES, k
            setattr(p, k, int(v))
        _ck(lib().sptmm_weights_set_plan(self.handle, M, int(bool(batched)), C.byref(p)))

    def get_plan(self, M: int, batched: bool) -> dict:
        p = PlanStruct()
        _ck(lib().sptmm_weights_get_plan(self.handle, M, int(bool(batched)), C.byref(p)))
        return {k: getattr(p, k) for k in PlanStruct.NAMES}

    def tune(self, M: int, batch: int = 0, act: int = 0):
        """Bounded on-device search for the launch shape of calls with M rows (batch = 0: lone launches, else launches of
        `batch` GEMVs; act 0 int8, 1 fp16, 2 fp32 rows, 3 / 4 the lone quantising call on fp16 / bf16 rows); the fastest plan is
        stored in the object.  -> (us per GEMV with the model's shape, with the plan kept, plan)."""
        a, b = C.c_double(), C.c_double()
        _ck(lib().sptmm_weights_tune(self.handle, M, batch, act, C.byref(a), C.byref(b)))
        return a.value, b.value, self.get_plan(M, batch > 0)

    # raw launches on device buffers (asynchronous on `stream`)
    def gemv_i8(self, X: DeviceBuffer, M: int, Cout: DeviceBuffer, stream: Stream | None = None):
        _ck(lib().sptmm_gemv_i8(self.handle, X.ptr, M, Cout.ptr, stream.handle if stream else None))

    def gemv_f16(self, X: DeviceBuffer, M: int, Cout: DeviceBuffer, stream: Stream | None = None):
        _ck(lib().sptmm_gemv_f16(self.handle, X.ptr, M, Cout.ptr, stream.handle if stream else None))

    def gemv_f32(self, X: DeviceBuffer, M: int, Cout: DeviceBuffer, stream: Stream | None = None):
        _ck(lib().sptmm_gemv_f32(self.handle, X.ptr, M, Cout.ptr, stream.handle if stream else None))

    def gemv_q8(self, X: DeviceBuffer, x_type: int, M: int, w_scale: float, Yout: DeviceBuffer, stream: Stream | None = None):
        """x_type 1 = fp16, 2 = bf16 (raw 16-bit patterns); Y = float32."""
        _ck(lib().sptmm_gemv_q8(self.handle, X.ptr, x_type, M, w_scale, Yout.ptr, stream.handle if stream else None))

    def q8_workspace_bytes(self, M: int) -> int:
        return int(lib().sptmm_gemv_q8_workspace_bytes(self.handle, M))

    def gemv_q8_ws(self, X: DeviceBuffer, x_type: int, M: int, w_scale: float, Yout: DeviceBuffer, workspace: DeviceBuffer | None,
                   workspace_bytes: int, stream: Stream | None = None):
        """gemv_q8 with a device workspace of q8_workspace_bytes(M): beyond four rows, quantise once, then the int8 GEMV."""
        _ck(lib().sptmm_gemv_q8_ws(self.handle, X.ptr, x_type, M, w_scale, Yout.ptr, workspace.ptr if workspace else None,
                                   workspace_bytes, stream.handle if stream else None))

    def gemv_i8_scaled(self, Xq: DeviceBuffer, inv: DeviceBuffer, M: int, w_scale: float, Yout: DeviceBuffer, stream: Stream | None = None):
        """int8 rows quantised beforehand + their 1/s (float32 [M]) -> Y = float32(C) * inv[m] * w_scale."""
        _ck(lib().sptmm_gemv_i8_scaled(self.handle, Xq.ptr, inv.ptr, M, w_scale, Yout.ptr, stream.handle if stream else None))

    def matmul_i8_scaled(self, Xq: np.ndarray, inv: np.ndarray, w_scale: float = 1.0) -> np.ndarray:
        i = self.info
        M, K = Xq.shape
        assert K == i["K"] and Xq.dtype == np.int8 and inv.dtype == np.float32 and inv.shape == (M,)
        xb, ib, yb = DeviceBuffer.from_numpy(Xq), DeviceBuffer.from_numpy(inv), DeviceBuffer(4 * M * i["N"])
        yb.fill(0xFF)
        try:
            self.gemv_i8_scaled(xb, ib, M, w_scale, yb)
            device_sync()
            return yb.to_numpy(np.float32, (M, i["N"]))
        finally:
            for o in (xb, ib, yb):
                o.free()

    def gemv_q8_static(self, X: DeviceBuffer, x_type: int, M: int, w_scale: float, Yout: DeviceBuffer, stream: Stream | None = None):
        """gemv_q8_ws on the library's static device scratch: allocates nothing; calls that overlap on one GPU race."""
        _ck(lib().sptmm_gemv_q8_static(self.handle, X.ptr, x_type, M, w_scale, Yout.ptr, stream.handle if stream else None))

    def matmul_q8(self, X: np.ndarray, w_scale: float = 1.0, bf16: bool = False, workspace: bool = False) -> np.ndarray:
        """Host convenience: X [M][K] float16 (or uint16 bf16 patterns with bf16=True) -> Y [M][N] float32.
        workspace=True: through gemv_q8_ws with a workspace allocated for the call."""
        i = self.info
        M, K = X.shape
        assert K == i["K"] and X.dtype == (np.uint16 if bf16 else np.float16)
        xb = DeviceBuffer.from_numpy(X)
        yb = DeviceBuffer(4 * M * i["N"])
        yb.fill(0xFF)
        ws = None
        try:
            if workspace:
                nbytes = self.q8_workspace_bytes(M)
                ws = DeviceBuffer(nbytes)
                ws.fill(0xA5)
                self.gemv_q8_ws(xb, 2 if bf16 else 1, M, w_scale, yb, ws, nbytes)
            else:
                self.gemv_q8(xb, 2 if bf16 else 1, M, w_scale, yb)
            device_sync()
            return yb.to_numpy(np.float32, (M, i["N"]))
        finally:
            xb.free()
            yb.free()
            if ws is not None:
                ws.free()

    def matmul(self, X: np.ndarray) -> np.ndarray:
        """Host convenience: upload X [M][K], run on the device, download C [M][N]."""
        i = self.info
        M, K = X.shape
        assert K == i["K"]
        xb = DeviceBuffer.from_numpy(X)
        cb = DeviceBuffer(4 * M * i["N"])
        cb.fill(0xFF)
        try:
            if X.dtype == np.int8:
                self.gemv_i8(xb, M, cb)
                out = np.int32
            elif X.dtype == np.float16:
                self.gemv_f16(xb, M, cb)
                out = np.float32
            elif X.dtype == np.float32:
                self.gemv_f32(xb, M, cb)
                out = np.float32
            else:
                raise TypeError("activations must be int8, float16 or float32")
            device_sync()
            return cb.to_numpy(out, (M, i["N"]))
        finally:
            xb.free()
            cb.free()

    def free(self):
        if self.handle:
            lib().sptmm_weights_free(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
