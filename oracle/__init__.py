"""CPU oracle for the MCCL hot path -- TEST INFRASTRUCTURE ONLY.

ctypes bindings over ``liboracle.so`` (the plain-C restatement in
``mccl_oracle.c``) and, when it has been built, over
``_ref/libmccl_ref_compression.so`` (the reference's own csrc/compression
sources compiled by ``make ref``).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the shipped library never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libmccl_ref_compression.so")

OP_SUM, OP_AVG, OP_PRODUCT, OP_MIN, OP_MAX = 0, 1, 2, 3, 4
U8, I32, I64, F16, F32, BOOL, BF16 = 0, 3, 4, 5, 6, 11, 15
RING_BASIC, RING_CHUNKED = 0, 1
OK, ERR_OP, ERR_DTYPE, ERR_CAPACITY, ERR_SIZE, ERR_INDEX, ERR_ARG = 0, -1, -2, -3, -4, -5, -6


def build(ref: bool = True) -> None:
    """Compile liboracle.so (always) and _ref (when the reference is present)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    if ref and os.path.isdir("/root/reference/csrc/compression"):
        subprocess.check_call(["make", "-s", "-C", _HERE, "ref"])


def _load():
    if not os.path.exists(_LIB_PATH):
        build(ref=False)
    lib = C.CDLL(_LIB_PATH)
    vp, i64, u64, i32, f32, f64 = C.c_void_p, C.c_int64, C.c_uint64, C.c_int, C.c_float, C.c_double
    sig = {
        "orc_f16_to_f32": (f32, [C.c_uint16]),
        "orc_f32_to_f16": (C.c_uint16, [f32]),
        "orc_bf16_to_f32": (f32, [C.c_uint16]),
        "orc_f32_to_bf16": (C.c_uint16, [f32]),
        "orc_convert": (i32, [vp, vp, i64, i32]),
        "orc_f32_to_f16_transport": (C.c_uint16, [f32]),
        "orc_fp16_compress": (i64, [vp, i64, vp, i64, i32]),
        "orc_fp16_decompress": (i32, [vp, i64, vp, i64, i32]),
        "orc_fold2_f32": (i32, [vp, vp, i64, i32, i32]),
        "orc_scale_f32": (i32, [vp, i64, f32, i32]),
        "orc_fold2_scale_f32": (i32, [vp, vp, i64, f32, i32]),
        "orc_fold2_h": (i32, [vp, vp, i64, i32, i32]),
        "orc_scale_h": (i32, [vp, i64, i32, f32]),
        "orc_fold2_scale_h": (i32, [vp, vp, i64, i32, f32]),
        "orc_fold2_int": (i32, [vp, vp, i64, i32, i32]),
        "orc_scale_int": (i32, [vp, i64, i32, f32, i32]),
        "orc_ring_chunks": (i32, [i32, i32]),
        "orc_ring_chunk_elems": (i64, [i64, i32, i32]),
        "orc_ring_first_rank": (i32, [i32, i32, i32]),
        "orc_ring_fold": (i32, [vp, vp, i32, i64, i32, i32, i32, i32, f32, i32]),
        "orc_ring_simulate_f32": (i32, [vp, vp, i32, i64, i32, i32]),
        "orc_topk_k": (C.c_uint32, [u64, f64]),
        "orc_topk_max_compressed_size": (u64, [u64, f64]),
        "orc_topk_compress": (i64, [vp, vp, u64, f64, vp, u64]),
        "orc_topk_decompress": (i32, [vp, u64, vp, u64]),
        "orc_sparse_accumulate": (i32, [vp, u64, vp, vp, i32, i32, f32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _p(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


_NP_DTYPE = {F32: np.float32, F16: np.uint16, BF16: np.uint16, I32: np.int32, I64: np.int64,
             U8: np.uint8, BOOL: np.uint8}


# ---- 16-bit conversions ------------------------------------------------------
def _convert(x: np.ndarray, kind: int, out_dtype) -> np.ndarray:
    x = np.ascontiguousarray(x)
    out = np.empty(x.shape, dtype=out_dtype)
    lib.orc_convert(_p(out), _p(x), x.size, kind)
    return out


def f16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return _convert(bits.astype(np.uint16, copy=False), 0, np.float32)


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    return _convert(x.astype(np.float32, copy=False), 1, np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return _convert(bits.astype(np.uint16, copy=False), 2, np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    return _convert(x.astype(np.float32, copy=False), 3, np.uint16)


# ---- FP16 compressor ----------------------------------------------------------
def fp16_compress(data: np.ndarray, dtype: int = F32, capacity=None):
    """Wire bytes (uint8 array), or the negative status."""
    data = np.ascontiguousarray(data)
    cap = data.nbytes if capacity is None else capacity
    out = np.zeros(max(cap, 1), dtype=np.uint8)
    rc = int(lib.orc_fp16_compress(_p(data), data.nbytes, _p(out), cap, dtype))
    return rc if rc < 0 else out[:rc].copy()


def fp16_decompress(wire: np.ndarray, count: int, dtype: int = F32, size=None):
    """(dense array of `count` elements, status)."""
    wire = np.ascontiguousarray(wire)
    dst = np.zeros(count, dtype=np.float32 if dtype == F32 else np.uint16)
    rc = int(lib.orc_fp16_decompress(_p(wire), wire.nbytes if size is None else size, _p(dst), dst.nbytes, dtype))
    return dst, rc


# ---- folds (in place on dst; dst is returned) -------------------------------
def fold2(dst: np.ndarray, src: np.ndarray, dtype: int, op: int, threads: int = 0) -> int:
    assert dst.shape == src.shape
    n = dst.size
    if dtype == F32:
        return lib.orc_fold2_f32(_p(dst), _p(src), n, op, threads)
    if dtype in (F16, BF16):
        return lib.orc_fold2_h(_p(dst), _p(src), n, dtype, op)
    return lib.orc_fold2_int(_p(dst), _p(src), n, dtype, op)


def scale(buf: np.ndarray, dtype: int, s: float, threads: int = 0, round_i32: bool = False) -> int:
    n = buf.size
    if dtype == F32:
        return lib.orc_scale_f32(_p(buf), n, s, threads)
    if dtype in (F16, BF16):
        return lib.orc_scale_h(_p(buf), n, dtype, s)
    return lib.orc_scale_int(_p(buf), n, dtype, s, int(round_i32))


def fold2_scale(dst: np.ndarray, src: np.ndarray, dtype: int, s: float, threads: int = 0) -> int:
    n = dst.size
    if dtype == F32:
        return lib.orc_fold2_scale_f32(_p(dst), _p(src), n, s, threads)
    if dtype in (F16, BF16):
        return lib.orc_fold2_scale_h(_p(dst), _p(src), n, dtype, s)
    return ERR_DTYPE


def _ptr_array(arrs):
    return (C.c_void_p * len(arrs))(*[_p(a) for a in arrs])


def ring_fold(ins, dtype: int, op: int, schedule: int = RING_BASIC, scale_by=None,
              stepwise: bool = False) -> np.ndarray:
    """Closed-form ring-order fold of len(ins) rank buffers."""
    n = ins[0].size
    out = np.empty_like(ins[0])
    rc = lib.orc_ring_fold(_p(out), _ptr_array(ins), len(ins), n, schedule, dtype, op,
                           0 if scale_by is None else 1, 0.0 if scale_by is None else scale_by,
                           int(stepwise))
    if rc != OK:
        raise ValueError(f"orc_ring_fold rc={rc}")
    return out


def ring_simulate_f32(ins, op: int, schedule: int = RING_BASIC) -> np.ndarray:
    n = ins[0].size
    out = np.empty_like(ins[0])
    rc = lib.orc_ring_simulate_f32(_p(out), _ptr_array(ins), len(ins), n, schedule, op)
    if rc != OK:
        raise ValueError(f"orc_ring_simulate_f32 rc={rc}")
    return out


# ---- top-k ------------------------------------------------------------------
def topk_k(count: int, ratio: float) -> int:
    return int(lib.orc_topk_k(count, ratio))


def topk_max_compressed_size(nbytes: int, ratio: float) -> int:
    return int(lib.orc_topk_max_compressed_size(nbytes, ratio))


def topk_compress(grad: np.ndarray, residual: np.ndarray, ratio: float, capacity=None):
    """Returns (wire bytes as uint8 array, rc). residual is updated in place."""
    assert grad.dtype == np.float32 and residual.dtype == np.float32
    cap = topk_max_compressed_size(grad.size * 4, ratio) if capacity is None else capacity
    out = np.zeros(max(cap, 1), dtype=np.uint8)
    rc = lib.orc_topk_compress(_p(grad), _p(residual), grad.size, ratio, _p(out), cap)
    if rc < 0:
        return None, int(rc)
    return out[:rc].copy(), int(rc)


def topk_decompress(wire: np.ndarray, count: int, size=None):
    dst = np.empty(count, dtype=np.float32)
    rc = lib.orc_topk_decompress(_p(wire), wire.size if size is None else size, _p(dst), count)
    return dst, int(rc)


def sparse_accumulate(wires, count: int, scale_by=None):
    acc = np.empty(count, dtype=np.float32)
    sizes = (C.c_uint64 * len(wires))(*[w.size for w in wires])
    rc = lib.orc_sparse_accumulate(_p(acc), count, _ptr_array(wires), sizes, len(wires),
                                   0 if scale_by is None else 1,
                                   0.0 if scale_by is None else scale_by)
    return acc, int(rc)


def parse_wire(wire: np.ndarray):
    """[u32 k][k x (u32 idx, f32 val)] -> (k, idx uint32[k], val float32[k])."""
    k = int(wire[:4].view("<u4")[0])
    body = wire[4:4 + 8 * k].view("<u4").reshape(k, 2)
    return k, body[:, 0].copy(), body[:, 1].copy().view(np.float32)


# ---- the reference's own compression code (oracle/_ref) --------------------
class RefCompressor:
    """mccl::make_compressor(mode, param) from the compiled reference sources."""

    _lib = None

    @classmethod
    def available(cls) -> bool:
        return os.path.exists(_REF_PATH)

    @classmethod
    def _get(cls):
        if cls._lib is None:
            l = C.CDLL(_REF_PATH)
            l.ref_make_compressor.restype = C.c_void_p
            l.ref_make_compressor.argtypes = [C.c_int, C.c_double]
            l.ref_free_compressor.argtypes = [C.c_void_p]
            l.ref_compress.restype = C.c_longlong
            l.ref_compress.argtypes = [C.c_void_p, C.c_void_p, C.c_ulonglong, C.c_void_p,
                                       C.c_ulonglong, C.c_int, C.c_ulonglong]
            l.ref_decompress.restype = C.c_int
            l.ref_decompress.argtypes = [C.c_void_p, C.c_void_p, C.c_ulonglong, C.c_void_p,
                                         C.c_ulonglong, C.c_int]
            l.ref_max_compressed_size.restype = C.c_ulonglong
            l.ref_max_compressed_size.argtypes = [C.c_void_p, C.c_ulonglong]
            l.ref_error_feedback_buffer_count.restype = C.c_ulonglong
            l.ref_error_feedback_buffer_count.argtypes = [C.c_void_p]
            l.ref_reset_error_feedback.argtypes = [C.c_void_p]
            l.ref_reset_error_feedback_for_tensor.argtypes = [C.c_void_p, C.c_ulonglong]
            cls._lib = l
        return cls._lib

    def __init__(self, mode: int = 2, param: float = 0.01):
        self.l = self._get()
        self.h = self.l.ref_make_compressor(mode, param)
        if not self.h:
            raise RuntimeError("reference make_compressor threw")

    def __del__(self):
        if getattr(self, "h", None):
            self.l.ref_free_compressor(self.h)
            self.h = None

    def max_compressed_size(self, nbytes: int) -> int:
        return int(self.l.ref_max_compressed_size(self.h, nbytes))

    def compress(self, data: np.ndarray, stable_id: int = 0, capacity=None, dtype: int = F32):
        cap = self.max_compressed_size(data.nbytes) if capacity is None else capacity
        out = np.zeros(max(cap, 1), dtype=np.uint8)
        rc = self.l.ref_compress(self.h, _p(data), data.nbytes, _p(out), cap, dtype, stable_id)
        if rc < 0:
            return None
        return out[:rc].copy()

    def decompress(self, wire: np.ndarray, count: int, size=None, dtype: int = F32):
        dst = np.zeros(count, dtype=np.uint16 if dtype == F16 else np.float32)
        rc = self.l.ref_decompress(self.h, _p(wire), wire.size if size is None else size,
                                   _p(dst), dst.nbytes, dtype)
        return dst, int(rc)

    def buffer_count(self) -> int:
        return int(self.l.ref_error_feedback_buffer_count(self.h))

    def reset(self) -> None:
        self.l.ref_reset_error_feedback(self.h)

    def reset_for(self, stable_id: int) -> None:
        self.l.ref_reset_error_feedback_for_tensor(self.h, stable_id)
