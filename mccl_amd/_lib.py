"""ctypes loader for ``libmccl_hip.so`` (the C ABI in ``include/mccl_hip.h``).

There is no CPU fallback: if the library has not been built, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# MCCL_HIP_LIBRARY selects another build of the same ABI (kernel tuning experiments)
LIB_PATH = os.environ.get("MCCL_HIP_LIBRARY") or os.path.join(_HERE, "libmccl_hip.so")

# (restype, argtypes) for every symbol include/mccl_hip.h declares
_vp, _u64, _u32, _i32, _f32, _f64 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int, C.c_float, C.c_double
SIGNATURES = {
    "mccl_hip_init": (_i32, []),
    "mccl_hip_abi_version": (_i32, []),
    "mccl_hip_strerror": (C.c_char_p, [_i32]),
    "mccl_hip_last_hip_error": (_i32, []),
    "mccl_hip_pointer_check": (_i32, [_vp, _u64, C.POINTER(_vp)]),
    "mccl_hip_fold2": (_i32, [_vp, _vp, _u64, _i32, _i32, _vp]),
    "mccl_hip_scale": (_i32, [_vp, _u64, _i32, _f32, _vp]),
    "mccl_hip_fold2_scale": (_i32, [_vp, _vp, _u64, _i32, _f32, _vp]),
    "mccl_hip_fold2_batch": (_i32, [_vp, _vp, _vp, _u32, _i32, _i32, _vp]),
    "mccl_hip_ring_fold": (_i32, [_vp, C.POINTER(_vp), _i32, _u64, _u64, _i32, _i32, _i32, _i32, _f32, _i32, _vp]),
    "mccl_hip_topk_k": (_u32, [_u64, _f64]),
    "mccl_hip_topk_max_compressed_size": (_u64, [_u64, _f64]),
    "mccl_hip_topk_workspace_bytes": (_u64, [_u64, _u64, _f64]),
    "mccl_hip_topk_compress": (_i32, [_vp, _vp, _u64, _u64, _f64, _vp, _u64, _vp, _u64, _vp, _vp]),
    "mccl_hip_topk_list_workspace_bytes": (_u64, [C.POINTER(_u64), _u32, _f64]),
    "mccl_hip_topk_compress_list": (_i32, [C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_u64), C.POINTER(_vp),
                                           C.POINTER(_u64), _u32, _f64, _vp, _u64, _vp, _vp]),
    "mccl_hip_topk_path_report": (_i32, [_vp, _u64, _u64, _f64, C.POINTER(_u32), C.POINTER(_u32), _vp]),
    "mccl_hip_topk_decompress": (_i32, [_vp, _u64, _vp, _u64, _vp, _vp]),
    "mccl_hip_sparse_accumulate": (_i32, [_vp, _u64, _u64, C.POINTER(_vp), _i32, _u64, _i32, _f32, _vp, _vp, _u64, _vp]),
    "mccl_hip_sparse_accumulate_workspace_bytes": (_u64, [_u64, _u64, _i32]),
    "mccl_hip_sparse_accumulate_static": (_i32, [_vp, _u64, _u64, C.POINTER(_vp), _i32, _u64, _i32, _f32, _vp, _vp]),
    "mccl_hip_cast_f32_to_f16": (_i32, [_vp, _vp, _u64, _vp]),
    "mccl_hip_cast_f16_to_f32": (_i32, [_vp, _vp, _u64, _vp]),
    "mccl_hip_fence_signal": (_i32, [_vp, C.POINTER(_u64)]),
    "mccl_hip_fence_wait": (_i32, [_u64, _i32]),
    "mccl_hip_fence_query": (_i32, [_u64]),
    "mccl_hip_fence_block_stream": (_i32, [_u64, _vp]),
    "mccl_hip_sync": (_i32, [_vp]),
    "mccl_hip_set_tuning": (_i32, [C.c_char_p, _i32]),
    "mccl_hip_get_tuning": (_i32, [C.c_char_p]),
}

_lib = None


def load() -> C.CDLL:
    """Returns the loaded library; raises if it was never built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m mccl_amd.build --lib` "
                "(there is no CPU fallback for the HIP kernels)")
        try:
            # torch ships its own HIP runtime under the same soname; load it
            # first so the process ends up with exactly one runtime
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class MCCLHipError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, code: int, where: str):
        self.code = code
        text = load().mccl_hip_strerror(code).decode()
        extra = ""
        if code == -7:
            extra = f" (hipError_t {load().mccl_hip_last_hip_error()})"
        super().__init__(f"[MCCL] {where}: {text}{extra}")


def check(code: int, where: str) -> None:
    if code != 0:
        raise MCCLHipError(code, where)
