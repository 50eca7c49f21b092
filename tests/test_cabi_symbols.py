"""The C-ABI library loads on a CPU-only host and exports every symbol that
include/mccl_hip.h declares (no compute call is made here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mccl_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mccl_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("mccl_hip_fold2", "mccl_hip_scale", "mccl_hip_fold2_scale", "mccl_hip_ring_fold",
                 "mccl_hip_topk_compress", "mccl_hip_topk_decompress", "mccl_hip_sparse_accumulate",
                 "mccl_hip_fence_signal", "mccl_hip_fence_wait", "mccl_hip_init"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from mccl_amd import _lib
    lib = _lib.load()
    for name in declared_symbols():
        assert hasattr(lib, name), name
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert lib.mccl_hip_abi_version() == 1


def test_host_only_entry_points_agree_with_the_reference_formulas():
    from mccl_amd import _lib
    lib = _lib.load()
    # k = max(1, uint32(count * ratio)); max size = 4 + 8 * (uint32(count * ratio) + 1)
    assert lib.mccl_hip_topk_k(6_553_600, 0.01) == 65_536
    assert lib.mccl_hip_topk_k(4_759_624, 0.01) == 47_596
    assert lib.mccl_hip_topk_k(10, 0.01) == 1
    assert lib.mccl_hip_topk_max_compressed_size(6_553_600 * 4, 0.01) == 4 + 8 * 65_537
    assert lib.mccl_hip_strerror(-5) == b"TopK decompress: index out of bounds"
    assert lib.mccl_hip_topk_workspace_bytes(96_510_024, 6_553_600, 0.01) > 0
    assert lib.mccl_hip_set_tuning(b"fold_blocks_per_cu", 4) == 0
    assert lib.mccl_hip_get_tuning(b"fold_blocks_per_cu") == 4
    assert lib.mccl_hip_set_tuning(b"fold_blocks_per_cu", 256) == 0
    assert lib.mccl_hip_set_tuning(b"no_such_key", 1) == -6


def test_argument_errors_need_no_gpu():
    from mccl_amd import _lib
    lib = _lib.load()
    assert lib.mccl_hip_fold2(None, None, 0, 6, 0, None) == 0          # empty: no-op
    assert lib.mccl_hip_fold2(None, None, 4, 6, 5, None) == -1         # BAND unsupported
    assert lib.mccl_hip_fold2(None, None, 4, 6, 0, None) == -6         # null pointer
    assert lib.mccl_hip_topk_decompress(ctypes.c_void_p(4096), 7, ctypes.c_void_p(4096), 8, None, None) == -4


def test_tensor_layer_rejects_host_buffers_before_any_call():
    # the ctypes layer knows the buffer sizes; host tensors and short buffers raise ValueError there
    import torch
    from mccl_amd import hip_ops as ops
    a = torch.zeros(8)
    for call in (lambda: ops.fold2(a, a.clone()), lambda: ops.scale(a, 0.5), lambda: ops.fold2_scale(a, a.clone(), 0.5),
                 lambda: ops.ring_fold(a, [a.clone(), a.clone()]),
                 lambda: ops.topk_compress(a, a.clone(), 0.5),
                 lambda: ops.topk_decompress(torch.zeros(12, dtype=torch.uint8), 12, 8),
                 lambda: ops.sparse_accumulate(a, [torch.zeros(12, dtype=torch.uint8)], 12),
                 lambda: ops.sparse_accumulate_static(a, [torch.zeros(12, dtype=torch.uint8)], 12),
                 lambda: ops.cast_f32_to_f16(a), lambda: ops.cast_f16_to_f32(a.half())):
        with pytest.raises(ValueError, match="must live on the GPU"):
            call()


def test_pointer_check_needs_arguments():
    from mccl_amd import _lib
    lib = _lib.load()
    out = ctypes.c_void_p(0)
    assert lib.mccl_hip_pointer_check(None, 16, ctypes.byref(out)) == -6
    assert lib.mccl_hip_strerror(-10) == b"pointer is not GPU-accessible memory"
