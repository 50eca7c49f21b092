"""Tensor-level calls into the C ABI (``include/mccl_hip.h``).

Every function takes ROCm torch tensors, passes ``data_ptr()`` and torch's
current HIP stream to the library, and only enqueues work.  Nothing here
computes on the host.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import torch

from . import _lib

SUM, AVG, PRODUCT, MIN, MAX = 0, 1, 2, 3, 4
RING_BASIC, RING_CHUNKED = 0, 1

# at::ScalarType values
_DTYPE_CODE = {
    torch.uint8: 0, torch.int32: 3, torch.int64: 4, torch.float16: 5,
    torch.float32: 6, torch.bool: 11, torch.bfloat16: 15,
}


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise _lib.MCCLHipError(-2, f"dtype {t.dtype}") from None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, what: str, dtype: Optional[torch.dtype] = None, min_numel: int = 0) -> None:
    """This layer is the only place buffer sizes are known: every tensor whose
    pointer goes to the library is checked for device, layout, element type and
    capacity here, so a short or host buffer raises instead of faulting the GPU."""
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{what} must be a tensor")
    if not t.is_cuda:
        raise ValueError(f"{what} must live on the GPU, got {t.device}")
    if not t.is_contiguous():
        raise ValueError(f"{what} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{what} must be {dtype}, got {t.dtype}")
    if t.numel() < min_numel:
        raise ValueError(f"{what} holds {t.numel()} elements, {min_numel} are needed")


def fold2(dst: torch.Tensor, src: torch.Tensor, op: int = SUM) -> torch.Tensor:
    _dev(dst, "dst"); _dev(src, "src")
    if dst.shape != src.shape or dst.dtype != src.dtype:
        raise ValueError("shape / dtype mismatch")
    rc = _lib.load().mccl_hip_fold2(dst.data_ptr(), src.data_ptr(), dst.numel(), dtype_code(dst), op, _stream())
    _lib.check(rc, "fold2")
    return dst


def fold2_batch(dsts: Sequence[torch.Tensor], srcs: Sequence[torch.Tensor], op: int = SUM) -> None:
    """dsts[i] (op)= srcs[i] for every i, in one launch per 128 folds.  The folds run in no
    particular order: a destination may not overlap any other fold's destination or source
    (the library refuses such a list)."""
    if len(dsts) != len(srcs):
        raise ValueError("as many sources as destinations")
    if not dsts:
        return
    for d, s_ in zip(dsts, srcs):
        _dev(d, "dst"); _dev(s_, "src")
        if d.shape != s_.shape or d.dtype != s_.dtype or d.dtype != dsts[0].dtype:
            raise ValueError("shape / dtype mismatch")
    counts = (C.c_uint64 * len(dsts))(*[d.numel() for d in dsts])
    rc = _lib.load().mccl_hip_fold2_batch(_ptrs(dsts), _ptrs(srcs), counts, len(dsts), dtype_code(dsts[0]), op, _stream())
    _lib.check(rc, "fold2_batch")


def scale(buf: torch.Tensor, s: float) -> torch.Tensor:
    _dev(buf, "buf")
    rc = _lib.load().mccl_hip_scale(buf.data_ptr(), buf.numel(), dtype_code(buf), s, _stream())
    _lib.check(rc, "scale")
    return buf


def fold2_scale(dst: torch.Tensor, src: torch.Tensor, s: float) -> torch.Tensor:
    _dev(dst, "dst"); _dev(src, "src")
    if dst.shape != src.shape or dst.dtype != src.dtype:
        raise ValueError("shape / dtype mismatch")
    rc = _lib.load().mccl_hip_fold2_scale(dst.data_ptr(), src.data_ptr(), dst.numel(), dtype_code(dst), s, _stream())
    _lib.check(rc, "fold2_scale")
    return dst


def _ptrs(tensors: Sequence[torch.Tensor]):
    return (C.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def ring_fold(out: torch.Tensor, ins: Sequence[torch.Tensor], op: int = SUM,
              schedule: int = RING_BASIC, bucket_elems: Optional[int] = None,
              scale_by: Optional[float] = None, stepwise: bool = False) -> torch.Tensor:
    _dev(out, "out")
    for t in ins:
        _dev(t, "in")
        if t.numel() != out.numel() or t.dtype != out.dtype:
            raise ValueError("shape / dtype mismatch")
    n = out.numel()
    if not ins:
        raise ValueError("ring_fold needs at least one rank buffer")
    rc = _lib.load().mccl_hip_ring_fold(
        out.data_ptr(), _ptrs(ins), len(ins), n, bucket_elems or max(n, 1), schedule, dtype_code(out), op,
        0 if scale_by is None else 1, 0.0 if scale_by is None else scale_by, int(stepwise), _stream())
    _lib.check(rc, "ring_fold")
    return out


def topk_k(count: int, ratio: float) -> int:
    return int(_lib.load().mccl_hip_topk_k(count, ratio))


def topk_max_compressed_size(nbytes: int, ratio: float) -> int:
    return int(_lib.load().mccl_hip_topk_max_compressed_size(nbytes, ratio))


def topk_wire_stride(bucket_elems: int, ratio: float) -> int:
    """Bytes reserved per bucket payload: the reference's max_compressed_size."""
    return topk_max_compressed_size(bucket_elems * 4, ratio)


def topk_workspace(n_total: int, bucket_elems: int, ratio: float, device) -> torch.Tensor:
    nbytes = int(_lib.load().mccl_hip_topk_workspace_bytes(n_total, bucket_elems, ratio))
    if nbytes == 0:
        raise _lib.MCCLHipError(-6, "topk_workspace_bytes")
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def topk_compress(grad: torch.Tensor, residual: torch.Tensor, ratio: float,
                  bucket_elems: Optional[int] = None, wire: Optional[torch.Tensor] = None,
                  workspace: Optional[torch.Tensor] = None, wire_stride: Optional[int] = None,
                  status: Optional[torch.Tensor] = None):
    """Returns (wire uint8 tensor [nbuckets * stride], stride). residual is updated.
    status: int32 device tensor of one element that receives ERR_TIMEOUT (caller zeroes it)."""
    _dev(grad, "grad"); _dev(residual, "residual")
    if grad.dtype != torch.float32 or residual.dtype != torch.float32:
        raise _lib.MCCLHipError(-2, "TopK compression currently supports float32 only")
    n = grad.numel()
    be = min(bucket_elems or n, n) if n else 1
    stride = wire_stride if wire_stride is not None else topk_wire_stride(be, ratio)
    nb = (n + be - 1) // be if n else 1
    if residual.numel() != n:
        raise ValueError(f"residual holds {residual.numel()} elements, the gradient {n}")
    if wire is None:
        wire = torch.empty(nb * stride, dtype=torch.uint8, device=grad.device)
    if workspace is None:
        workspace = topk_workspace(max(n, 1), be, ratio, grad.device)
    _dev(wire, "wire", torch.uint8, nb * stride)
    _dev(workspace, "workspace", torch.uint8)
    if status is not None:
        _dev(status, "status", torch.int32, 1)
    rc = _lib.load().mccl_hip_topk_compress(grad.data_ptr(), residual.data_ptr(), n, be, ratio,
                                           wire.data_ptr(), stride, workspace.data_ptr(),
                                           workspace.numel(), status.data_ptr() if status is not None else None,
                                           _stream())
    _lib.check(rc, "topk_compress")
    return wire, stride


def topk_compress_list(grads: Sequence[torch.Tensor], residuals: Sequence[torch.Tensor], ratio: float,
                       wires: Optional[Sequence[torch.Tensor]] = None, workspace: Optional[torch.Tensor] = None,
                       status: Optional[torch.Tensor] = None):
    """Top-k payloads of a list of separate buckets in one call; returns the list of wire tensors
    (each max_compressed_size bytes, the payload at its front).  residuals are updated."""
    nb = len(grads)
    if nb == 0 or nb != len(residuals):
        raise ValueError("one residual per gradient bucket, at least one bucket")
    for i, (g, r) in enumerate(zip(grads, residuals)):
        _dev(g, f"grads[{i}]", torch.float32, 1)
        _dev(r, f"residuals[{i}]", torch.float32)
        if r.numel() != g.numel():
            raise ValueError(f"residuals[{i}] holds {r.numel()} elements, the bucket {g.numel()}")
    if wires is None:
        wires = [torch.empty(topk_wire_stride(g.numel(), ratio), dtype=torch.uint8, device=g.device) for g in grads]
    for i, w in enumerate(wires):
        _dev(w, f"wires[{i}]", torch.uint8)
    counts = (C.c_uint64 * nb)(*[g.numel() for g in grads])
    caps = (C.c_uint64 * nb)(*[w.numel() for w in wires])
    if workspace is None:
        nbytes = int(_lib.load().mccl_hip_topk_list_workspace_bytes(counts, nb, ratio))
        if nbytes == 0:
            raise _lib.MCCLHipError(-6, "topk_list_workspace_bytes")
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=grads[0].device)
    _dev(workspace, "workspace", torch.uint8)
    if status is not None:
        _dev(status, "status", torch.int32, 1)
    rc = _lib.load().mccl_hip_topk_compress_list(_ptrs(grads), _ptrs(residuals), counts, _ptrs(wires), caps, nb,
                                                ratio, workspace.data_ptr(), workspace.numel(),
                                                status.data_ptr() if status is not None else None, _stream())
    _lib.check(rc, "topk_compress_list")
    return list(wires)


def topk_path_report(workspace: torch.Tensor, n_total: int, bucket_elems: int, ratio: float):
    """(buckets finished by the single-pass path, buckets) of the last compress call."""
    ok, nb = C.c_uint32(0), C.c_uint32(0)
    rc = _lib.load().mccl_hip_topk_path_report(workspace.data_ptr(), n_total, bucket_elems, ratio,
                                               C.byref(ok), C.byref(nb), _stream())
    _lib.check(rc, "topk_path_report")
    return int(ok.value), int(nb.value)


def topk_decompress(wire: torch.Tensor, wire_bytes: int, count: int,
                    dense: Optional[torch.Tensor] = None, status: Optional[torch.Tensor] = None):
    _dev(wire, "wire", torch.uint8, wire_bytes)
    if dense is None:
        dense = torch.empty(count, dtype=torch.float32, device=wire.device)
    _dev(dense, "dense", torch.float32, count)
    if status is not None:
        _dev(status, "status", torch.int32, 1)
    rc = _lib.load().mccl_hip_topk_decompress(wire.data_ptr(), wire_bytes, dense.data_ptr(), count,
                                             None if status is None else status.data_ptr(), _stream())
    _lib.check(rc, "topk_decompress")
    return dense


def _check_payload_sets(wires, n: int, bucket_elems: int, wire_stride: int, status) -> None:
    be = max(1, min(bucket_elems, n))
    nb = (n + be - 1) // be
    for r, w in enumerate(wires):
        _dev(w, f"wires[{r}]", torch.uint8, nb * wire_stride)
    if status is not None:
        _dev(status, "status", torch.int32, 1)


def sparse_workspace(n_total: int, bucket_elems: int, ws: int, device) -> torch.Tensor:
    nbytes = int(_lib.load().mccl_hip_sparse_accumulate_workspace_bytes(n_total, bucket_elems, ws))
    if nbytes == 0:
        raise _lib.MCCLHipError(-6, "sparse_accumulate_workspace_bytes")
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def sparse_accumulate(acc: torch.Tensor, wires: Sequence[torch.Tensor], wire_stride: int,
                      bucket_elems: Optional[int] = None, scale_by: Optional[float] = None,
                      status: Optional[torch.Tensor] = None, workspace="auto") -> torch.Tensor:
    """workspace: "auto" allocates the scratch, None selects the scratch-free kernel."""
    _dev(acc, "acc", torch.float32)
    n = acc.numel()
    be = bucket_elems or max(n, 1)
    _check_payload_sets(wires, n, be, wire_stride, status)
    if isinstance(workspace, str):
        workspace = sparse_workspace(n, be, len(wires), acc.device)
    if workspace is not None:
        _dev(workspace, "workspace", torch.uint8)
    rc = _lib.load().mccl_hip_sparse_accumulate(
        acc.data_ptr(), n, be, _ptrs(wires), len(wires), wire_stride,
        0 if scale_by is None else 1, 0.0 if scale_by is None else scale_by,
        None if status is None else status.data_ptr(),
        None if workspace is None else workspace.data_ptr(), 0 if workspace is None else workspace.numel(),
        _stream())
    _lib.check(rc, "sparse_accumulate")
    return acc


def sparse_accumulate_static(acc: torch.Tensor, wires: Sequence[torch.Tensor], wire_stride: int,
                             bucket_elems: Optional[int] = None, scale_by: Optional[float] = None,
                             status: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sparse_accumulate on the library's static scratch: the call allocates nothing."""
    _dev(acc, "acc", torch.float32)
    n = acc.numel()
    _check_payload_sets(wires, n, bucket_elems or max(n, 1), wire_stride, status)
    rc = _lib.load().mccl_hip_sparse_accumulate_static(
        acc.data_ptr(), n, bucket_elems or max(n, 1), _ptrs(wires), len(wires), wire_stride,
        0 if scale_by is None else 1, 0.0 if scale_by is None else scale_by,
        None if status is None else status.data_ptr(), _stream())
    _lib.check(rc, "sparse_accumulate_static")
    return acc


def cast_f32_to_f16(src: torch.Tensor, dst: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(src, "src", torch.float32)
    if dst is None:
        dst = torch.empty(src.numel(), dtype=torch.float16, device=src.device)
    _dev(dst, "dst", torch.float16, src.numel())
    _lib.check(_lib.load().mccl_hip_cast_f32_to_f16(src.data_ptr(), dst.data_ptr(), src.numel(), _stream()),
               "cast_f32_to_f16")
    return dst


def cast_f16_to_f32(src: torch.Tensor, dst: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(src, "src", torch.float16)
    if dst is None:
        dst = torch.empty(src.numel(), dtype=torch.float32, device=src.device)
    _dev(dst, "dst", torch.float32, src.numel())
    _lib.check(_lib.load().mccl_hip_cast_f16_to_f32(src.data_ptr(), dst.data_ptr(), src.numel(), _stream()),
               "cast_f16_to_f32")
    return dst


def fence_signal() -> int:
    t = C.c_uint64(0)
    _lib.check(_lib.load().mccl_hip_fence_signal(_stream(), C.byref(t)), "fence_signal")
    return int(t.value)


def fence_wait(ticket: int, timeout_ms: int = 0) -> None:
    _lib.check(_lib.load().mccl_hip_fence_wait(ticket, timeout_ms), "fence_wait")


def fence_query(ticket: int) -> bool:
    rc = _lib.load().mccl_hip_fence_query(ticket)
    if rc < 0:
        raise _lib.MCCLHipError(rc, "fence_query")
    return bool(rc)


def set_tuning(key: str, value: int) -> None:
    _lib.check(_lib.load().mccl_hip_set_tuning(key.encode(), value), f"set_tuning({key})")
