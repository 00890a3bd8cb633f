"""quik.symmetric: symmetric quantize / dequantize ops on MI355X.

Same names and keyword names as the reference's pybind module
(src/symmetric/symmetric.cpp:108-136).  The reference's own caller omits `bits`
(experiments/qlinear.py:103,142) although the binding requires it; here `bits` defaults to
the value that caller means (4 for quantize, 32 for dequantize), so both spellings work.
"""
from __future__ import annotations

import torch

from . import _lib as L

__all__ = ["quantize", "dequantize", "int4FusedDequantize", "int8FusedDequantize", "quantize_mapped"]


def quantize(src: torch.Tensor, scale: torch.Tensor, bits: int = 4) -> torch.Tensor:
    """q = rne_int(fp16(src / scale[row])); uint8 [M, ceil(K/2)] nibbles (bits=4, low four bits
    kept, no clamp) or int8 [M, K] (bits=8, wraps)."""
    L.check_cuda_contiguous("quantize", src=src, scale=scale)
    if bits not in (4, 8):
        raise RuntimeError("Unsupported data type")
    L.dtype_id(src, "quantize", allow_bf16=False)
    L.dtype_id(scale, "quantize", allow_bf16=False)
    rows, cols = src.shape
    if scale.size(0) != rows:
        raise RuntimeError(f"quantize: expected scale to have size {rows} at dimension 0, got {scale.size(0)}")
    lib = L.load()
    with L.device_guard(src.device):
        if bits == 4:
            dst = torch.empty((rows, (cols + 1) // 2), dtype=torch.uint8, device=src.device)
        else:
            dst = torch.empty((rows, cols), dtype=torch.int8, device=src.device)
        L.check(lib.quik_sym_quantize(L.ptr(src), L.ptr(scale), rows, cols, bits, L.ptr(dst), L.stream()), "quantize")
    return dst


_X_DTYPE = {8: torch.int8, 16: torch.float16, 32: torch.int32}


def dequantize(x: torch.Tensor, scale_row: torch.Tensor, scale_col: torch.Tensor, y: torch.Tensor,
               bits: int = 32) -> torch.Tensor:
    """out = fp16(fp16(fp16(fp16(x) * scale_row) * scale_col) + y); `bits` names x's type:
    8 int8, 16 float16, 32 int32.  scale_row has size(0) == M and scale_col size(1) == N."""
    L.check_cuda_contiguous("dequantize", x=x, scale_row=scale_row, scale_col=scale_col, y=y)
    if bits not in _X_DTYPE:
        raise RuntimeError("Unsupported data type")
    if x.dtype != _X_DTYPE[bits]:
        raise RuntimeError(f"dequantize: bits={bits} expects x of dtype {_X_DTYPE[bits]} but got {x.dtype}")
    if x.shape != y.shape:
        raise RuntimeError(f"dequantize: expected x and y to have the same size, got {tuple(x.shape)} and "
                           f"{tuple(y.shape)}")
    rows, cols = x.shape
    if scale_row.size(0) != rows:
        raise RuntimeError(f"dequantize: expected scale_row to have size {rows} at dimension 0")
    if scale_col.dim() < 2 or scale_col.size(1) != cols:
        raise RuntimeError(f"dequantize: expected scale_col to have size {cols} at dimension 1")
    for name, t in (("scale_row", scale_row), ("scale_col", scale_col), ("y", y)):
        L.dtype_id(t, "dequantize", allow_bf16=False)
    lib = L.load()
    with L.device_guard(x.device):
        out = torch.empty_like(y)
        L.check(lib.quik_sym_dequantize(L.ptr(x), bits, L.ptr(scale_row), L.ptr(scale_col), L.ptr(y), rows, cols,
                                        L.ptr(out), L.stream()), "dequantize")
    return out


def _fused_dequantize(op, bits, A, B, scale_row, scale_col, y):
    L.check_cuda_contiguous(op, A=A, B=B, scale_row=scale_row, scale_col=scale_col, y=y)
    want = torch.uint8 if bits == 4 else torch.int8
    if A.dtype != want or B.dtype != want:
        raise RuntimeError(f"{op}: expected {want} operands but got {A.dtype} and {B.dtype}")
    if A.dim() != 2 or B.dim() != 2 or A.size(1) != B.size(1):
        raise RuntimeError(f"{op}: A [M, K] and B [N, K] must agree in K, got {tuple(A.shape)} and {tuple(B.shape)}")
    M, N, K = A.size(0), B.size(0), A.size(1) * (2 if bits == 4 else 1)
    for name, t, n in (("scale_row", scale_row, M), ("scale_col", scale_col, N), ("y", y, M * N)):
        L.dtype_id(t, op, allow_bf16=False)
        if t.numel() != n:
            raise RuntimeError(f"{op}: expected {name} to have {n} elements but got {t.numel()}")
    lib = L.load()
    with L.device_guard(A.device):
        # one launch, no int32 matrix; only calls of at most 32 rows (weight-streaming kernel) need the workspace
        acc = torch.empty((M, N), dtype=torch.int32, device=A.device) \
            if lib.quik_fused_dequantize_workspace_bytes(M, N) else None
        out = torch.empty((M, N), dtype=torch.float16, device=A.device)
        L.check(lib.quik_sym_fused_dequantize(L.ptr(A), L.ptr(B), L.ptr(scale_row), L.ptr(scale_col), L.ptr(y), M, N, K,
                                              bits, L.ptr(acc), L.ptr(out), L.stream()), op)
    return out


def int4FusedDequantize(A, B, scale_row, scale_col, y):
    """out = int4(A) @ int4(B)^T * scale_row * scale_col + y, left to right in fp16
    (src/symmetric/symmetric.cpp:44-57).  A [M, K/2], B [N, K/2] uint8; scale_row [M, 1], scale_col [1, N], y [M, N] fp16."""
    return _fused_dequantize("int4FusedDequantize", 4, A, B, scale_row, scale_col, y)


def int8FusedDequantize(A, B, scale_row, scale_col, y):
    """int8 operands [M, K] / [N, K]; otherwise as int4FusedDequantize (src/symmetric/symmetric.cpp:59-72)."""
    return _fused_dequantize("int8FusedDequantize", 8, A, B, scale_row, scale_col, y)


def quantize_mapped(src: torch.Tensor, colmap: torch.Tensor, num_int: int, num_fp: int, bits: int, divisor: float,
                    tiled: bool):
    """MixedQLinear's symmetric activation branch (experiments/qlinear.py:97-103) in one kernel: outlier gather,
    scale = fp16(max|x[:, int]| / divisor) and rne(fp16(x / scale)) codes.  fp16 only; the column map must select
    the streaming kernel (asymmetric.colmap_streams).  Returns (q, scale [rows, 1], fp_x) with q / fp_x as
    symmetric.quantize would give them, or, with tiled=True, (operand buffer, scale, None) for
    matmul.mixed_linear_fp6 (bits=4) / matmul.mixed_linear_tile8 (bits=8)."""
    from .asymmetric import check_mapped_args
    if bits not in (4, 8):
        raise RuntimeError("Unsupported data type")
    rows, cols = check_mapped_args("quantize", src, colmap, num_int, num_fp, need_streaming=True)
    L.dtype_id(src, "quantize", allow_bf16=False)
    lib = L.load()
    with L.device_guard(src.device):
        if tiled:
            nbytes = (lib.quik_fp6_operand_bytes if bits == 4 else lib.quik_tile8_operand_bytes)(max(rows, 1), num_int,
                                                                                                  num_fp)
            if nbytes == 0:
                raise RuntimeError("quantize: shape not supported by the tile-ordered operand format")
            dst = torch.empty((nbytes,), dtype=torch.uint8, device=src.device)
            fp_x = None
        else:
            dst = torch.empty((rows, num_int // 2) if bits == 4 else (rows, num_int),
                              dtype=torch.uint8 if bits == 4 else torch.int8, device=src.device)
            fp_x = torch.empty((rows, num_fp), dtype=src.dtype, device=src.device)
        scale = torch.empty((rows, 1), dtype=torch.float16, device=src.device)
        L.check(lib.quik_sym_quantize_mapped(L.ptr(src), rows, cols, L.ptr(colmap), num_int, num_fp, bits,
                                             float(divisor), 1 if tiled else 0, L.ptr(dst), L.ptr(scale),
                                             L.ptr(fp_x) if fp_x is not None and num_fp else None, L.stream()),
                "quantize")
    return dst, scale, fp_x
