"""quik.asymmetric: per-token asymmetric quantize / dequantize ops on MI355X.

Same names, argument order and keyword names as the reference's pybind module
(src/asymmetric/asymmetric.cpp:134-180 of the reference): quantize, dequantize, find_meta,
quantizeOld.  Every op allocates and returns new tensors on the device of its first argument
and runs on torch's current stream.
"""
from __future__ import annotations

import torch

from . import _lib as L

__all__ = ["int4FusedDequantize", "int8FusedDequantize", "quantize", "dequantize", "find_meta", "quantizeOld",
           "build_colmap", "quantize_mapped", "quantize_mapped_fp6", "quantize_mapped_tile8", "colmap_streams",
           "check_mapped_args"]


def _check_bits(bits):
    if bits not in (4, 8):
        raise RuntimeError("bits argument must be either 4 or 8")


def build_colmap(int_indices: torch.Tensor, fp_indices: torch.Tensor, cols: int) -> torch.Tensor:
    """Compact column map for quantize_mapped (uint8 blob on the indices' device).

    Build it once per layer; it depends only on the two index tensors."""
    L.check_cuda_contiguous("quantize", int_indices=int_indices, fp_indices=fp_indices)
    if int_indices.dtype != torch.int64 or fp_indices.dtype != torch.int64:
        raise RuntimeError("quantize: int_indices and fp_indices must be int64 tensors")
    lib = L.load()
    num_int, num_fp = int_indices.numel(), fp_indices.numel()
    if num_fp + num_int != cols:
        raise RuntimeError("Quantize: number of fp and int columns is not equal to total number of columns")
    nbytes = lib.quik_colmap_bytes(cols, num_int, num_fp)
    with L.device_guard(int_indices.device):
        cm = torch.empty(nbytes, dtype=torch.uint8, device=int_indices.device)
        L.check(lib.quik_colmap_build(L.ptr(int_indices), num_int, L.ptr(fp_indices) if num_fp else None, num_fp,
                                      cols, L.ptr(cm), L.stream()), "quantize")
    return cm


def check_mapped_args(op: str, src: torch.Tensor, colmap: torch.Tensor, num_int: int, num_fp: int,
                      need_streaming: bool = False):
    """Argument checks shared by the ops that take a prebuilt column map; returns (rows, cols).

    The column map must be the blob `build_colmap` made for these (cols, num_int, num_fp): a map of another shape has
    its sections at other offsets.  need_streaming: the op exists on the streaming kernel only (tile-ordered output,
    symmetric activations); a map built from int_indices in any other than ascending order is refused here, before
    anything is launched (checked once per column map, the answer is kept on the tensor)."""
    L.check_cuda_contiguous(op, src=src, colmap=colmap)
    if src.dim() != 2:
        raise RuntimeError(f"{op}: expected a 2-D src but got {src.dim()} dimensions")
    rows, cols = src.shape
    if num_fp + num_int != cols:
        raise RuntimeError("Quantize: number of fp and int columns is not equal to total number of columns")
    if getattr(colmap, "_quik_shape", None) != (cols, num_int, num_fp):      # first use of this map with this shape
        if colmap.dtype != torch.uint8:
            raise RuntimeError(f"{op}: the column map is a uint8 blob from build_colmap, got {colmap.dtype}")
        if colmap.numel() != L.load().quik_colmap_bytes(cols, num_int, num_fp):
            raise RuntimeError(f"{op}: the column map was not built for {num_int} integer and {num_fp} outlier "
                               "columns")
        colmap._quik_shape = (cols, num_int, num_fp)
        colmap._quik_streams = None
    if need_streaming:
        if colmap._quik_streams is None:
            colmap._quik_streams = colmap_streams(colmap, num_int, num_fp)
        if not colmap._quik_streams:
            raise RuntimeError(f"{op}: this op needs ascending int_indices that partition the columns with fp_indices "
                               "(and a multiple of 8 columns, at most 32768): the column map does not select the "
                               "streaming kernel")
    return rows, cols


def quantize_mapped(src: torch.Tensor, colmap: torch.Tensor, num_int: int, num_fp: int, bits: int):
    """quantize() with a prebuilt column map: one kernel launch."""
    _check_bits(bits)
    rows, cols = check_mapped_args("quantize", src, colmap, num_int, num_fp)
    dt = L.dtype_id(src, "quantize", allow_bf16=True)
    if num_int % 2 != 0:
        raise RuntimeError("Quantize: number of int columns has to be even (implementation detail)")
    lib = L.load()
    with L.device_guard(src.device):
        if bits == 4:
            dst = torch.empty((rows, num_int // 2), dtype=torch.uint8, device=src.device)
        else:
            dst = torch.empty((rows, num_int), dtype=torch.int8, device=src.device)
        meta = torch.empty((2 * rows,), dtype=src.dtype, device=src.device)
        fp_x = torch.empty((rows, num_fp), dtype=src.dtype, device=src.device)
        L.check(lib.quik_asym_quantize(L.ptr(src), dt, rows, cols, L.ptr(colmap), num_int, num_fp, bits, L.ptr(dst),
                                       L.ptr(meta), L.ptr(fp_x), L.stream()), "quantize")
    return dst, meta, fp_x


def colmap_streams(colmap: torch.Tensor, num_int: int, num_fp: int) -> bool:
    """True if the column map selects the streaming kernel (ascending int_indices that partition the
    columns with fp_indices, cols % 8 == 0, cols <= 32768).  Synchronises once: call per layer, not per step."""
    lib = L.load()
    with L.device_guard(colmap.device):
        rc = lib.quik_colmap_streaming(L.ptr(colmap), num_int + num_fp, num_int, num_fp, L.stream())
    if rc < 0:
        L.check(rc, "colmap_streams")
    return rc == 1


def quantize_mapped_fp6(src: torch.Tensor, colmap: torch.Tensor, num_int: int, num_fp: int):
    """quantize_mapped with bits = 4 whose codes and outlier values go to an operand buffer for
    matmul.mixed_linear_fp6 (internal format, see include/quik_hip.h).  Returns (x6 uint8 buffer, meta)."""
    rows, cols = check_mapped_args("quantize", src, colmap, num_int, num_fp, need_streaming=True)
    dt = L.dtype_id(src, "quantize", allow_bf16=True)
    lib = L.load()
    nbytes = lib.quik_fp6_operand_bytes(max(rows, 1), num_int, num_fp)
    if nbytes == 0:
        raise RuntimeError("quantize: the 6-bit operand format needs a multiple of 128 integer columns and a "
                           "multiple of 32 outlier columns")
    with L.device_guard(src.device):
        x6 = torch.empty((nbytes,), dtype=torch.uint8, device=src.device)
        meta = torch.empty((2 * rows,), dtype=src.dtype, device=src.device)
        L.check(lib.quik_asym_quantize_fp6(L.ptr(src), dt, rows, cols, L.ptr(colmap), num_int, num_fp, L.ptr(x6),
                                           L.ptr(meta), L.stream()), "quantize")
    return x6, meta


def quantize_mapped_tile8(src: torch.Tensor, colmap: torch.Tensor, num_int: int, num_fp: int):
    """quantize_mapped with bits = 8 whose codes and outlier values go to a tile-ordered operand buffer for
    matmul.mixed_linear_tile8 (internal format, see include/quik_hip.h).  Returns (x8 uint8 buffer, meta)."""
    rows, cols = check_mapped_args("quantize", src, colmap, num_int, num_fp, need_streaming=True)
    dt = L.dtype_id(src, "quantize", allow_bf16=True)
    lib = L.load()
    nbytes = lib.quik_tile8_operand_bytes(max(rows, 1), num_int, num_fp)
    if nbytes == 0:
        raise RuntimeError("quantize: the tile-ordered int8 format needs a multiple of 64 integer columns and a "
                           "multiple of 32 outlier columns")
    with L.device_guard(src.device):
        x8 = torch.empty((nbytes,), dtype=torch.uint8, device=src.device)
        meta = torch.empty((2 * rows,), dtype=src.dtype, device=src.device)
        L.check(lib.quik_asym_quantize_tile8(L.ptr(src), dt, rows, cols, L.ptr(colmap), num_int, num_fp, L.ptr(x8),
                                             L.ptr(meta), L.stream()), "quantize")
    return x8, meta


def quantize(src: torch.Tensor, int_indices: torch.Tensor, fp_indices: torch.Tensor, bits: int):
    """(dst, meta, fp_x) = quantize(src [M, in], int_indices [K] int64, fp_indices [F] int64, bits).

    dst: uint8 [M, K/2] (bits=4, low nibble = even element) or int8 [M, K]; meta: [2M]
    interleaved (scale, zero) in src's dtype; fp_x[r, j] = src[r, fp_indices[j]]."""
    _check_bits(bits)
    L.check_cuda_contiguous("quantize", src=src)
    L.check_cuda_contiguous("quantize", int_indices=int_indices)
    L.check_cuda_contiguous("quantize", fp_indices=fp_indices)
    if src.dim() != 2:
        raise RuntimeError(f"quantize: expected a 2-D src but got {src.dim()} dimensions")
    colmap = build_colmap(int_indices, fp_indices, src.shape[1])
    return quantize_mapped(src, colmap, int_indices.numel(), fp_indices.numel(), bits)


def dequantize(x: torch.Tensor, meta: torch.Tensor, scale_col: torch.Tensor, wReduced: torch.Tensor,
               y: torch.Tensor, bits: int) -> torch.Tensor:
    """out = dtype(f32(x) * (s_row * s_col) + ((zero + 2^(bits-1) * s_row) * wReduced + y)).

    x int32 [M, N]; meta [2M]; scale_col with size(0) == N; wReduced with size(1) == N; y [M, N]."""
    L.check_cuda_contiguous("dequantize", x=x, meta=meta, scale_col=scale_col, y=y)
    L.check_cuda_contiguous("dequantize", wReduced=wReduced.contiguous())
    _check_bits(bits)
    if x.dtype != torch.int32:
        raise RuntimeError(f"dequantize: expected an int32 x but got {x.dtype}")
    if x.numel() != y.numel():
        raise RuntimeError(f"Expected tensor for x to have same number of elements as tensor for y; but "
                           f"{x.numel()} does not equal {y.numel()} (while checking arguments for dequantize)")
    rows, cols = x.shape
    if meta.size(0) != 2 * rows:
        raise RuntimeError(f"dequantize: expected meta to have size {2 * rows} at dimension 0, got {meta.size(0)}")
    if scale_col.size(0) != cols:
        raise RuntimeError(f"dequantize: expected scale_col to have size {cols} at dimension 0, "
                           f"got {scale_col.size(0)}")
    if wReduced.dim() < 2 or wReduced.size(1) != cols:
        raise RuntimeError(f"dequantize: expected wReduced to have size {cols} at dimension 1")
    dt = L.dtype_id(y, "dequantize", allow_bf16=True)
    for name, t in (("meta", meta), ("scale_col", scale_col), ("wReduced", wReduced)):
        if t.dtype != y.dtype:
            raise RuntimeError(f"dequantize: expected {name} to have dtype {y.dtype} but got {t.dtype}")
    lib = L.load()
    with L.device_guard(x.device):
        out = torch.empty_like(y)
        L.check(lib.quik_asym_dequantize(L.ptr(x), L.ptr(meta), L.ptr(scale_col), L.ptr(wReduced.contiguous()),
                                         L.ptr(y), dt, rows, cols, bits, L.ptr(out), L.stream()), "dequantize")
    return out


def find_meta(src: torch.Tensor, bits: int) -> torch.Tensor:
    """meta [2M] fp16: per-row (scale, zero) over all columns of an fp16 src."""
    L.check_cuda_contiguous("find_meta", src=src)
    _check_bits(bits)
    L.dtype_id(src, "find_meta", allow_bf16=False)
    rows, cols = src.shape
    lib = L.load()
    with L.device_guard(src.device):
        meta = torch.empty((2 * rows,), dtype=torch.float16, device=src.device)
        L.check(lib.quik_asym_find_meta(L.ptr(src), rows, cols, bits, L.ptr(meta), L.stream()), "find_meta")
    return meta


def quantizeOld(src: torch.Tensor, meta: torch.Tensor, bits: int) -> torch.Tensor:
    """Quantise every column of an fp16 src with given meta [2M]."""
    L.check_cuda_contiguous("quantize", src=src, meta=meta)
    _check_bits(bits)
    L.dtype_id(src, "quantize", allow_bf16=False)
    L.dtype_id(meta, "quantize", allow_bf16=False)
    rows, cols = src.shape
    if meta.size(0) != 2 * rows:
        raise RuntimeError(f"quantize: expected meta to have size {2 * rows} at dimension 0, got {meta.size(0)}")
    lib = L.load()
    with L.device_guard(src.device):
        if bits == 4:
            dst = torch.empty((rows, (cols + 1) // 2), dtype=torch.uint8, device=src.device)
        else:
            dst = torch.empty((rows, cols), dtype=torch.int8, device=src.device)
        L.check(lib.quik_asym_quantize_old(L.ptr(src), L.ptr(meta), rows, cols, bits, L.ptr(dst), L.stream()),
                "quantize")
    return dst


def _fused_operands(op, A, B, bits):
    want = torch.uint8 if bits == 4 else torch.int8
    if A.dtype != want or B.dtype != want:
        raise RuntimeError(f"{op}: expected {want} operands but got {A.dtype} and {B.dtype}")
    if A.dim() != 2 or B.dim() != 2 or A.size(1) != B.size(1):
        raise RuntimeError(f"{op}: A [M, K] and B [N, K] must agree in K, got {tuple(A.shape)} and {tuple(B.shape)}")
    return A.size(0), B.size(0), A.size(1) * (2 if bits == 4 else 1)


def _fused_dequantize(op, bits, A, B, scale_row, scale_col, shift_value, zero_row, w_reduced, y):
    L.check_cuda_contiguous(op, A=A, B=B, scale_row=scale_row, scale_col=scale_col, zero_row=zero_row,
                            w_reduced=w_reduced, y=y)
    M, N, K = _fused_operands(op, A, B, bits)
    for name, t, n in (("scale_row", scale_row, M), ("zero_row", zero_row, M), ("scale_col", scale_col, N),
                       ("w_reduced", w_reduced, N), ("y", y, M * N)):
        L.dtype_id(t, op, allow_bf16=False)
        if t.numel() != n:
            raise RuntimeError(f"{op}: expected {name} to have {n} elements but got {t.numel()}")
    lib = L.load()
    with L.device_guard(A.device):
        # one launch, no int32 matrix; only calls of at most 32 rows (weight-streaming kernel) need the workspace
        acc = torch.empty((M, N), dtype=torch.int32, device=A.device) \
            if lib.quik_fused_dequantize_workspace_bytes(M, N) else None
        out = torch.empty((M, N), dtype=torch.float16, device=A.device)
        L.check(lib.quik_asym_fused_dequantize(L.ptr(A), L.ptr(B), L.ptr(scale_row), L.ptr(scale_col),
                                               float(shift_value), L.ptr(zero_row), L.ptr(w_reduced), L.ptr(y), M, N,
                                               K, bits, L.ptr(acc), L.ptr(out), L.stream()), op)
    return out


def int4FusedDequantize(A, B, scale_row, scale_col, shift_value, zero_row, w_reduced, y):
    """out = int4(A) @ int4(B)^T * scale_col * scale_row + (zero_row + shift_value * scale_row) * w_reduced + y,
    evaluated left to right in fp16 like the reference's epilogue (src/asymmetric/asymmetric.cpp:46-65).
    A [M, K/2], B [N, K/2] uint8; scale_row, zero_row [M, 1]; scale_col, w_reduced [1, N]; y [M, N]; all fp16."""
    return _fused_dequantize("int4FusedDequantize", 4, A, B, scale_row, scale_col, shift_value, zero_row, w_reduced, y)


def int8FusedDequantize(A, B, scale_row, scale_col, shift_value, zero_row, w_reduced, y):
    """int8 operands [M, K] / [N, K]; otherwise as int4FusedDequantize (src/asymmetric/asymmetric.cpp:67-88)."""
    return _fused_dequantize("int8FusedDequantize", 8, A, B, scale_row, scale_col, shift_value, zero_row, w_reduced, y)
