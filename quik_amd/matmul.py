"""quik.matmul: exact integer GEMMs on MI355X matrix cores.

Same names and keyword names as the reference's pybind module (src/matmul/matmul.cpp:78-109):
int4Matmul(A, B), int8Matmul(A, B) -> int32 [M, N] = A @ B^T.  The 2:4-sparse and cuSPARSELt
entry points of the reference are NVIDIA sparse-tensor-core formats and are not provided.
mixed_linear is the one-launch fused tail of MixedQLinear.forward (no reference counterpart
as a separate op; it computes what experiments/qlinear.py:122-145 computes in three ops).
"""
from __future__ import annotations

import threading

import torch

from . import _lib as L

__all__ = ["int4Matmul", "int8Matmul", "mixed_linear", "pack_weight_fp6", "mixed_linear_fp6", "pack_weight_tile8",
           "mixed_linear_tile8"]


def _matmul(op, A, B, want_dtype, sym, kmul):
    L.check_cuda_contiguous(op, A=A, B=B)
    if A.dtype != want_dtype or B.dtype != want_dtype:
        raise RuntimeError(f"{op}: expected {want_dtype} operands but got {A.dtype} and {B.dtype}")
    if A.dim() != 2 or B.dim() != 2 or A.size(1) != B.size(1):
        raise RuntimeError(f"{op}: A [M, K] and B [N, K] must agree in K, got {tuple(A.shape)} and {tuple(B.shape)}")
    M, N, K = A.size(0), B.size(0), A.size(1) * kmul
    lib = L.load()
    with L.device_guard(A.device):
        C = torch.empty((M, N), dtype=torch.int32, device=A.device)
        L.check(getattr(lib, sym)(L.ptr(A), L.ptr(B), L.ptr(C), M, N, K, L.stream()), op)
    return C


def int4Matmul(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """A uint8 [M, K/2], B uint8 [N, K/2], nibble-packed int4 (low nibble = even element)."""
    return _matmul("int4Matmul", A, B, torch.uint8, "quik_int4_matmul", 2)


def int8Matmul(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """A int8 [M, K], B int8 [N, K]."""
    return _matmul("int8Matmul", A, B, torch.int8, "quik_int8_matmul", 1)


def mixed_linear(qx, int_weight, meta, weights_scales, reduced_w, fp_x, fp_weight, bias, bits, out_dtype):
    """Fused outlier GEMM + integer GEMM + dequantize: returns [M, N] in out_dtype.

    reduced_w=None selects the symmetric form (meta = per-row scales, no zero-point term)."""
    if bits not in (4, 8):
        raise RuntimeError("bits argument must be either 4 or 8")
    tensors = dict(qx=qx, int_weight=int_weight, meta=meta, weights_scales=weights_scales)
    for name, t in (("reduced_w", reduced_w), ("fp_x", fp_x), ("fp_weight", fp_weight), ("bias", bias)):
        if t is not None and t.numel() > 0:
            tensors[name] = t
    L.check_cuda_contiguous("mixed_linear", **tensors)
    want = torch.uint8 if bits == 4 else torch.int8
    if qx.dtype != want or int_weight.dtype != want:
        raise RuntimeError(f"mixed_linear: bits={bits} expects {want} operands")
    if out_dtype == torch.float16:
        dt = L.QUIK_F16
    elif out_dtype == torch.bfloat16:
        dt = L.QUIK_BF16
    else:
        raise RuntimeError(f"mixed_linear: unsupported dtype {out_dtype}")
    for name, t in tensors.items():
        if name not in ("qx", "int_weight") and t.dtype != out_dtype:
            raise RuntimeError(f"mixed_linear: expected {name} of dtype {out_dtype} but got {t.dtype}")
    M, N = qx.size(0), int_weight.size(0)
    if qx.size(1) != int_weight.size(1):
        raise RuntimeError("mixed_linear: qx and int_weight disagree in K")
    K = qx.size(1) * (2 if bits == 4 else 1)
    F = 0 if "fp_x" not in tensors else fp_x.size(1)
    if F and (fp_weight.size(0) != N or fp_weight.size(1) != F or fp_x.size(0) != M):
        raise RuntimeError("mixed_linear: fp_x [M, F] and fp_weight [N, F] sizes are inconsistent")
    if meta.numel() != (2 * M if reduced_w is not None else M) or weights_scales.numel() != N:
        raise RuntimeError("mixed_linear: meta / weights_scales sizes are inconsistent with M, N")
    if reduced_w is not None and reduced_w.numel() != N:
        raise RuntimeError("mixed_linear: reduced_w must have N elements")
    if "bias" in tensors and bias.numel() != N:
        raise RuntimeError("mixed_linear: bias must have N elements")
    lib = L.load()
    with L.device_guard(qx.device):
        out = torch.empty((M, N), dtype=out_dtype, device=qx.device)
        L.check(lib.quik_mixed_linear_fwd(L.ptr(qx), L.ptr(int_weight), L.ptr(meta), L.ptr(weights_scales),
                                          L.ptr(reduced_w), L.ptr(fp_x) if F else None,
                                          L.ptr(fp_weight) if F else None, L.ptr(tensors.get("bias")), dt, M, N, K,
                                          F, bits, L.ptr(out), L.stream()), "mixed_linear")
    return out


# K split of the tile-ordered GEMMs (few token rows, few output columns, long K) needs a zeroed workspace (arrival
# counters, which every launch leaves at zero, and partial sums).  Launches that overlap on one GPU must not share
# one, so there is one per (GPU, stream), made by the first eager call on that stream that can use it, shared by all
# layers, and one more per GPU for calls recorded into HIP graphs (made together with the GPU's first eager one: a
# capture cannot allocate).  Graphs that are replayed on different streams at the same time would share that one:
# set split_k = False while capturing such graphs.  Beyond _MAX_STREAMS streams per GPU further streams run without
# the K split (same output bits, the unsplit kernel).
split_k = True
_SPLITK_BYTES = 4096 + 256 * 128 * 128 * 4   # the largest request: 256 workgroups of one 128x128 tile each
_MAX_STREAMS = 8
_splitk_workspaces = {}
_splitk_needed = {}
_splitk_lock = threading.Lock()


def _splitk_workspace(device, M, N, K, bits):
    if not split_k:
        return None, 0
    key = (M, N, K, bits)
    need = _splitk_needed.get(key)
    if need is None:
        need = _splitk_needed[key] = L.load().quik_splitk_workspace_bytes(M, N, K, bits)
    if need == 0:
        return None, 0
    capturing = torch.cuda.is_current_stream_capturing()
    slot = (device.index, "graphs" if capturing else torch.cuda.current_stream(device).cuda_stream)
    ws = _splitk_workspaces.get(slot)
    if ws is None:
        if capturing:                                   # no allocation that a graph's pool would own
            return None, 0
        with _splitk_lock:
            ws = _splitk_workspaces.get(slot)
            if ws is None:
                if sum(1 for d, _ in _splitk_workspaces if d == device.index) > _MAX_STREAMS:
                    return None, 0
                if (device.index, "graphs") not in _splitk_workspaces:
                    _splitk_workspaces[(device.index, "graphs")] = torch.zeros(_SPLITK_BYTES, dtype=torch.uint8,
                                                                               device=device)
                ws = _splitk_workspaces[slot] = torch.zeros(_SPLITK_BYTES, dtype=torch.uint8, device=device)
    return ws, ws.numel()


def pack_weight_fp6(int_weight: torch.Tensor, fp_weight: torch.Tensor, colmap: torch.Tensor) -> torch.Tensor:
    """Nibble-packed int4 weights [N, K/2] and outlier weights [N, F] -> operand buffer for mixed_linear_fp6
    (once per layer).  `colmap` is the layer's column map (asymmetric.build_colmap): the operand buffers of this
    path keep the integer columns in the map's in-place order, weights and activations alike."""
    L.check_cuda_contiguous("pack_weight_fp6", int_weight=int_weight, fp_weight=fp_weight, colmap=colmap)
    if int_weight.dtype != torch.uint8 or int_weight.dim() != 2:
        raise RuntimeError("pack_weight_fp6: expected a uint8 [N, K/2] int_weight")
    if fp_weight.dtype not in (torch.float16, torch.bfloat16) or fp_weight.dim() != 2 or \
            fp_weight.size(0) != int_weight.size(0):
        raise RuntimeError("pack_weight_fp6: expected an fp16/bf16 [N, F] fp_weight")
    N, K, F = int_weight.size(0), int_weight.size(1) * 2, fp_weight.size(1)
    lib = L.load()
    nbytes = lib.quik_fp6_operand_bytes(N, K, F)
    if nbytes == 0:
        raise RuntimeError("pack_weight_fp6: K must be a multiple of 128 and F a multiple of 32")
    if colmap.dtype != torch.uint8 or colmap.numel() != lib.quik_colmap_bytes(K + F, K, F):
        raise RuntimeError(f"pack_weight_fp6: the column map was not built for {K} integer and {F} outlier columns")
    from .asymmetric import colmap_streams
    if getattr(colmap, "_quik_streams", None) is None:
        colmap._quik_shape = (K + F, K, F)
        colmap._quik_streams = colmap_streams(colmap, K, F)
    if not colmap._quik_streams:
        raise RuntimeError("pack_weight_fp6: the column map does not select the streaming kernel (ascending "
                           "int_indices that partition the columns with fp_indices)")
    with L.device_guard(int_weight.device):
        out = torch.empty((nbytes,), dtype=torch.uint8, device=int_weight.device)
        L.check(lib.quik_fp6_pack_weight(L.ptr(int_weight), L.ptr(fp_weight) if F else None, N, K, F, L.ptr(colmap),
                                         L.ptr(out), L.stream()), "pack_weight_fp6")
    return out


def mixed_linear_fp6(x6, w6, meta, weights_scales, reduced_w, bias, M, N, K, F, out_dtype):
    """mixed_linear (asymmetric, 4 bits) on operand buffers (asymmetric.quantize_mapped_fp6, pack_weight_fp6):
    the int4 products run on the E2M3 matrix-core path at twice the int8 rate; same result bit for bit."""
    tensors = dict(x6=x6, w6=w6, meta=meta, weights_scales=weights_scales)
    symmetric = reduced_w is None      # meta then holds one scale per row and there is no zero-point term
    if not symmetric:
        tensors["reduced_w"] = reduced_w
    if bias is not None and bias.numel() > 0:
        tensors["bias"] = bias
    L.check_cuda_contiguous("mixed_linear_fp6", **tensors)
    dt = L.QUIK_F16 if out_dtype == torch.float16 else L.QUIK_BF16 if out_dtype == torch.bfloat16 else None
    if dt is None:
        raise RuntimeError(f"mixed_linear_fp6: unsupported dtype {out_dtype}")
    for name, t in tensors.items():
        if name not in ("x6", "w6") and t.dtype != out_dtype:
            raise RuntimeError(f"mixed_linear_fp6: expected {name} of dtype {out_dtype} but got {t.dtype}")
    lib = L.load()
    if x6.numel() != lib.quik_fp6_operand_bytes(M, K, F) or w6.numel() != lib.quik_fp6_operand_bytes(N, K, F):
        raise RuntimeError("mixed_linear_fp6: operand buffers do not match M, N, K, F")
    if meta.numel() != (M if symmetric else 2 * M) or weights_scales.numel() != N or \
            (not symmetric and reduced_w.numel() != N):
        raise RuntimeError("mixed_linear_fp6: meta / weights_scales / reduced_w sizes are inconsistent with M, N")
    with L.device_guard(x6.device):
        out = torch.empty((M, N), dtype=out_dtype, device=x6.device)
        ws, ws_bytes = _splitk_workspace(x6.device, M, N, K, 4)
        L.check(lib.quik_mixed_linear_fwd_fp6_ws(L.ptr(x6), L.ptr(w6), L.ptr(meta), L.ptr(weights_scales),
                                                 L.ptr(tensors.get("reduced_w")), L.ptr(tensors.get("bias")), dt, M, N, K,
                                                 F, L.ptr(out), L.ptr(ws), ws_bytes, L.stream()), "mixed_linear_fp6")
    return out


def pack_weight_tile8(int_weight: torch.Tensor, fp_weight: torch.Tensor) -> torch.Tensor:
    """int8 weights [N, K] and outlier weights [N, F] -> tile-ordered operand buffer for mixed_linear_tile8
    (once per layer)."""
    L.check_cuda_contiguous("pack_weight_tile8", int_weight=int_weight, fp_weight=fp_weight)
    if int_weight.dtype != torch.int8 or int_weight.dim() != 2:
        raise RuntimeError("pack_weight_tile8: expected an int8 [N, K] int_weight")
    if fp_weight.dtype not in (torch.float16, torch.bfloat16) or fp_weight.dim() != 2 or \
            fp_weight.size(0) != int_weight.size(0):
        raise RuntimeError("pack_weight_tile8: expected an fp16/bf16 [N, F] fp_weight")
    N, K, F = int_weight.size(0), int_weight.size(1), fp_weight.size(1)
    lib = L.load()
    nbytes = lib.quik_tile8_operand_bytes(N, K, F)
    if nbytes == 0:
        raise RuntimeError("pack_weight_tile8: K must be a multiple of 64 and F a multiple of 32")
    with L.device_guard(int_weight.device):
        out = torch.empty((nbytes,), dtype=torch.uint8, device=int_weight.device)
        L.check(lib.quik_tile8_pack_weight(L.ptr(int_weight), L.ptr(fp_weight) if F else None, N, K, F, L.ptr(out),
                                           L.stream()), "pack_weight_tile8")
    return out


def mixed_linear_tile8(x8, w8, meta, weights_scales, reduced_w, bias, M, N, K, F, out_dtype):
    """mixed_linear (asymmetric, 8 bits) on tile-ordered operand buffers (asymmetric.quantize_mapped_tile8,
    pack_weight_tile8): same result bit for bit, every operand cache line fetched once per tile."""
    tensors = dict(x8=x8, w8=w8, meta=meta, weights_scales=weights_scales)
    symmetric = reduced_w is None      # meta then holds one scale per row and there is no zero-point term
    if not symmetric:
        tensors["reduced_w"] = reduced_w
    if bias is not None and bias.numel() > 0:
        tensors["bias"] = bias
    L.check_cuda_contiguous("mixed_linear_tile8", **tensors)
    dt = L.QUIK_F16 if out_dtype == torch.float16 else L.QUIK_BF16 if out_dtype == torch.bfloat16 else None
    if dt is None:
        raise RuntimeError(f"mixed_linear_tile8: unsupported dtype {out_dtype}")
    for name, t in tensors.items():
        if name not in ("x8", "w8") and t.dtype != out_dtype:
            raise RuntimeError(f"mixed_linear_tile8: expected {name} of dtype {out_dtype} but got {t.dtype}")
    lib = L.load()
    if x8.numel() != lib.quik_tile8_operand_bytes(M, K, F) or w8.numel() != lib.quik_tile8_operand_bytes(N, K, F):
        raise RuntimeError("mixed_linear_tile8: operand buffers do not match M, N, K, F")
    if meta.numel() != (M if symmetric else 2 * M) or weights_scales.numel() != N or \
            (not symmetric and reduced_w.numel() != N):
        raise RuntimeError("mixed_linear_tile8: meta / weights_scales / reduced_w sizes are inconsistent with M, N")
    with L.device_guard(x8.device):
        out = torch.empty((M, N), dtype=out_dtype, device=x8.device)
        ws, ws_bytes = _splitk_workspace(x8.device, M, N, K, 8)
        L.check(lib.quik_mixed_linear_fwd_tile8_ws(L.ptr(x8), L.ptr(w8), L.ptr(meta), L.ptr(weights_scales),
                                                   L.ptr(tensors.get("reduced_w")), L.ptr(tensors.get("bias")), dt, M, N,
                                                   K, F, L.ptr(out), L.ptr(ws), ws_bytes, L.stream()),
                "mixed_linear_tile8")
    return out
