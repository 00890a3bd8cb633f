"""ctypes binding of libquik_hip.so (declarations: include/quik_hip.h)."""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libquik_hip.so")

QUIK_F16, QUIK_BF16 = 0, 1

_vp, _i64, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

# name -> (restype, argtypes); one entry per symbol declared in include/quik_hip.h
SIGNATURES = {
    "quik_status_string": (ctypes.c_char_p, [_int]),
    "quik_last_hip_error": (ctypes.c_char_p, []),
    "quik_abi_version": (_int, []),
    "quik_colmap_bytes": (_i64, [_i64, _i64, _i64]),
    "quik_colmap_build": (_int, [_vp, _i64, _vp, _i64, _i64, _vp, _vp]),
    "quik_asym_quantize": (_int, [_vp, _int, _i64, _i64, _vp, _i64, _i64, _int, _vp, _vp, _vp, _vp]),
    "quik_asym_find_meta": (_int, [_vp, _i64, _i64, _int, _vp, _vp]),
    "quik_asym_quantize_old": (_int, [_vp, _vp, _i64, _i64, _int, _vp, _vp]),
    "quik_asym_dequantize": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _int, _vp, _vp]),
    "quik_sym_quantize": (_int, [_vp, _vp, _i64, _i64, _int, _vp, _vp]),
    "quik_sym_dequantize": (_int, [_vp, _int, _vp, _vp, _vp, _i64, _i64, _vp, _vp]),
    "quik_asym_fused_dequantize": (_int, [_vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _i64, _i64, _i64, _int,
                                          _vp, _vp, _vp]),
    "quik_sym_fused_dequantize": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp, _vp, _vp]),
    "quik_fused_dequantize_workspace_bytes": (_i64, [_i64, _i64]),
    "quik_fp6_operand_bytes": (_i64, [_i64, _i64, _i64]),
    "quik_fp6_pack_weight": (_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "quik_colmap_streaming": (_int, [_vp, _i64, _i64, _i64, _vp]),
    "quik_asym_quantize_fp6": (_int, [_vp, _int, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _vp]),
    "quik_mixed_linear_fwd_fp6": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp]),
    "quik_sym_quantize_mapped": (_int, [_vp, _i64, _i64, _vp, _i64, _i64, _int, ctypes.c_float, _int, _vp, _vp, _vp,
                                        _vp]),
    "quik_tile8_operand_bytes": (_i64, [_i64, _i64, _i64]),
    "quik_tile8_pack_weight": (_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "quik_asym_quantize_tile8": (_int, [_vp, _int, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _vp]),
    "quik_mixed_linear_fwd_tile8": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp]),
    "quik_splitk_workspace_bytes": (_i64, [_i64, _i64, _i64, _int]),
    "quik_mixed_linear_fwd_fp6_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp, _i64,
                                            _vp]),
    "quik_mixed_linear_fwd_tile8_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp, _i64,
                                              _vp]),
    "quik_layer_workspace_bytes": (_i64, [_vp, _i64]),
    "quik_layer_forward": (_int, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp]),
    "quik_layer_set_one_launch": (None, [_int]),
    "quik_sim_act_fake_quant": (_int, [_vp, _int, _i64, _i64, _vp, _int, _vp, _vp]),
    "quik_mixed_linear_fwd_tile8_noalloc": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp]),
    "quik_int4_matmul": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "quik_int8_matmul": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "quik_mixed_linear_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _int,
                                     _vp, _vp]),
}



class QuikLayer(ctypes.Structure):
    """struct quik_layer of include/quik_hip.h."""
    _fields_ = [("struct_bytes", ctypes.c_int32), ("bits", ctypes.c_int32), ("dtype", ctypes.c_int32),
                ("symmetric", ctypes.c_int32), ("in_features", _i64), ("num_int", _i64), ("num_fp", _i64),
                ("out_features", _i64), ("sym_divisor", ctypes.c_float), ("colmap_streams", ctypes.c_int32),
                ("tiled_min_rows", ctypes.c_int32), ("reserved", ctypes.c_int32), ("colmap", _vp), ("int_weight", _vp),
                ("weights_scales", _vp), ("reduced_w", _vp), ("fp_weight", _vp), ("bias", _vp), ("tiled_weight", _vp)]


_lib = None


def load():
    """Load the HIP library; there is no fallback when it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C quik_amd/csrc` (or __graft_entry__.build()); "
                "quik_amd has no CPU or PyTorch fallback")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status: int, op: str):
    if status != 0:
        lib = load()
        msg = lib.quik_status_string(status).decode()
        if status == -7:
            msg += ": " + lib.quik_last_hip_error().decode()
        raise RuntimeError(f"{op}: {msg}")


def ptr(t):
    """Device address of a tensor as ctypes takes it for a void* argument (None -> NULL)."""
    return None if t is None else t.data_ptr()


def stream():
    """torch's current stream on the current device, as a raw hipStream_t value."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device: torch.device):
    """`with device_guard(t.device):` makes the tensor's GPU current for the launch, as the reference's CUDAGuard
    does (asymmetric.cu:179,322,495); free when it already is (the usual case: this sits on every forward)."""
    if device.index is None or device.index == torch._C._cuda_getDevice():
        return _NO_GUARD
    return torch.cuda.device(device)


def dtype_id(t: torch.Tensor, op: str, allow_bf16: bool) -> int:
    if t.dtype == torch.float16:
        return QUIK_F16
    if t.dtype == torch.bfloat16 and allow_bf16:
        return QUIK_BF16
    want = "float16 or bfloat16" if allow_bf16 else "float16"
    raise RuntimeError(f"{op}: expected a {want} tensor but got {t.dtype}")


def check_cuda_contiguous(op: str, **tensors):
    """The checks the reference's host functions make before launching:
    torch::checkAllContiguous and torch::checkDeviceType(..., CUDA)."""
    dev = None
    for name, t in tensors.items():
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{op}(): argument '{name}' must be a torch.Tensor, not {type(t).__name__}")
        if not t.is_cuda:
            raise RuntimeError(f"{op}: expected tensor for argument '{name}' to be on a CUDA (HIP) device, "
                               f"but it is on {t.device}")
        if not t.is_contiguous():
            raise RuntimeError(f"{op}: expected tensor for argument '{name}' to be contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"{op}: expected all tensors on the same GPU, but '{name}' is on {t.device} "
                               f"and another argument is on {dev}")
    return dev
