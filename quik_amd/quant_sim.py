"""The reference's simulated ("fake-quant") activation path on MI355X.

`ActQuantWrapper` has the interface of the class of the same name in the reference's experiments/quant_sim.py
(:193-256): it wraps a Linear, `quantizer.configure(bits)` sets the activation width, `fp_features_configure(scales,
fp_features)` picks the `fp_features` columns with the largest scales as outliers (torch.sort order, :224-225), and
`forward` fake-quantizes the other columns per token, passes the outliers through and calls the wrapped module.
The reference does this with a dozen tensor ops per call; here the fake-quant is ONE HIP kernel
(quik_sim_act_fake_quant), the wrapped Linear stays a library GEMM.  Used for accuracy cross-checks of the kernel
path (MixedQLinear), which follows a different zero-point convention and agrees with this path to quantisation noise.
"""
from __future__ import annotations

import torch

from . import _lib as L

__all__ = ["ActQuantWrapper", "ActQuantizer", "act_fake_quant", "outlier_mask"]


def outlier_mask(cols: int, fp_feature_idx, device) -> torch.Tensor:
    """One bit per column (bit c % 32 of word c / 32), set for the outlier columns; int32 tensor on `device`."""
    bits = torch.zeros((cols + 31) // 32 * 32, dtype=torch.int64)
    if fp_feature_idx is not None and len(fp_feature_idx):
        bits[torch.as_tensor(fp_feature_idx).cpu().long()] = 1
    words = (bits.reshape(-1, 32) << torch.arange(32)).sum(1)
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.to(torch.int32).to(device)


def act_fake_quant(x: torch.Tensor, mask: torch.Tensor, bits: int) -> torch.Tensor:
    """Per-token asymmetric fake-quant of the columns whose mask bit is clear (experiments/quant_sim.py:5-7,
    167-188); the others are copied.  x: fp16 / bf16 on the GPU, any leading shape; returns a tensor like x."""
    L.check_cuda_contiguous("act_fake_quant", x=x, mask=mask)
    dt = L.dtype_id(x, "act_fake_quant", allow_bf16=True)
    cols = x.shape[-1]
    if mask.dtype != torch.int32 or mask.numel() != (cols + 31) // 32:
        raise RuntimeError("act_fake_quant: mask must hold one bit per column in int32 words (outlier_mask)")
    if not 2 <= bits <= 8:
        raise RuntimeError("act_fake_quant: bits must be between 2 and 8")
    rows = x.numel() // cols
    lib = L.load()
    with L.device_guard(x.device):
        out = torch.empty_like(x)
        L.check(lib.quik_sim_act_fake_quant(L.ptr(x), dt, rows, cols, L.ptr(mask), bits, L.ptr(out), L.stream()),
                "act_fake_quant")
    return out


class ActQuantizer(torch.nn.Module):
    """Holds the activation width (experiments/quant_sim.py:144-165); 16 bits means no quantisation."""

    def __init__(self):
        super().__init__()
        self.bits = 16
        self.configured = False

    def configure(self, bits):
        self.bits = bits
        self.configured = True


class ActQuantWrapper(torch.nn.Module):
    """experiments/quant_sim.py:193-256 with the fake-quant as one kernel."""

    def __init__(self, module):
        super().__init__()
        self.module = module
        self.quantizer = ActQuantizer()
        self.fp_features_num = 0
        self.act_scales = None
        self.fp_feature_idx = None
        self.quantized_feature_idx = None
        self._mask = None

    def extra_repr(self) -> str:
        return f'Act. Bits: {self.quantizer.bits}, FP features: {self.fp_features_num}'

    def fp_features_configure(self, scales, fp_features):
        self.act_scales = scales
        self.fp_features_num = fp_features
        order = torch.sort(scales)[1]
        if fp_features == 0:
            self.quantized_feature_idx = torch.arange(scales.shape[0])
            self.fp_feature_idx = None
        else:
            self.fp_feature_idx = order[-fp_features:]
            self.quantized_feature_idx = order[:-fp_features]
        self._mask = None

    def forward(self, x):
        x_dtype = x.dtype
        if self.quantizer.bits == 16:
            return self.module(x).to(x_dtype)
        if not x.is_cuda:
            raise RuntimeError("ActQuantWrapper.forward needs a tensor on the GPU; there is no CPU path")
        # (the reference asserts batch size 1 for 3-D inputs, :173-174; rows are independent, any batch works here)
        if self._mask is None or self._mask.device != x.device:
            self._mask = outlier_mask(x.shape[-1], self.fp_feature_idx, x.device)
        xc = x if x.is_contiguous() else x.contiguous()
        return self.module(act_fake_quant(xc, self._mask, self.quantizer.bits)).to(x_dtype)
