"""CPU restatement of the reference's fake-quant ("simulated") activation path.

TEST / BENCH INFRASTRUCTURE ONLY (the cpu_baseline leg of bench.py and the tests).
It follows experiments/quant_sim.py of the reference:
  asymmetric_quantize      :5-7     q = clamp(round(x/scale) + zero, 0, maxq); scale*(q - zero)
  ActQuantizer.find_params :167-188 xmin = min(row_min, 0), xmax = max(row_max, 0),
                                    all-zero row -> (-1, +1); scale = (xmax-xmin)/maxq;
                                    zero = round(-xmin/scale)
  ActQuantWrapper.forward  :227-256 outlier columns pass through, the rest is fake
                                    quantised, then the wrapped nn.Linear runs.
This path uses a different zero-point convention from the kernels, so it agrees with
the kernel path only to quantisation noise; it is the timed CPU baseline, not the
bit-exact oracle.  Storage is fp16, arithmetic fp32 (CPU BLAS has no fast half GEMM).
"""
from __future__ import annotations

import torch


def act_fake_quant(q_features: torch.Tensor, bits: int) -> torch.Tensor:
    """find_params + forward of ActQuantizer on a 2-D fp32 tensor (quant_sim.py:5-7,167-188)."""
    maxq = float(2 ** bits - 1)
    zero_t = torch.zeros(q_features.shape[0], dtype=q_features.dtype)
    xmin = torch.minimum(q_features.min(1)[0], zero_t)
    xmax = torch.maximum(q_features.max(1)[0], zero_t)
    both = (xmin == 0) & (xmax == 0)
    xmin[both] = -1
    xmax[both] = +1
    scale = ((xmax - xmin) / maxq).unsqueeze(1)
    zero = torch.round(-xmin.unsqueeze(1) / scale)
    q = torch.clamp(torch.round(q_features / scale) + zero, 0, maxq)
    return scale * (q - zero)


def sim_mixed_linear(x: torch.Tensor, weight: torch.Tensor, int_idx: torch.Tensor, fp_idx: torch.Tensor,
                     bits: int, bias: torch.Tensor | None = None,
                     weight_f32: torch.Tensor | None = None) -> torch.Tensor:
    """ActQuantWrapper.forward (quant_sim.py:227-256) around F.linear with the fake-quant weight.

    x [M, in] and weight [N, in] are fp16 (storage); compute in fp32; result fp16.  `weight_f32`
    may carry the weight already widened to fp32 so that a timing loop excludes that copy."""
    xf = x.float()
    mixed = torch.zeros_like(xf)
    mixed[:, int_idx] = act_fake_quant(xf[:, int_idx], bits).to(x.dtype).float()
    if fp_idx.numel():
        mixed[:, fp_idx] = xf[:, fp_idx]
    w32 = weight.float() if weight_f32 is None else weight_f32
    out = torch.nn.functional.linear(mixed, w32, None if bias is None else bias.float())
    return out.to(x.dtype)
