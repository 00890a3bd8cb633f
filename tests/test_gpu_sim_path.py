"""The reference's simulated (fake-quant) activation path on the GPU (quik_amd/quant_sim.py, one HIP kernel)
against its CPU restatement oracle/sim_path.py (experiments/quant_sim.py:5-7,167-188,227-256): the fake-quantized
activation bit for bit (both evaluate the same IEEE fp32 expression and round once to the storage type), the
wrapped Linear's output within the fp16 tolerance of a library GEMM."""
import numpy as np
import pytest
import torch

from oracle import sim_path

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _inputs(M, n_in, F, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, n_in, generator=g)
    scales = torch.rand(n_in, generator=g)
    fp_idx = torch.sort(scales)[1][-F:] if F else torch.tensor([], dtype=torch.long)
    x[:, fp_idx] *= 50
    x[0] = 0.0                                     # all-zero row: (xmin, xmax) = (-1, +1)
    x[1] = x[1].abs() + 0.5                        # all positive: xmin = 0
    x[2] = -x[2].abs() - 0.5                       # all negative: xmax = 0
    x[3] *= 1e-4
    return x.to(dtype), scales, fp_idx


@pytest.mark.parametrize("M,n_in,F", [(40, 512, 32), (9, 1000, 13), (300, 8192, 256), (5, 100, 0), (7, 4100, 64)])
@pytest.mark.parametrize("bits", [4, 8, 3])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_act_fake_quant_equals_the_cpu_restatement(M, n_in, F, bits, dtype):
    from quik_amd import quant_sim
    x, scales, fp_idx = _inputs(M, n_in, F, M + n_in + bits, dtype)
    keep = torch.ones(n_in, dtype=torch.bool)
    keep[fp_idx] = False
    int_idx = torch.arange(n_in)[keep]
    want = torch.zeros(M, n_in)
    want[:, int_idx] = sim_path.act_fake_quant(x.float()[:, int_idx], bits)
    want = want.to(dtype)
    want[:, fp_idx] = x[:, fp_idx]
    mask = quant_sim.outlier_mask(n_in, fp_idx, DEV)
    got = quant_sim.act_fake_quant(x.to(DEV), mask, bits).cpu()
    assert got.dtype == dtype and torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("bits", [4, 8])
def test_act_quant_wrapper_forward(bits):
    """ActQuantWrapper with the reference's interface: configure, fp_features_configure (outliers = the columns
    with the largest scales), forward on 2-D and (1, S, in) inputs; 16 bits and zero outliers are pass-through
    / quantize-everything corner cases (experiments/quant_sim.py:227-236)."""
    from quik_amd.quant_sim import ActQuantWrapper
    M, n_in, N, F = 64, 1024, 96, 64
    x, scales, fp_idx = _inputs(M, n_in, F, 11 + bits, torch.float16)
    g = torch.Generator().manual_seed(3)
    lin = torch.nn.Linear(n_in, N, bias=True)
    lin.weight.data = (0.02 * torch.randn(N, n_in, generator=g))
    lin.bias.data = torch.randn(N, generator=g)
    lin = lin.half().requires_grad_(False)
    wrap = ActQuantWrapper(lin.to(DEV))
    assert torch.equal(wrap(x.to(DEV)).cpu(), lin.to(DEV)(x.to(DEV)).cpu())            # 16 bits: untouched
    wrap.quantizer.configure(bits)
    wrap.fp_features_configure(scales, F)
    assert torch.equal(torch.sort(wrap.fp_feature_idx)[0], torch.sort(fp_idx)[0])
    keep = torch.ones(n_in, dtype=torch.bool)
    keep[fp_idx] = False
    int_idx = torch.arange(n_in)[keep]
    want = sim_path.sim_mixed_linear(x, lin.weight.data.cpu(), int_idx, fp_idx, bits, lin.bias.data.cpu()).double()
    for xin in (x.to(DEV), x.to(DEV).reshape(1, M, n_in)):
        got = wrap(xin).reshape(M, N).cpu().double()
        rms = float(torch.sqrt((want ** 2).mean()))
        assert float((got - want).abs().max()) <= 1e-2 * rms
    wrap.fp_features_configure(scales, 0)                                                # quantize every column
    want0 = sim_path.sim_mixed_linear(x, lin.weight.data.cpu(), torch.arange(n_in), torch.tensor([], dtype=torch.long),
                                      bits, lin.bias.data.cpu()).double()
    got0 = wrap(x.to(DEV)).cpu().double()
    assert float((got0 - want0).abs().max()) <= 1e-2 * float(torch.sqrt((want0 ** 2).mean()))
    assert "FP features: 0" in wrap.extra_repr()


def test_kernel_path_and_simulated_path_on_the_gpu_agree_to_quantisation_noise():
    """MixedQLinear (kernel path) against ActQuantWrapper around the float Linear with the fake-quant weight
    (simulated path), both on the GPU, at a Llama-7B-sized layer: their errors against the float64 layer on the
    exact activation are of the same size (different zero-point conventions, same quantisation step)."""
    from quik_amd.qlinear import MixedQLinear
    from quik_amd.quant_sim import ActQuantWrapper
    M, n_in, N, F, bits = 512, 4096, 1024, 256, 4
    g = torch.Generator().manual_seed(9)
    x = torch.randn(M, n_in, generator=g)
    fp_idx = torch.randperm(n_in, generator=g)[:F]
    x[:, fp_idx] *= 50
    x = x.half()
    keep = torch.ones(n_in, dtype=torch.bool)
    keep[fp_idx] = False
    int_idx = torch.arange(n_in)[keep]
    s_w = (torch.rand(N, 1, generator=g) * 0.009 + 0.001).half()
    W = torch.empty(N, n_in, dtype=torch.float16)
    W[:, int_idx] = (torch.randint(-8, 8, (N, n_in - F), generator=g).float() * s_w.float()).half()
    W[:, fp_idx] = (0.02 * torch.randn(N, F, generator=g)).half()
    lin = torch.nn.Linear(n_in, N, bias=False).half().requires_grad_(False)
    lin.weight.data = W.clone()
    kern = MixedQLinear.from_float(lin, W, s_w, None, fp_idx, bits=bits).to(DEV)
    sim = ActQuantWrapper(lin.to(DEV))
    sim.quantizer.configure(bits)
    scales = torch.zeros(n_in)
    scales[fp_idx] = 1.0
    sim.fp_features_configure(scales, F)
    out_k = kern(x.to(DEV))[0].double().cpu()
    out_s = sim(x.to(DEV)).double().cpu()
    ref = x.double() @ W.double().T
    ek, es = float((out_k - ref).pow(2).mean().sqrt()), float((out_s - ref).pow(2).mean().sqrt())
    rms = float(ref.pow(2).mean().sqrt())
    assert ek < 0.25 * rms and es < 0.25 * rms       # 4-bit activations: both far from exact, by the same amount
    assert 0.5 < ek / es < 2.0
    assert float((out_k - out_s).pow(2).mean().sqrt()) < 2.0 * max(ek, es)
