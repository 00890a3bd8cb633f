"""The route MixedQLinear.forward takes by default, at the full sizes of the benchmark configurations.

A module built with `from_float` is called as `mod(x)`, so the dispatch of the module decides the kernels:
tile-ordered operands on the 6-bit matrix-core GEMM (W4A4) or the tile-ordered int8 GEMM (W8A8) above 32 token
rows, their K split where the tiles are few, the wide + narrow tile plan in one launch.  Checks per shape:
  * output bits equal those of the same module on the row-major int8-MFMA kernels (`six_bit_path = False`),
    which tests/test_gpu_parity.py::test_full_size_properties holds against the oracle at the same shapes
    through exact row / column checksums of the integer GEMM;
  * the oracle's MixedQLinear forward (experiments/qlinear.py:80-148 restated on the CPU) on three spot tiles
    and on the first and last rows, within 1e-2 x output RMS (max abs), the stated tolerance, and within a
    few fp16 ulps of the largest term in practice.
"""
import numpy as np
import pytest
import torch

from oracle import quik_oracle as qo

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _lib():
    from quik_amd import _lib as L
    L.load()
    assert torch.cuda.is_available()
    yield


def _bits(t):
    return t.detach().contiguous().view(torch.int16)


def make_full_size_layer(M, n_in, N, F, bits, symm, kind, seed, dtype=torch.float16):
    """Inputs of the measurement protocol, made on the device: x ~ N(0, 1) (or Student-t, 3 degrees of freedom) with
    the outlier columns scaled up, W = codes x per-row scale on the integer columns, N(0, 0.02) on the outlier
    columns.  Returns the module (through from_float), x and the float weight matrix / scales / outlier indices."""
    from quik_amd.qlinear import MixedQLinear
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn(M, n_in, generator=g, device=DEV)
    if kind == "student":
        chi2 = torch.zeros(M, n_in, device=DEV)
        for _ in range(3):
            chi2 += torch.randn(M, n_in, generator=g, device=DEV) ** 2
        x = x / torch.sqrt(chi2 / 3)
    fi = torch.randperm(n_in, generator=g, device=DEV)[:F]
    x[:, fi] *= 20 if kind == "student" else 50
    x = x.clamp(-6e4, 6e4).to(dtype)
    keep = torch.ones(n_in, dtype=torch.bool, device=DEV)
    keep[fi] = False
    ii = torch.arange(n_in, device=DEV)[keep]
    K = n_in - F
    lo, hi = (-8, 8) if bits == 4 else (-127, 128)
    s_w = (torch.rand(N, 1, generator=g, device=DEV) * 0.009 + 0.001).to(dtype)
    W = torch.empty(N, n_in, dtype=dtype, device=DEV)
    for s in range(0, N, 4096):
        e = min(N, s + 4096)
        codes = torch.randint(lo, hi, (e - s, K), generator=g, device=DEV).float()
        W[s:e, ii] = (codes * s_w[s:e].float()).to(dtype)      # the codes survive the rounding of the product
        W[s:e, fi] = (0.02 * torch.randn(e - s, F, generator=g, device=DEV)).to(dtype)
    lin = torch.nn.Linear(n_in, N, bias=False, dtype=dtype, device="meta")
    mod = MixedQLinear.from_float(lin, W, s_w.cpu(), None, fi.cpu(), symm=symm, bits=bits).to(DEV)
    return mod, x, W, s_w, fi


def check_against_oracle(out, x, W, s_w, fi, bits, symm, tiles):
    """out [M, N] (device) against the oracle's forward on row / column index sets `tiles`."""
    fin = fi.cpu().numpy()
    bf16 = out.dtype == torch.bfloat16
    dt = qo.BF16 if bf16 else qo.F16
    host = (lambda t: t.float().cpu().numpy()) if bf16 else (lambda t: t.cpu().numpy())
    for rows, cols in tiles:
        omod = qo.from_float(host(W[cols]), host(s_w[cols]), fin, bits, symm=symm, dtype=dt)
        want, inter = qo.mixed_qlinear_forward(host(x[rows]), omod, bits, None, symm=symm, dtype=dt)
        got = out[rows][:, cols].float().cpu().numpy().astype(np.float64)
        w64 = want.astype(np.float64)
        assert np.isfinite(w64).all()
        if bf16:
            # one bf16 ulp of the output exceeds 1e-2 x RMS for the larger outputs, and the oracle (like the
            # reference) rounds the outlier product to bf16 before the final sum: one ulp of each
            y64 = np.abs(np.asarray(inter["fp_result"], np.float64))
            assert (np.abs(got - w64) <= (np.abs(w64) + y64) * 2.0 ** -7).all(), (rows[0], cols[0])
            continue
        err = np.abs(got - w64).max()
        assert err <= 1e-2 * np.sqrt((w64 ** 2).mean()), (err, rows[0], cols[0])
        assert err <= 4 * np.abs(w64).max() * 2.0 ** -10, (err, rows[0], cols[0])


def spot_tiles(M, N):
    th, tw = min(48, M), min(64, N)
    r = lambda a: np.arange(a, a + th)
    c = lambda a: np.arange(a, a + tw)
    mid_c = min(N - tw, (N // 2 // 256) * 256 + 200)     # straddles a 256-column tile boundary
    edge = np.r_[0:min(4, M), max(M - 4, 0):M]          # first and last rows ...
    return [(r(0), c(0)), (r((M - th) // 2), c(mid_c)), (r(M - th), c(N - tw)),
            (np.unique(edge), np.r_[0:8, N // 2:N // 2 + 8, N - 8:N])]   # ... over the first, middle and last columns


DEFAULT_ROUTE = [
    # tokens, in, out, outliers, bits, symmetric, activations
    (2048, 8192, 28672, 256, 4, False, "x50"),      # Llama-2-70B gate/up: the benchmark's shape and its tile plan
    (2048, 8192, 28672, 256, 4, True, "x50"),       # ... symmetric activations
    (8192, 8192, 28672, 256, 4, False, "x50"),      # ... 16 x 512 tokens, the decoder block's prefill
    (2048, 28672, 8192, 256, 8, False, "x50"),      # Llama-2-70B down_proj, W8A8
    (2048, 8192, 8192, 256, 4, False, "x50"),       # Llama-2-70B q/o
    (2048, 8192, 8192, 256, 4, True, "x50"),        # ... symmetric
    (2048, 8192, 1024, 256, 4, False, "x50"),       # Llama-2-70B k/v (GQA)
    (2048, 4096, 11008, 256, 4, False, "x50"),      # Llama-2-7B gate/up
    (2048, 4096, 4096, 256, 4, False, "x50"),       # Llama-2-7B q/k/v/o
    (2048, 11008, 4096, 256, 8, False, "x50"),      # Llama-2-7B down_proj, W8A8
    (2048, 5120, 13824, 256, 4, False, "student"),  # Llama-2-13B gate/up
    (2048, 13824, 5120, 256, 8, False, "student"),  # Llama-2-13B down_proj, W8A8
    (128, 5120, 13824, 256, 4, False, "student"),   # Llama-2-13B gate/up, 128 tokens
    (128, 13824, 5120, 256, 8, False, "student"),   # Llama-2-13B down_proj, 128 tokens: K split
    (128, 5120, 5120, 256, 4, False, "student"),    # Llama-2-13B q/k/v/o, 128 tokens
    (64, 28672, 8192, 256, 8, False, "x50"),        # Llama-2-70B down_proj, 64 single-token rows: K split
    (2049, 8192, 28672, 256, 4, False, "x50"),      # Llama-2-70B gate/up, one row more than the tiles hold: ragged last row block
    (2048, 8192, 28672, 256, 4, False, "x50", torch.bfloat16),     # Llama-2-70B gate/up, bf16 activations and weights
    (2048, 13824, 5120, 256, 8, False, "student", torch.bfloat16),  # Llama-2-13B down_proj, W8A8, bf16
    (512, 4096, 4096, 128, 4, False, "x50"),        # the single-layer configuration of the CPU simulated path: 512 tokens, 128 outliers
    (512, 4096, 4096, 128, 4, True, "x50"),         # ... symmetric activations
]


@pytest.mark.parametrize("case", DEFAULT_ROUTE)
def test_default_route_at_benchmark_shapes(case):
    M, n_in, N, F, bits, symm, kind = case[:7]
    dtype = case[7] if len(case) > 7 else torch.float16
    mod, x, W, s_w, fi = make_full_size_layer(M, n_in, N, F, bits, symm, kind, seed=sum(case[:5]) + symm, dtype=dtype)
    assert mod._six_bit_ok(M)                      # the shape is one the tile-ordered path takes
    out = mod(x)
    assert mod._w6 is not None                     # ... and it did run
    assert out.shape == (1, M, N) and out.dtype == dtype
    out = out[0]
    assert torch.isfinite(out).all()
    mod.six_bit_path = False
    mod._w6 = None
    ref = mod(x)[0]                                # row-major operands, int8 MFMA
    assert mod._w6 is None
    assert torch.equal(_bits(out), _bits(ref))
    del ref
    check_against_oracle(out, x, W, s_w, fi, bits, symm, spot_tiles(M, N))


def test_default_route_random_shapes_against_the_oracle():
    """Seeded sweep over module calls of any size: row counts on both sides of every switch of kernels, ragged N,
    K and F at the granularity the GEMM's row alignment allows (shapes the tile-ordered paths refuse included),
    W4A4 / W8A8 / symmetric, fp16 against the oracle's forward on the whole output, bf16 against the row-major
    route of the same module bit for bit.  Elementwise bound: 1e-2 x output RMS, or two fp16 ulps of the element
    where that is larger (heavy-tailed outputs)."""
    from quik_amd.qlinear import MixedQLinear
    rng = np.random.default_rng(4242)
    done = 0
    while done < 40:
        bits = int(rng.choice([4, 8]))
        symm = bits == 4 and rng.random() < 0.2
        bf16 = (not symm) and rng.random() < 0.25
        M = int(rng.choice([1, 2, 3, 16, 32, 33, 48, 64, 65, 100, 128, 129, 256, 257, 300, 511, 700, 1100]))
        K = (32 if bits == 4 else 16) * int(rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 31, 32, 40, 64, 77, 128]))
        F = 8 * int(rng.choice([0, 0, 1, 2, 4, 8, 9, 16, 32, 33]))
        N = int(rng.choice([5, 8, 31, 64, 100, 130, 256, 513, 1000, 2048, 4100]))
        if M * N < 64 or M * N * K > 2e9:
            continue
        done += 1
        n_in = K + F
        fi = rng.permutation(n_in)[:F].astype(np.int64)
        keep = np.ones(n_in, bool)
        keep[fi] = False
        ii = np.arange(n_in)[keep]
        lo, hi = (-8, 8) if bits == 4 else (-127, 128)
        s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
        W = np.zeros((N, n_in), np.float16)
        W[:, ii] = (rng.integers(lo, hi, (N, K)) * s_w.astype(np.float32)).astype(np.float16)
        W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
        bias = (0.1 * rng.standard_normal(N)).astype(np.float16) if rng.random() < 0.5 else None
        lin = torch.nn.Linear(n_in, N, bias=bias is not None)
        if bias is not None:
            lin.bias.data = torch.from_numpy(bias.astype(np.float32))
        x = rng.standard_normal((M, n_in)).astype(np.float32)
        if rng.random() < 0.5:
            x[:, fi] *= 50
        elif F:
            x[:, fi] = np.clip(20 * rng.standard_t(3, (M, F)), -6e4, 6e4)
        x = x.astype(np.float16)
        case = (done, M, N, K, F, bits, bool(symm), bool(bf16), bias is not None)
        mod = MixedQLinear.from_float(lin, torch.from_numpy(W), torch.from_numpy(s_w), None,
                                      torch.from_numpy(fi) if F else None, symm=bool(symm), bits=bits).to(DEV)
        if bf16:
            mod = mod.to(torch.bfloat16)
            xt = torch.from_numpy(x).to(DEV).to(torch.bfloat16)
            out = mod(xt)[0]
            mod.six_bit_path = False
            assert torch.equal(_bits(out), _bits(mod(xt)[0])), case
            continue
        omod = qo.from_float(W, s_w, fi, bits, symm=bool(symm))
        want, _ = qo.mixed_qlinear_forward(x, omod, bits, bias, symm=bool(symm))
        w64 = want.astype(np.float64)
        fin = np.isfinite(w64)
        rms = np.sqrt((w64[fin] ** 2).mean()) + 1e-30
        xt = torch.from_numpy(x).to(DEV)
        got = mod(xt)[0]
        d = np.abs(got.float().cpu().numpy().astype(np.float64) - w64)[fin]
        assert not (d > np.maximum(1e-2 * rms, 2.0 ** -9 * np.abs(w64[fin]))).any(), (case, d.max(), rms)
        if M > 32 and not symm:
            mod.six_bit_path = False
            assert torch.equal(_bits(got), _bits(mod(xt)[0])), case


def test_default_route_three_dimensional_prefill_input():
    """The decoder block's prefill hands (16, 512, 8192); the module flattens it and returns (16, 512, N)."""
    M, n_in, N, F, bits = 8192, 8192, 1024, 256, 4
    mod, x, W, s_w, fi = make_full_size_layer(M, n_in, N, F, bits, False, "x50", seed=5)
    out = mod(x.reshape(16, 512, n_in))
    assert out.shape == (16, 512, N)
    flat = mod(x)[0]
    assert torch.equal(_bits(out.reshape(M, N)), _bits(flat))
    check_against_oracle(flat, x, W, s_w, fi, bits, False, spot_tiles(M, N))


def _oracle_module_slice(mod, cols):
    """The oracle's view of output columns `cols` of a MixedQLinear, from the module's own packed buffers."""
    c = torch.as_tensor(cols, device=mod.int_weight.device)
    return {
        "weights_scales": mod.weights_scales[c].cpu().numpy(),
        "int_weight": mod.int_weight[c].cpu().numpy(),
        "int_indices": mod.int_indices.cpu().numpy(),
        "fp_indices": mod.fp_indices.cpu().numpy(),
        "fp_weight": mod.fp_weight[c].cpu().numpy(),
        "reduced_w": mod.reduced_w[:, c].cpu().numpy(),
    }


@pytest.mark.parametrize("B,S,past", [(16, 512, 0), (64, 1, 512)])
def test_decoder_block_at_llama2_70b_dims(B, S, past):
    """The full decoder block of the benchmark (bench.DecoderBlock: hidden 8192, 64 heads, 8 KV heads, MLP 28672;
    seven MixedQLinear, q/k/v and gate/up sharing their quantized inputs, W8A8 down_proj; norms / attention /
    SiLU in PyTorch), prefill of 16 x 512 tokens and a decode step of 64 single tokens over a 512-token cache.
    Every linear's output is checked on spot tiles against the oracle's forward of the very tensor that linear
    consumed (experiments/qlinear.py:80-148 restated on the CPU), and the block with q/k/v and gate/up as fused
    groups gives the same bits."""
    import bench
    blk = bench.DecoderBlock(torch.device(DEV), seed=B)
    x, cache = blk.inputs(B, S, past)
    seen = {}

    def hook(name, mod, inp, out):
        M = B * S
        assert out.shape == (B, S, mod.out_features) and out.dtype == torch.float16
        x2, o2 = inp.reshape(M, -1), out.reshape(M, -1)
        bits = mod.bits
        for rows, cols in spot_tiles(M, mod.out_features)[:3]:
            omod = _oracle_module_slice(mod, cols)
            want, _ = qo.mixed_qlinear_forward(x2[rows].cpu().numpy(), omod, bits)
            got = o2[rows][:, cols].float().cpu().numpy().astype(np.float64)
            w64 = want.astype(np.float64)
            err = np.abs(got - w64).max()
            assert err <= 1e-2 * np.sqrt((w64 ** 2).mean()), (name, err)
        seen[name] = True

    out = blk.forward(x, False, cache, hook)
    assert sorted(seen) == ["down", "gate", "k", "o", "q", "up", "v"]
    assert torch.isfinite(out).all()
    out_f = blk.forward(x, True, cache)
    assert torch.equal(_bits(out), _bits(out_f))
