"""MixedQLinear forward for one or two token rows: ONE launch (the weight-streaming matrix-vector kernel quantises
the rows itself) against the two-launch form (quik_asym_quantize / quik_sym_quantize_mapped + quik_mixed_linear_fwd)
and against the oracle.

The one-launch form uses the quantize kernels' own arithmetic on the same inputs, so codes and scales, and with them
the outputs, must be bit-identical to the two-launch form; that form is switched on through
quik_layer_set_one_launch(0) (reference op sequence: experiments/qlinear.py:114-145).  That the first call really
was one launch is read off the workspace the caller hands over: the one-launch form never writes it.
Against the oracle the usual tolerance of the fused forward applies (1e-2 x output RMS; the outlier sum's order is
not defined by the reference).
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import quik_oracle as qo

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _lib():
    from quik_amd import _lib as L
    lib = L.load()
    assert torch.cuda.is_available()
    yield
    lib.quik_layer_set_one_launch(1)


def _layer(rng, N, n_in, F, bits, dtype, runs, symm=False):
    from quik_amd.qlinear import MixedQLinear
    if runs and F:
        starts = rng.permutation(n_in // 32)[:F // 4] * 32 + rng.integers(0, 20, F // 4)
        fi = (starts[:, None] + np.arange(4)[None, :]).ravel().astype(np.int64)
        fi[:4] = [0, 1, n_in - 1, n_in - 2] if 0 not in fi and n_in - 1 not in fi else fi[:4]
        fi = np.unique(fi)
        fi = np.concatenate([fi, np.setdiff1d(np.arange(40, 40 + 4 * F), fi)[:F - len(fi)]])
    else:
        fi = rng.permutation(n_in)[:F].astype(np.int64)
    mask = np.ones(n_in, bool)
    mask[fi] = False
    ii = np.arange(n_in)[mask]
    lo, hi = (-8, 8) if bits == 4 else (-128, 128)
    codes = rng.integers(lo, hi, (N, n_in - F))
    s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    W = np.zeros((N, n_in), np.float16)
    W[:, ii] = (codes * s_w.astype(np.float32)).astype(np.float16)
    W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
    bias = (0.1 * rng.standard_normal(N)).astype(np.float16)
    lin = torch.nn.Linear(n_in, N, bias=True)
    lin.bias.data = torch.from_numpy(bias.astype(np.float32))
    mod = MixedQLinear.from_float(lin, torch.from_numpy(W), torch.from_numpy(s_w), None, torch.from_numpy(fi),
                                  symm=symm, bits=bits).to(DEV)
    if dtype == torch.bfloat16:
        mod = mod.to(torch.bfloat16)
    return mod, W, s_w, fi, ii, bias


def _call(mod, x, sentinel):
    """quik_layer_forward through the C ABI with a workspace filled with `sentinel`; returns (out, workspace)."""
    from quik_amd import _lib as L
    lib = L.load()
    rows = x.shape[0]
    desc, _ = mod._descriptor(False)
    nbytes = lib.quik_layer_workspace_bytes(ctypes.byref(desc), rows)
    ws = torch.full((nbytes,), sentinel, dtype=torch.uint8, device=DEV)
    out = torch.empty((rows, mod.out_features), dtype=x.dtype, device=DEV)
    L.check(lib.quik_layer_forward(ctypes.byref(desc), x.data_ptr(), rows, ws.data_ptr(), nbytes, None, 0,
                                   out.data_ptr(), None, L.stream()), "forward")
    torch.cuda.synchronize()
    return out, ws


# rows, N, in, F, bits, dtype, outlier columns in runs
CASES = [
    (1, 13824, 5120, 256, 4, torch.float16, False),      # Llama-2-13B gate_proj, one token
    (2, 13824, 5120, 256, 4, torch.float16, True),
    (1, 5120, 13824, 256, 8, torch.float16, False),      # 13B down_proj W8A8
    (2, 4096, 11008, 256, 8, torch.float16, True),
    (1, 1000, 1024 + 64, 64, 4, torch.float16, True),    # N not a multiple of the waves per workgroup
    (2, 520, 2048, 0, 4, torch.float16, False),          # no outlier columns
    (1, 320, 544, 32, 8, torch.float16, False),
    (1, 2048, 4096 + 128, 128, 4, torch.bfloat16, True),
    (2, 1024, 2048 + 64, 64, 8, torch.bfloat16, False),
    (1, 8192, 28672, 256, 8, torch.float16, False),      # 70B down_proj: the longest rows
    (2, 1001, 1024 + 64, 64, 4, torch.float16, False),   # ragged N: odd row stride of the output
    (1, 5, 128 + 32, 32, 4, torch.float16, False),       # fewer columns than waves, the shortest K
    (2, 77, 256 + 32, 32, 8, torch.bfloat16, True),
]


@pytest.mark.parametrize("rows,N,n_in,F,bits,dtype,runs", CASES)
def test_one_launch_equals_two_launches_and_the_oracle(rows, N, n_in, F, bits, dtype, runs):
    from quik_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(rows * 7 + N + n_in + F + bits)
    mod, W, s_w, fi, ii, bias = _layer(rng, N, n_in, F, bits, dtype, runs)
    x = rng.standard_normal((rows, n_in)).astype(np.float32)
    x[:, fi] *= 50
    xt = torch.from_numpy(x).to(DEV, dtype)
    lib.quik_layer_set_one_launch(1)
    out1, ws1 = _call(mod, xt, 0x5A)
    assert bool((ws1 == 0x5A).all()), "the one-launch form does not touch the workspace"
    lib.quik_layer_set_one_launch(0)
    out2, ws2 = _call(mod, xt, 0x5A)
    lib.quik_layer_set_one_launch(1)
    assert not bool((ws2 == 0x5A).all())
    assert torch.equal(out1.view(torch.int16), out2.view(torch.int16))
    # oracle (fp16 arithmetic of the reference's kernels; bf16 inputs are compared through their fp32 values)
    if dtype == torch.float16:
        omod = qo.from_float(W, s_w, fi, bits)
        want, _ = qo.mixed_qlinear_forward(xt.cpu().numpy(), omod, bits, bias=bias)
        got = out1.float().cpu().numpy()
        rms = float(np.sqrt((want.astype(np.float64) ** 2).mean()))
        assert np.abs(got - want.astype(np.float64)).max() <= 1e-2 * rms


def test_edge_rows_in_one_launch():
    """Constant, all-zero, overflowing-range and NaN rows: the quantize inside the kernel takes the same decisions
    (scale floor, division path, NaN codes) as the quantize kernel."""
    from quik_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(11)
    mod, W, s_w, fi, ii, bias = _layer(rng, 640, 1024 + 64, 64, 4, torch.float16, True)
    rows = []
    r = rng.standard_normal(1088).astype(np.float16)
    for kind in range(6):
        x = r.copy()
        if kind == 0:
            x[:] = 1.5
        elif kind == 1:
            x[:] = 0
        elif kind == 2:
            x[ii[3]], x[ii[4]] = 65504.0, -65504.0
        elif kind == 3:
            x[ii[6]] = np.nan
        elif kind == 4:
            x *= np.float16(1e-7)
        else:
            x[ii[5]] = np.inf
        rows.append(x)
    for a, b in ((0, 1), (2, 3), (4, 5)):
        xt = torch.from_numpy(np.stack([rows[a], rows[b]])).to(DEV)
        lib.quik_layer_set_one_launch(1)
        out1, _ = _call(mod, xt, 0)
        lib.quik_layer_set_one_launch(0)
        out2, _ = _call(mod, xt, 0)
        lib.quik_layer_set_one_launch(1)
        assert torch.equal(out1.view(torch.int16), out2.view(torch.int16)), (a, b)


@pytest.mark.parametrize("rows,N,n_in,F", [(1, 13824, 5120, 256), (2, 1000, 1024 + 64, 64), (1, 520, 2048, 0),
                                           (2, 77, 256 + 32, 32)])
def test_symmetric_layer_in_one_launch(rows, N, n_in, F):
    """Symmetric activations (fp16, 4 bits: scale = max |x| / 4 as the reference's expression evaluates,
    experiments/qlinear.py:97-103) take the same single launch: bit-identical to quik_sym_quantize_mapped + the fused
    GEMM, within the fused forward's tolerance of the oracle's fp16-chain result; rows that hold a NaN, an infinity
    or nothing but zeros included."""
    from quik_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(rows + N + n_in + F)
    mod, W, s_w, fi, ii, bias = _layer(rng, N, n_in, F, 4, torch.float16, F > 0, symm=True)
    x = rng.standard_normal((rows, n_in)).astype(np.float32)
    x[:, fi] *= 50
    variants = [x.astype(np.float16)]
    for kind in range(3):
        y = x.astype(np.float16).copy()
        if kind == 0:
            y[0, ii[3]] = np.nan
        elif kind == 1:
            y[rows - 1, ii[5]] = np.inf
        else:
            y[0, :] = 0
        variants.append(y)
    for k, xv in enumerate(variants):
        xt = torch.from_numpy(xv).to(DEV)
        lib.quik_layer_set_one_launch(1)
        out1, ws1 = _call(mod, xt, 0x5A)
        assert bool((ws1 == 0x5A).all()), "the one-launch form does not touch the workspace"
        lib.quik_layer_set_one_launch(0)
        out2, ws2 = _call(mod, xt, 0x5A)
        lib.quik_layer_set_one_launch(1)
        assert not bool((ws2 == 0x5A).all())
        assert torch.equal(out1.view(torch.int16), out2.view(torch.int16)), k
        if k == 0:
            omod = qo.from_float(W, s_w, fi, 4, symm=True)
            want, _ = qo.mixed_qlinear_forward(xv, omod, 4, bias=bias, symm=True)
            w64 = want.astype(np.float64)
            rms = float(np.sqrt((w64 ** 2).mean()))
            assert np.abs(out1.float().cpu().numpy() - w64).max() <= 1e-2 * rms


def test_three_rows_keep_two_launches():
    from quik_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(12)
    mod, W, s_w, fi, ii, bias = _layer(rng, 512, 1024 + 64, 64, 4, torch.float16, False)
    xt = torch.from_numpy(rng.standard_normal((3, 1088)).astype(np.float16)).to(DEV)
    _, ws = _call(mod, xt, 0x5A)
    assert not bool((ws == 0x5A).all())


def test_decode_sizes_random_shapes_against_the_oracle():
    """Seeded sweep over calls of 1 .. 32 rows: ragged N and K, with and without outlier columns and bias, both
    widths.  Whatever kernel the library picks (matrix-vector kernel in one or two launches, MFMA weight-streaming
    kernel with the token rows streamed or resident in LDS), the module's output stays within the fused forward's
    tolerance of the oracle, and equals the two-launch form bit for bit where the one-launch form applies."""
    from quik_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(777)
    for it in range(28):
        bits = int(rng.choice([4, 8]))
        rows = int(rng.choice([1, 1, 2, 2, 3, 4, 5, 8, 13, 16, 17, 31, 32]))
        F = int(rng.choice([0, 8, 16, 32, 64, 72, 256]))
        K = int(rng.choice([32, 64, 96, 128, 256, 384, 640, 992, 1024, 2048, 4864]))    # (K % 32 == 0 and F % 8 == 0: the GEMM's row alignment)
        N = int(rng.choice([1, 7, 8, 33, 100, 256, 513, 1000, 2048, 8200, 9000]))
        n_in = K + F
        with_bias = bool(rng.integers(0, 2))
        case = (it, rows, N, n_in, F, bits, with_bias)
        mod, W, s_w, fi, ii, bias = _layer(rng, N, n_in, F, bits, torch.float16, bool(rng.integers(0, 2)) and F >= 8 and n_in >= 8 * F + 64)
        if not with_bias:
            mod.bias = None
            bias = None
        x = rng.standard_normal((rows, n_in)).astype(np.float32)
        x[:, fi] *= 50
        xt = torch.from_numpy(x).to(DEV, torch.float16)
        lib.quik_layer_set_one_launch(1)
        out1 = mod(xt)[0]
        lib.quik_layer_set_one_launch(0)
        out2 = mod(xt)[0]
        lib.quik_layer_set_one_launch(1)
        if rows <= 2:
            assert torch.equal(out1.view(torch.int16), out2.view(torch.int16)), case
        omod = qo.from_float(W, s_w, fi, bits)
        want, _ = qo.mixed_qlinear_forward(xt.cpu().numpy(), omod, bits, bias=bias)
        w64 = want.astype(np.float64)
        rms = float(np.sqrt((w64 ** 2).mean())) + 1e-30
        for got in (out1, out2):
            err = np.abs(got.float().cpu().numpy() - w64).max()
            assert err <= 1e-2 * rms, (case, err, rms)
