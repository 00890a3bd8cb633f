"""quik_layer_forward: one library call per MixedQLinear forward (quantize launch + fused GEMM launch).

The entry point replaces the op sequence of MixedQLinear.forward (experiments/qlinear.py:80-148 of the reference)
for callers that want one crossing into the library per layer.  Checks:
  * through the C ABI, with a descriptor and a workspace built by the test, the output bits equal those of the
    stand-alone entry points called one after the other (which tests/test_gpu_parity.py holds against the oracle);
  * `MixedQLinear.forward` takes this path by default and gives the bits of the module's op-by-op route;
  * the oracle's forward on the same inputs, within 1e-2 x output RMS;
  * the profiling event is recorded between the two launches, on the launch stream.
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
    L.load()
    assert torch.cuda.is_available()
    yield


def _bits(t):
    return t.detach().contiguous().view(torch.int16)


def _layer(rng, N, n_in, F, bits):
    fi = np.sort(rng.permutation(n_in)[:F]).astype(np.int64)
    keep = np.ones(n_in, bool)
    keep[fi] = False
    ii = np.arange(n_in)[keep]
    lo, hi = (-8, 8) if bits == 4 else (-127, 128)
    s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    W = np.zeros((N, n_in), np.float16)
    W[:, ii] = (rng.integers(lo, hi, (N, n_in - F)) * s_w.astype(np.float32)).astype(np.float16)
    W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
    return W, s_w, fi


def _module(W, s_w, fi, bits, bias, symm, dtype=torch.float16):
    from quik_amd.qlinear import MixedQLinear
    N, n_in = W.shape
    lin = torch.nn.Linear(n_in, N, bias=bias is not None)
    if bias is not None:
        lin.bias.data = torch.from_numpy(bias)
    mod = MixedQLinear.from_float(lin, torch.from_numpy(W).to(dtype), torch.from_numpy(s_w).to(dtype), None,
                                  torch.from_numpy(fi) if fi.size else None, symm=symm, bits=bits)
    return mod.to(DEV)


CASES = [
    # rows, out, in, outliers, bits, symmetric, bias
    (1, 384, 1024, 64, 4, False, False),      # decode kernel
    (20, 200, 1056, 32, 4, False, True),
    (32, 256, 2048 + 256, 256, 8, False, False),
    (33, 300, 1024 + 64, 64, 4, False, True),  # first row count on the tile-ordered path
    (200, 520, 4096 + 128, 128, 4, False, False),
    (260, 300, 1280 + 256, 256, 8, False, True),
    (48, 256, 1024 + 32, 32, 4, True, False),  # symmetric activations, tile-ordered
    (8, 256, 1024 + 32, 32, 4, True, True),    # symmetric activations, decode kernel
    (100, 128, 1000, 40, 4, False, True),      # K % 128 != 0: row-major operands at any row count
    (64, 128, 512, 0, 4, False, True),         # no outliers
]


@pytest.mark.parametrize("case", CASES)
def test_module_forward_is_one_call_and_matches_the_op_sequence(case, monkeypatch):
    M, N, n_in, F, bits, symm, with_bias = case
    rng = np.random.default_rng(sum(case[:5]) + symm)
    W, s_w, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16) if with_bias else None
    x = rng.standard_normal((M, n_in)).astype(np.float32)
    x[:, fi] *= 50
    x = x.astype(np.float16)
    mod = _module(W, s_w, fi, bits, bias, symm)
    xt = torch.from_numpy(x).to(DEV)

    from quik_amd import _lib as L
    calls = []
    real = L.load().quik_layer_forward
    monkeypatch.setattr(L.load(), "quik_layer_forward", lambda *a: calls.append(a[2]) or real(*a))
    out = mod(xt)
    assert calls == [M]                          # the module went through the one-call entry point
    assert out.shape == (1, M, N) and out.dtype == torch.float16

    monkeypatch.setattr(type(mod), "_forward_one_call", lambda self, x2: None)
    ref = mod(xt)                                # the module's op-by-op route: two library calls
    assert calls == [M]
    assert torch.equal(_bits(out), _bits(ref))

    omod = qo.from_float(W, s_w, fi, bits, symm=symm)
    want, _ = qo.mixed_qlinear_forward(x, omod, bits, bias, symm=symm)
    w64 = want.astype(np.float64)
    err = np.abs(out[0].float().cpu().numpy().astype(np.float64) - w64).max()
    assert err <= 1e-2 * np.sqrt((w64 ** 2).mean())
    assert err <= 4 * np.abs(w64).max() * 2.0 ** -10


def test_bfloat16_module_takes_the_one_call_path():
    M, N, n_in, F, bits = 70, 256, 2048 + 64, 64, 4
    rng = np.random.default_rng(3)
    W, s_w, fi = _layer(rng, N, n_in, F, bits)
    mod = _module(W, s_w, fi, bits, None, False, dtype=torch.bfloat16)
    x = torch.from_numpy(rng.standard_normal((M, n_in)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    out = mod(x)
    assert out.dtype == torch.bfloat16
    type(mod)._forward_one_call, keep = (lambda self, x2: None), type(mod)._forward_one_call
    try:
        ref = mod(x)
    finally:
        type(mod)._forward_one_call = keep
    assert torch.equal(_bits(out), _bits(ref))


@pytest.mark.parametrize("M,bits", [(16, 4), (96, 4), (96, 8)])
def test_layer_forward_through_the_c_abi(M, bits):
    """Descriptor, workspace and call made by hand, as a C caller would; against the stand-alone entry points."""
    from quik_amd import _lib as L, asymmetric, matmul
    lib = L.load()
    N, n_in, F = 320, 2048 + 64, 64
    K = n_in - F
    rng = np.random.default_rng(M + bits)
    W, s_w, fi = _layer(rng, N, n_in, F, bits)
    mod = _module(W, s_w, fi, bits, None, False)
    x = torch.from_numpy(rng.standard_normal((M, n_in)).astype(np.float16)).to(DEV)
    colmap = asymmetric.build_colmap(mod.int_indices, mod.fp_indices, n_in)
    assert asymmetric.colmap_streams(colmap, K, F)
    tiled = M >= 33
    w_t = None
    if tiled:
        w_t = matmul.pack_weight_fp6(mod.int_weight, mod.fp_weight, colmap) if bits == 4 else \
            matmul.pack_weight_tile8(mod.int_weight, mod.fp_weight)

    d = L.QuikLayer()
    d.struct_bytes = ctypes.sizeof(L.QuikLayer)
    d.bits, d.dtype, d.symmetric = bits, L.QUIK_F16, 0
    d.in_features, d.num_int, d.num_fp, d.out_features = n_in, K, F, N
    d.sym_divisor, d.colmap_streams, d.tiled_min_rows = 4.0, 1, 33
    d.colmap, d.int_weight, d.weights_scales = colmap.data_ptr(), mod.int_weight.data_ptr(), mod.weights_scales.data_ptr()
    d.reduced_w, d.fp_weight = mod.reduced_w.data_ptr(), mod.fp_weight.data_ptr()
    d.tiled_weight = w_t.data_ptr() if tiled else None
    nbytes = lib.quik_layer_workspace_bytes(ctypes.byref(d), M)
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    out = torch.empty(M, N, dtype=torch.float16, device=DEV)
    before, mid, after = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    mid.record()                                 # an event has a handle once it has been recorded
    torch.cuda.synchronize()
    before.record()
    rc = lib.quik_layer_forward(ctypes.byref(d), x.data_ptr(), M, ws.data_ptr(), nbytes, None, 0, out.data_ptr(),
                                mid.cuda_event, L.stream())
    after.record()
    assert rc == 0, lib.quik_status_string(rc)
    torch.cuda.synchronize()
    # the event sits between the two launches on the launch stream: recorded by this call (its time lies between
    # the two events around the call), and each of the two intervals holds one kernel
    assert before.elapsed_time(mid) >= 0 and mid.elapsed_time(after) >= 0
    assert before.elapsed_time(mid) + mid.elapsed_time(after) > 0

    if tiled and bits == 4:
        q, meta = asymmetric.quantize_mapped_fp6(x, colmap, K, F)
        ref = matmul.mixed_linear_fp6(q, w_t, meta, mod.weights_scales, mod.reduced_w, None, M, N, K, F, torch.float16)
    elif tiled:
        q, meta = asymmetric.quantize_mapped_tile8(x, colmap, K, F)
        ref = matmul.mixed_linear_tile8(q, w_t, meta, mod.weights_scales, mod.reduced_w, None, M, N, K, F, torch.float16)
    else:
        q, meta, fp = asymmetric.quantize_mapped(x, colmap, K, F, bits)
        ref = matmul.mixed_linear(q, mod.int_weight, meta, mod.weights_scales, mod.reduced_w, fp, mod.fp_weight, None,
                                  bits, torch.float16)
    assert torch.equal(_bits(out), _bits(ref))
    # a workspace one byte short is refused before anything is launched
    assert lib.quik_layer_forward(ctypes.byref(d), x.data_ptr(), M, ws.data_ptr(), nbytes - 1, None, 0, out.data_ptr(),
                                  None, L.stream()) == -6


@pytest.mark.parametrize("bits,symm,n_in,F", [(4, False, 2048 + 64, 64), (8, False, 1280 + 256, 256),
                                              (4, True, 1024 + 32, 32)])
def test_one_resident_copy_of_the_weights(bits, symm, n_in, F):
    """release_row_major_weights(): the module keeps the tile-ordered copy only and serves every row count from
    it; release_tiled_weights(): the reference's buffers only.  Above 32 rows all three give the same bits; up to
    32 rows the tile-ordered kernels add the fp32 terms in another order than the weight-streaming kernel:
    equal within rounding, and within 1e-2 x RMS of the oracle."""
    N = 384
    rng = np.random.default_rng(bits + F)
    W, s_w, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16)
    omod = qo.from_float(W, s_w, fi, bits, symm=symm)
    both = _module(W, s_w, fi, bits, bias, symm)
    tiled_only = _module(W, s_w, fi, bits, bias, symm)
    rows_only = _module(W, s_w, fi, bits, bias, symm)
    rows_only.release_tiled_weights()
    xs = {}
    for M in (1, 20, 32, 33, 200):
        x = rng.standard_normal((M, n_in)).astype(np.float32)
        x[:, fi] *= 50
        xs[M] = x.astype(np.float16)
    ref = {M: both(torch.from_numpy(x).to(DEV)) for M, x in xs.items()}
    wb = both.weight_bytes()
    assert wb["row_major"] == wb["reference_layout"] == N * ((n_in - F) * bits // 8 + F * 2)
    assert wb["tiled"] >= N * ((n_in - F) * (6 if bits == 4 else 8) // 8 + F * 2)
    tiled_only.release_row_major_weights()
    wt = tiled_only.weight_bytes()
    assert wt["row_major"] == 0 and wt["tiled"] == wb["tiled"]
    assert rows_only.weight_bytes()["tiled"] == 0
    for M, x in xs.items():
        xt = torch.from_numpy(x).to(DEV)
        got_t, got_r = tiled_only(xt), rows_only(xt)
        assert rows_only._w6 is None
        assert torch.equal(_bits(got_r), _bits(ref[M]))
        want, _ = qo.mixed_qlinear_forward(x, omod, bits, bias, symm=symm)
        w64 = want.astype(np.float64)
        if M > 32:
            assert torch.equal(_bits(got_t), _bits(ref[M]))
        err = np.abs(got_t[0].float().cpu().numpy().astype(np.float64) - w64).max()
        assert err <= 1e-2 * np.sqrt((w64 ** 2).mean())
        assert err <= 4 * np.abs(w64).max() * 2.0 ** -10
    with pytest.raises(RuntimeError):
        tiled_only.release_tiled_weights()


@pytest.mark.parametrize("bits,symm,n_in,F", [(4, False, 2048 + 64, 64), (8, False, 1280 + 256, 256),
                                              (4, True, 1024 + 32, 32)])
def test_transient_tile_ordered_copy(bits, symm, n_in, F, monkeypatch):
    """transient_tiled_copy: calls of more than 32 rows repack the reference's buffers into a temporary operand
    buffer and run the same tile-ordered GEMM.  Same output bits as the default module at every row count (the
    small calls are untouched), nothing tile-ordered kept between calls, one packing launch per large call; the
    same under HIP graph replays."""
    from quik_amd import matmul
    N = 384
    rng = np.random.default_rng(bits + F + 1)
    W, s_w, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16)
    both = _module(W, s_w, fi, bits, bias, symm)
    lean = _module(W, s_w, fi, bits, bias, symm)
    lean.transient_tiled_copy = True
    packs = []
    for name in ("pack_weight_fp6", "pack_weight_tile8"):
        orig = getattr(matmul, name)
        monkeypatch.setattr(matmul, name, lambda *a, _o=orig, **k: (packs.append(1), _o(*a, **k))[1])
    for M in (1, 32, 33, 200, 33):
        x = rng.standard_normal((M, n_in)).astype(np.float32)
        x[:, fi] *= 50
        xt = torch.from_numpy(x.astype(np.float16)).to(DEV)
        want = both(xt)
        n0 = len(packs)
        got = lean(xt)
        assert torch.equal(_bits(got), _bits(want)), M
        assert len(packs) - n0 == (1 if M > 32 else 0)
        wb = lean.weight_bytes()
        assert wb["tiled"] == 0 and wb["row_major"] == wb["reference_layout"] and lean._w6 is None
    with pytest.raises(RuntimeError):
        lean.release_row_major_weights()
    # graph replays: the packing launch is part of the graph
    xt = torch.from_numpy((rng.standard_normal((70, n_in)) * 1.0).astype(np.float16)).to(DEV)
    want = both(xt).clone()
    lean(xt)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        lean(xt)
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = lean(xt)
    for _ in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(out), _bits(want))


# ------------------------------------------------------------------------------ shared-input groups
@pytest.mark.parametrize("rows,bits,symm,bias", [(200, 4, False, False), (16, 4, False, True), (72, 4, True, False),
                                                 (130, 8, False, False), (1, 8, False, False)])
def test_shared_input_group_is_one_quantize_and_one_gemm(rows, bits, symm, bias, monkeypatch):
    """Layers wired as the reference wires q/k/v (experiments/llama.py:402-437: one SharedQuantizedInput(3), every
    member built by from_float with it) run as ONE library call for the whole group; each member's output has the
    bits the member gives on its own, and equals the oracle's forward within the stated tolerance."""
    from quik_amd import _lib as L
    from quik_amd.qlinear import MixedQLinear, SharedQuantizedInput
    rng = np.random.default_rng(rows + bits)
    n_in, F = 1024 + 64, 64
    sizes = [512, 128, 192]                  # q wider than k / v, as with grouped-query attention
    fi = np.sort(rng.permutation(n_in)[:F]).astype(np.int64)
    shared = SharedQuantizedInput(len(sizes))
    members, alone, parts = [], [], []
    for N in sizes:
        W, s_w, _ = _layer(rng, N, n_in, F, bits)
        # the outlier columns of a group are the same for every member (they come from the shared input's statistics)
        keep = np.ones(n_in, bool)
        keep[fi] = False
        lo, hi = (-8, 8) if bits == 4 else (-127, 128)
        W = np.zeros((N, n_in), np.float16)
        W[:, keep] = (rng.integers(lo, hi, (N, n_in - F)) * s_w.astype(np.float32)).astype(np.float16)
        W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
        b = (0.1 * rng.standard_normal(N)).astype(np.float16) if bias else None
        lin = torch.nn.Linear(n_in, N, bias=bias)
        if bias:
            lin.bias.data = torch.from_numpy(b)
        mk = lambda sh: MixedQLinear.from_float(lin, torch.from_numpy(W), torch.from_numpy(s_w), sh,
                                                torch.from_numpy(fi), symm=symm, bits=bits).to(DEV)
        members.append(mk(shared))
        alone.append(mk(None))
        parts.append((W, s_w, b))
    x = rng.standard_normal((rows, n_in)).astype(np.float32)
    x[:, fi] *= 50
    xt = torch.from_numpy(x.astype(np.float16)).to(DEV)

    lib = L.load()
    calls = []
    real = lib.quik_layer_forward

    class Spy:
        def __getattr__(self, name):
            if name == "quik_layer_forward":
                def counted(*a):
                    calls.append(a[2])
                    return real(*a)
                return counted
            return getattr(lib, name)
    monkeypatch.setattr(L, "load", lambda: Spy())
    for rep in range(2):                      # the second pass reuses the fused weights
        calls.clear()
        outs = [m(xt) for m in members]       # the call order of the reference's decoder layer: one after the other
        torch.cuda.synchronize()
        assert calls == [rows]                # one quantize + one GEMM for the three layers
        assert shared.cur_group_elem == 0 and shared._outs is None
    monkeypatch.undo()
    for m, a, o, (W, s_w, b) in zip(members, alone, outs, parts):
        assert o.shape == (1, rows, m.out_features)
        want_bits = a(xt)
        assert torch.equal(_bits(o), _bits(want_bits))
        omod = qo.from_float(W, s_w, fi, bits, symm=symm)
        want, _ = qo.mixed_qlinear_forward(x.astype(np.float16), omod, bits, b, symm=symm)
        got = o[0].float().cpu().numpy().astype(np.float64)
        w64 = want.astype(np.float64)
        assert np.abs(got - w64).max() <= 1e-2 * np.sqrt((w64 ** 2).mean())
    # the members' buffers are slices of the group's: one copy of the weights, and the state dict is the members' own
    assert members[1].int_weight.data_ptr() == shared._fused.int_weight[sizes[0]:].data_ptr()
    for m, a in zip(members, alone):
        sd_m, sd_a = m.state_dict(), a.state_dict()
        assert sorted(sd_m) == sorted(sd_a)
        assert all(torch.equal(sd_m[k], sd_a[k]) for k in sd_m)
    # switched off: the reference's protocol, one library crossing sequence per member, same bits
    MixedQLinear.fuse_shared_groups = False
    try:
        outs2 = [m(xt) for m in members]
    finally:
        MixedQLinear.fuse_shared_groups = True
    assert all(torch.equal(_bits(o), _bits(o2)) for o, o2 in zip(outs, outs2))


def test_shared_input_group_with_different_outlier_columns_is_not_fused():
    """Members whose outlier columns differ cannot share one GEMM: the group falls back to the reference's protocol
    (which shares the first member's quantized activation, whatever the later members' columns are)."""
    from quik_amd.qlinear import MixedQLinear, SharedQuantizedInput
    rng = np.random.default_rng(5)
    n_in, F, bits = 512 + 32, 32, 4
    shared = SharedQuantizedInput(2)
    mods = []
    for k in range(2):
        W, s_w, fi = _layer(rng, 96, n_in, F, bits)
        lin = torch.nn.Linear(n_in, 96, bias=False)
        mods.append(MixedQLinear.from_float(lin, torch.from_numpy(W), torch.from_numpy(s_w), shared,
                                            torch.from_numpy(fi), bits=bits).to(DEV))
    xt = torch.from_numpy(rng.standard_normal((40, n_in)).astype(np.float16)).to(DEV)
    outs = [m(xt) for m in mods]
    assert shared._fused is False and shared.cur_group_elem == 0
    assert all(torch.isfinite(o).all() for o in outs)
