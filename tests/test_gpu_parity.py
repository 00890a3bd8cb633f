"""GPU parity: every op of the C ABI (through the quik Python surface) against the CPU oracle.

Bar: integer codes, packed bytes, metadata and int32 accumulators are bit-exact; fp16/bf16
outputs of the stand-alone dequantize ops are bit-exact against the oracle's association
order and within 1 output ulp of a float64 evaluation; the fused forward is within
1e-2 x output RMS (max abs) of the oracle, the tolerance the task states, and in practice
within a few output ulps.
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


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t.to(DEV) if dtype is None else t.to(DEV, dtype)


def _bf16_t(a32):
    """float32 numpy array holding bf16-representable values -> bf16 tensor on the GPU."""
    return torch.from_numpy(np.ascontiguousarray(a32, np.float32)).to(torch.bfloat16).to(DEV)


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _split(rng, n_in, F, shuffle=False):
    fp_idx = rng.permutation(n_in)[:F].astype(np.int64)
    mask = np.ones(n_in, bool)
    mask[fp_idx] = False
    ii = np.arange(n_in, dtype=np.int64)[mask]
    if shuffle:
        ii = rng.permutation(ii)
    return ii, fp_idx


def _acts(rng, M, n_in, fp_idx, kind="x50"):
    x = rng.standard_normal((M, n_in)).astype(np.float32)
    if kind == "x50":
        x[:, fp_idx] *= 50
    elif kind == "student":
        x[:, fp_idx] = np.clip(20 * rng.standard_t(3, (M, len(fp_idx))), -6e4, 6e4)
    elif kind == "uniform":
        x = rng.random((M, n_in)).astype(np.float32)
    return x


def _edge_rows(x, ii):
    """Overwrite the first rows with edge cases (needs M >= 8, K >= 16)."""
    x[0, :] = 1.5                                   # constant row: scale clamps at 1e-6
    x[1, ii[:8]] = [0, 0.5, 1.5, 2.5, 3.5, 4.5, 15, 7.5]
    x[2, :] *= 1e-7                                 # fp16 subnormals
    x[3, ii[3]] = 65504.0
    x[3, ii[4]] = -65504.0                          # range overflows fp16
    x[4, ii[5]] = np.inf
    x[5, ii[6]] = np.nan
    x[6, :] = 0.0
    x[7, ii] = np.nan                               # all-NaN row
    return x


# ------------------------------------------------------------------------------ asym quantize
QCASES = [
    # M, in, F, kind, shuffle
    (33, 512, 32, "x50", False),
    (9, 4096, 128, "student", False),
    (64, 1024, 0, "x50", False),
    (17, 100, 10, "x50", True),        # row length not a multiple of 8: scalar load path
    (40, 384, 32, "uniform", True),    # int_indices in arbitrary order
    (12, 2050, 2, "x50", False),
    (20, 520, 6, "x50", False),        # K = 514: not a multiple of 16, scalar tail of the packed output
    (300, 8192, 256, "x50", False),    # several rows per workgroup (register prefetch of the next row)
    (70, 28672, 256, "student", False),
    (530, 8192, 256, "x50", False),    # 512 rows or more: one wave per row, 16 groups per lane
    (600, 2056, 300, "student", False),  # ... 8 groups per lane, more dirty groups than lanes
    (515, 520, 6, "x50", False),       # ... 4 groups per lane, scalar tail of the packed output
    (40, 12288, 64, "x50", False),     # four waves per row, 8 groups per lane
]


@pytest.mark.parametrize("case", QCASES)
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("bf16", [False, True])
def test_asym_quantize_bit_exact(case, bits, bf16):
    import quik
    M, n_in, F, kind, shuffle = case
    rng = np.random.default_rng(hash((M, n_in, F, bits, bf16)) % 2 ** 31)
    ii, fi = _split(rng, n_in, F, shuffle)
    x32 = _edge_rows(_acts(rng, M, n_in, fi, kind), ii)
    if bf16:
        xs = qo.bf16_round(x32)
        xt = _bf16_t(xs)
        dst, meta, fp_x = qo.asym_quantize(xs, ii, fi, bits, qo.BF16)
        meta_b, fp_b = qo.f32_to_bf16_bits(meta), qo.f32_to_bf16_bits(fp_x)
    else:
        with np.errstate(over="ignore"):
            xs = x32.astype(np.float16)
        xt = _t(xs)
        dst, meta, fp_x = qo.asym_quantize(xs, ii, fi, bits, qo.F16)
        meta_b, fp_b = meta.view(np.uint16), fp_x.view(np.uint16)
    q, m, f = quik.asymmetric.quantize(xt, _t(ii), _t(fi), bits)
    assert q.dtype == (torch.uint8 if bits == 4 else torch.int8)
    assert m.shape == (2 * M,) and f.shape == (M, F) and m.dtype == xt.dtype
    got_m = _bits(m)
    # scale bit-exact; zero bit-exact except that -0/+0 and NaN payloads are not distinguished
    want_f = np.asarray(meta, np.float32)
    got_f = m.float().cpu().numpy()
    assert np.array_equal(got_m[0::2], meta_b[0::2])
    assert np.array_equal(np.nan_to_num(got_f[1::2], nan=12345.0), np.nan_to_num(want_f[1::2], nan=12345.0))
    assert np.array_equal(q.cpu().numpy(), dst)
    assert np.array_equal(_bits(f), fp_b)


def test_asym_quantize_config1_shape_and_reference_invariants():
    """The reference-sized single layer (512 x 4096, 128 outliers x50) plus the reference's own checks
    (test/python/test_quant.py:24-39): indexed quantize == find_meta + quantizeOld on the gathered
    columns, fp_x == x[:, fp_indices]."""
    import quik
    g = torch.Generator().manual_seed(0)
    M, n_in, F = 512, 4096, 128
    x = torch.randn(M, n_in, generator=g)
    fi = torch.randperm(n_in, generator=g)[:F]
    x[:, fi] *= 50
    x = x.half()
    ii = torch.arange(n_in)
    ii = ii[~torch.isin(ii, fi)]
    xd = x.to(DEV)
    for bits in (4, 8):
        q, meta, fp = quik.asymmetric.quantize(xd, ii.to(DEV), fi.to(DEV), bits)
        int_t = xd[:, ii.to(DEV)].contiguous()
        meta_base = quik.asymmetric.find_meta(int_t, bits)
        q_base = quik.asymmetric.quantizeOld(int_t, meta_base, bits)
        assert torch.equal(meta, meta_base) and torch.equal(q, q_base)
        assert torch.equal(fp, xd[:, fi.to(DEV)])
        dst, m, f = qo.asym_quantize(x.numpy(), ii.numpy(), fi.numpy(), bits)
        assert np.array_equal(q.cpu().numpy(), dst)
        assert np.array_equal(_bits(meta), m.view(np.uint16))


def test_quotient_exhaustive_numerators():
    """Every non-negative fp16 numerator (finite, inf, NaN) against 300 scales, through
    quantizeOld with zero = 0: pins storage(d / scale) -> rne -> clamp for the whole domain."""
    import quik
    num = np.arange(0, 0x8000, dtype=np.uint16).view(np.float16)       # 0 .. +inf .. NaN
    rng = np.random.default_rng(11)
    scales = np.concatenate([
        np.array([1.0133e-6, 6e-8, 1.0, 0.5, 3.0, 65504.0, 4368.0, 0.1, 1 / 3], np.float32),
        np.exp(rng.uniform(np.log(1e-6), np.log(6e4), 291)).astype(np.float32)]).astype(np.float16)
    R = scales.size
    x = np.broadcast_to(num, (R, num.size)).copy()
    meta = np.zeros(2 * R, np.float16)
    meta[0::2] = scales
    for bits in (8, 4):
        got = quik.asymmetric.quantizeOld(_t(x), _t(meta), bits).cpu().numpy()
        want = qo.quantize_old(x, meta, bits)
        assert np.array_equal(got, want)


def test_fast_quotient_path_exhaustive_rows():
    """The row kernel's reciprocal + correction quotient: rows that contain every fp16 value in
    [0, hi] so that x - zero runs over all numerators for a fixed scale."""
    import quik
    rng = np.random.default_rng(12)
    rows = []
    for hi_bits in [0x3C00, 0x4B80, 0x5BF8, 0x7BFF, 0x0400, 0x2E66, 0x5640] + list(rng.integers(0x0400, 0x7BFF, 40)):
        vals = np.arange(0, int(hi_bits) + 1, dtype=np.uint16)
        row = np.zeros(0x7C00, np.uint16)
        row[:vals.size] = vals
        rows.append(row)
    x = np.stack(rows).view(np.float16)
    n_in = x.shape[1]
    ii = np.arange(n_in, dtype=np.int64)
    fi = np.zeros(0, np.int64)
    for bits in (4, 8):
        q, m, _ = quik.asymmetric.quantize(_t(x), _t(ii), _t(fi), bits)
        dst, meta, _ = qo.asym_quantize(x, ii, fi, bits)
        assert np.array_equal(_bits(m), meta.view(np.uint16))
        assert np.array_equal(q.cpu().numpy(), dst)


def test_streaming_quotient_full_domain_on_device():
    """Every fp16 scale the row kernel can produce against every numerator: one row per row maximum
    hi in [2^-14, 65504) holding all fp16 values 0 .. hi, zero = 0, so d = x and the scale is
    fp16(hi / maxq).  Expected codes come from IEEE float64 division on the device (the quotient of
    two fp16 numbers rounds to fp16 the same way from float64 as from the exact value); the 47-row
    test above ties the same arithmetic to the oracle."""
    import quik
    n_in = 0x7C00
    ii = torch.arange(n_in, device=DEV)
    fi = torch.zeros(0, dtype=torch.int64, device=DEV)
    cols = torch.arange(n_in, device=DEV, dtype=torch.int32)
    his = torch.arange(0x0400, 0x7BFF, device=DEV, dtype=torch.int32)
    for bits in (4, 8):
        maxq = float(2 ** bits - 1)
        for lo in range(0, his.numel(), 4096):
            hi = his[lo:lo + 4096]
            xb = torch.where(cols[None, :] <= hi[:, None], cols[None, :], torch.zeros_like(cols[None, :]))
            x = xb.to(torch.int16).view(torch.float16)
            q, m, _ = quik.asymmetric.quantize(x, ii, fi, bits)
            scale = (hi.to(torch.int16).view(torch.float16).float() / maxq).clamp_min(1e-6).half()
            assert torch.equal(m[0::2], scale) and not m[1::2].any()
            t = (x.double() / scale.double()[:, None]).half()
            lvl = t.float().clamp(0, maxq).round().to(torch.int32) - 2 ** (bits - 1)
            if bits == 4:
                want = ((lvl[:, 0::2] & 0xF) | ((lvl[:, 1::2] & 0xF) << 4)).to(torch.uint8)
            else:
                want = lvl.to(torch.int8)
            assert torch.equal(q, want), (bits, lo)


def test_asym_quantize_argument_errors():
    import quik
    x = torch.randn(4, 64, dtype=torch.float16, device=DEV)
    ii = torch.arange(62, device=DEV)
    fi = torch.tensor([62, 63], device=DEV)
    with pytest.raises(RuntimeError, match="either 4 or 8"):
        quik.asymmetric.quantize(x, ii, fi, 5)
    with pytest.raises(RuntimeError, match="not equal to total number of columns"):
        quik.asymmetric.quantize(x, ii[:-2], fi, 4)
    with pytest.raises(RuntimeError, match="has to be even"):
        quik.asymmetric.quantize(x, torch.arange(61, device=DEV), torch.tensor([61, 62, 63], device=DEV), 4)
    with pytest.raises(RuntimeError, match="contiguous"):
        quik.asymmetric.quantize(x.t().contiguous().t(), ii, fi, 4)
    with pytest.raises(RuntimeError, match="CUDA"):
        quik.asymmetric.quantize(x.cpu(), ii, fi, 4)
    with pytest.raises(RuntimeError, match="float16"):
        quik.asymmetric.quantize(x.float(), ii, fi, 4)
    with pytest.raises(TypeError):
        quik.asymmetric.quantize(x, ii, fi)
    q, m, f = quik.asymmetric.quantize(x[:0], ii, fi, 4)   # empty batch
    assert q.shape == (0, 31) and m.shape == (0,) and f.shape == (0, 2)


# ------------------------------------------------------------------------------ integer GEMM
MM_CASES = [
    # M, N, K
    (512, 32, 512),      # the reference's test_matmul.py case
    (1, 128, 3968),
    (16, 300, 96),
    (100, 40, 32),
    (257, 384, 3840),
    (128, 512, 4864),
    (300, 260, 7936),
    (512, 1024, 3968),
    # at most 32 token rows: the weight-streaming kernel (slabs of 32 columns, 128-byte K chunks per wave)
    (5, 40, 32),         # one chunk, fewer chunks than waves, ragged last slab
    (32, 8200, 4864),    # more slabs than resident workgroups: several slabs per workgroup
    (17, 96, 4096 + 32), # 8 waves per slab (long K, few slabs), K tail of half a 32-byte step for int4
]


@pytest.mark.parametrize("M,N,K", MM_CASES)
def test_int4_matmul_exact(M, N, K):
    import quik
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a = rng.integers(-8, 8, (M, K)).astype(np.int8)
    b = rng.integers(-8, 8, (N, K)).astype(np.int8)
    if M >= 2 and N >= 2:
        a[0, :] = -8
        b[0, :] = -8      # largest magnitude accumulators: 64 * K
        a[1, :] = 7
        b[1, :] = -8
    want = qo.int_matmul(a, b)
    c = quik.matmul.int4Matmul(_t(qo.pack_i4(a)), _t(qo.pack_i4(b)))
    assert c.dtype == torch.int32 and c.shape == (M, N)
    assert np.array_equal(c.cpu().numpy(), want)


@pytest.mark.parametrize("M,N,K", [(512, 32, 512), (1, 128, 13568), (16, 300, 16), (100, 40, 48),
                                     (257, 384, 10752), (300, 260, 2048), (2, 2, 28416),
                                     (3, 31, 16 * 11), (32, 8200, 2048), (17, 96, 4096 + 16)])
def test_int8_matmul_exact(M, N, K):
    import quik
    rng = np.random.default_rng(M * 5 + N * 11 + K)
    a = rng.integers(-128, 128, (M, K)).astype(np.int8)
    b = rng.integers(-128, 128, (N, K)).astype(np.int8)
    if M >= 2 and N >= 2:
        a[0, :] = -128
        b[0, :] = -128
        a[1, :] = 127
        b[1, :] = -128
    want = qo.int_matmul(a, b)
    c = quik.matmul.int8Matmul(_t(a), _t(b))
    assert np.array_equal(c.cpu().numpy(), want)


def test_matmul_reference_known_answer():
    """test/python/test_matmul.py:16-26 as written there: randint(-8, 7), float bmm, round, int32."""
    import quik
    from quik_amd.qlinear import pack_to_i4
    torch.manual_seed(0)
    B, M, K, N = 1, 512, 512, 32
    a = torch.randint(-8, 7, (B, M, K), dtype=torch.int8).to(DEV)
    b = torch.randint(-8, 7, (B, N, K), dtype=torch.int8).to(DEV)
    c_gt = torch.bmm(a.float(), b.float().transpose(1, 2)).round().to(torch.int32)
    c = quik.matmul.int4Matmul(pack_to_i4(a[0]), pack_to_i4(b[0]))
    assert torch.equal(c, c_gt[0])


def test_matmul_argument_errors():
    import quik
    a = torch.zeros((4, 16), dtype=torch.uint8, device=DEV)
    with pytest.raises(RuntimeError, match="alignment"):
        quik.matmul.int4Matmul(a[:, :8].contiguous(), a[:, :8].contiguous())     # K = 16 int4, not % 32
    with pytest.raises(RuntimeError, match="agree in K"):
        quik.matmul.int4Matmul(a, torch.zeros((4, 32), dtype=torch.uint8, device=DEV))
    with pytest.raises(RuntimeError, match="contiguous"):
        quik.matmul.int4Matmul(torch.zeros((16, 4), dtype=torch.uint8, device=DEV).t(), a)
    with pytest.raises(RuntimeError, match="CUDA"):
        quik.matmul.int4Matmul(a.cpu(), a.cpu())
    with pytest.raises(RuntimeError, match="expected torch.int8"):
        quik.matmul.int8Matmul(a, a)
    assert quik.matmul.int4Matmul(a[:0], a).shape == (0, 4)


# ------------------------------------------------------------------------------ dequantize
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("M,N", [(24, 40), (33, 100), (256, 1024), (5, 7)])
def test_asym_dequantize(bits, bf16, M, N):
    import quik
    rng = np.random.default_rng(M + N + bits)
    dt = qo.BF16 if bf16 else qo.F16
    rnd = (lambda v: qo.bf16_round(v.astype(np.float32))) if bf16 else (lambda v: v.astype(np.float16))
    tt = _bf16_t if bf16 else _t
    acc = rng.integers(-500000, 500000, (M, N)).astype(np.int32)
    acc[0, 0] = 2 ** 31 - 1
    acc[-1, -1] = -2 ** 31
    meta = rnd(np.stack([rng.uniform(0.01, 0.3, M), rng.uniform(-3, 0, M)], 1).reshape(-1))
    scol = rnd(rng.uniform(0.001, 0.01, (N, 1)))
    wred = rnd(rng.standard_normal((1, N)))
    y = rnd(rng.standard_normal((M, N)) * 3)
    out = quik.asymmetric.dequantize(_t(acc), tt(meta), tt(scol), tt(wred), tt(y), bits)
    want = qo.asym_dequantize(acc, meta, scol, wred, y, bits, dt)
    want_b = qo.f32_to_bf16_bits(want) if bf16 else want.view(np.uint16)
    assert out.dtype == (torch.bfloat16 if bf16 else torch.float16)
    assert np.array_equal(_bits(out), want_b)
    ref = qo.asym_dequantize_f64(acc, meta, scol, wred, y, bits, dt)
    ulp = np.maximum(np.abs(ref), 2.0 ** -14) * (2.0 ** -7 if bf16 else 2.0 ** -10)
    got = out.float().cpu().numpy().astype(np.float64)
    fin = np.isfinite(got)
    assert (np.abs(got - ref)[fin] <= ulp[fin]).all()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("cols", [128, 130, 127])
def test_sym_quantize_bit_exact(bits, cols):
    import quik
    torch.manual_seed(1)
    src = torch.randn(48, cols, dtype=torch.float16)
    scale = torch.randn(48, 1, dtype=torch.float16)
    src[0, :4] = torch.tensor([float("inf"), float("nan"), 65504.0, -65504.0], dtype=torch.float16)
    got = quik.symmetric.quantize(src.to(DEV), scale.to(DEV), bits).cpu().numpy()
    want = qo.sym_quantize(src.numpy(), scale.numpy(), bits)
    assert np.array_equal(got, want)
    if bits == 8:
        # the reference's own assertion (test/python/test_cuaprseLt.py:21-23) where it is defined
        ref = (src / scale).round()
        ok = (ref.abs() <= 127).numpy()
        assert np.array_equal(got[ok], ref.to(torch.int8).numpy()[ok])


@pytest.mark.parametrize("bits", [8, 16, 32])
def test_sym_dequantize_bit_exact(bits):
    """test/python/test_cuaprseLt.py:45-47: c * scale_row * scale_col + y in torch fp16, bit-equal."""
    import quik
    torch.manual_seed(2)
    M, N = 37, 53
    sr = torch.randn(M, 1, dtype=torch.float16)
    sc = torch.randn(1, N, dtype=torch.float16)
    y = torch.randn(M, N, dtype=torch.float16)
    if bits == 16:
        c = (torch.randn(M, N) * 100).half()
        ch = c
    elif bits == 8:
        c = torch.randint(-128, 128, (M, N), dtype=torch.int8)
        ch = c.half()
    else:
        c = torch.randint(-70000, 70000, (M, N), dtype=torch.int32)
        ch = c.half()
    out = quik.symmetric.dequantize(c.to(DEV), sr.to(DEV), sc.to(DEV), y.to(DEV), bits).cpu()
    ref = ch * sr * sc + y
    fin = torch.isfinite(ref)
    assert torch.equal(out[fin], ref[fin]) and torch.equal(torch.isnan(out), torch.isnan(ref))
    want = qo.sym_dequantize(c.numpy(), sr.numpy(), sc.numpy(), y.numpy(), bits)
    assert np.array_equal(out.numpy()[fin.numpy()], want[fin.numpy()])


# ------------------------------------------------------------------------------ MixedQLinear
def _layer(rng, N, n_in, F, bits):
    ii, fi = _split(rng, n_in, F)
    lo, hi = (-8, 8) if bits == 4 else (-127, 128)
    codes = rng.integers(lo, hi, (N, n_in - F))
    s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    W = np.zeros((N, n_in), np.float16)
    W[:, ii] = (codes * s_w.astype(np.float32)).astype(np.float16)
    W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
    return W, s_w, ii, fi


def _module(W, s_w, fi, bits, bias=None, symm=False, fused=True, shared=None):
    from quik_amd.qlinear import MixedQLinear
    N, n_in = W.shape
    lin = torch.nn.Linear(n_in, N, bias=bias is not None)
    if bias is not None:
        lin.bias.data = torch.from_numpy(bias)
    mod = MixedQLinear.from_float(lin, torch.from_numpy(W), torch.from_numpy(s_w), shared,
                                  torch.from_numpy(fi) if fi.size else None, symm=symm, bits=bits, fused=fused)
    return mod.to(DEV)


FWD_CASES = [
    # M, N, in, F, bits, bias, kind
    (32, 64, 512, 32, 4, False, "x50"),
    (100, 200, 1024, 64, 4, True, "student"),
    (300, 520, 4096, 128, 4, False, "x50"),
    (16, 256, 2048, 256, 8, False, "x50"),
    (260, 300, 1280, 256, 8, True, "x50"),
    (64, 128, 512, 0, 4, True, "x50"),
    (1, 384, 1024, 64, 4, False, "x50"),
    (5, 40, 72, 8, 4, True, "x50"),          # decode kernel: one K chunk, half an outlier piece, ragged slab
    (7, 100, 200, 8, 8, True, "student"),
    (32, 8200, 1056, 32, 4, False, "x50"),   # decode kernel: several slabs per workgroup
    (20, 64, 8192 + 520, 520, 8, True, "x50"),  # decode kernel: 8 waves per slab, more outlier pieces than prefetched
    (9, 8300, 1000, 40, 4, True, "x50"),     # decode kernel, token rows in LDS: last K chunk and last outlier piece cut short
    (12, 70, 456, 24, 8, False, "student"),  # decode kernel, token rows streamed: the same for int8
]


@pytest.mark.parametrize("case", FWD_CASES)
def test_mixed_qlinear_forward(case):
    M, N, n_in, F, bits, with_bias, kind = case
    rng = np.random.default_rng(sum(case[:5]))
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16) if with_bias else None
    x = _acts(rng, M, n_in, fi, kind).astype(np.float16)
    omod = qo.from_float(W, s_w, fi, bits)
    want, inter = qo.mixed_qlinear_forward(x, omod, bits, bias)
    mod = _module(W, s_w, fi, bits, bias)
    # from_float buffers are those of the oracle
    assert np.array_equal(mod.int_weight.cpu().numpy(), omod["int_weight"])
    assert np.array_equal(mod.int_indices.cpu().numpy(), omod["int_indices"])
    assert np.array_equal(mod.reduced_w.cpu().numpy(), omod["reduced_w"])
    out = mod(_t(x))
    assert out.shape == (1, M, N) and out.dtype == torch.float16
    got = out[0].float().cpu().numpy().astype(np.float64)
    w64 = want.astype(np.float64)
    rms = np.sqrt((w64 ** 2).mean())
    err = np.abs(got - w64).max()
    assert err <= 1e-2 * rms, (err, rms)
    # much tighter in practice: a few output ulps of the largest term
    assert err <= 4 * np.abs(w64).max() * 2.0 ** -10
    # unfused op sequence: integer stages bit-exact, output = oracle up to the outlier GEMM's order
    mod_u = _module(W, s_w, fi, bits, bias, fused=False)
    out_u = mod_u(_t(x))[0].float().cpu().numpy().astype(np.float64)
    assert np.abs(out_u - w64).max() <= 4 * np.abs(w64).max() * 2.0 ** -10
    # the algebraic identity against a float64 linear layer on the dequantised activation
    xd = qo.dequantized_activation_f64(x, ii, fi, bits)
    ref = xd @ W.astype(np.float64).T + (0 if bias is None else bias.astype(np.float64))
    assert np.abs(got - ref).max() <= 1e-2 * np.sqrt((ref ** 2).mean())


def test_mixed_qlinear_bf16_and_3d_input():
    from quik_amd.qlinear import MixedQLinear
    rng = np.random.default_rng(21)
    N, n_in, F, bits = 192, 768, 64, 4
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    Wb = torch.from_numpy(W.astype(np.float32)).to(torch.bfloat16)
    sb = torch.from_numpy(s_w.astype(np.float32)).to(torch.bfloat16)
    # rebuild W so that codes * scale round-trips in bf16
    codes = (torch.from_numpy(W[:, ii].astype(np.float32)) / torch.from_numpy(s_w.astype(np.float32))).round()
    Wb[:, torch.from_numpy(ii)] = (codes * sb.float()).to(torch.bfloat16)
    lin = torch.nn.Linear(n_in, N, bias=False)
    mod = MixedQLinear.from_float(lin, Wb, sb, None, torch.from_numpy(fi), bits=bits).to(DEV)
    x = torch.from_numpy(_acts(rng, 2 * 48, n_in, fi)).to(torch.bfloat16).reshape(2, 48, n_in)
    out = mod(x.to(DEV))
    assert out.shape == (2, 48, N) and out.dtype == torch.bfloat16
    xs = x.reshape(-1, n_in).float().numpy()
    omod = qo.from_float(Wb.float().numpy(), sb.float().numpy(), fi, bits, dtype=qo.BF16)
    want, inter = qo.mixed_qlinear_forward(xs, omod, bits, None, dtype=qo.BF16)
    got = out.reshape(-1, N).float().cpu().numpy().astype(np.float64)
    w64 = want.astype(np.float64)
    # bf16 keeps 8 significant bits: one output ulp (2^-7 relative) already exceeds 1e-2 x RMS for the
    # larger outputs, and the oracle (like the reference) rounds the outlier product to bf16 before the
    # final sum.  Bound: one bf16 ulp of the output plus one of that intermediate; then the stated
    # tolerance against the unrounded float64 result.
    y64 = np.abs(inter["fp_result"].astype(np.float64))
    assert (np.abs(got - w64) <= (np.abs(w64) + y64) * 2.0 ** -7).all()
    xd = qo.dequantized_activation_f64(xs, omod["int_indices"], fi, bits, qo.BF16)
    ref = xd @ Wb.double().numpy().T
    rms = np.sqrt((ref ** 2).mean())
    assert (np.abs(got - ref) <= 1e-2 * rms + np.abs(ref) * 2.0 ** -8).all()


def test_shared_quantized_input_group():
    """q/k/v-style group (experiments/llama.py:402-411): the first member quantizes, all reuse."""
    from quik_amd.qlinear import SharedQuantizedInput
    rng = np.random.default_rng(22)
    n_in, F, bits, M = 512, 32, 4, 40
    shared = SharedQuantizedInput(3)
    mods, omods = [], []
    fi = None
    for N in (64, 96, 128):
        W, s_w, ii, fi_new = _layer(np.random.default_rng(5), N, n_in, F, bits)   # same split for the group
        fi = fi_new
        mods.append(_module(W, s_w, fi, bits, shared=shared))
        omods.append(qo.from_float(W, s_w, fi, bits))
    x = _acts(rng, M, n_in, fi).astype(np.float16)
    xt = _t(x)
    from quik_amd.qlinear import MixedQLinear
    # the reference's protocol (the shared quantized activation is held until the last member has run), and the
    # default here: one quantize + one GEMM for the group, the other members' columns held instead
    for fuse in (False, True):
        MixedQLinear.fuse_shared_groups = fuse
        try:
            for i, (m, om) in enumerate(zip(mods, omods)):
                out = m(xt)[0].float().cpu().numpy()
                want, _ = qo.mixed_qlinear_forward(x, om, bits)
                assert np.abs(out - want).max() <= 1e-2 * np.sqrt((want.astype(np.float64) ** 2).mean())
                held = shared._outs if fuse else shared.qint_x
                assert (held is None) == (i == 2)
        finally:
            MixedQLinear.fuse_shared_groups = True


@pytest.mark.parametrize("tokens,bits", [(300, 4), (8, 4), (40, 8)])
def test_fused_group_equals_member_layers(tokens, bits):
    """q/k/v-style group as ONE GEMM over concatenated output columns: bit-identical to the members run
    one by one (same per-column arithmetic), for the large-tile, mid-tile and decode kernels."""
    from quik_amd.qlinear import FusedMixedQLinearGroup
    rng = np.random.default_rng(40 + tokens)
    n_in, F = 1024, 64
    mods = []
    fi = None
    for i, N in enumerate((512, 128, 160)):
        W, s_w, ii, fi = _layer(np.random.default_rng(9), N, n_in, F, bits)        # same column split
        W2, s_w2, _, _ = _layer(np.random.default_rng(100 + i), N, n_in, F, bits)  # different weights
        codes = np.random.default_rng(200 + i).integers(-8 if bits == 4 else -127, 8 if bits == 4 else 128,
                                                        (N, n_in - F))
        Wm = np.zeros((N, n_in), np.float16)
        Wm[:, ii] = (codes * s_w2.astype(np.float32)).astype(np.float16)
        Wm[:, fi] = (0.02 * np.random.default_rng(300 + i).standard_normal((N, F))).astype(np.float16)
        bias = np.random.default_rng(400 + i).standard_normal(N).astype(np.float16)
        mods.append(_module(Wm, s_w2, fi, bits, bias))
    x = _t(_acts(rng, tokens, n_in, fi).astype(np.float16))
    group = FusedMixedQLinearGroup(mods)
    outs = group(x)
    assert len(outs) == 3
    for m, o in zip(mods, outs):
        assert torch.equal(o, m(x))


def test_packed_state_dict_round_trip():
    """The packed module is its own checkpoint format: buffers under the reference's names
    (experiments/qlinear.py:53-78), saved with torch.save and loaded into a freshly constructed
    module (no from_float) reproduce the forward bit for bit."""
    import io
    from quik_amd.qlinear import MixedQLinear
    rng = np.random.default_rng(77)
    N, n_in, F = 192, 640, 64
    for bits, with_bias in ((4, True), (8, False)):
        W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
        bias = rng.standard_normal(N).astype(np.float16) if with_bias else None
        mod = _module(W, s_w, fi, bits, bias)
        sd = mod.state_dict()
        names = {"weights_scales", "int_weight", "int_indices", "fp_indices", "fp_weight", "reduced_w"}
        assert set(sd) == names | ({"bias"} if with_bias else set())
        assert sd["int_weight"].dtype == (torch.uint8 if bits == 4 else torch.int8)
        buf = io.BytesIO()
        torch.save(sd, buf)
        buf.seek(0)
        loaded = torch.load(buf, weights_only=True)
        fresh = MixedQLinear(n_in, N, None, fp_features_num=F, symm=False, bits=bits, dtype=torch.float16)
        if not with_bias:
            fresh.bias = None
        fresh.load_state_dict(loaded)
        fresh = fresh.to(DEV)
        x = _t(_acts(rng, 37, n_in, fi).astype(np.float16))
        assert torch.equal(fresh(x), mod(x))


@pytest.mark.parametrize("bits,bf16", [(4, False), (8, False), (4, True)])
def test_kernel_path_vs_simulated_path(bits, bf16):
    """Accuracy cross-check of the two ways the reference evaluates a QUIK layer: the kernel path
    (the HIP kernels, on the GPU) against the fake-quant simulated path (experiments/quant_sim.py:193-256,
    restated in oracle/sim_path.py).  The two use different zero-point conventions, so they agree to
    quantisation noise only: both errors against the unquantised float64 layer must be of the same
    size, and 8 bits must be far more accurate than 4."""
    from oracle import sim_path
    from quik_amd.qlinear import MixedQLinear
    rng = np.random.default_rng(50 + bits)
    M, N, n_in, F = 256, 384, 2048, 128
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    x = _acts(rng, M, n_in, fi, "student").astype(np.float16)
    dt = torch.bfloat16 if bf16 else torch.float16
    Wt, st, xt = torch.from_numpy(W).to(dt), torch.from_numpy(s_w).to(dt), torch.from_numpy(x).to(dt)
    if bf16:   # codes * scale must round-trip in the storage type
        codes = (torch.from_numpy(W[:, ii].astype(np.float32)) / torch.from_numpy(s_w.astype(np.float32))).round()
        Wt[:, torch.from_numpy(ii)] = (codes * st.float()).to(dt)
    lin = torch.nn.Linear(n_in, N, bias=False)
    mod = MixedQLinear.from_float(lin, Wt, st, None, torch.from_numpy(fi), bits=bits).to(DEV)
    out = mod(xt.to(DEV))[0].double().cpu().numpy()
    sim = sim_path.sim_mixed_linear(xt, Wt, torch.from_numpy(ii),
                                    torch.from_numpy(fi), bits).double().numpy()
    full = xt.double().numpy() @ Wt.double().numpy().T
    rms = np.sqrt((full ** 2).mean())
    e_ker = np.sqrt(((out - full) ** 2).mean()) / rms
    e_sim = np.sqrt(((sim - full) ** 2).mean()) / rms
    assert 0.5 < e_sim / e_ker < 2.0, (e_sim, e_ker)
    assert e_ker < (0.2 if bits == 4 else 0.02), e_ker


# 6-bit matrix-core path (two tile plans), weight-streaming MFMA kernel, matrix-vector kernel behind a quantize
# launch (K = 960 is not a multiple of 128) and with the quantize inside (one launch)
@pytest.mark.parametrize("tokens,n_in", [(300, 1024), (40, 1024), (4, 1024), (2, 1024), (1, 1088), (2, 1088)])
def test_forward_under_hip_graph_replays(tokens, n_in):
    """The forward (quantize + GEMM, no allocation or synchronisation inside the library) captured in a
    HIP graph: every replay, with new input contents and eager work in between, equals the eager result."""
    rng = np.random.default_rng(60 + tokens)
    N, F, bits = 384, 64, 4
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    mod = _module(W, s_w, fi, bits, rng.standard_normal(N).astype(np.float16))
    static_x = _t(_acts(rng, tokens, n_in, fi).astype(np.float16))
    mod(static_x)                                   # warm up: column map built, kernel attributes set
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            mod(static_x)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = mod(static_x)
    for rep in range(4):
        new_x = _t(_acts(rng, tokens, n_in, fi).astype(np.float16))
        static_x.copy_(new_x)
        graph.replay()
        torch.cuda.synchronize()
        got = static_out.clone()
        want = mod(new_x)                           # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep


def test_symmetric_mixed_qlinear():
    """Symmetric activations (scale = max|x| / 4 as the reference's expression evaluates):
    codes bit-exact with the oracle; fused fp32 epilogue within tolerance of the fp16-chain op."""
    rng = np.random.default_rng(23)
    M, N, n_in, F, bits = 48, 96, 512, 32, 4
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    x = _acts(rng, M, n_in, fi).astype(np.float16)
    omod = qo.from_float(W, s_w, fi, bits, symm=True)
    want, inter = qo.mixed_qlinear_forward(x, omod, bits, None, symm=True)
    mod_u = _module(W, s_w, fi, bits, symm=True, fused=False)
    out_u = mod_u(_t(x))[0].cpu().numpy()
    fin = np.isfinite(want)
    rms = np.sqrt((want[fin].astype(np.float64) ** 2).mean())
    assert np.abs(out_u[fin].astype(np.float64) - want[fin]).max() <= 1e-2 * rms
    mod = _module(W, s_w, fi, bits, symm=True, fused=True)
    out = mod(_t(x))[0].float().cpu().numpy()
    assert np.abs(out[fin].astype(np.float64) - want[fin]).max() <= 1e-2 * rms


# ------------------------------------------------------------------------------ full-size properties
def _full_size_check(M, n_in, N, F, bits, kind="x50", oracle_rows=256):
    """Layer shapes too large for a CPU product: the quantize kernel is compared with the oracle on a
    sample of rows, the integer GEMM through size-independent identities (row and column checksums,
    exact in float64) and exact spot tiles, and the fused output against the oracle's dequantize
    applied to the exact accumulators on the same tiles."""
    import quik
    g = torch.Generator().manual_seed(M + n_in + N + bits)
    K = n_in - F
    x = torch.randn(M, n_in, generator=g)
    if kind == "student":   # heavy tails: Student-t with 3 degrees of freedom, seeded
        chi2 = (torch.randn(3, M, n_in, generator=g) ** 2).sum(0)
        x = x / torch.sqrt(chi2 / 3)
    fi = torch.randperm(n_in, generator=g)[:F]
    x[:, fi] *= 20 if kind == "student" else 50
    x = x.half()
    ii = torch.arange(n_in)
    ii = ii[~torch.isin(ii, fi)]
    xd, iid, fid = x.to(DEV), ii.to(DEV), fi.to(DEV)
    q, meta, fp = quik.asymmetric.quantize(xd, iid, fid, bits)
    rows = np.unique(np.concatenate([np.arange(min(M, 8)), np.arange(max(M - 8, 0), M),
                                     np.random.default_rng(1).integers(0, M, oracle_rows)]))
    dst, m, f = qo.asym_quantize(x.numpy()[rows], ii.numpy(), fi.numpy(), bits)
    assert np.array_equal(q.cpu().numpy()[rows], dst)
    assert np.array_equal(_bits(meta).reshape(M, 2)[rows], m.view(np.uint16).reshape(-1, 2))
    assert torch.equal(fp.cpu(), x[:, fi])

    if bits == 4:
        qw = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g).to(DEV)
        c = quik.matmul.int4Matmul(q, qw)

        def unpack(p):  # uint8 [R, K/2] -> float64 [R, K] on the GPU
            lo = (p & 0xF).to(torch.int16)
            hi = (p >> 4).to(torch.int16)
            lo = torch.where(lo >= 8, lo - 16, lo)
            hi = torch.where(hi >= 8, hi - 16, hi)
            return torch.stack([lo, hi], dim=2).reshape(p.shape[0], -1).double()
        cpu_mm = qo.int4_matmul
    else:
        qw = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g).to(DEV)
        c = quik.matmul.int8Matmul(q, qw)

        def unpack(p):
            return p.double()
        cpu_mm = qo.int8_matmul

    a64 = unpack(q)
    step = 2048
    colsum_b = torch.zeros(K, dtype=torch.float64, device=DEV)
    for s in range(0, N, step):
        colsum_b += unpack(qw[s:s + step]).sum(0)
    assert torch.equal(c.double().sum(1), a64 @ colsum_b)            # sum_n C[m, n]
    rowsum_a = a64.sum(0)
    for s in range(0, N, step):
        assert torch.equal(c[:, s:s + step].double().sum(0), unpack(qw[s:s + step]) @ rowsum_a)   # sum_m C[m, n]
    # exact spot tiles against the oracle
    th, tw = min(64, M), 64
    spots = [(0, 0), ((M - th) // 2, (N // 2 // 8) * 8), (M - th, N - tw)]
    qn, cn = q.cpu().numpy(), None
    for (r0, c0) in spots:
        want = cpu_mm(qn[r0:r0 + th], qw[c0:c0 + tw].cpu().numpy())
        assert np.array_equal(c[r0:r0 + th, c0:c0 + tw].cpu().numpy(), want)

    s_w = (torch.rand(N, 1, generator=g) * 0.009 + 0.001).half().to(DEV)
    wred = torch.randn(1, N, generator=g).half().to(DEV)
    fpw = (0.02 * torch.randn(N, F, generator=g)).half().to(DEV)
    out = quik.matmul.mixed_linear(q, qw, meta, s_w, wred, fp, fpw, None, bits, torch.float16)
    mn, fn = meta.cpu().numpy(), fp.cpu().numpy()
    for (r0, c0) in spots:
        y = qo.fp_linear(fn[r0:r0 + th], fpw[c0:c0 + tw].cpu().numpy(), None)
        want = qo.asym_dequantize(c[r0:r0 + th, c0:c0 + tw].cpu().numpy(), mn[2 * r0:2 * (r0 + th)],
                                  s_w[c0:c0 + tw].cpu().numpy(), wred[:, c0:c0 + tw].cpu().numpy(), y, bits)
        got = out[r0:r0 + th, c0:c0 + tw].float().cpu().numpy()
        w64 = want.astype(np.float64)
        assert np.abs(got - w64).max() <= 1e-2 * np.sqrt((w64 ** 2).mean())
        assert np.abs(got - w64).max() <= 4 * np.abs(w64).max() * 2.0 ** -10


FULL_SIZE = [
    # tokens, in, out, outliers, bits
    (2048, 8192, 28672, 256, 4, "x50"),      # Llama-2-70B gate/up (the benchmark workload)
    (2048, 8192, 1024, 256, 4, "x50"),       # Llama-2-70B k/v (GQA)
    (2048, 28672, 8192, 256, 8, "x50"),      # Llama-2-70B down_proj, int8
    (2048, 4096, 11008, 256, 4, "x50"),      # Llama-2-7B gate/up
    (2048, 11008, 4096, 256, 8, "x50"),      # Llama-2-7B down_proj, int8
    (2048, 5120, 13824, 256, 4, "student"),  # Llama-2-13B gate/up, prefill
    (128, 13824, 5120, 256, 8, "student"),   # Llama-2-13B down_proj, int8, 128 tokens
    (16, 5120, 5120, 256, 4, "student"),     # Llama-2-13B q/k/v/o, 16 tokens
    (1, 5120, 13824, 256, 4, "student"),     # Llama-2-13B gate/up, single-token decode
    (16, 5120, 13824, 256, 4, "student"),    # Llama-2-13B gate/up, 16 tokens: token rows resident in LDS
    (32, 8192, 10240, 256, 4, "x50"),        # Llama-2-70B q+k+v, 32 tokens: the largest resident token operand
]


@pytest.mark.parametrize("case", FULL_SIZE)
def test_full_size_properties(case):
    _full_size_check(*case)


DECODE_RESIDENT = [
    # M, N, in, F, bits: N > 8192, so a workgroup of the weight-streaming kernel walks over several slabs
    (16, 8192 + 4128, 1024 + 64, 64, 4),
    (32, 8192 + 167, 2048 + 32, 32, 8),
    (7, 9000, 512, 0, 4),
    (32, 8320, 8192, 256, 4),
    (4, 8224, 28672, 256, 8),      # int8 rows of a down_proj: four of them still fit
]


@pytest.mark.parametrize("case", DECODE_RESIDENT)
def test_decode_kernel_with_token_rows_resident_in_lds(case):
    """At most 32 token rows and more than 8192 output columns: the weight-streaming kernel keeps the token rows in
    LDS.  Its output must have the bits of the same layer cut into column halves of at most 8192 columns (which
    stream the token rows from L2), and agree with the oracle."""
    M, N, n_in, F, bits = case
    rng = np.random.default_rng(sum(case))
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16)
    x = _acts(rng, M, n_in, fi).astype(np.float16)
    out = _module(W, s_w, fi, bits, bias)(_t(x))[0]
    half = N // 2
    lo = _module(W[:half], s_w[:half], fi, bits, bias[:half])(_t(x))[0]
    hi = _module(W[half:], s_w[half:], fi, bits, bias[half:])(_t(x))[0]
    assert np.array_equal(_bits(out), np.concatenate([_bits(lo), _bits(hi)], axis=1))
    cols = np.r_[0:64, N - 64:N]
    omod = qo.from_float(W[cols], s_w[cols], fi, bits)
    want, _ = qo.mixed_qlinear_forward(x, omod, bits, bias[cols])
    got = out.float().cpu().numpy()[:, cols]
    rms = np.sqrt((want.astype(np.float64) ** 2).mean())
    assert np.abs(got.astype(np.float64) - want).max() <= 1e-2 * rms


# ------------------------------------------------------------------------------ decoder block chain
@pytest.mark.parametrize("tokens", [(2, 24), (5, 1)])     # prefill (batch x seq), then single-token decode
def test_decoder_block_linears_chained(tokens):
    """All seven linears of a Llama-style decoder block (GQA: narrower k/v; int8 down_proj) replaced by
    MixedQLinear as experiments/llama.py:394-440 does it: q/k/v share one quantized input, gate/up
    another, down_proj is W8A8.  Dims are scaled down so that the oracle can follow; every layer's
    output is compared with the oracle's forward of the very tensor the GPU layer consumed, so the
    check is per layer and the chain exercises the plumbing between them."""
    from quik_amd.qlinear import SharedQuantizedInput
    B, S = tokens
    hidden, kv, mlp, F = 512, 128, 1536, 32
    rng = np.random.default_rng(31 + B)
    shared_qkv, shared_mlp = SharedQuantizedInput(3), SharedQuantizedInput(2)
    _, _, _, fi_h = _layer(rng, 8, hidden, F, 4)            # one outlier set per input space
    _, _, _, fi_m = _layer(rng, 8, mlp, F, 8)

    def make(N, n_in, fi, bits, shared=None):
        ii = np.setdiff1d(np.arange(n_in), fi)
        lo, hi = (-8, 8) if bits == 4 else (-127, 128)
        s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
        W = np.zeros((N, n_in), np.float16)
        W[:, ii] = (rng.integers(lo, hi, (N, ii.size)) * s_w.astype(np.float32)).astype(np.float16)
        W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
        return _module(W, s_w, fi, bits, shared=shared), qo.from_float(W, s_w, fi, bits)

    layers = {
        "q": make(hidden, hidden, fi_h, 4, shared_qkv), "k": make(kv, hidden, fi_h, 4, shared_qkv),
        "v": make(kv, hidden, fi_h, 4, shared_qkv), "o": make(hidden, hidden, fi_h, 4),
        "gate": make(mlp, hidden, fi_h, 4, shared_mlp), "up": make(mlp, hidden, fi_h, 4, shared_mlp),
        "down": make(hidden, mlp, fi_m, 8),
    }

    def run(name, x):          # x: torch fp16 [B, S, in] on the device
        mod, omod = layers[name]
        out = mod(x)
        assert out.shape == (B, S, mod.out_features) and out.dtype == torch.float16
        bits = 8 if name == "down" else 4
        want, _ = qo.mixed_qlinear_forward(x.reshape(B * S, -1).cpu().numpy(), omod, bits)
        w64 = want.astype(np.float64)
        got = out.reshape(B * S, -1).float().cpu().numpy()
        assert np.abs(got - w64).max() <= 1e-2 * np.sqrt((w64 ** 2).mean()), name
        return out

    h = _t(_acts(rng, B * S, hidden, fi_h).astype(np.float16)).reshape(B, S, hidden)
    q, k, v = run("q", h), run("k", h), run("v", h)
    assert shared_qkv.qint_x is None                        # released after the third member
    # stand-in for attention (left to PyTorch in the reference as well): mix v into q's shape
    att = torch.tanh(q) + v.repeat(1, 1, hidden // kv) * torch.sigmoid(k.repeat(1, 1, hidden // kv))
    h2 = h + run("o", att.half())
    g, u = run("gate", h2), run("up", h2)
    assert shared_mlp.qint_x is None
    out = h2 + run("down", (torch.nn.functional.silu(g) * u).half())
    assert torch.isfinite(out).all()


# ------------------------------------------------------------------------------ fused GEMM + dequantize ops
def _fused_operands(bits, M, N, K, spread, seed):
    torch.manual_seed(seed)
    a_ref = torch.randint(-spread, spread, (M, K), dtype=torch.int8)
    b_ref = torch.randint(-spread, spread, (N, K), dtype=torch.int8)
    if bits == 4:
        a, b = _t(qo.pack_i4(a_ref.numpy())), _t(qo.pack_i4(b_ref.numpy()))
    else:
        a, b = a_ref.to(DEV), b_ref.to(DEV)
    return a_ref.to(DEV), b_ref.to(DEV), a, b


@pytest.mark.parametrize("bits", [4, 8])
def test_fused_dequantize_reference_known_answers(bits):
    """The reference's own known-answer tests for the fused ops, same shapes, distributions and
    formulas (test/python/test_fused.py:16-67 int4, :130-177 int8), evaluated by torch on the device."""
    import quik
    M, N, K = 1024, 5120, 2048
    a_ref, b_ref, a, b = _fused_operands(bits, M, N, K, 3, 1)
    scale_row = torch.rand(M, 1, dtype=torch.float16).to(DEV)
    scale_col = torch.rand(1, N, dtype=torch.float16).to(DEV)
    y = torch.rand(M, N).to(torch.float16).to(DEV)
    c_int = torch.matmul(a_ref.float(), b_ref.float().transpose(1, 0)).round().to(torch.int32)
    sym = quik.symmetric.int4FusedDequantize if bits == 4 else quik.symmetric.int8FusedDequantize
    c = sym(a, b, scale_row, scale_col, y)
    assert torch.equal(c, c_int * scale_row * scale_col + y)

    shift_value = 0.6394267984578837          # random.random() under seed 42
    zero_row = torch.rand(M, 1, dtype=torch.float16).to(DEV)
    w_reduce = torch.rand(1, N, dtype=torch.float16).to(DEV)
    c_ref = c_int * scale_col * scale_row + \
        (zero_row + torch.tensor([shift_value], dtype=torch.float16).item() * scale_row) * w_reduce + y
    asym = quik.asymmetric.int4FusedDequantize if bits == 4 else quik.asymmetric.int8FusedDequantize
    c = asym(a, b, scale_row, scale_col, shift_value, zero_row, w_reduce, y)
    assert torch.equal(c, c_ref)


@pytest.mark.parametrize("bits,spread", [(4, 8), (8, 128)])
def test_fused_dequantize_vs_oracle_full_operand_range(bits, spread):
    """Full-range operands: accumulators far beyond 2048, so the int32 -> fp16 conversion rounds and,
    for int8, overflows to inf; bit-exact against the oracle (NaN positions equal, payloads ignored)."""
    import quik
    M, N, K = 70, 200, 1024
    a_ref, b_ref, a, b = _fused_operands(bits, M, N, K, spread, 5)
    rng = np.random.default_rng(7)
    scale_row = rng.uniform(0, 1, (M, 1)).astype(np.float16)
    scale_col = rng.uniform(0, 1, (1, N)).astype(np.float16)
    zero_row = rng.standard_normal((M, 1)).astype(np.float16)
    w_reduce = rng.standard_normal((1, N)).astype(np.float16)
    y = rng.standard_normal((M, N)).astype(np.float16)
    acc = qo.int_matmul(a_ref.cpu().numpy(), b_ref.cpu().numpy())
    sym = quik.symmetric.int4FusedDequantize if bits == 4 else quik.symmetric.int8FusedDequantize
    asym = quik.asymmetric.int4FusedDequantize if bits == 4 else quik.asymmetric.int8FusedDequantize
    got = sym(a, b, _t(scale_row), _t(scale_col), _t(y)).cpu().numpy()
    want = qo.sym_dequantize(acc, scale_row, scale_col, y, 32)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(want)].view(np.uint16), want[~np.isnan(want)].view(np.uint16))
    got = asym(a, b, _t(scale_row), _t(scale_col), 8.0, _t(zero_row), _t(w_reduce), _t(y)).cpu().numpy()
    want = qo.asym_fused_dequantize(acc, scale_row, scale_col, 8.0, zero_row, w_reduce, y)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(want)].view(np.uint16), want[~np.isnan(want)].view(np.uint16))


@pytest.mark.parametrize("M,N,K", [(33, 40, 64), (100, 130, 96), (257, 300, 512), (300, 8200, 128),
                                   (2048, 2048 + 136, 256), (1000, 520, 160), (16, 200, 256), (1, 64, 4096)])
@pytest.mark.parametrize("bits", [4, 8])
def test_fused_dequantize_is_one_launch_on_every_tile_plan(M, N, K, bits, monkeypatch):
    """The fused GEMM + dequantize ops run the integer product and the fp16-arithmetic epilogue in ONE launch
    (src/asymmetric/fused_dequantize.cu:9-119, src/symmetric/fused_dequantize.cu:9-107 of the reference do the
    same) on every tile shape of the plan, ragged M and N, K that only the plain (non-pipelined) tiles accept; no
    M x N int32 matrix is allocated.  Calls of at most 32 rows keep the two-launch form (weight-streaming kernel +
    epilogue kernel).  Bit-exact against the oracle either way."""
    import quik
    from quik_amd import _lib as L
    spread = 8 if bits == 4 else 128
    a_ref, b_ref, a, b = _fused_operands(bits, M, N, K, spread, M + N + K)
    rng = np.random.default_rng(M + K)
    scale_row = rng.uniform(0, 0.1, (M, 1)).astype(np.float16)
    scale_col = rng.uniform(0, 0.1, (1, N)).astype(np.float16)
    zero_row = rng.standard_normal((M, 1)).astype(np.float16)
    w_reduce = rng.standard_normal((1, N)).astype(np.float16)
    y = rng.standard_normal((M, N)).astype(np.float16)
    need = L.load().quik_fused_dequantize_workspace_bytes(M, N)
    assert (need > 0) == (M <= 32)
    int32_allocs = []
    real_empty = torch.empty

    def spy(*args, **kw):
        if kw.get("dtype") == torch.int32:
            int32_allocs.append(args)
        return real_empty(*args, **kw)
    monkeypatch.setattr(torch, "empty", spy)
    acc = qo.int_matmul(a_ref.cpu().numpy(), b_ref.cpu().numpy())
    sym = quik.symmetric.int4FusedDequantize if bits == 4 else quik.symmetric.int8FusedDequantize
    asym = quik.asymmetric.int4FusedDequantize if bits == 4 else quik.asymmetric.int8FusedDequantize
    got_s = sym(a, b, _t(scale_row), _t(scale_col), _t(y)).cpu().numpy()
    got_a = asym(a, b, _t(scale_row), _t(scale_col), float(2 ** (bits - 1)), _t(zero_row), _t(w_reduce), _t(y)).cpu().numpy()
    assert (len(int32_allocs) == 0) == (M > 32)
    for got, want in ((got_s, qo.sym_dequantize(acc, scale_row, scale_col, y, 32)),
                      (got_a, qo.asym_fused_dequantize(acc, scale_row, scale_col, float(2 ** (bits - 1)), zero_row,
                                                       w_reduce, y))):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~np.isnan(want)].view(np.uint16), want[~np.isnan(want)].view(np.uint16))


# ------------------------------------------------------------------------------ 6-bit matrix-core path
def _decode_operand6(buf, rows, K, F):
    """Operand buffer of the 6-bit path -> (levels [rows, K], outlier bit patterns [rows, F], level sums [rows]),
    following the layout documented in quik_amd/csrc/fp6_format.h (restated here, not imported)."""
    steps, fsteps, blocks = K // 64, F // 16, (rows + 63) // 64
    block_bytes = (steps + fsteps) * 3072
    assert buf.size == blocks * block_bytes + 4 * rows
    levels = np.zeros((rows, K), np.int64)
    outl = np.zeros((rows, F), np.uint16)
    for r in range(rows):
        base = (r >> 6) * block_bytes
        head_row = ((r >> 5) & 1) * 1024 + (r & 31) * 32
        swap = (r >> 3) & 1
        for s in range(steps):
            for h in range(2):
                head = buf[base + s * 3072 + head_row + ((h ^ swap) << 4):][:16]
                tail = buf[base + s * 3072 + 2048 + h * 512 + (r & 63) * 8:][:8]
                word = int.from_bytes(bytes(head) + bytes(tail), "little")
                levels[r, s * 64 + h * 32: s * 64 + h * 32 + 32] = [(word >> (6 * e)) & 63 for e in range(32)]
        for t in range(fsteps):
            for c in range(2):
                chunk = buf[base + (steps + t) * 3072 + head_row + ((c ^ swap) << 4):][:16]
                outl[r, t * 16 + c * 8: t * 16 + c * 8 + 8] = np.frombuffer(bytes(chunk), np.uint16)
    sums = np.frombuffer(bytes(buf[blocks * block_bytes:]), np.int32)
    return levels, outl, sums


def _in_place_order(ii, fi, n_in):
    """Position k of the 6-bit operand buffers -> index into ascending int_indices (restated from the rule in
    quik_amd/csrc/colmap.h): source column k keeps its place when it is an integer column; the outlier columns among
    the first K columns (holes, ascending) are filled by the integer columns of the last F columns (ascending)."""
    K = len(ii)
    outlier = np.zeros(n_in, bool)
    outlier[fi] = True
    holes = [c for c in range(K) if outlier[c]]
    fillers = [c for c in range(K, n_in) if not outlier[c]]
    assert len(holes) == len(fillers)
    col = np.arange(K)
    col[holes] = fillers
    return np.searchsorted(np.sort(ii), col)


@pytest.mark.parametrize("rows,K,F,bf16", [(70, 256, 32, False), (130, 128, 64, True), (64, 384, 0, False),
                                           (9, 2048 + 128, 160, False), (200, 8192 + 2048, 512 + 64, False)])
def test_six_bit_operand_buffers_hold_the_int4_codes(rows, K, F, bf16):
    """quantize_mapped_fp6 and pack_weight_fp6 write the codes of quantize_mapped / int_weight (bit-exact against
    the oracle elsewhere) as levels code + 8, the outlier values and the level sums, in the documented layout,
    with the integer columns in the column map's in-place order (the last cases: several fragments per lane, more
    holes than a lane keeps in registers, rows longer than the double-buffered kernel takes)."""
    from quik_amd import asymmetric, matmul
    rng = np.random.default_rng(rows + K + F)
    n_in = K + F
    ii, fi = _split(rng, n_in, F)
    x = _acts(rng, rows, n_in, fi).astype(np.float16)
    if rows >= 8:
        x = _edge_rows(x, ii)
    xt = _bf16_t(x.astype(np.float32)) if bf16 else _t(x)
    colmap = asymmetric.build_colmap(_t(ii), _t(fi), n_in)
    assert asymmetric.colmap_streams(colmap, K, F)
    q, meta, fp_x = asymmetric.quantize_mapped(xt, colmap, K, F, 4)
    x6, meta6 = asymmetric.quantize_mapped_fp6(xt, colmap, K, F)
    assert np.array_equal(_bits(meta), _bits(meta6))
    qn = q.cpu().numpy()
    want = np.empty((rows, K), np.int64)
    want[:, 0::2] = (qn & 0xF) ^ 8
    want[:, 1::2] = (qn >> 4) ^ 8
    order = _in_place_order(ii, fi, n_in)
    levels, outl, sums = _decode_operand6(x6.cpu().numpy(), rows, K, F)
    assert np.array_equal(levels, want[:, order])
    assert np.array_equal(outl, _bits(fp_x).reshape(rows, F))
    assert np.array_equal(sums, want.sum(1))
    # weights
    N = rows
    qw = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    fpw = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
    fpw_t = _bf16_t(fpw.astype(np.float32)) if bf16 else _t(fpw)
    w6 = matmul.pack_weight_fp6(_t(qw), fpw_t, colmap)
    want = np.empty((N, K), np.int64)
    want[:, 0::2] = (qw & 0xF) ^ 8
    want[:, 1::2] = (qw >> 4) ^ 8
    levels, outl, sums = _decode_operand6(w6.cpu().numpy(), N, K, F)
    assert np.array_equal(levels, want[:, order])
    assert np.array_equal(outl, _bits(fpw_t).reshape(N, F))
    assert np.array_equal(sums, want.sum(1))


def test_tile8_operand_buffers_hold_the_int8_codes():
    """quantize_mapped_tile8 / pack_weight_tile8: the int8 codes of quantize_mapped / int_weight and the outlier
    values, at the documented places (quik_amd/csrc/gemm_tile8.h)."""
    from quik_amd import asymmetric, matmul
    rng = np.random.default_rng(8)
    rows, K, F = 100, 192, 32
    n_in = K + F
    ii, fi = _split(rng, n_in, F)
    x = _edge_rows(_acts(rng, rows, n_in, fi).astype(np.float16), ii)
    colmap = asymmetric.build_colmap(_t(ii), _t(fi), n_in)
    q, meta, fp_x = asymmetric.quantize_mapped(_t(x), colmap, K, F, 8)
    x8, meta8 = asymmetric.quantize_mapped_tile8(_t(x), colmap, K, F)
    assert np.array_equal(_bits(meta), _bits(meta8))
    qw = rng.integers(-128, 128, (rows, K)).astype(np.int8)
    fpw = (0.02 * rng.standard_normal((rows, F))).astype(np.float16)
    w8 = matmul.pack_weight_tile8(_t(qw), _t(fpw))

    def decode(buf):
        steps, fsteps = K // 32, F // 16
        block_bytes = (steps + fsteps) * 2048
        assert buf.size == ((rows + 63) // 64) * block_bytes
        codes, outl = np.zeros((rows, K), np.int8), np.zeros((rows, F), np.uint16)
        for r in range(rows):
            base = (r >> 6) * block_bytes + ((r >> 5) & 1) * 1024 + (r & 31) * 32
            for s_ in range(steps + fsteps):
                for h in range(2):
                    chunk = bytes(buf[base + s_ * 2048 + ((h ^ ((r >> 3) & 1)) << 4):][:16])
                    if s_ < steps:
                        codes[r, s_ * 32 + h * 16: s_ * 32 + h * 16 + 16] = np.frombuffer(chunk, np.int8)
                    else:
                        t = s_ - steps
                        outl[r, t * 16 + h * 8: t * 16 + h * 8 + 8] = np.frombuffer(chunk, np.uint16)
        return codes, outl

    codes, outl = decode(x8.cpu().numpy())
    assert np.array_equal(codes, q.cpu().numpy()) and np.array_equal(outl, _bits(fp_x).reshape(rows, F))
    codes, outl = decode(w8.cpu().numpy())
    assert np.array_equal(codes, qw) and np.array_equal(outl, fpw.view(np.uint16))


SIX_CASES = [
    # M, N, in, F, bias, kind: K = in - F a multiple of 128, F a multiple of 32, M > 32
    (33, 200, 544, 32, True, "x50"),          # smallest row count of the path
    (100, 1056, 1024 + 64, 64, False, "student"),
    (256, 256, 384, 128, True, "x50"),        # one 128x128-tile round, two integer steps
    (300, 520, 1088, 64, False, "student"),   # ragged M and N
    (257, 130, 544, 32, True, "x50"),         # two outlier steps, N below a tile
    (512, 1024, 1024, 0, True, "x50"),        # no outlier columns
    (1000, 4160, 4096, 256, True, "x50"),     # 256x256 and 256x128 tiles in one launch, ragged M, N = 32.5 tiles
    (2048, 1280, 2048 + 96, 96, False, "x50"),
    (2048, 8192, 1024 + 128, 128, True, "x50"),   # one full round of 256x256 tiles: the eight-wave tile
    (2040, 8192 - 64, 512 + 32, 32, False, "x50"),   # eight-wave tiles, ragged last tile row and column
]


@pytest.mark.parametrize("case", SIX_CASES)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("bits", [4, 8])
def test_six_bit_path_is_bit_identical_to_the_int8_path(case, bf16, bits):
    """MixedQLinear on the tile-ordered operands (4 bits: 6-bit E2M3 matrix-core GEMM; 8 bits: int8 MFMA) against
    the same layer on the row-major int8-MFMA kernels (which the other tests hold against the oracle): identical
    output bits, NaN / Inf rows included."""
    from quik_amd.qlinear import MixedQLinear
    M, N, n_in, F, with_bias, kind = case
    rng = np.random.default_rng(sum(case[:4]) + bf16 + bits)
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16) if with_bias else None
    x = _edge_rows(_acts(rng, M, n_in, fi, kind).astype(np.float16), ii)
    mods = []
    for six in (True, False):
        mod = _module(W, s_w, fi, bits, bias)
        if bf16:
            mod = mod.to(torch.bfloat16)
            mod.dtype = torch.bfloat16
        mod.six_bit_path = six
        mods.append(mod)
    xt = _bf16_t(x.astype(np.float32)) if bf16 else _t(x)
    out6, out8 = mods[0](xt), mods[1](xt)
    assert mods[0]._w6 is not None and mods[1]._w6 is None      # the paths that were meant to run did run
    assert out6.shape == out8.shape == (1, M, N)
    assert np.array_equal(_bits(out6), _bits(out8))
    if not bf16:                                                # and against the oracle, on a slice of the rows
        omod = qo.from_float(W, s_w, fi, bits)
        rows = np.r_[0:24, M - 8:M]
        want, _ = qo.mixed_qlinear_forward(x[rows], omod, bits, bias)
        got = out6[0].float().cpu().numpy()[rows]
        fin = np.isfinite(want)
        assert np.array_equal(np.isfinite(got), fin)
        rms = np.sqrt((want[fin].astype(np.float64) ** 2).mean())
        assert np.abs(got[fin].astype(np.float64) - want[fin]).max() <= 1e-2 * rms


SYM_QUANT_CASES = [(40, 160, 32), (300, 1088, 64), (77, 512, 0), (1000, 4096, 256), (64, 8192 + 1024, 1024)]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("case", SYM_QUANT_CASES)
def test_sym_quantize_mapped_is_the_op_sequence_in_one_kernel(case, bits):
    """symmetric.quantize_mapped against the module's op sequence (experiments/qlinear.py:97-103: gather, max|x| /
    divisor in fp16, symmetric.quantize) and against the oracle's symmetric quantizer on the scale it produced:
    scale, codes and outlier values bit-equal, zero / subnormal / overflowing / Inf / NaN rows included."""
    import quik
    from quik_amd import asymmetric, symmetric
    M, n_in, F = case
    K = n_in - F
    rng = np.random.default_rng(M + n_in + F + bits)
    ii, fi = _split(rng, n_in, F)
    x = _edge_rows(_acts(rng, M, n_in, fi).astype(np.float16), ii)
    x[8, :] = 6e-8                                   # scale underflows to zero
    x[9, :] = -3.0
    xt, iit, fit = _t(x), _t(ii), _t(fi)
    divisor = 1 << ((bits - 1) - 1)
    colmap = asymmetric.build_colmap(iit, fit, n_in)
    assert asymmetric.colmap_streams(colmap, K, F)
    int_x = xt[:, iit].contiguous()
    scale = (torch.max(torch.abs(int_x), dim=1)[0].unsqueeze(1) / divisor).to(torch.float16)
    q = quik.symmetric.quantize(int_x, scale, bits)
    q2, scale2, fp2 = symmetric.quantize_mapped(xt, colmap, K, F, bits, divisor, False)
    nan_rows = torch.isnan(scale.float()).flatten().cpu().numpy()
    assert np.array_equal(_bits(scale)[~nan_rows], _bits(scale2)[~nan_rows])
    assert torch.isnan(scale2.float()).flatten().cpu().numpy()[nan_rows].all()
    assert np.array_equal(q.cpu().numpy(), q2.cpu().numpy())
    assert np.array_equal(_bits(fp2), x[:, fi].view(np.uint16))
    want = qo.sym_quantize(x[:, ii], scale2.cpu().numpy(), bits)
    assert np.array_equal(q2.cpu().numpy(), want)


SYM_SIX_CASES = [
    # M, N, in, F, bias
    (33, 200, 544, 32, True),
    (300, 520, 1088, 64, False),
    (512, 1024, 1024, 0, True),
    (1000, 4160, 4096, 256, True),
    (2048, 8192, 1024 + 128, 128, False),
]


@pytest.mark.parametrize("case", SYM_SIX_CASES)
def test_symmetric_module_on_tile_ordered_operands(case):
    """A symmetric MixedQLinear (4 bits, the only width from_float accepts) on the tile-ordered path (one quantize
    kernel into the 6-bit operand buffer, E2M3 matrix-core GEMM with the symmetric epilogue) against the same
    layer on the row-major kernels: identical output bits; and against the oracle within the fp16 tolerance."""
    M, N, n_in, F, with_bias = case
    bits = 4
    rng = np.random.default_rng(sum(case[:4]) + 5)
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16) if with_bias else None
    x = _edge_rows(_acts(rng, M, n_in, fi).astype(np.float16), ii)
    mods = []
    for six in (True, False):
        mod = _module(W, s_w, fi, bits, bias, symm=True)
        mod.six_bit_path = six
        mods.append(mod)
    out6, out8 = mods[0](_t(x)), mods[1](_t(x))
    assert mods[0]._w6 is not None and mods[1]._w6 is None
    assert out6.shape == out8.shape == (1, M, N)
    got6, got8 = _bits(out6).reshape(M, N), _bits(out8).reshape(M, N)
    nan_rows = np.isnan(x[:, ii].astype(np.float32)).any(1)
    assert np.array_equal(got6[~nan_rows], got8[~nan_rows])
    assert torch.isnan(out6[0].float()).cpu().numpy()[nan_rows].all()
    rows = np.r_[8:32, M - 1:M]                       # finite rows
    omod = qo.from_float(W, s_w, fi, bits, symm=True)
    want, _ = qo.mixed_qlinear_forward(x[rows], omod, bits, bias, symm=True)
    got = out6[0].float().cpu().numpy()[rows]
    rms = np.sqrt((want.astype(np.float64) ** 2).mean())
    assert np.abs(got.astype(np.float64) - want).max() <= 1e-2 * rms


SPLIT_K_CASES = [
    # M, N, in, F, bits, symm, bf16: few 128x128 tiles and a long K
    (64, 512, 8192 + 64, 64, 4, False, False),
    (64, 1024, 8192, 256, 4, False, True),
    (100, 640, 4096 + 32, 32, 8, False, False),
    (256, 520, 2048 + 64, 64, 8, False, True),      # ragged N
    (64, 384, 8192, 0, 4, False, False),            # no outlier columns
    (33, 130, 8192 + 64, 64, 4, True, False),       # symmetric activations, ragged M and N
    (200, 8192, 28672, 256, 8, False, False),       # Llama-2-70B down_proj at 200 tokens
]


@pytest.mark.parametrize("case", SPLIT_K_CASES)
def test_split_k_gives_the_same_bits(case):
    """Tile-ordered GEMMs with K split over several workgroups per tile (partial sums through a workspace, the last
    workgroup to arrive finishes the tile) against the same layer without the split: identical output bits, on
    repeated calls (the arrival counters return to zero) and with edge-case rows."""
    from quik_amd import _lib, matmul
    M, N, n_in, F, bits, symm, bf16 = case
    K = n_in - F
    assert _lib.load().quik_splitk_workspace_bytes(M, N, K, bits) > 0       # the shape does split
    rng = np.random.default_rng(sum(case[:5]))
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16)
    x = _edge_rows(_acts(rng, M, n_in, fi).astype(np.float16), ii)
    mod = _module(W, s_w, fi, bits, bias, symm=symm)
    if bf16:
        mod = mod.to(torch.bfloat16)
        mod.dtype = torch.bfloat16
    xt = _bf16_t(x.astype(np.float32)) if bf16 else _t(x)
    assert matmul.split_k
    try:
        got = [_bits(mod(xt)) for _ in range(3)]
        matmul.split_k = False
        want = _bits(mod(xt))
    finally:
        matmul.split_k = True
    nan_rows = np.isnan(x[:, ii].astype(np.float32)).any(1) if symm else np.zeros(M, bool)
    for g in got:
        assert np.array_equal(g[0][~nan_rows], want[0][~nan_rows])
    ws = matmul._splitk_workspaces[(torch.cuda.current_device(), torch.cuda.current_stream().cuda_stream)]
    assert int(ws[:4096].view(torch.int32).abs().sum()) == 0               # counters are back at zero
    # a second stream gets a workspace of its own (launches on two streams may overlap), same bits
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        other = _bits(mod(xt))
        assert matmul._splitk_workspaces[(torch.cuda.current_device(), side.cuda_stream)] is not ws
    side.synchronize()
    assert np.array_equal(other[0][~nan_rows], want[0][~nan_rows])
    del matmul._splitk_workspaces[(torch.cuda.current_device(), side.cuda_stream)]   # (the number per GPU is bounded)


@pytest.mark.parametrize("M,tiled", [(16, False), (24, True), (32, False), (32, True), (33, True)])
def test_int8_layers_around_the_switch_of_paths(M, tiled):
    """W8A8 at small row counts: up to 32 rows the weight-streaming kernel runs, above it the tile-ordered path
    (with its K split), which also accepts fewer rows when asked (`tile8_min_rows`).  Both against the oracle
    (their fp32 sums differ in order, so they are not compared bit for bit with each other)."""
    from quik_amd.qlinear import MixedQLinear
    N, n_in, F, bits = 520, 4096 + 64, 64, 8
    rng = np.random.default_rng(M)
    W, s_w, ii, fi = _layer(rng, N, n_in, F, bits)
    bias = rng.standard_normal(N).astype(np.float16)
    x = _acts(rng, M, n_in, fi).astype(np.float16)
    mod = _module(W, s_w, fi, bits, bias)
    assert MixedQLinear.tile8_min_rows == 33
    if tiled:
        mod.tile8_min_rows = 1
    out = mod(_t(x))[0].float().cpu().numpy()
    assert (mod._w6 is not None) == tiled
    omod = qo.from_float(W, s_w, fi, bits)
    want, _ = qo.mixed_qlinear_forward(x, omod, bits, bias)
    rms = np.sqrt((want.astype(np.float64) ** 2).mean())
    assert np.abs(out.astype(np.float64) - want).max() <= 1e-2 * rms


def test_six_bit_path_shared_input_and_fallbacks():
    """A q/k/v-style group on the 6-bit path quantizes once into the operand format; a member with the path
    switched off, or a call with fewer rows than the threshold, takes the int4 path, with the same results."""
    from quik_amd.qlinear import SharedQuantizedInput
    rng = np.random.default_rng(77)
    n_in, F, M = 1024 + 64, 64, 320
    shared = SharedQuantizedInput(3)
    mods, singles = [], []
    for N in (256, 128, 384):
        W, s_w, ii, fi = _layer(np.random.default_rng(6), N, n_in, F, 4)
        mods.append(_module(W, s_w, fi, 4, shared=shared))
        single = _module(W, s_w, fi, 4)
        single.six_bit_path = False
        singles.append(single)
    xt = _t(_acts(rng, M, n_in, fi).astype(np.float16))
    from quik_amd.qlinear import MixedQLinear
    for i, (m, s) in enumerate(zip(mods, singles)):            # the default: one GEMM for the group
        out = m(xt)
        assert (shared._outs is None) == (i == 2) and shared.x6 is None and shared.qint_x is None
        assert torch.equal(out, s(xt))
    MixedQLinear.fuse_shared_groups = False                    # member by member, as the reference runs a group
    try:
        for i, (m, s) in enumerate(zip(mods, singles)):
            out = m(xt)
            assert (shared.x6 is None) == (i == 2) and shared.qint_x is None
            assert torch.equal(out, s(xt))
        mods[1].six_bit_path = False                           # mixed group: member 1 re-quantizes to int4
        for i, (m, s) in enumerate(zip(mods, singles)):
            assert torch.equal(m(xt), s(xt))
        assert shared.x6 is None and shared.qint_x is None
        small = xt[:20].contiguous()                           # decode size: int4 path, weight-streaming kernel
        assert torch.equal(mods[0](small), singles[0](small))
        shared.finish(), shared.finish()
    finally:
        MixedQLinear.fuse_shared_groups = True
    # a group whose members disagree about the tile-ordered path is not fused, and still gives the members' bits
    for i, (m, s) in enumerate(zip(mods, singles)):
        assert torch.equal(m(xt), s(xt))
    assert shared._fused is False and shared.x6 is None and shared.qint_x is None


def test_tile_ordered_paths_random_shapes():
    """Op-level sweep of the two tile-ordered paths (quantize + fused GEMM) against the row-major kernels over random
    shapes, ragged in M and N, both dtypes, with and without bias and outliers: identical bits."""
    from quik_amd import asymmetric, matmul
    rng = np.random.default_rng(2024)
    for it in range(16):
        bits = int(rng.choice([4, 8]))
        K = (128 if bits == 4 else 64) * int(rng.integers(1, 24))
        F = 32 * int(rng.integers(0, 6))
        M = int(rng.choice([33, 65, 129, 200, 257, 511, 777, 1500, 2049]))
        N = int(rng.choice([8, 100, 130, 384, 520, 1000, 2048, 4160]))
        dt = torch.bfloat16 if rng.integers(0, 2) else torch.float16
        g = torch.Generator().manual_seed(it)
        n_in = K + F
        x = torch.randn(M, n_in, generator=g)
        fi = torch.randperm(n_in, generator=g)[:F]
        x[:, fi] *= 50
        x = x.to(dt).to(DEV)
        keep = torch.ones(n_in, dtype=torch.bool)
        keep[fi] = False
        ii = torch.arange(n_in)[keep]
        cm = asymmetric.build_colmap(ii.to(DEV), fi.to(DEV), n_in)
        if bits == 4:
            qw = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g).to(DEV)
        else:
            qw = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g).to(DEV)
        s_w = (torch.rand(N, 1, generator=g) * 0.009 + 0.001).to(dt).to(DEV)
        wred = torch.randn(1, N, generator=g).to(dt).to(DEV)
        fpw = (0.02 * torch.randn(N, F, generator=g)).to(dt).to(DEV)
        bias = torch.randn(N, generator=g).to(dt).to(DEV) if rng.integers(0, 2) else None
        q, meta, fp = asymmetric.quantize_mapped(x, cm, K, F, bits)
        want = matmul.mixed_linear(q, qw, meta, s_w, wred, fp if F else None, fpw if F else None, bias, bits, dt)
        if bits == 4:
            xb, meta2 = asymmetric.quantize_mapped_fp6(x, cm, K, F)
            got = matmul.mixed_linear_fp6(xb, matmul.pack_weight_fp6(qw, fpw, cm), meta2, s_w, wred, bias, M, N, K, F, dt)
        else:
            xb, meta2 = asymmetric.quantize_mapped_tile8(x, cm, K, F)
            got = matmul.mixed_linear_tile8(xb, matmul.pack_weight_tile8(qw, fpw), meta2, s_w, wred, bias, M, N, K, F, dt)
        case = (it, bits, M, N, K, F, dt)
        assert np.array_equal(_bits(meta), _bits(meta2)), case
        assert np.array_equal(_bits(got), _bits(want)), case


def test_tile_ordered_ops_refuse_a_column_map_that_does_not_stream():
    """int_indices in any other than ascending order (which the reference's quantize accepts, and the row-major
    op serves through the gather kernel) have no tile-ordered form: the wrappers raise before anything is launched,
    for a wrong-size column map as well, and the row-major op still agrees with the oracle."""
    import quik
    from quik_amd import asymmetric, symmetric
    rng = np.random.default_rng(99)
    M, n_in, F = 64, 1024 + 64, 64
    K = n_in - F
    ii, fi = _split(rng, n_in, F, shuffle=True)
    x = _acts(rng, M, n_in, fi).astype(np.float16)
    xt = _t(x)
    cm = asymmetric.build_colmap(_t(ii), _t(fi), n_in)
    assert not asymmetric.colmap_streams(cm, K, F)
    for bits, fn in ((4, asymmetric.quantize_mapped_fp6), (8, asymmetric.quantize_mapped_tile8)):
        with pytest.raises(RuntimeError, match="streaming kernel"):
            fn(xt, cm, K, F)
    for tiled in (False, True):
        with pytest.raises(RuntimeError, match="streaming kernel"):
            symmetric.quantize_mapped(xt, cm, K, F, 4, 4.0, tiled)
    q, meta, fp = asymmetric.quantize_mapped(xt, cm, K, F, 4)          # the gather kernel serves this order
    dst, m, f = qo.asym_quantize(x, ii, fi, 4)
    assert np.array_equal(q.cpu().numpy(), dst) and np.array_equal(_bits(fp), f.view(np.uint16))
    ii2, fi2 = _split(rng, n_in, F)
    cm_ok = asymmetric.build_colmap(_t(ii2), _t(fi2), n_in)
    with pytest.raises(RuntimeError, match="column map was not built"):
        asymmetric.quantize_mapped_fp6(xt[:, :1024 + 32].contiguous(), cm_ok, 1024, 32)
    with pytest.raises(RuntimeError, match="uint8 blob"):
        asymmetric.quantize_mapped(xt, cm_ok.view(torch.int8), K, F, 4)
    with pytest.raises(RuntimeError, match="CUDA"):
        asymmetric.quantize_mapped_fp6(xt, cm_ok.cpu(), K, F)
    # the C entry points themselves refuse such a map (QUIK_ERR_COLMAP = -8) and launch nothing
    from quik_amd import _lib as L
    lib = L.load()
    ERR_COLMAP = -8
    assert b"column map" in lib.quik_status_string(ERR_COLMAP)

    def c_calls(colmap):
        """return codes of the four entry points that exist on the streaming kernel only; none may write"""
        nbytes = lib.quik_fp6_operand_bytes(M, K, F)
        buf = torch.full((max(nbytes, lib.quik_tile8_operand_bytes(M, K, F)),), 0x5A, dtype=torch.uint8, device=DEV)
        meta6 = torch.zeros(2 * M, dtype=torch.float16, device=DEV)
        qw = torch.zeros((M, K // 2), dtype=torch.uint8, device=DEV)
        fpw = torch.zeros((M, F), dtype=torch.float16, device=DEV)
        rcs = [lib.quik_asym_quantize_fp6(L.ptr(xt), L.QUIK_F16, M, n_in, L.ptr(colmap), K, F, L.ptr(buf), L.ptr(meta6), L.stream()),
               lib.quik_asym_quantize_tile8(L.ptr(xt), L.QUIK_F16, M, n_in, L.ptr(colmap), K, F, L.ptr(buf), L.ptr(meta6), L.stream()),
               lib.quik_sym_quantize_mapped(L.ptr(xt), M, n_in, L.ptr(colmap), K, F, 4, 4.0, 1, L.ptr(buf), L.ptr(meta6), None, L.stream()),
               lib.quik_fp6_pack_weight(L.ptr(qw), L.ptr(fpw), M, K, F, L.ptr(colmap), L.ptr(buf), L.stream())]
        torch.cuda.synchronize()
        assert bool((buf == 0x5A).all()) and bool((meta6 == 0).all())
        return rcs

    assert c_calls(cm) == [ERR_COLMAP] * 4
    # ascending int_indices that overlap fp_indices (same counts, but no partition): refused as well, although the
    # ascending order and the number of distinct outlier columns alone would pass
    ii_bad = ii2.copy()                              # ascending (from _split)
    pos = int(np.searchsorted(ii_bad, fi2.max()))    # the integer column just below the largest outlier column ...
    assert pos > 0
    ii_bad[pos - 1] = fi2.max()                      # ... is replaced by that outlier column: still ascending
    assert np.all(np.diff(ii_bad) > 0) and np.intersect1d(ii_bad, fi2).size == 1
    cm_overlap = asymmetric.build_colmap(_t(ii_bad), _t(fi2), n_in)
    assert not asymmetric.colmap_streams(cm_overlap, K, F)
    assert c_calls(cm_overlap) == [ERR_COLMAP] * 4
    # the library forgets what it knew about an address when a new map is built there
    assert asymmetric.colmap_streams(cm_ok, K, F)
    rc = lib.quik_colmap_build(L.ptr(_t(ii)), K, L.ptr(_t(fi)), F, n_in, L.ptr(cm_ok), L.stream())
    assert rc == 0 and lib.quik_colmap_streaming(L.ptr(cm_ok), n_in, K, F, L.stream()) == 0
    # one call per layer forward: a descriptor that claims a streaming map for one that is not gets the same refusal
    desc = L.QuikLayer()
    import ctypes
    desc.struct_bytes = ctypes.sizeof(L.QuikLayer)
    desc.bits, desc.dtype, desc.symmetric = 4, L.QUIK_F16, 0
    desc.in_features, desc.num_int, desc.num_fp, desc.out_features = n_in, K, F, 64
    desc.colmap_streams, desc.tiled_min_rows = 1, 1
    junk = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    desc.colmap, desc.weights_scales, desc.reduced_w, desc.tiled_weight = L.ptr(cm), L.ptr(junk), L.ptr(junk), L.ptr(junk)
    nws = lib.quik_layer_workspace_bytes(ctypes.byref(desc), M)
    ws = torch.zeros(nws, dtype=torch.uint8, device=DEV)
    out = torch.full((M, 64), 7.0, dtype=torch.float16, device=DEV)
    rc = lib.quik_layer_forward(ctypes.byref(desc), L.ptr(xt), M, L.ptr(ws), nws, None, 0, L.ptr(out), None, L.stream())
    torch.cuda.synchronize()
    assert rc == ERR_COLMAP and bool((out == 7.0).all())
