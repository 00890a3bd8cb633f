"""Pins the CPU oracle (oracle/quik_oracle.py) before anything is compared with it.

The reference holds no stored golden vectors for this path; its tests are formulas
evaluated at run time (test/python/test_quant.py, test_matmul.py, test_cuaprseLt.py).
Each check below is either one of those formulas evaluated with an independent routine
(torch CPU half arithmetic, integer matmul), a closed-form known answer, an invariant of
the mathematics, or the independently written scalar C restatement.
"""
import numpy as np
import pytest
import torch

from oracle import quik_oracle as qo


def _rng(seed=0):
    return np.random.default_rng(seed)


def _x_with_outliers(rng, M, n_in, fp_idx, heavy=False):
    x = rng.standard_normal((M, n_in)).astype(np.float32)
    if heavy:
        x[:, fp_idx] = np.clip(20 * rng.standard_t(3, (M, len(fp_idx))), -6e4, 6e4)
    else:
        x[:, fp_idx] *= 50
    return x.astype(np.float16)


def _split(rng, n_in, F):
    fp_idx = rng.permutation(n_in)[:F].astype(np.int64)
    mask = np.ones(n_in, bool)
    mask[fp_idx] = False
    return np.arange(n_in, dtype=np.int64)[mask], fp_idx


# ----------------------------------------------------------------------------- packing
def test_pack_known_bytes_and_roundtrip():
    # element 0 in the low nibble, two's complement nibbles (qlinear.py:11-18)
    assert qo.pack_i4(np.array([[-8, 7]])).tolist() == [[0x78]]
    assert qo.pack_i4(np.array([[1, -1, 0, -8]])).tolist() == [[0xF1, 0x80]]
    allb = np.arange(256, dtype=np.uint8).reshape(1, 256)
    assert np.array_equal(qo.pack_i4(qo.unpack_i4(allb)), allb)
    u = qo.unpack_i4(allb)
    assert u.min() == -8 and u.max() == 7
    # torch restatement of the reference's pack_to_i4 expression on the same data
    X = torch.from_numpy(u.astype(np.int8))
    tc = torch.where(X < 0, 2 ** 4 + X, X).to(torch.uint8)
    ref = (tc[:, 0::2] | (tc[:, 1::2] << 4)).numpy()
    assert np.array_equal(ref, allb)


# ----------------------------------------------------------------------------- asym quantize KATs
def test_asym_quantize_known_answers():
    K = 16
    ii = np.arange(K)
    fi = np.array([], dtype=np.int64)
    # ramp 0..15: scale exactly 1, zero 0, codes -8..7
    ramp = np.arange(16, dtype=np.float16).reshape(1, 16)
    dst, meta, _ = qo.asym_quantize(ramp, ii, fi, 4)
    assert meta[0] == 1.0 and meta[1] == 0.0
    assert qo.unpack_i4(dst).tolist() == [list(range(-8, 8))]
    # constant row: scale clamps at 1e-6f -> binary16 subnormal 0x0011; all codes -8
    const = np.full((1, 16), 3.25, np.float16)
    dst, meta, _ = qo.asym_quantize(const, ii, fi, 4)
    assert meta.view(np.uint16)[0] == 0x0011 and meta[1] == np.float16(3.25)
    assert (qo.unpack_i4(dst) == -8).all()
    # ties go to even: (x - 0)/1 with x = .5, 1.5, 2.5, 3.5 -> 0, 2, 2, 4
    row = np.array([[0, 0.5, 1.5, 2.5, 3.5, 15] + [0] * 10], np.float16)
    dst, meta, _ = qo.asym_quantize(row, ii, fi, 4)
    assert meta[0] == 1.0
    assert qo.unpack_i4(dst)[0, :6].tolist() == [-8, -8, -6, -6, -4, 7]
    # 8 bit: ramp 0..255 -> scale 1, codes -128..127
    ramp8 = np.arange(256, dtype=np.float16).reshape(1, 256)
    dst, meta, _ = qo.asym_quantize(ramp8, np.arange(256), fi, 8)
    assert meta[0] == 1.0 and dst.tolist() == [list(range(-128, 128))]
    # NaN is skipped by min/max and quantises to code -8; +inf makes the scale inf
    row = np.array([[np.nan, 0, 15] + [1] * 13], np.float16)
    dst, meta, _ = qo.asym_quantize(row, ii, fi, 4)
    assert meta[0] == 1.0 and meta[1] == 0.0
    assert qo.unpack_i4(dst)[0, :3].tolist() == [-8, -8, 7]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("heavy", [False, True])
def test_asym_quantize_vs_torch_half_formula(bits, heavy):
    """The per-element arithmetic evaluated by torch's CPU half kernels, an independent routine.

    The divide-and-round semantic is the one test/python/test_cuaprseLt.py:21-23 pins
    ((src / scale).round() in torch fp16)."""
    rng = _rng(1)
    M, n_in, F = 33, 512, 32
    ii, fi = _split(rng, n_in, F)
    x = _x_with_outliers(rng, M, n_in, fi, heavy)
    dst, meta, fp_x = qo.asym_quantize(x, ii, fi, bits)
    xt = torch.from_numpy(x)[:, torch.from_numpy(ii)]
    mx, mn = xt.max(1)[0], xt.min(1)[0]
    scale = torch.clamp((mx.float() - mn.float()) / float(2 ** bits - 1), min=1e-6).half()
    assert torch.equal(torch.from_numpy(meta[0::2].copy()), scale)
    assert torch.equal(torch.from_numpy(meta[1::2].copy()), mn)
    d = ((xt - mn[:, None]) / scale[:, None])
    assert d.dtype == torch.float16
    q = torch.clamp(d.round(), 0, 2 ** bits - 1).to(torch.int32) - 2 ** (bits - 1)
    got = qo.unpack_i4(dst) if bits == 4 else dst
    assert np.array_equal(got, q.numpy().astype(np.int8))
    assert np.array_equal(fp_x, x[:, fi])


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("heavy", [False, True])
def test_asym_quantize_bf16_vs_torch_bfloat16_formula(bits, heavy):
    """The bf16 mode of the oracle against torch's CPU bfloat16 kernels, which round every operation to bfloat16
    (the semantic of __hsub / __hdiv on __nv_bfloat16 and of __bfloat162int_rn, include/util.h:45-110;
    dispatch src/asymmetric/asymmetric.cu:531-579): scale, zero and every code bit-equal, edge rows included."""
    rng = _rng(11 + bits)
    M, n_in, F = 40, 512, 32
    ii, fi = _split(rng, n_in, F)
    x32 = _x_with_outliers(rng, M, n_in, fi, heavy).astype(np.float32)
    x32[0, :] = 1.5                                             # constant row: the scale clamps at 1e-6
    x32[1, ii[:8]] = [0, 0.5, 1.5, 2.5, 3.5, 4.5, 15, 7.5]      # exact ties
    x32[2, :] *= 1e-7
    x32[3, ii[3]], x32[3, ii[4]] = 3e38, -3e38                  # the range overflows fp32: scale = inf
    x32[4, ii[5]] = np.inf
    x32[5, ii[6]] = np.nan
    x32[6, :] = 0.0
    xb = torch.from_numpy(x32).to(torch.bfloat16)               # round-to-nearest-even, torch's own conversion
    xs = xb.float().numpy()
    assert np.array_equal(qo.bf16_round(x32)[~np.isnan(x32)], xs[~np.isnan(x32)])
    dst, meta, fp_x = qo.asym_quantize(xs, ii, fi, bits, qo.BF16)
    xi = xb[:, torch.from_numpy(ii)]
    # torch.max / min propagate NaN where __hmax / __hmin skip it: take them over the non-NaN entries
    big = torch.tensor(float("inf"), dtype=torch.bfloat16)
    mx = torch.where(torch.isnan(xi), -big, xi).max(1)[0]
    mn = torch.where(torch.isnan(xi), big, xi).min(1)[0]
    scale = torch.clamp((mx.float() - mn.float()) / float(2 ** bits - 1), min=1e-6).to(torch.bfloat16)
    got_scale = torch.from_numpy(meta[0::2].copy()).to(torch.bfloat16)
    got_zero = torch.from_numpy(meta[1::2].copy()).to(torch.bfloat16)
    assert torch.equal(got_scale.view(torch.int16), scale.view(torch.int16))
    assert torch.equal(got_zero.view(torch.int16), mn.view(torch.int16))
    assert np.array_equal(meta[0::2], scale.float().numpy())   # the oracle's meta is exactly bf16-representable
    d = xi - mn[:, None]
    assert d.dtype == torch.bfloat16
    t = d / scale[:, None]
    assert t.dtype == torch.bfloat16
    r = torch.nan_to_num(t.float().round(), nan=0.0, posinf=2.0 ** 31, neginf=-2.0 ** 31)   # NaN -> 0, as the intrinsic
    q = torch.clamp(r, 0, 2 ** bits - 1).to(torch.int32) - 2 ** (bits - 1)
    got = qo.unpack_i4(dst) if bits == 4 else dst
    assert np.array_equal(got, q.numpy().astype(np.int8))
    assert np.array_equal(fp_x, xs[:, fi])


@pytest.mark.parametrize("bits", [4, 8])
def test_asym_dequantize_bf16_vs_torch(bits):
    """asym_dequantize in bf16 mode: fp32 arithmetic in the reference's association order (asymmetric.cu:134-163)
    evaluated by torch fp32 ops on bfloat16-stored inputs, one rounding to bfloat16 by torch's conversion."""
    rng = _rng(17 + bits)
    M, N = 24, 40
    acc = rng.integers(-3_000_000, 3_000_000, (M, N)).astype(np.int32)
    acc[0, :4] = [0, 1, -1, 2 ** 24 + 1]
    bf = lambda a: torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16)
    meta = bf(np.stack([rng.uniform(1e-3, 0.2, M), rng.standard_normal(M)], 1).reshape(-1))
    s_col = bf(rng.uniform(1e-3, 1e-2, N))
    w_red = bf(rng.standard_normal(N) * 3)
    y = bf(rng.standard_normal((M, N)))
    got = qo.asym_dequantize(acc, meta.float().numpy(), s_col.float().numpy(), w_red.float().numpy(),
                             y.float().numpy(), bits, qo.BF16)
    s, z = meta.float()[0::2][:, None], meta.float()[1::2][:, None]
    shift = 8.0 if bits == 4 else 128.0
    t = torch.from_numpy(acc).float() * (s * s_col.float()[None, :])
    t = t + ((z + shift * s) * w_red.float()[None, :] + y.float())
    want = t.to(torch.bfloat16)
    assert np.array_equal(qo.f32_to_bf16_bits(got), want.view(torch.int16).numpy().view(np.uint16))


@pytest.mark.parametrize("bits", [4, 8])
def test_asym_quantize_invariants(bits):
    """test/python/test_quant.py: meta vs torch to 3 places; indexed == gather-then-quantise;
    plus: row minimum -> lowest code, row maximum -> highest code when the scale is not
    clamped; codes are monotone in x; dequantised codes lie within scale/2 (+fp16 slack) of x."""
    rng = _rng(2)
    M, n_in, F = 16, 1024, 64
    ii, fi = _split(rng, n_in, F)
    x = rng.random((M, n_in)).astype(np.float16)
    dst, meta, fp_x = qo.asym_quantize(x, ii, fi, bits)
    xi = x[:, ii].astype(np.float32)
    unit = np.maximum((xi.max(1) - xi.min(1)) / (2 ** bits - 1), 1e-6)
    assert np.abs(meta[0::2].astype(np.float32) - unit).max() < 1e-3
    assert np.abs(meta[1::2].astype(np.float32) - xi.min(1)).max() == 0
    q = (qo.unpack_i4(dst) if bits == 4 else dst).astype(np.int32)
    # gather-then-quantise with the found meta (quantizeOld) gives the same codes
    q2 = qo.quantize_old(x[:, ii], qo.find_meta(x[:, ii], bits), bits)
    assert np.array_equal(q2, dst)
    lo, hi = -(2 ** (bits - 1)), 2 ** (bits - 1) - 1
    r = np.arange(M)
    assert (q[r, xi.argmin(1)] == lo).all() and (q[r, xi.argmax(1)] == hi).all()
    order = np.argsort(xi, axis=1, kind="stable")
    assert (np.diff(np.take_along_axis(q, order, 1), axis=1) >= 0).all()
    s = meta[0::2].astype(np.float64)[:, None]
    z = meta[1::2].astype(np.float64)[:, None]
    recon = s * (q - lo) + z
    assert (np.abs(recon - xi) <= 0.5 * s * 1.02 + 1e-3).all()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("is_bf16", [False, True])
def test_asym_quantize_numpy_vs_c(bits, is_bf16, c_oracle):
    rng = _rng(3 + bits + is_bf16)
    M, n_in, F = 40, 384, 32
    ii, fi = _split(rng, n_in, F)
    ii = rng.permutation(ii)  # any order is allowed by the op
    x32 = rng.standard_normal((M, n_in)).astype(np.float32)
    x32[:, fi] *= 50
    x32[0, :] = 1.5          # constant row
    x32[1, ii[:8]] = [0, 0.5, 1.5, 2.5, 3.5, 4.5, 15, 7.5]
    x32[2, :] *= 1e-7        # subnormal range in fp16
    x32[3, ii[3]] = 6e4      # large dynamic range
    if is_bf16:
        xs = qo.bf16_round(x32)
        bits_in = qo.f32_to_bf16_bits(xs)
        dst, meta, fp_x = qo.asym_quantize(xs, ii, fi, bits, qo.BF16)
        meta_bits, fp_bits = qo.f32_to_bf16_bits(meta), qo.f32_to_bf16_bits(fp_x)
    else:
        xs = x32.astype(np.float16)
        bits_in = xs.view(np.uint16)
        dst, meta, fp_x = qo.asym_quantize(xs, ii, fi, bits, qo.F16)
        meta_bits, fp_bits = meta.view(np.uint16), fp_x.view(np.uint16)
    cd, cm, cf = c_oracle.asym_quantize(bits_in, ii, fi, bits, is_bf16)
    assert np.array_equal(cm, meta_bits)
    assert np.array_equal(cd, dst)
    assert np.array_equal(cf, fp_bits)


def test_half_conversions_exhaustive(c_oracle):
    lib = c_oracle.lib()
    allh = np.arange(65536, dtype=np.uint16)
    f = allh.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 7):
        v = lib.qo_half_to_float(h)
        if np.isnan(f[h]):
            assert np.isnan(v)
        else:
            assert v == f[h]
            assert lib.qo_double_to_half(float(f[h])) == h
    rng = _rng(5)
    d = np.concatenate([rng.standard_normal(2000) * s for s in (1e-7, 1e-4, 1, 300, 7e4)])
    mid = (f[0x3C00:0x3C10].astype(np.float64) + f[0x3C01:0x3C11]) / 2  # exact ties
    d = np.concatenate([d, mid, [65519.99, 65520.0, 2 ** -25, 2 ** -24 * 1.5]])
    with np.errstate(over="ignore"):
        want = d.astype(np.float16).view(np.uint16)
    got = np.array([lib.qo_double_to_half(float(v)) for v in d], dtype=np.uint16)
    assert np.array_equal(got, want)
    f32 = (rng.standard_normal(3000) * 10).astype(np.float32)
    want = torch.from_numpy(f32).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(np.array([lib.qo_float_to_bf16(float(v)) for v in f32], np.uint16), want)
    assert np.array_equal(qo.f32_to_bf16_bits(qo.bf16_round(f32)), want)


# ----------------------------------------------------------------------------- integer GEMM
def test_int_matmul_exact(c_oracle):
    rng = _rng(6)
    M, N, K = 7, 5, 64
    a = rng.integers(-8, 8, (M, K)).astype(np.int8)
    b = rng.integers(-8, 8, (N, K)).astype(np.int8)
    brute = np.array([[sum(int(a[m, k]) * int(b[n, k]) for k in range(K)) for n in range(N)] for m in range(M)])
    got = qo.int4_matmul(qo.pack_i4(a), qo.pack_i4(b))
    assert got.dtype == np.int32 and np.array_equal(got, brute)
    assert np.array_equal(c_oracle.int4_matmul(qo.pack_i4(a), qo.pack_i4(b)), brute)
    # the reference's own definition (test/python/test_matmul.py:20-26): float bmm, round, int32
    ta, tb = torch.from_numpy(a), torch.from_numpy(b)
    ref = torch.matmul(ta.float(), tb.float().T).round().to(torch.int32).numpy()
    assert np.array_equal(got, ref)
    a8 = rng.integers(-128, 128, (M, 96)).astype(np.int8)
    b8 = rng.integers(-128, 128, (N, 96)).astype(np.int8)
    ref8 = (torch.from_numpy(a8).long() @ torch.from_numpy(b8).long().T).numpy()
    assert np.array_equal(qo.int8_matmul(a8, b8), ref8)
    assert np.array_equal(c_oracle.int8_matmul(a8, b8), ref8)
    # extreme operands at a long K stay exact
    ext = np.full((2, 28416), -128, np.int8)
    assert (qo.int8_matmul(ext, ext) == 128 * 128 * 28416).all()


# ----------------------------------------------------------------------------- asym dequantize
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("is_bf16", [False, True])
def test_asym_dequantize(bits, is_bf16, c_oracle):
    rng = _rng(7)
    M, N = 24, 40
    dt = qo.BF16 if is_bf16 else qo.F16
    rnd = (lambda v: qo.bf16_round(v.astype(np.float32))) if is_bf16 else (lambda v: v.astype(np.float16))
    acc = rng.integers(-60000, 60000, (M, N)).astype(np.int32)
    meta = rnd(np.stack([rng.uniform(0.01, 0.3, M), rng.uniform(-3, 0, M)], 1).reshape(-1))
    scol = rnd(rng.uniform(0.001, 0.01, (N, 1)))
    wred = rnd(rng.standard_normal((1, N)))
    y = rnd(rng.standard_normal((M, N)) * 3)
    out = qo.asym_dequantize(acc, meta, scol, wred, y, bits, dt)
    ref = qo.asym_dequantize_f64(acc, meta, scol, wred, y, bits, dt)
    o64 = out.astype(np.float64)
    ulp = np.maximum(np.abs(ref), 2.0 ** -14) * (2.0 ** -7 if is_bf16 else 2.0 ** -10)
    assert (np.abs(o64 - ref) <= ulp).all()
    # zero accumulators and zero y leave exactly the zero-point correction term
    z = np.zeros_like(acc)
    zy = rnd(np.zeros((M, N)))
    o2 = qo.asym_dequantize(z, meta, scol, wred, zy, bits, dt).astype(np.float64)
    m64 = meta.astype(np.float64)
    corr = (m64[1::2, None] + (8 if bits == 4 else 128) * m64[0::2, None]) * wred.astype(np.float64)
    assert (np.abs(o2 - corr) <= np.maximum(np.abs(corr), 2.0 ** -14) * (2.0 ** -7 if is_bf16 else 2.0 ** -10)).all()
    # independent scalar C restatement, same association order: bit-equal
    tob = qo.f32_to_bf16_bits if is_bf16 else (lambda v: v.view(np.uint16))
    cb = c_oracle.asym_dequantize(acc, tob(meta), tob(scol), tob(wred), tob(y), bits, is_bf16)
    assert np.array_equal(cb, tob(out))


# ----------------------------------------------------------------------------- symmetric
@pytest.mark.parametrize("bits", [4, 8])
def test_sym_quantize_vs_reference_formula(bits, c_oracle):
    """test/python/test_cuaprseLt.py:21-23: qb == (src / scale).round().to(int8) in torch fp16."""
    torch.manual_seed(1)
    N, K = 48, 130 if bits == 8 else 128
    src = torch.randn(N, K, dtype=torch.float16)
    scale = torch.randn(N, 1, dtype=torch.float16)
    if bits == 4:
        scale = scale.abs() + 0.5
    q = qo.sym_quantize(src.numpy(), scale.numpy(), bits)
    ref = (src / scale).round()
    if bits == 8:
        # restrict the comparison to in-range quotients; out-of-range wraps (C conversion)
        ok = (ref.abs() <= 127).numpy()
        assert ok.mean() > 0.9
        assert np.array_equal(q[ok], ref.to(torch.int8).numpy()[ok])
        wrapped = (ref.float().numpy().astype(np.int64) & 0xFF).astype(np.uint8).view(np.int8)
        fin = np.isfinite(ref.float().numpy())
        assert np.array_equal(q[fin], wrapped[fin])
    else:
        codes = ref.to(torch.int32).numpy()
        assert np.array_equal(qo.unpack_i4(q).astype(np.int32) & 0xF, codes & 0xF)
    cq = c_oracle.sym_quantize(src.numpy().view(np.uint16), scale.numpy().view(np.uint16), bits)
    assert np.array_equal(cq, q)


def test_sym_quantize_odd_columns_and_scale():
    x = np.array([[1.0, -2.0, 3.0]], np.float16)
    q = qo.sym_quantize(x, np.array([[1.0]], np.float16), 4)
    assert q.shape == (1, 2) and q.tolist() == [[0xE1, 0x03]]
    # experiments/qlinear.py:101-102: divisor is 1 << ((bits-1)-1) = 4 for bits=4
    assert qo.sym_act_scale(np.array([[2.0, -8.0]], np.float16), 4).tolist() == [[2.0]]


@pytest.mark.parametrize("bits", [8, 16, 32])
def test_sym_dequantize_vs_reference_formula(bits, c_oracle):
    """test/python/test_cuaprseLt.py:45-47: c * scale_row * scale_col + y evaluated in torch fp16."""
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
        c = torch.randint(-70000, 70000, (M, N), dtype=torch.int32)  # beyond 65504: overflows to inf
        ch = c.half()
    ref = ch * sr * sc + y
    out = qo.sym_dequantize(c.numpy(), sr.numpy(), sc.numpy(), y.numpy(), bits)
    assert np.array_equal(out.view(np.uint16), ref.numpy().view(np.uint16))
    cx = c.numpy().view(np.uint16) if bits == 16 else c.numpy()
    co = c_oracle.sym_dequantize(cx, bits, sr.numpy().view(np.uint16), sc.numpy().view(np.uint16),
                                 y.numpy().view(np.uint16))
    fin = np.isfinite(out)
    assert np.array_equal(co[fin], out.view(np.uint16)[fin])
    assert (np.isnan(out[~fin]) == np.isnan(co[~fin].view(np.float16))).all()


# ----------------------------------------------------------------------------- MixedQLinear
def _layer(rng, N, n_in, F, bits):
    ii, fi = _split(rng, n_in, F)
    lo, hi = (-8, 8) if bits == 4 else (-127, 128)
    codes = rng.integers(lo, hi, (N, n_in - F))
    s_w = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    W = np.zeros((N, n_in), np.float16)
    W[:, ii] = (codes * s_w.astype(np.float32)).astype(np.float16)
    W[:, fi] = (0.02 * rng.standard_normal((N, F))).astype(np.float16)
    return W, s_w, codes, ii, fi


@pytest.mark.parametrize("bits", [4, 8])
def test_from_float_roundtrip(bits):
    rng = _rng(8)
    N, n_in, F = 48, 256, 32
    W, s_w, codes, ii, fi = _layer(rng, N, n_in, F, bits)
    mod = qo.from_float(W, s_w, fi, bits)
    got = qo.unpack_i4(mod["int_weight"]) if bits == 4 else mod["int_weight"]
    # fp16(code*s)/s rounds back to the code (|code| <= 127 needs < 2^-8 relative error)
    assert np.array_equal(got, codes.astype(np.int8))
    assert np.array_equal(mod["int_indices"], ii)
    assert np.array_equal(mod["fp_weight"], W[:, fi])
    red = W[:, ii].astype(np.float32).sum(1, dtype=np.float32).astype(np.float16)
    assert np.array_equal(mod["reduced_w"], red.reshape(1, N))
    # torch restatement of qlinear.py:178-186 on the same data
    Wt = torch.from_numpy(W)
    r = (Wt[:, torch.from_numpy(ii)] / torch.from_numpy(s_w)).round().to(torch.int8).numpy()
    assert np.array_equal(r, got)


@pytest.mark.parametrize("bits,heavy", [(4, False), (4, True), (8, False)])
def test_mixed_forward_identity(bits, heavy):
    """out ~= x_deq W^T with x_deq = s(q + 2^(b-1)) + zero on int columns, x on outliers (float64);
    tolerance: max abs error <= 1e-2 * output RMS."""
    rng = _rng(9)
    M, N, n_in, F = 32, 64, 512, 32
    W, s_w, codes, ii, fi = _layer(rng, N, n_in, F, bits)
    x = _x_with_outliers(rng, M, n_in, fi, heavy)
    mod = qo.from_float(W, s_w, fi, bits)
    out, inter = qo.mixed_qlinear_forward(x, mod, bits)
    xd = qo.dequantized_activation_f64(x, ii, fi, bits)
    ref = xd @ W.astype(np.float64).T
    rms = np.sqrt((ref ** 2).mean())
    assert np.abs(out.astype(np.float64) - ref).max() <= 1e-2 * rms
    # and the quantised layer approximates the float layer to quantisation noise
    full = x.astype(np.float64) @ W.astype(np.float64).T
    rel = np.sqrt(((ref - full) ** 2).mean()) / np.sqrt((full ** 2).mean())
    assert rel < (0.5 if bits == 4 else 0.05)


def test_sim_path_agrees_to_quantisation_noise():
    from oracle import sim_path
    rng = _rng(10)
    M, N, n_in, F = 32, 64, 512, 32
    W, s_w, codes, ii, fi = _layer(rng, N, n_in, F, 4)
    x = _x_with_outliers(rng, M, n_in, fi)
    mod = qo.from_float(W, s_w, fi, 4)
    out, _ = qo.mixed_qlinear_forward(x, mod, 4)
    sim = sim_path.sim_mixed_linear(torch.from_numpy(x), torch.from_numpy(W), torch.from_numpy(ii),
                                    torch.from_numpy(fi), 4).float().numpy()
    full = x.astype(np.float64) @ W.astype(np.float64).T
    e_sim = np.sqrt(((sim - full) ** 2).mean())
    e_ker = np.sqrt(((out.astype(np.float64) - full) ** 2).mean())
    assert 0.5 < e_sim / e_ker < 2.0
    # closed-form check of the sim quantiser on one row: grid contains zero exactly
    q = sim_path.act_fake_quant(torch.tensor([[-1.0, 0.0, 0.4, 2.0]]), 4)
    scale = 3.0 / 15
    assert torch.allclose(q, torch.tensor([[-1.0, 0.0, 0.4, 2.0]]), atol=scale / 2 + 1e-6)
    assert q[0, 1] == 0 and abs(q[0, 0] + 1.0) < 1e-6


def test_sim_quantiser_on_half_input_is_a_float32_evaluation():
    """The reference's fake-quant runs on half tensors, but not in half arithmetic: find_params compares the row
    minima with `torch.zeros(rows)`, a float32 tensor (experiments/quant_sim.py:178-180), so xmin, xmax, scale and
    zero are float32 by type promotion, and `x / scale` in asymmetric_quantize (:5-7) promotes the half input as
    well; the only rounding to half is the `.to(x_dtype)` of ActQuantWrapper.forward (:248).  The op sequence is
    spelled out here on a half input, dtype for dtype, and must equal the oracle's float32 evaluation rounded
    once, bit for bit (edge rows: all zero, all positive, all negative, ties at .5 of the grid)."""
    from oracle import sim_path
    g = torch.Generator().manual_seed(3)
    for bits in (4, 8):
        x = (torch.randn(64, 256, generator=g) * 3).half()
        x[0] = 0
        x[1] = x[1].abs() + 1
        x[2] = -x[2].abs() - 1
        x[3, :16] = torch.arange(16).half() * 0.5          # scale 0.5 for 4 bits: every second value is a tie
        x[3, 16:] = 0
        x[3, 16] = 7.5
        maxq = torch.tensor(2 ** bits - 1)
        tmp = torch.zeros(x.shape[0])                       # float32, as in the reference
        xmin = torch.minimum(x.min(1)[0], tmp)
        xmax = torch.maximum(x.max(1)[0], tmp)
        assert xmin.dtype == torch.float32
        both = (xmin == 0) & (xmax == 0)
        xmin[both] = -1
        xmax[both] = +1
        scale = (xmax - xmin) / maxq
        zero = torch.round(-xmin / scale)
        scale = scale.unsqueeze(1).repeat(1, x.shape[-1]).reshape(x.shape)
        zero = zero.unsqueeze(1).repeat(1, x.shape[-1]).reshape(x.shape)
        q = torch.clamp(torch.round(x / scale) + zero, 0, maxq)
        assert q.dtype == torch.float32
        literal = (scale * (q - zero)).to(x.dtype)
        ours = sim_path.act_fake_quant(x.float(), bits).to(x.dtype)
        assert torch.equal(literal.view(torch.int16), ours.view(torch.int16))


# ---------------------------------------------------------------------------- fused dequantize ops
@pytest.mark.parametrize("spread", [3, 8, 128])
def test_fused_dequantize_epilogues_vs_reference_known_answer_formula(spread):
    """The reference pins its fused GEMM + dequantize ops by evaluating the formula with torch tensor
    arithmetic (test/python/test_fused.py:33-37 symmetric, :56-62 asymmetric): int32 times fp16 tensors
    promote to fp16 and every operation rounds to fp16.  The same expressions, evaluated here by torch
    on the CPU, must equal the oracle bit for bit; `spread` widens the operands beyond the reference's
    randint(-3, 3) so that the int32 -> fp16 conversion rounds (|acc| > 2048) and overflows."""
    g = torch.Generator().manual_seed(spread)
    M, N, K = 48, 80, 256
    a = torch.randint(-spread, spread, (M, K), generator=g, dtype=torch.int32)
    b = torch.randint(-spread, spread, (N, K), generator=g, dtype=torch.int32)
    c_ref = a @ b.t()
    scale_row = torch.rand(M, 1, generator=g).half()
    scale_col = torch.rand(1, N, generator=g).half()
    zero_row = torch.rand(M, 1, generator=g).half()
    w_reduce = torch.rand(1, N, generator=g).half()
    y = torch.rand(M, N, generator=g).half()
    shift_value = 0.7371
    want_sym = c_ref * scale_row * scale_col + y
    want_asym = c_ref * scale_col * scale_row + \
        (zero_row + torch.tensor([shift_value], dtype=torch.float16).item() * scale_row) * w_reduce + y
    assert want_sym.dtype == torch.float16 and want_asym.dtype == torch.float16
    got_sym = qo.sym_dequantize(c_ref.numpy(), scale_row.numpy(), scale_col.numpy(), y.numpy(), 32)
    got_asym = qo.asym_fused_dequantize(c_ref.numpy(), scale_row.numpy(), scale_col.numpy(), shift_value,
                                        zero_row.numpy(), w_reduce.numpy(), y.numpy())
    assert np.array_equal(got_sym.view(np.uint16), want_sym.numpy().view(np.uint16))
    assert np.array_equal(got_asym.view(np.uint16), want_asym.numpy().view(np.uint16))
    if spread == 128:
        assert np.isinf(got_asym).any()       # the overflow case is really exercised
