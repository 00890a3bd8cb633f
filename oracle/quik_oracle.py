"""CPU oracle for the QUIK MixedQLinear forward path (numpy).

TEST INFRASTRUCTURE ONLY.  This module restates, on the CPU, the arithmetic of the
reference's CUDA kernels so that the HIP kernels can be checked against it.  It is
imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg,
and by nothing else: the shipped library never routes through it.

Every function cites the reference source it follows (paths relative to the
reference checkout).  "fp16 op" means: evaluate in >= fp32 and round the result to
IEEE binary16, ties to even.  numpy float16 arithmetic does exactly that per
operation; for + - * / an fp32 intermediate makes the second rounding innocuous
because 24 >= 2*11 + 2.  bfloat16 values are carried as float32 arrays whose low
16 mantissa bits are zero; `bf16_round` performs the ties-to-even rounding.

How each function is pinned (none is "parity unpinned"):
  pack_i4 / unpack_i4      closed form + exhaustive round trip over all 256 bytes
  asym_quantize            known-answer rows (constant row, 15-step ramp, ties),
                           invariants from test/python/test_quant.py, an
                           independent scalar C restatement (oracle/quik_oracle.c)
  int_matmul               exact integers; brute force triple loop on tiny cases,
                           definition from test/python/test_matmul.py:16-26
  asym_dequantize          fp64 evaluation within 1 output ulp, zero-acc identity
  sym_quantize             test/python/test_cuaprseLt.py:21-23 (torch fp16 divide)
  sym_dequantize           test/python/test_cuaprseLt.py:45-47 (torch fp16 chain)
  from_float               exact code*scale round trip (experiments/qlinear.py)
  mixed_qlinear_forward    algebraic identity against a float64 linear layer
The outlier GEMM (torch.nn.functional.linear in experiments/qlinear.py:124) has no
defined summation order in the reference; it is compared with a tolerance only.
"""
from __future__ import annotations

import numpy as np

F16 = "f16"
BF16 = "bf16"


# --------------------------------------------------------------------------- #
# storage-type helpers
# --------------------------------------------------------------------------- #
def bf16_round(x):
    """float32 -> nearest bfloat16 (ties to even), returned as float32.

    Mirrors __float2bfloat16_rn (include/util.h:84-87): NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    r = r.astype(np.uint32)
    nan = np.isnan(x)
    out = r.view(np.float32).copy()
    out[nan] = np.nan
    return out.reshape(x.shape)


def bf16_bits_to_f32(bits):
    """uint16 bfloat16 bit patterns -> float32 values."""
    b = np.ascontiguousarray(bits).view(np.uint16).astype(np.uint32) << 16
    return b.view(np.float32)


def f32_to_bf16_bits(x):
    """float32 values that are bfloat16-representable -> uint16 bit patterns."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (x.view(np.uint32) >> 16).astype(np.uint16)


def _round_to(x32, dtype):
    """Round float32 to the storage type; result as float16 array or bf16-in-f32."""
    if dtype == F16:
        with np.errstate(over="ignore"):
            return np.asarray(x32, dtype=np.float32).astype(np.float16)
    return bf16_round(x32)


def _as_f32(x, dtype):
    if dtype == F16:
        return np.asarray(x, dtype=np.float16).astype(np.float32)
    return np.asarray(x, dtype=np.float32)


def _rne_to_int(d32):
    """__half2int_rn / __bfloat162int_rn (include/util.h:45-58): round to nearest
    even, NaN -> 0, +-inf saturate."""
    d = np.asarray(d32, dtype=np.float64)
    r = np.rint(d)
    r = np.where(np.isnan(r), 0.0, r)
    r = np.clip(r, -2147483648.0, 2147483647.0)
    return r.astype(np.int64)


# --------------------------------------------------------------------------- #
# int4 packing (experiments/qlinear.py:11-18, include/int4.h:78-98)
# --------------------------------------------------------------------------- #
def pack_i4(q):
    """Signed codes in [-8,7], shape [R, K] with K even -> uint8 [R, K/2].

    Element k lives in byte k//2; even k in the low nibble (qlinear.py:15-18)."""
    q = np.asarray(q)
    assert q.shape[-1] % 2 == 0
    u = (q.astype(np.int16) & 0xF).astype(np.uint8)
    return (u[..., 0::2] | (u[..., 1::2] << 4)).astype(np.uint8)


def unpack_i4(p):
    """Inverse of pack_i4: uint8 [R, K/2] -> int8 [R, K] sign-extended."""
    p = np.asarray(p, dtype=np.uint8)
    lo = (p & 0xF).astype(np.int8)
    hi = (p >> 4).astype(np.int8)
    lo = np.where(lo >= 8, lo - 16, lo).astype(np.int8)
    hi = np.where(hi >= 8, hi - 16, hi).astype(np.int8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.int8)
    out[..., 0::2] = lo
    out[..., 1::2] = hi
    return out


# --------------------------------------------------------------------------- #
# asymmetric per-token quantisation
# --------------------------------------------------------------------------- #
def find_meta_rows(xi, bits, dtype=F16):
    """Per-row (scale, zero) over the columns of `xi`.

    src/asymmetric/asymmetric.cu:340-381 (FindMetaParallelIndexed) and :263-301:
    max / min with __hmax / __hmin (NaN operands are skipped), then
    scale = float2type(fmaxf((max_f - min_f) / divisor, 1e-6)), zero = min."""
    x32 = _as_f32(xi, dtype)
    with np.errstate(invalid="ignore", over="ignore"):
        mx = np.fmax.reduce(x32, axis=1)
        mn = np.fmin.reduce(x32, axis=1)
        div = np.float32((1 << bits) - 1)
        s32 = np.fmax((mx - mn).astype(np.float32) / div, np.float32(1e-6)).astype(np.float32)
    scale = _round_to(s32, dtype)
    zero = _round_to(mn, dtype)  # exact: mn is already a storage-type value
    return scale, zero


def quantize_codes_with_meta(xi, scale, zero, bits, dtype=F16):
    """Codes for already-gathered columns with given per-row meta.

    src/asymmetric/asymmetric.cu:33-39, 392-398, 424-429:
    data = hdiv(hsub(x, zero), scale); val = type2int_rn(data);
    val = min(max(val, 0), 2^bits - 1) - 2^(bits-1)."""
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        if dtype == F16:
            x = np.asarray(xi, dtype=np.float16)
            d = (x - np.asarray(zero, np.float16)[:, None]).astype(np.float16)
            d = (d / np.asarray(scale, np.float16)[:, None]).astype(np.float16)
            d32 = d.astype(np.float32)
        else:
            x = np.asarray(xi, dtype=np.float32)
            d = bf16_round(x - np.asarray(zero, np.float32)[:, None])
            d32 = bf16_round(d / np.asarray(scale, np.float32)[:, None])
    v = _rne_to_int(d32)
    hi = (1 << bits) - 1
    q = np.clip(v, 0, hi) - (1 << (bits - 1))
    return q.astype(np.int8)


def _interleave_meta(scale, zero, dtype):
    m = np.empty(2 * scale.shape[0], dtype=np.float16 if dtype == F16 else np.float32)
    m[0::2] = scale
    m[1::2] = zero
    return m


def asym_quantize(x, int_indices, fp_indices, bits, dtype=F16):
    """quik.asymmetric.quantize: returns (dst, meta, fp_x).

    src/asymmetric/asymmetric.cu:448-490 (kernel), :492-584 (host):
    dst is uint8 [M, K/2] nibble-packed for bits=4 or int8 [M, K] for bits=8,
    meta is [2M] interleaved (scale, zero), fp_x[r, j] = x[r, fp_indices[j]]."""
    int_indices = np.asarray(int_indices, dtype=np.int64)
    fp_indices = np.asarray(fp_indices, dtype=np.int64)
    assert bits in (4, 8)
    assert x.shape[1] == int_indices.size + fp_indices.size  # asymmetric.cu:519-521
    assert int_indices.size % 2 == 0                          # asymmetric.cu:522-524
    xs = np.asarray(x, dtype=np.float16) if dtype == F16 else np.asarray(x, dtype=np.float32)
    xi = xs[:, int_indices]
    scale, zero = find_meta_rows(xi, bits, dtype)
    q = quantize_codes_with_meta(xi, scale, zero, bits, dtype)
    dst = pack_i4(q) if bits == 4 else q
    meta = _interleave_meta(scale, zero, dtype)
    fp_x = xs[:, fp_indices].copy()
    return dst, meta, fp_x


def find_meta(x, bits):
    """quik.asymmetric.find_meta (fp16 only, all columns).

    src/asymmetric/asymmetric.cu:263-338."""
    scale, zero = find_meta_rows(np.asarray(x, np.float16), bits, F16)
    return _interleave_meta(scale, zero, F16)


def quantize_old(x, meta, bits):
    """quik.asymmetric.quantizeOld (fp16 only): quantise every column with given meta.

    src/asymmetric/asymmetric.cu:13-117.  For bits=4 an odd column count leaves the
    high nibble of the last byte of a row zero (colsDst = ceil(cols/2), :97); the
    4-bit kernel indexes the source as idx*2+i over the flattened array (:25-43),
    which equals row-wise packing only when the column count is even."""
    x = np.asarray(x, np.float16)
    meta = np.asarray(meta, np.float16)
    assert meta.size == 2 * x.shape[0]                         # asymmetric.cu:71-72
    q = quantize_codes_with_meta(x, meta[0::2], meta[1::2], bits, F16)
    if bits == 8:
        return q
    assert x.shape[1] % 2 == 0, "oracle restates the even-column case only"
    return pack_i4(q)


# --------------------------------------------------------------------------- #
# integer GEMM (src/matmul/matmul.cu:17-55, 98-136)
# --------------------------------------------------------------------------- #
def int_matmul(a_codes, b_codes):
    """C[m, n] = sum_k a[m, k] * b[n, k], exact, int32.

    float64 BLAS is exact here: every partial sum is an integer below 2^53."""
    a = np.asarray(a_codes, dtype=np.float64)
    b = np.asarray(b_codes, dtype=np.float64)
    c = a @ b.T
    assert np.all(np.abs(c) < 2 ** 31)
    return c.astype(np.int64).astype(np.int32)


def int4_matmul(a_packed, b_packed):
    """quik.matmul.int4Matmul on nibble-packed operands (matmul.cu:17-55)."""
    return int_matmul(unpack_i4(a_packed), unpack_i4(b_packed))


def int8_matmul(a, b):
    """quik.matmul.int8Matmul (matmul.cu:98-136)."""
    return int_matmul(np.asarray(a, np.int8), np.asarray(b, np.int8))


# --------------------------------------------------------------------------- #
# asymmetric dequantise (src/asymmetric/asymmetric.cu:119-173, 175-233)
# --------------------------------------------------------------------------- #
def asym_dequantize(acc, meta, scale_col, w_reduced, y, bits, dtype=F16):
    """out = storage( f32(acc) * (s_row * s_col) + ((zero + shift * s_row) * w_red + y) ).

    All fp32, in the reference's association order (asymmetric.cu:138-146); nvcc may
    contract the multiply-adds, so the last fp32 ulp is not defined by the source."""
    acc = np.asarray(acc, dtype=np.int32)
    m32 = _as_f32(meta, dtype)
    s = m32[0::2][:, None]
    z = m32[1::2][:, None]
    c = _as_f32(scale_col, dtype).reshape(1, -1)
    w = _as_f32(w_reduced, dtype).reshape(1, -1)
    y32 = _as_f32(y, dtype)
    shift_value = np.float32(8.0 if bits == 4 else 128.0)
    with np.errstate(over="ignore", invalid="ignore"):
        t = acc.astype(np.float32)
        shift = ((z + shift_value * s).astype(np.float32) * w).astype(np.float32)
        t = (t * (s * c).astype(np.float32)).astype(np.float32)
        t = (t + (shift + y32).astype(np.float32)).astype(np.float32)
    return _round_to(t, dtype)


def asym_dequantize_f64(acc, meta, scale_col, w_reduced, y, bits, dtype=F16):
    """Same formula in float64, unrounded: the yardstick for tolerance checks."""
    m = _as_f32(meta, dtype).astype(np.float64)
    s = m[0::2][:, None]
    z = m[1::2][:, None]
    c = _as_f32(scale_col, dtype).astype(np.float64).reshape(1, -1)
    w = _as_f32(w_reduced, dtype).astype(np.float64).reshape(1, -1)
    shift_value = 8.0 if bits == 4 else 128.0
    return np.asarray(acc, np.float64) * (s * c) + (z + shift_value * s) * w + _as_f32(y, dtype).astype(np.float64)


def asym_fused_dequantize(acc, scale_row, scale_col, shift_value, zero_row, w_reduced, y):
    """Epilogue of quik.asymmetric.int{4,8}FusedDequantize, fp16 arithmetic, one rounding per op:

        ((h(acc) * scale_col) * scale_row + (zero_row + h(shift) * scale_row) * w_reduced) + y

    include/asymmetric/epilogue/thread/linear_combination_dequant.h:155-162 (c10::Half operators:
    fp32 op, result rounded to half; `row_vec` is bound to scale_col and `col_vec` to scale_row,
    src/asymmetric/fused_dequantize.cu:46-57); the same expression is the reference's own
    known-answer formula, test/python/test_fused.py:56-62."""
    h = np.float16
    with np.errstate(over="ignore", invalid="ignore"):
        a = np.asarray(acc, np.int32).astype(np.float64).astype(h)       # exact int -> one rounding to half
        sr = np.asarray(scale_row, h).reshape(-1, 1)
        sc = np.asarray(scale_col, h).reshape(1, -1)
        z = np.asarray(zero_row, h).reshape(-1, 1)
        w = np.asarray(w_reduced, h).reshape(1, -1)
        sh = h(np.float32(shift_value))
        t = ((a * sc).astype(h) * sr).astype(h)
        u = ((z + (sh * sr).astype(h)).astype(h) * w).astype(h)
        return ((t + u).astype(h) + np.asarray(y, h)).astype(h)


# --------------------------------------------------------------------------- #
# symmetric variants (src/symmetric/symmetric.cu)
# --------------------------------------------------------------------------- #
def sym_act_scale(int_x, bits=4):
    """Caller-side per-row scale of MixedQLinear's symmetric branch.

    experiments/qlinear.py:101-102: max|x| / (1 << (bits - 1) - 1) where Python
    precedence makes the divisor 1 << ((bits-1)-1), i.e. 4 for bits=4.  The division
    happens in fp16 (torch half / python int), then `.to(float16)`."""
    x = np.asarray(int_x, np.float16)
    amax = np.abs(x).max(axis=1, keepdims=True)
    div = np.float16(1 << ((bits - 1) - 1))
    return (amax / div).astype(np.float16)


def sym_quantize(x, scale, bits):
    """quik.symmetric.quantize: q = half2int_rn(hdiv(x, scale[row])).

    src/symmetric/symmetric.cu:6-28 (int4: the low four bits are kept, no clamp;
    odd column counts leave the last high nibble zero), :50-61 (int8: C conversion
    int -> int8_t, i.e. wrap)."""
    x = np.asarray(x, np.float16)
    s = np.asarray(scale, np.float16).reshape(-1, 1)
    assert s.shape[0] == x.shape[0]                           # symmetric.cu:33-34
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        d = (x / s).astype(np.float16).astype(np.float32)
    v = _rne_to_int(d)
    if bits == 8:
        return (v & 0xFF).astype(np.uint8).view(np.int8)
    assert bits == 4
    u = (v & 0xF).astype(np.uint8)
    if u.shape[1] % 2:
        u = np.concatenate([u, np.zeros((u.shape[0], 1), np.uint8)], axis=1)
    return (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)


def sym_dequantize(x, scale_row, scale_col, y, bits):
    """quik.symmetric.dequantize: fp16 chain.

    src/symmetric/symmetric.cu:81-113: xh = int2half_rn(x) (or x itself for
    bits=16); out = hmul(hmul(xh, sRow[r]), sCol[c]) + y, the final add being
    torch::Half operator+ (fp32 add rounded to fp16).  `bits` selects the type of
    x: 8 -> int8, 16 -> half, 32 -> int32 (symmetric.cpp:32-41)."""
    assert bits in (8, 16, 32)
    sr = np.asarray(scale_row, np.float16).reshape(-1, 1)
    sc = np.asarray(scale_col, np.float16).reshape(1, -1)
    y = np.asarray(y, np.float16)
    with np.errstate(over="ignore", invalid="ignore"):
        if bits == 16:
            xh = np.asarray(x, np.float16)
        else:
            xh = np.asarray(x).astype(np.float64).astype(np.float16)  # exact int -> one RNE rounding
        t = (xh * sr).astype(np.float16)
        t = (t * sc).astype(np.float16)
        out = (t.astype(np.float32) + y.astype(np.float32)).astype(np.float16)
    return out


# --------------------------------------------------------------------------- #
# MixedQLinear (experiments/qlinear.py)
# --------------------------------------------------------------------------- #
def from_float(weight, weights_scales, fp_indices, bits=4, symm=False, dtype=F16):
    """MixedQLinear.from_float buffers (experiments/qlinear.py:150-199).

    int_indices = ascending complement of fp_indices (:163-167);
    int_weight = pack(round(W[:, int] / s_w)) with the divide in the weight dtype (:178-182);
    reduced_w[0, n] = dtype(sum_k f32(W[n, int_k])) (:185-186);
    fp_weight = W[:, fp_indices] (:198)."""
    w = np.asarray(weight, np.float16) if dtype == F16 else np.asarray(weight, np.float32)
    n_out, n_in = w.shape
    fp_indices = np.asarray([] if fp_indices is None else fp_indices, dtype=np.int64)
    mask = np.ones(n_in, bool)
    mask[fp_indices] = False
    int_indices = np.arange(n_in, dtype=np.int64)[mask]
    assert int_indices.size + fp_indices.size == n_in
    s = np.asarray(weights_scales).reshape(n_out, 1)
    wi = w[:, int_indices]
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        if dtype == F16:
            r = np.rint((wi / s.astype(np.float16)).astype(np.float16).astype(np.float32))
        else:
            r = np.rint(bf16_round(wi / s.astype(np.float32)))
    codes = r.astype(np.int64).astype(np.int8)
    out = {
        "weights_scales": _round_to(s.astype(np.float32), dtype),
        "int_weight": pack_i4(codes) if bits == 4 else codes,
        "int_indices": int_indices,
        "fp_indices": fp_indices,
        "fp_weight": w[:, fp_indices].copy(),
    }
    if not symm:
        red = _as_f32(wi, dtype).sum(axis=1, dtype=np.float32)
        out["reduced_w"] = _round_to(red, dtype).reshape(1, n_out)
    return out


def fp_linear(fp_x, fp_weight, bias, dtype=F16):
    """torch.nn.functional.linear(fp_x, fp_weight, bias) (experiments/qlinear.py:123-124).

    BLAS summation order is unspecified in the reference; this restatement
    accumulates in float64, adds the bias and rounds once to the storage type."""
    acc = _as_f32(fp_x, dtype).astype(np.float64) @ _as_f32(fp_weight, dtype).astype(np.float64).T
    if bias is not None:
        acc = acc + _as_f32(bias, dtype).astype(np.float64).reshape(1, -1)
    return _round_to(acc.astype(np.float32), dtype)


def mixed_qlinear_forward(x, mod, bits=4, bias=None, symm=False, dtype=F16):
    """MixedQLinear.forward on a 2-D input (experiments/qlinear.py:80-148).

    `mod` is the dict from from_float.  Returns (out [M, N], intermediates)."""
    K = mod["int_indices"].size
    M = x.shape[0]
    N = mod["weights_scales"].shape[0]
    inter = {}
    if symm:
        xs = np.asarray(x, np.float16)
        int_x = xs[:, mod["int_indices"]]
        fp_x = xs[:, mod["fp_indices"]]
        qscale = sym_act_scale(int_x, bits)
        qx = sym_quantize(int_x, qscale, bits)
        inter.update(qscale=qscale)
    else:
        qx, meta, fp_x = asym_quantize(x, mod["int_indices"], mod["fp_indices"], bits, dtype)
        inter.update(meta=meta)
    if mod["fp_indices"].size > 0:
        fp_result = fp_linear(fp_x, mod["fp_weight"], bias, dtype)
    elif bias is not None:
        fp_result = np.repeat(np.asarray(bias).reshape(1, -1), M, axis=0)
    else:
        fp_result = np.zeros((M, N), np.float16 if dtype == F16 else np.float32)
    acc = int4_matmul(qx, mod["int_weight"]) if bits == 4 else int8_matmul(qx, mod["int_weight"])
    if symm:
        out = sym_dequantize(acc, qscale, mod["weights_scales"].reshape(1, -1), fp_result, 32)
    else:
        out = asym_dequantize(acc, meta, mod["weights_scales"], mod["reduced_w"], fp_result, bits, dtype)
    inter.update(qx=qx, fp_x=fp_x, fp_result=fp_result, acc=acc)
    return out, inter


def dequantized_activation_f64(x, int_indices, fp_indices, bits, dtype=F16):
    """x_deq[:, int] = s*(q + 2^(bits-1)) + zero, x_deq[:, fp] = x[:, fp], float64.

    The algebraic identity behind the zero-point correction:
    x W^T = s_row s_col sum(q qw) + (2^(b-1) s_row + zero) s_col sum(qw)."""
    qx, meta, fp_x = asym_quantize(x, int_indices, fp_indices, bits, dtype)
    q = unpack_i4(qx) if bits == 4 else qx
    m = _as_f32(meta, dtype).astype(np.float64)
    xd = np.zeros(x.shape, np.float64)
    xd[:, int_indices] = m[0::2][:, None] * (q.astype(np.float64) + (1 << (bits - 1))) + m[1::2][:, None]
    xd[:, fp_indices] = _as_f32(fp_x, dtype).astype(np.float64)
    return xd
