"""CPU check of the arithmetic shortcut of the fp16 streaming quantize kernel.

The kernel computes the level as rne_int(clamp(fp16(f32(d) * r))) with r = fp32(1 / scale), where the
contract asks for rne_int(clamp(fp16(d / scale))) (reference: src/asymmetric/asymmetric.cu:340-435).
The two fp16 values may differ in the last place; the level may not.  A level can only change when
the quotient sits next to a k + 1/2 boundary, so for every fp16 scale >= 1e-6 this test takes, for
every boundary, the fp16 numerators around (k + 1/2) * scale and compares the levels.  Both possible
hardware roundings of the product are modelled: fp32 then fp16, and fp16 directly.  (The full
32k x 32k domain gives zero level differences as well; it takes minutes on a CPU, so the GPU suite
covers it on the device.)"""
import numpy as np


def _levels(t16, maxq):
    return np.rint(np.clip(t16.astype(np.float32), 0, maxq))


def test_uncorrected_reciprocal_product_never_changes_a_level():
    allh = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)
    scales = allh[allh >= np.float16(1e-6)]
    bounds = np.arange(255, dtype=np.float64) + 0.5                       # covers 4 and 8 bits
    offs = np.arange(-3, 4, dtype=np.int32)
    for i in range(0, scales.size, 512):
        s = scales[i:i + 512]
        s64 = s.astype(np.float64)[:, None]
        with np.errstate(over="ignore"):
            near = (s64 * bounds[None, :]).astype(np.float16)             # fp16 next to (k + 1/2) * scale
        bits = near.view(np.uint16).astype(np.int32)[:, :, None] + offs[None, None, :]
        bits = np.clip(bits, 0, 0x7BFF).astype(np.uint16)                 # finite, non-negative numerators
        d = bits.view(np.float16).reshape(s.size, -1)
        r = (np.float32(1.0) / s.astype(np.float32)[:, None]).astype(np.float32)
        with np.errstate(over="ignore", invalid="ignore"):
            want = (d.astype(np.float64) / s64).astype(np.float16)
            two_step = (d.astype(np.float32) * r).astype(np.float16)
            one_step = (d.astype(np.float64) * r.astype(np.float64)).astype(np.float16)
        for maxq in (15, 255):
            assert np.array_equal(_levels(two_step, maxq), _levels(want, maxq))
            assert np.array_equal(_levels(one_step, maxq), _levels(want, maxq))
    # every numerator against a sample of scales: the fp16 quotients do differ here and there (so the
    # shortcut is not the identity and the level check above is not vacuous), the levels never do
    rng = np.random.default_rng(5)
    s = rng.choice(scales, 1500, replace=False)
    r = (np.float32(1.0) / s.astype(np.float32)[:, None]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = (allh.astype(np.float64)[None, :] / s.astype(np.float64)[:, None]).astype(np.float16)
        two_step = (allh.astype(np.float32)[None, :] * r).astype(np.float16)
    assert (two_step != want).sum() > 0
    for maxq in (15, 255):
        assert np.array_equal(_levels(two_step, maxq), _levels(want, maxq))


def test_four_bit_quotient_never_reaches_the_upper_clamp_on_the_fast_path():
    """The kernel that writes the 6-bit operand buffers drops the upper clamp min(t, 15) for rows with a finite
    range.  That is safe if fp16(d * r) < 15.5 for every numerator d = fp16(x - zero) a row can hold.  d is at most
    the fp16 round-up of the row's range, and the scale is fp16(max(range / 15, 1e-6)): for every fp16 scale this
    takes the largest range that still rounds to that scale (plus the slack of the fp32 division) and the largest
    numerator it allows, and evaluates the quotient both ways.  The largest value, 15.47, belongs to the smallest,
    subnormal scale, whose rounding error is the largest relative to its size."""
    pat = np.arange(0x0011, 0x7C00, dtype=np.uint16)                    # fp16(1e-6) = 0x0011 is the smallest scale
    assert np.float16(1e-6).view(np.uint16) == 0x0011
    s = pat.view(np.float16).astype(np.float64)
    nxt = (pat + 1).view(np.float16).astype(np.float64)
    nxt[-1] = 65536.0
    hi = (s + nxt) / 2                                                  # fp32 values up to here round to s
    r_max = 15 * hi * (1 + 2.0 ** -22)
    keep = r_max <= 65504.0 * (1 + 2.0 ** -10)                          # a larger range takes the IEEE-divide path
    with np.errstate(over="ignore"):
        d = r_max.astype(np.float32).astype(np.float16)
        d = np.where(d.astype(np.float64) < r_max, np.nextafter(d, np.float16(np.inf)), d).astype(np.float16)
    keep &= np.isfinite(d)
    d64, s64 = d.astype(np.float64)[keep], s[keep]
    r = (1.0 / s64).astype(np.float32).astype(np.float64)
    two_step = (d64 * r).astype(np.float32).astype(np.float16).astype(np.float64)
    one_step = (d64 * r).astype(np.float16).astype(np.float64)
    exact = (d64 / s64).astype(np.float16).astype(np.float64)
    top = np.maximum(np.maximum(two_step, one_step), exact)
    assert keep.sum() > 25000 and top.max() < 15.5
    assert top.max() > 15.4 and s64[top.argmax()] == np.float16(1e-6)    # the bound is tight where the text says
    # symmetric activations: scale = fp16(max|x| / 4) >= 1e-6 on the fast path, so |t| stays near 4
    a = np.arange(0x0001, 0x7C00, dtype=np.uint16).view(np.float16)
    sc = (a.astype(np.float32) / np.float32(4)).astype(np.float16)
    ok = sc >= np.float16(1e-6)
    t = (a[ok].astype(np.float64) * (1.0 / sc[ok].astype(np.float64)).astype(np.float32)).astype(np.float16)
    assert np.abs(t.astype(np.float64)).max() < 4.5
