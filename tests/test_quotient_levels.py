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
