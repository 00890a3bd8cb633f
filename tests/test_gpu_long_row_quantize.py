"""Rows of more than 8192 columns -> int8 operand buffer in tile order (quik_asym_quantize_tile8).

fp16 rows of that length go through a kernel of their own (the row is copied global -> LDS into a ring of two
slots, one or two workgroups of eight waves per CU); every other case keeps the streaming kernel.  The buffer is decoded
here from the documented layout (quik_amd/csrc/gemm_tile8.h, restated) and compared, code for code and bit for bit,
with the oracle's per-token quantize (src/asymmetric/asymmetric.cu:15-108 with the reference's index gather,
quik/asymmetric.py), at every group count per lane the kernel is built for, with ragged row counts, edge rows
(constant, subnormal, overflowing range, infinity, NaN, all-NaN), outlier columns next to each other and at both
ends of the row, no outlier columns at all, and more rows than one pass of the persistent grid takes.
Signalling-NaN bit patterns, which no arithmetic produces but a caller may hand over, are skipped by min / max like
every other NaN (the reference's __hmin / __hmax): checked for this kernel and for the 6-bit one.
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


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def decode_tile8(buf, rows, K, F):
    """operand buffer -> int8 codes [rows, K], outlier bit patterns [rows, F]: rows in blocks of 64, per block
    K / 32 integer steps then F / 16 outlier steps of 2 KB; row r of a block at 1024 ((r >> 5) & 1) + 32 (r & 31),
    16-byte chunk h of the step in slot h ^ ((r >> 3) & 1)."""
    steps, fsteps = K // 32, F // 16
    block_bytes = (steps + fsteps) * 2048
    assert buf.size == ((rows + 63) // 64) * block_bytes
    s = np.arange(steps + fsteps)[None, :, None]
    h = np.arange(2)[None, None, :]
    codes, outl = np.empty((rows, K), np.int8), np.empty((rows, F), np.uint16)
    for r0 in range(0, rows, 64):                                             # block by block: small index arrays
        r = np.arange(r0, min(r0 + 64, rows))[:, None, None]
        off = (r >> 6) * block_bytes + ((r >> 5) & 1) * 1024 + (r & 31) * 32 + s * 2048 + ((h ^ ((r >> 3) & 1)) << 4)
        chunks = buf[(off[..., None] + np.arange(16)).reshape(r.shape[0], -1)]  # [rows of the block, (steps + fsteps) * 32]
        codes[r0:r0 + 64] = chunks[:, :steps * 32].view(np.int8)
        outl[r0:r0 + 64] = np.ascontiguousarray(chunks[:, steps * 32:]).view(np.uint16)
    return codes, outl


def _case(rng, rows, n_in, fi):
    fi = np.asarray(fi, np.int64)
    mask = np.ones(n_in, bool)
    mask[fi] = False
    ii = np.arange(n_in, dtype=np.int64)[mask]
    x = rng.standard_normal((rows, n_in)).astype(np.float32)
    x[:, fi] *= 50
    x = x.astype(np.float16)
    x[0, :] = 1.5                                   # constant row: scale clamps at 1e-6
    x[1, ii[:8]] = [0, 0.5, 1.5, 2.5, 3.5, 4.5, 15, 7.5]
    x[2, :] *= 1e-7                                 # fp16 subnormals
    x[3, ii[3]], x[3, ii[4]] = 65504.0, -65504.0    # range overflows fp16: the division path
    x[4, ii[5]] = np.inf
    x[5, ii[6]] = np.nan
    x[6, :] = 0.0
    x[7, ii] = np.nan                               # all-NaN row
    x[8, ii[-1]], x[8, ii[0]] = 300.0, -200.0       # extremes in the first and the last group of the row
    return x, ii, fi


def _check(x, ii, fi, n_in):
    from quik_amd import asymmetric
    rows, K, F = x.shape[0], len(ii), len(fi)
    cm = asymmetric.build_colmap(_t(ii), _t(fi), n_in)
    assert asymmetric.colmap_streams(cm, K, F)
    x8, meta = asymmetric.quantize_mapped_tile8(_t(x), cm, K, F)
    torch.cuda.synchronize()
    want_q, want_meta, want_fp = qo.asym_quantize(x, ii, fi, 8)
    got_meta = meta.cpu().contiguous().view(torch.int16).numpy().view(np.uint16).reshape(rows, 2)
    want_bits = want_meta.view(np.uint16).reshape(rows, 2)
    nan_zero = np.isnan(want_meta.reshape(rows, 2)[:, 1].astype(np.float32))
    assert np.array_equal(got_meta[:, 0], want_bits[:, 0])
    assert np.array_equal(got_meta[~nan_zero, 1], want_bits[~nan_zero, 1])
    assert np.isnan(meta.float().cpu().numpy().reshape(rows, 2)[nan_zero, 1]).all()
    codes, outl = decode_tile8(x8.cpu().numpy(), rows, K, F)
    bad = np.argwhere(codes != want_q)
    assert bad.size == 0, (bad[:5], codes[tuple(bad[0])], want_q[tuple(bad[0])])
    assert np.array_equal(outl, want_fp.view(np.uint16).reshape(rows, F))


# rows, in_features, outlier columns: in / 8 / 512 rounded up = groups per lane (3 .. 8)
@pytest.mark.parametrize("rows,n_in,F", [
    (300, 11008, 256),         # Llama-2-7B down_proj: 3 groups per lane, two workgroups per CU
    (2048 + 7, 13824, 256),    # Llama-2-13B down_proj: 4; every workgroup takes several rows
    (40, 8192 + 64, 64),       # the shortest row of the kernel
    (37, 8192, 256),           # one column group fewer: the streaming kernel
    (70, 28672, 256),          # Llama-2-70B down_proj: 7 groups per lane, exactly
    (2100, 28672, 256),        # more rows than the grid's first pass, ragged last block
    (41, 16384 + 64, 64),      # 5 groups per lane, most of the fifth past the row's end
    (64, 24576, 128),          # 6
    (33, 31744, 256),          # 8: the longest row whose ring fits LDS
    (40, 20480 - 64, 0),       # no outlier columns; row length not a multiple of the 1 KB copies
    (36, 28672, 512),          # as many outlier columns as lanes
])
def test_long_rows_against_the_oracle(rows, n_in, F):
    rng = np.random.default_rng(rows + n_in + F)
    fi = rng.permutation(n_in)[:F]
    if F >= 64:
        # outlier columns next to each other, in one group of 8, and at both ends of the row
        fi[:16] = [0, 1, 2, 3, 4, 5, 6, 7, 8, 17, n_in - 1, n_in - 2, n_in - 9, 4096, 4097, 4103]
        fi = np.unique(fi)
        extra = np.setdiff1d(np.arange(100, 100 + 4 * F), fi)[:F - len(fi)]
        fi = rng.permutation(np.concatenate([fi, extra]))
    x, ii, fi = _case(rng, rows, n_in, fi)
    _check(x, ii, fi, n_in)


@pytest.mark.parametrize("seed", range(12))
def test_long_rows_random_shapes(seed):
    """Seeded random shapes over the kernel's whole range: 8224 .. 31744 columns in steps of 32, 0 .. 512 outlier
    columns (in runs, clustered at one end, or spread), 1 .. 300 rows."""
    rng = np.random.default_rng(1000 + seed)
    F = 32 * int(rng.integers(0, 17))
    k64 = int(rng.integers((8224 - F + 63) // 64, (31744 - F) // 64 + 1))
    n_in = 64 * k64 + F
    rows = int(rng.integers(9, 300))
    kind = seed % 3
    if kind == 0 or F == 0:
        fi = rng.permutation(n_in)[:F]
    elif kind == 1:                                        # runs of adjacent outlier columns
        starts = rng.permutation(n_in // 64)[:F // 8] * 64 + rng.integers(0, 50, F // 8)
        fi = (starts[:, None] + np.arange(8)[None, :]).ravel()
    else:                                                  # all of them in the last columns of the row
        fi = n_in - 1 - rng.permutation(2 * F)[:F]
    assert len(np.unique(fi)) == F
    x, ii, fi = _case(rng, rows, n_in, fi)
    _check(x, ii, fi, n_in)


def test_every_group_holds_an_outlier_column_falls_back():
    """More groups with outlier columns than the ring kernel keeps per lane (512): the streaming kernel serves the
    shape, same results."""
    rng = np.random.default_rng(5)
    n_in, F = 28672, 1024
    fi = np.arange(F) * 8 + rng.integers(0, 8, F)       # one outlier column in each of the first 1024 groups
    x, ii, fi = _case(rng, 34, n_in, fi)
    _check(x, ii, fi, n_in)


@pytest.mark.parametrize("bits", [4, 8])
def test_signalling_nans_are_skipped_like_quiet_ones(bits):
    from quik_amd import asymmetric
    rng = np.random.default_rng(bits)
    rows, n_in, F = 48, (28672 if bits == 8 else 8192), 256
    fi = rng.permutation(n_in)[:F]
    x, ii, fi = _case(rng, rows, n_in, fi)
    xb = x.view(np.uint16)
    for r in range(9, rows):
        cols = ii[rng.integers(0, len(ii), 6)]
        xb[r, cols] = [0x7C01, 0x7D00, 0xFC01, 0x7DFF, 0x7E00, 0xFDAB]       # signalling (quiet bit clear) and quiet
    # a signalling NaN right after the row's minimum and right before its maximum, inside one group
    xb[10, ii[64:72]] = np.array([-900.0, 0, 0, 0, 0, 0, 0, 0], np.float16).view(np.uint16)
    xb[10, ii[65]] = 0x7C01
    xb[11, ii[128:136]] = np.array([0, 0, 0, 0, 0, 0, 0, 900.0], np.float16).view(np.uint16)
    xb[11, ii[134]] = 0xFD55
    if bits == 8:
        _check(x, ii, fi, n_in)
        return
    K = len(ii)
    cm = asymmetric.build_colmap(_t(ii), _t(fi), n_in)
    x6, meta = asymmetric.quantize_mapped_fp6(_t(x), cm, K, F)
    q, _, _ = asymmetric.quantize_mapped(_t(x), cm, K, F, 4)        # the row-major kernel, oracle-checked elsewhere
    want_q, want_meta, _ = qo.asym_quantize(x, ii, fi, 4)
    assert np.array_equal(q.cpu().numpy(), want_q)
    got = meta.cpu().contiguous().view(torch.int16).numpy().view(np.uint16).reshape(rows, 2)
    want = want_meta.view(np.uint16).reshape(rows, 2)
    ok = ~np.isnan(want_meta.reshape(rows, 2)[:, 1].astype(np.float32))       # (the all-NaN row's zero is a NaN)
    assert np.array_equal(got[:, 0], want[:, 0]) and np.array_equal(got[ok, 1], want[ok, 1])
