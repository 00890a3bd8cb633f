"""The integer accumulator of the 6-bit matrix-core path, read directly.

`quik_mixed_linear_fwd_fp6` (and its K-split form `..._ws`) recovers sum_k a_k w_k from fp32 sums of E2M3
products and per-row / per-column level sums.  Every other test of that path compares rounded fp16 / bf16
outputs, in which an error of one unit of the accumulator (s_row * s_col, about 1e-3) hides below the output's
ulp.  Here the epilogue is made the identity: scale 1, zero -8, column scales 1, w_reduced = 0 (not NULL: the
asymmetric epilogue), no outliers, no bias, so that out = fp16(f32(acc)).
  * sparse weights (|acc| <= 2048): every integer in that range is an fp16 number, so out == acc, element for
    element, against the oracle's integer matmul (src/matmul/matmul.cu:17-55, test/python/test_matmul.py:16-26);
  * full-range codes: out == fp16(acc) bit for bit, one known rounding (float32 holds |acc| <= 64 K exactly),
    including the overflow to infinity of the all-extreme rows.
The activation operand buffer is written here, from the documented layout (quik_amd/csrc/fp6_format.h restated,
not imported), so the test does not lean on the quantize kernel; the weight buffer comes from pack_weight_fp6,
whose contents tests/test_gpu_parity.py decodes and checks.
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


def encode_operand6(levels):
    """levels [rows, K] (0 .. 15) -> operand buffer without outlier steps: per 64-row block and 64-element step a
    3 KB unit (heads of rows 0..31, heads of rows 32..63, tails), 32 six-bit fields per 24-byte fragment (16-byte
    head + 8-byte tail), head slot swapped by bit 3 of the row; one int32 level sum per row at the end."""
    rows, K = levels.shape
    steps, blocks = K // 64, (rows + 63) // 64
    block_bytes = steps * 3072
    buf = np.zeros(blocks * block_bytes + 4 * rows, np.uint8)
    # element e of a fragment occupies bits [6 e, 6 e + 6) of its 192 bits, little-endian
    bits = ((levels.astype(np.uint8)[:, :, None] >> np.arange(6, dtype=np.uint8)) & 1).astype(np.uint8)
    frag = np.packbits(bits.reshape(rows, steps, 2, 192), axis=-1, bitorder="little")        # [rows, steps, h, 24]
    r = np.arange(rows)[:, None, None]
    s = np.arange(steps)[None, :, None]
    h = np.arange(2)[None, None, :]
    unit = (r >> 6) * block_bytes + s * 3072
    head = unit + ((r >> 5) & 1) * 1024 + (r & 31) * 32 + ((h ^ ((r >> 3) & 1)) << 4)
    tail = unit + 2048 + h * 512 + (r & 63) * 8
    buf[(head[..., None] + np.arange(16)).ravel()] = frag[..., :16].ravel()
    buf[(tail[..., None] + np.arange(8)).ravel()] = frag[..., 16:].ravel()
    buf[blocks * block_bytes:] = np.frombuffer(levels.sum(1).astype(np.int32).tobytes(), np.uint8)
    return buf


def run_identity_epilogue(a_codes, w_codes, use_workspace):
    """fp16 output of the 6-bit GEMM with an identity epilogue, as float64, for signed int4 codes a [M, K], w [N, K]."""
    from quik_amd import _lib as L
    from quik_amd import asymmetric, matmul
    M, K = a_codes.shape
    N = w_codes.shape[0]
    lib = L.load()
    ii = np.arange(K, dtype=np.int64)
    colmap = asymmetric.build_colmap(_t(ii), _t(np.zeros(0, np.int64)), K)
    w6 = matmul.pack_weight_fp6(_t(qo.pack_i4(w_codes)), torch.empty((N, 0), dtype=torch.float16, device=DEV), colmap)
    x6 = _t(encode_operand6(a_codes.astype(np.int64) + 8))
    assert x6.numel() == lib.quik_fp6_operand_bytes(M, K, 0)
    meta = np.empty(2 * M, np.float16)
    meta[0::2], meta[1::2] = 1.0, -8.0
    s_col = _t(np.ones((N, 1), np.float16))
    w_red = _t(np.zeros((1, N), np.float16))
    want_split = lib.quik_splitk_workspace_bytes(M, N, K, 4) > 0
    old = matmul.split_k
    matmul.split_k = use_workspace
    try:
        out = matmul.mixed_linear_fp6(x6, w6, _t(meta), s_col, w_red, None, M, N, K, 0, torch.float16)
    finally:
        matmul.split_k = old
    torch.cuda.synchronize()
    return out.cpu().numpy(), want_split


# M, N, K: every tile plan of the 6-bit path (128x64, 128x128, K split, 256x256 with eight waves, 256x256 + 256x128)
SHAPES = [
    (40, 96, 128), (130, 200, 7936), (64, 1024, 7936), (300, 640, 128), (512, 4096, 256),
    (2048, 8192, 128), (2048, 28672, 128), (2049, 28672 + 64, 128),
]


def _exact_product(a, w):
    if a.shape[0] * w.shape[0] * a.shape[1] <= 1 << 28:
        return qo.int_matmul(a, w).astype(np.int64)
    # float64 holds these sums exactly (|acc| <= 64 K): one BLAS call instead of an int64 product of 10^10 terms
    acc = (a.astype(np.float64) @ w.astype(np.float64).T)
    sample = np.random.default_rng(0).integers(0, a.shape[0], 16)
    assert np.array_equal(acc[sample].astype(np.int64), qo.int_matmul(a[sample], w).astype(np.int64))
    return acc.astype(np.int64)


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_six_bit_path_returns_the_integer_accumulator(M, N, K):
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-8, 8, (M, K)).astype(np.int8)
    # sparse weights: at most 32 non-zero codes per output column, so |acc| <= 32 * 64 = 2048 (exact in fp16)
    w = np.zeros((N, K), np.int8)
    for n in range(N):
        idx = rng.choice(K, 32, replace=False)
        w[n, idx] = rng.integers(-8, 8, 32)
    a[0, :] = -8                       # extreme rows: every product of the non-zero weights at its largest
    a[M - 1, :] = 7
    acc = _exact_product(a, w)
    assert np.abs(acc).max() <= 2048
    for use_ws in (True, False):
        out, split = run_identity_epilogue(a, w, use_ws)
        if (M, N, K) == (64, 1024, 7936):
            assert split                                     # with a workspace this shape is split over K
        assert np.array_equal(out.astype(np.int64), acc), (use_ws, np.abs(out.astype(np.int64) - acc).max())


@pytest.mark.parametrize("M,N,K", [(40, 96, 128), (130, 200, 7936), (64, 1024, 7936), (300, 640, 2048),
                                   (2048, 2048 + 128, 7936)])
def test_six_bit_path_full_range_codes_round_once(M, N, K):
    rng = np.random.default_rng(M * 3 + N + K)
    a = rng.integers(-8, 8, (M, K)).astype(np.int8)
    w = rng.integers(-8, 8, (N, K)).astype(np.int8)
    a[0, :], a[1, :] = -8, 7
    w[0, :], w[1, :], w[N - 1, :] = -8, 7, -8        # acc = +-64 K, 56 K ...: beyond fp16 for K = 7936 (infinity)
    acc = _exact_product(a, w)
    assert np.abs(acc).max() == 64 * K
    with np.errstate(over="ignore"):
        want = acc.astype(np.float32).astype(np.float16)         # |acc| < 2^24: the float32 step is exact
    for use_ws in (True, False):
        out, _ = run_identity_epilogue(a, w, use_ws)
        assert np.array_equal(out.view(np.uint16), want.view(np.uint16)), use_ws
