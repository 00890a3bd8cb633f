"""quik_mixed_linear_fwd_tile8_noalloc (K-split workspace in a device array inside the library, no allocation in
the call) against quik_mixed_linear_fwd_tile8_ws with a caller workspace: identical output bits, on two calls in
a row, the second with a smaller input, plus a shape that does not split.  Through the C ABI."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _operands(M, N, K, F, seed):
    """Random tile-ordered int8 operands through the library's own quantize / pack entry points."""
    from quik_amd import asymmetric, matmul
    g = torch.Generator().manual_seed(seed)
    n_in = K + F
    x = torch.randn(M, n_in, generator=g)
    fi = torch.randperm(n_in, generator=g)[:F]
    x[:, fi] *= 50
    keep = torch.ones(n_in, dtype=torch.bool)
    keep[fi] = False
    ii = torch.arange(n_in)[keep]
    x = x.half().to(DEV)
    cm = asymmetric.build_colmap(ii.to(DEV), fi.to(DEV), n_in)
    x8, meta = asymmetric.quantize_mapped_tile8(x, cm, K, F)
    qw = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g).to(DEV)
    fpw = (0.02 * torch.randn(N, F, generator=g)).half().to(DEV)
    w8 = matmul.pack_weight_tile8(qw, fpw)
    s_w = (torch.rand(N, generator=g) * 0.009 + 0.001).half().to(DEV)
    wred = torch.randn(N, generator=g).half().to(DEV)
    bias = torch.randn(N, generator=g).half().to(DEV)
    return x8, w8, meta, s_w, wred, bias


def _run_pair(lib, L, M, N, K, F, seed):
    x8, w8, meta, s_w, wred, bias = _operands(M, N, K, F, seed)
    need = lib.quik_splitk_workspace_bytes(M, N, K, 8)
    ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=DEV)
    want = torch.empty((M, N), dtype=torch.float16, device=DEV)
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    st = L.stream()
    rc = lib.quik_mixed_linear_fwd_tile8_ws(L.ptr(x8), L.ptr(w8), L.ptr(meta), L.ptr(s_w), L.ptr(wred), L.ptr(bias),
                                            L.QUIK_F16, M, N, K, F, L.ptr(want), L.ptr(ws) if need else None, need, st)
    assert rc == 0
    rc = lib.quik_mixed_linear_fwd_tile8_noalloc(L.ptr(x8), L.ptr(w8), L.ptr(meta), L.ptr(s_w), L.ptr(wred),
                                                 L.ptr(bias), L.QUIK_F16, M, N, K, F, L.ptr(got), st)
    assert rc == 0, lib.quik_status_string(rc)
    torch.cuda.synchronize()
    assert torch.isfinite(want).all()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K, F)
    return need


def test_no_alloc_entry_point_matches_the_workspace_entry_point():
    from quik_amd import _lib as L
    lib = L.load()
    # first call: 4 tiles x 8 splits; then a smaller input that still splits (stale partial sums of the first
    # call lie in the array); then the first again; then a shape without a K split (no scratch involved)
    need1 = _run_pair(lib, L, 200, 256, 8192, 64, 1)
    need2 = _run_pair(lib, L, 64, 130, 2048, 32, 2)
    assert need1 > need2 > 4096
    _run_pair(lib, L, 200, 256, 8192, 64, 3)
    assert _run_pair(lib, L, 300, 4160, 1024, 64, 4) == 0
    # argument checks come before anything is launched
    one = 256
    assert lib.quik_mixed_linear_fwd_tile8_noalloc(one, one, one, one, one, None, 0, 64, 256, 2048 + 32, 32, one, None) == -4
    assert lib.quik_mixed_linear_fwd_tile8_noalloc(one, one, None, one, one, None, 0, 64, 256, 2048, 32, one, None) == -5
    assert lib.quik_mixed_linear_fwd_tile8_noalloc(one, one, one, one, one, None, 7, 64, 256, 2048, 32, one, None) == -3
