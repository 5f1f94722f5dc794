"""The allocation-free GEMV entry point (flute_gemv_noalloc) against flute_gemv, through the
C ABI: same kernels, so the outputs must be bit-identical.  Two calls in a row on the
same device, the second with a smaller input (the fixed scratch array keeps the first
call's contents), in configurations that use the scratch: a K split (partial sums and
tickets), a residual (coefficients) and a rotated weight with a residual (pre-rotated
input)."""
import ctypes

import pytest
import torch

import flute_oracle as O
from flute_extended import _lib
from _util import make_weight, make_x

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _desc(w, signs=None):
    d = _lib.FluteLinear()
    d.q1, d.lut1, d.q1_bytes = w["blob_d"].data_ptr(), w["lut_d"].data_ptr(), w["blob_d"].numel()
    d.N, d.K, d.b1, d.group_size = w["N"], w["K"], w["bits"], w["gs"]
    d.lut_rows = w["lut"].shape[0]
    d.lut_dtype = _lib.F16 if w["lut"].dtype == torch.float16 else _lib.BF16
    if w["resA"] is not None:
        d.resA, d.resB, d.R = w["resA_d"].data_ptr(), w["resB_d"].data_ptr(), w["resA"].shape[1]
    if w["bias"] is not None:
        d.bias = w["bias_d"].data_ptr()
    if signs is not None:
        d.signs = signs.data_ptr()
    return d


def _call(fn, d, x, N, split):
    y = torch.full((1, N), float("nan"), dtype=x.dtype, device=DEV)
    st = fn(ctypes.byref(d), x.data_ptr(), y.data_ptr(),
            _lib.F16 if x.dtype == torch.float16 else _lib.BF16, split,
            torch.cuda.current_stream().cuda_stream)
    assert st == 0, _lib.last_error()
    return y


@pytest.mark.parametrize("split,rank,rotate", [(4, 0, False), (1, 8, False), (8, 16, True), (2, 4, False)])
def test_noalloc_matches_gemv_on_two_calls_in_a_row(split, rank, rotate):
    big = make_weight(2048, 4096, seed=31, rank=rank, bias=True, device=DEV)
    small = make_weight(256, 1024, seed=32, rank=rank, bias=True, device=DEV)
    for w in (big, small):                              # the second call is the smaller one
        N, K = w["N"], w["K"]
        x = make_x(1, K, seed=33 + N).to(DEV)
        signs = O.rotation_signs(K, 5).to(DEV) if rotate else None
        d = _desc(w, signs)
        want = _call(_lib.lib.flute_gemv, d, x, N, split)
        got = _call(_lib.lib.flute_gemv_noalloc, d, x, N, split)
        torch.cuda.synchronize()
        assert not torch.isnan(got).any()
        assert torch.equal(got, want)
        assert torch.equal(_call(_lib.lib.flute_gemv_noalloc, d, x, N, split), want)


def test_noalloc_refuses_what_does_not_fit():
    N, K, split = 262144, 256, 4                         # 4 * N floats of partial sums > the array
    g = torch.Generator().manual_seed(34)
    blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, generator=g).to(DEV)
    lut = (torch.randn(N // 128, 16, generator=g) * 0.02).half().to(DEV)
    x = make_x(1, K, seed=35).to(DEV)
    d = _lib.FluteLinear()
    d.q1, d.lut1, d.q1_bytes = blob.data_ptr(), lut.data_ptr(), blob.numel()
    d.N, d.K, d.b1, d.group_size, d.lut_rows, d.lut_dtype = N, K, 4, 128, N // 128, _lib.F16
    y = torch.zeros(1, N, dtype=torch.float16, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    st = _lib.lib.flute_gemv_noalloc(ctypes.byref(d), x.data_ptr(), y.data_ptr(), _lib.F16, split,
                                     stream)
    assert st == _lib.FLUTE_ERR_UNSUPPORTED
    assert "scratch" in _lib.last_error()
    # without a split the same weight needs no scratch at all and is served
    assert _lib.lib.flute_gemv_noalloc(ctypes.byref(d), x.data_ptr(), y.data_ptr(), _lib.F16, 1,
                                       stream) == 0, _lib.last_error()
    want = torch.zeros_like(y)
    assert _lib.lib.flute_gemv(ctypes.byref(d), x.data_ptr(), want.data_ptr(), _lib.F16, 1,
                               stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(y, want)


def test_noalloc_under_graph_capture():
    """The entry point records no allocation and no memset node: it can be captured, and
    every replay gives the eager result."""
    w = make_weight(512, 2048, seed=36, rank=8, device=DEV)
    x = make_x(1, 2048, seed=37).to(DEV)
    d = _desc(w)
    want = _call(_lib.lib.flute_gemv, d, x, 512, 4)
    y = torch.zeros(1, 512, dtype=torch.float16, device=DEV)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        _call(_lib.lib.flute_gemv_noalloc, d, x, 512, 4)          # warm-up on the side stream
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            st = _lib.lib.flute_gemv_noalloc(ctypes.byref(d), x.data_ptr(), y.data_ptr(), _lib.F16, 4,
                                             torch.cuda.current_stream().cuda_stream)
            assert st == 0, _lib.last_error()
    for _ in range(3):
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
