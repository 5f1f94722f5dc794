"""GPU parity of the LUT grouped along K: one row of sixteen values per (output row, 128-wide
K group), W[n, k] = LUT[n, k // 128, idx[n, k]].

No upstream kernel, artifact or test has this form, so there is no upstream vector to pin it;
its definition is the closed form above, evaluated here with a numpy gather on the logical
(unpacked) indices.  The blob is the ordinary 4-bit idxN blob, whose packing the oracle tests
pin.  The dequantisation must match bit for bit; the GEMV is held to the benchmark's tolerance
(relative L2 <= 1e-3 against the fp64 product rounded once to the output type), and a one-hot
input must return the dequantised column exactly, which checks every lookup's K group.
"""
import ctypes

import numpy as np
import pytest
import torch

import flute_extended as fx
import flute_oracle as O
from _util import make_x, rel_l2
from flute_extended import _C, _lib, idxN

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-3


def make_kgroup(N, K, seed, lut_dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    lut = (torch.randn(N, K // 128, 16, generator=g) * 0.02).sort(dim=2).values.to(lut_dtype)
    blob = torch.from_numpy(idxN.pack_idxn(idx.numpy(), 4))
    return idx, lut, blob


def dense(idx, lut):
    """The closed form: W[n, k] = lut[n, k // 128, idx[n, k]], in the LUT's dtype."""
    N, K = idx.shape
    n = np.arange(N)[:, None]
    k = np.arange(K)[None, :]
    return lut[torch.from_numpy(np.broadcast_to(n, (N, K)).copy()),
               torch.from_numpy(np.broadcast_to(k // 128, (N, K)).copy()), idx.long()]


def exact(x, W, bias=None):
    y = x.double() @ W.double().t()
    if bias is not None:
        y = y + bias.double()
    return y


@pytest.mark.parametrize("N,K", [(128, 128), (256, 512), (384, 1024)])
@pytest.mark.parametrize("lut_dtype", [torch.float16, torch.bfloat16])
def test_dequant_is_bit_exact(N, K, lut_dtype):
    idx, lut, blob = make_kgroup(N, K, N + K, lut_dtype)
    W = fx.dequant_kgroup(blob.to(DEV), lut.to(DEV), K).cpu()
    assert W.dtype == lut_dtype
    assert torch.equal(W.view(torch.int16), dense(idx, lut).view(torch.int16))


SHAPES = [
    (128, 512), (256, 1024), (512, 2048), (1024, 4096), (4096, 4096), (12288, 4096),
    (4096, 12288), (512, 8192), (2048, 1024), (8192, 512),
]


@pytest.mark.parametrize("N,K", SHAPES)
def test_gemv_fp16(N, K):
    idx, lut, blob = make_kgroup(N, K, N * 3 + K)
    x = make_x(1, K, seed=11)
    y = fx.qgemm_gemv_kgroup(x.to(DEV), blob.to(DEV), lut.to(DEV)).cpu()
    assert y.shape == (1, N) and y.dtype == torch.float16
    assert rel_l2(y, exact(x, dense(idx, lut)).half()) <= TOL
    assert torch.equal(y, fx.qgemm_gemv_kgroup(x.to(DEV), blob.to(DEV), lut.to(DEV)).cpu())


@pytest.mark.parametrize("lut_dtype", [torch.float16, torch.bfloat16])
def test_gemv_bf16_activations_and_bias(lut_dtype):
    N, K = 1024, 4096
    idx, lut, blob = make_kgroup(N, K, 5, lut_dtype)
    g = torch.Generator().manual_seed(6)
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16()
    x = make_x(1, K, seed=12, dtype=torch.bfloat16)
    y = fx.qgemm_gemv_kgroup(x.to(DEV), blob.to(DEV), lut.to(DEV), bias=bias.to(DEV)).cpu()
    assert y.dtype == torch.bfloat16
    assert rel_l2(y, exact(x, dense(idx, lut), bias).bfloat16()) <= TOL


@pytest.mark.parametrize("N,K", [(256, 512), (512, 1024), (128, 4096)])
def test_one_hot_input_returns_the_dequantised_column(N, K):
    """y = W[:, k] exactly when x = e_k, for a k in every K group and both tiles of a group."""
    idx, lut, blob = make_kgroup(N, K, N + 2 * K)
    W = dense(idx, lut)
    blob_d, lut_d = blob.to(DEV), lut.to(DEV)
    ks = sorted({(g * 128 + (37 * g + 5) % 128) for g in range(K // 128)} | {0, 63, 64, 127, K - 1})
    for k in ks:
        x = torch.zeros(1, K, dtype=torch.float16)
        x[0, k] = 1.0
        y = fx.qgemm_gemv_kgroup(x.to(DEV), blob_d, lut_d).cpu()
        assert torch.equal(y[0].view(torch.int16), W[:, k].view(torch.int16)), k


@pytest.mark.parametrize("N,K,split", [(512, 4096, 2), (512, 4096, 4), (256, 8192, 8), (1024, 2048, 2)])
def test_k_splits_agree(N, K, split):
    idx, lut, blob = make_kgroup(N, K, 17 + split)
    x = make_x(1, K, seed=13)
    y = fx.qgemm_gemv_kgroup(x.to(DEV), blob.to(DEV), lut.to(DEV), split=split).cpu()
    assert rel_l2(y, exact(x, dense(idx, lut)).half()) <= TOL
    assert torch.equal(y, fx.qgemm_gemv_kgroup(x.to(DEV), blob.to(DEV), lut.to(DEV), split=split).cpu())


@pytest.mark.parametrize("block", [0, 128])
def test_fused_rotation(block):
    """The rotation is applied to the input only, so it is independent of the LUT's grouping: the
    fused launch must agree with the oracle's rotation followed by the closed-form product."""
    N, K = 512, 4096
    idx, lut, blob = make_kgroup(N, K, 23)
    x = make_x(1, K, seed=14)
    signs = O.rotation_signs(K, 3)
    xr = O.block_fht_reference(x, block, signs) if block else O.fht_reference(x, signs)
    y = fx.qgemm_gemv_kgroup(x.to(DEV), blob.to(DEV), lut.to(DEV), signs=signs.to(DEV),
                             rot_block=block).cpu()
    assert rel_l2(y, exact(xr.half(), dense(idx, lut)).half()) <= TOL


@pytest.mark.parametrize("rot", [False, True])
def test_residual_bias_and_rotation_through_the_descriptor(rot):
    """The low-rank residual, the bias and the rotation do not depend on how the LUT is grouped:
    a descriptor that carries all of them must give x_rot . W^T + (x_rot . resB^T) . resA^T + bias."""
    N, K, R = 512, 2048, 8
    idx, lut, blob = make_kgroup(N, K, 37)
    g = torch.Generator().manual_seed(38)
    resB = (torch.randn(R, K, generator=g) * 0.05).half()
    resA = (torch.randn(N, R, generator=g) * 0.05).half()
    bias = (torch.randn(N, generator=g) * 0.1).half()
    x = make_x(1, K, seed=17)
    signs = O.rotation_signs(K, 5)
    xr = O.fht_reference(x, signs).half() if rot else x
    want = exact(xr, dense(idx, lut), bias) + (xr.double() @ resB.double().t()) @ resA.double().t()
    xd, blob_d, lut_d = x.to(DEV), blob.to(DEV), lut.to(DEV)
    keep = [resB.to(DEV), resA.to(DEV), bias.to(DEV), signs.to(DEV)]
    w, _, keep2 = _C._describe_kgroup("test", xd, K, blob_d, lut_d, bias=keep[2],
                                      signs=keep[3] if rot else None)
    w.resB, w.resA, w.R = keep[0].data_ptr(), keep[1].data_ptr(), R
    out = torch.empty(1, N, dtype=torch.float16, device=DEV)
    _lib.check(_lib.lib.flute_gemv(ctypes.byref(w), xd.data_ptr(), out.data_ptr(), _lib.F16, 0,
                                   torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rel_l2(out.cpu(), want.half()) <= TOL


def test_noalloc_entry_replays_from_a_graph():
    """The allocation-free entry with a K split (tickets and partial sums in its fixed array),
    captured once and replayed: every replay must equal the eager result."""
    N, K, split = 256, 4096, 2
    idx, lut, blob = make_kgroup(N, K, 41)
    x = make_x(1, K, seed=18).to(DEV)
    blob_d, lut_d = blob.to(DEV), lut.to(DEV)
    want = fx.qgemm_gemv_kgroup(x, blob_d, lut_d, split=split)
    w, _, keep = _C._describe_kgroup("test", x, K, blob_d, lut_d)
    out = torch.zeros_like(want)

    def call():
        _lib.check(_lib.lib.flute_gemv_noalloc(ctypes.byref(w), x.data_ptr(), out.data_ptr(), _lib.F16,
                                               split, torch.cuda.current_stream().cuda_stream))
    call()                                             # resolves the array's address outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_noalloc_entry_matches():
    N, K, split = 512, 4096, 4
    idx, lut, blob = make_kgroup(N, K, 29)
    x = make_x(1, K, seed=15).to(DEV)
    blob_d, lut_d = blob.to(DEV), lut.to(DEV)
    want = fx.qgemm_gemv_kgroup(x, blob_d, lut_d, split=split)
    w, _, keep = _C._describe_kgroup("test", x, K, blob_d, lut_d)
    out = torch.empty_like(want)
    _lib.check(_lib.lib.flute_gemv_noalloc(ctypes.byref(w), x.data_ptr(), out.data_ptr(), _lib.F16,
                                           split, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(out, want)


def test_other_entry_points_refuse():
    N, K = 256, 512
    idx, lut, blob = make_kgroup(N, K, 31)
    x = make_x(4, K, seed=16).to(DEV)
    blob_d, lut_d = blob.to(DEV), lut.to(DEV)
    w, _, keep = _C._describe_kgroup("test", x[:1].contiguous(), K, blob_d, lut_d)
    out = torch.empty(4, N, dtype=torch.float16, device=DEV)
    st = _lib.lib.flute_gemm(ctypes.byref(w), x.data_ptr(), out.data_ptr(), 4, K, N, _lib.F16,
                             torch.cuda.current_stream().cuda_stream)
    assert st == _lib.FLUTE_ERR_UNSUPPORTED
    assert b"grouped along K" in _lib.lib.flute_last_error()
