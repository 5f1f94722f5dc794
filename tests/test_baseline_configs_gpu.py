"""GPU parity at the full sizes of the benchmark configurations, through the
flute_extended op surface (which calls the C ABI).

The oracle gathers and multiplies on the CPU, so at full size it is evaluated on a
few whole 128-row tiles (first, one inside, last): a tile's bytes are contiguous in
the blob, so the tiles picked form a valid blob of their own.  The comparison is the
upstream reference forward on the same inputs, `x.float() @ W.t()` rounded once to
x's dtype (scripts/palettized_modules.py:1241-1251), relative L2 <= 1e-3, and the
fp64 closed form rounded to the output type.
"""
import ctypes

import pytest
import torch

import flute_extended as fx
import flute_oracle as O
from flute_extended import _lib
from _util import make_x, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-3


def _full_weight(N, K, seed, lut_dtype):
    """Random 4-bit blob (any byte string is a valid idx4 blob), sorted N(0, 0.02) LUT rows."""
    g = torch.Generator().manual_seed(seed)
    blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, generator=g)
    lut = (torch.randn(N // 128, 16, generator=g) * 0.02).sort(dim=1).values.to(lut_dtype)
    return blob, lut


def _tile_rows(blob, lut, N, K, tiles):
    """(sub-blob, sub-LUT, row index) of the listed 128-row tiles at group size 128."""
    per_tile = K // 64 * 4096
    sub = torch.cat([blob[t * per_tile:(t + 1) * per_tile] for t in tiles])
    rows = torch.cat([torch.arange(t * 128, (t + 1) * 128) for t in tiles])
    return sub, lut[list(tiles)], rows


def _check_rows(y, x, blob, lut, N, K, tiles, tol=TOL):
    sub, sublut, rows = _tile_rows(blob, lut, N, K, tiles)
    n = len(tiles) * 128
    ref = O.linear_reference(x, sub.numpy(), sublut, n, K, 128, 4)          # upstream's forward
    exact = O.linear_exact(x, sub.numpy(), sublut, n, K, 128, 4).to(x.dtype)
    got = y[:, rows]
    assert got.dtype == x.dtype
    assert rel_l2(got, ref) <= tol, "against the reference forward (same rounding point)"
    assert rel_l2(got, exact) <= rel_l2(ref, exact) + tol / 4, \
        "no further from the exact result than the reference forward is"


def test_config0_single_linear_4096x4096_fp16():
    """BASELINE configs[0]: M = 1, K = 4096 -> N = 4096, fp16 LUT and activations."""
    N = K = 4096
    blob, lut = _full_weight(N, K, 40, torch.float16)
    x = make_x(1, K, seed=41)
    y = fx.qgemm_gemv_splitk_stream(x.to(DEV), blob.to(DEV), lut.to(DEV), 4, 128).cpu()
    assert y.shape == (1, N) and y.dtype == torch.float16
    _check_rows(y, x, blob, lut, N, K, range(N // 128))                    # every row
    y2 = fx.qgemm_gemv_stream(x.to(DEV), blob.to(DEV), lut.to(DEV), 4, 128).cpu()
    assert torch.equal(y, y2)


@pytest.mark.parametrize("M", [16, 64, 256, 1024])
@pytest.mark.parametrize("N,K", [(12288, 4096), (4096, 12288)])
def test_config4_prefill_gemm_bf16(N, K, M):
    """BASELINE configs[4]: both shapes, every M, bf16 LUT dequantised to bf16 operands,
    bf16 activations, fp32 accumulate, bf16 out."""
    blob, lut = _full_weight(N, K, N // 128 + M, torch.bfloat16)
    x = make_x(M, K, seed=M, dtype=torch.bfloat16)
    bd, ld = blob.to(DEV), lut.to(DEV)
    y = fx.qgemm_per_group_lut(x.to(DEV), bd, ld, bitwidth=4, group_size=128,
                               indices_layout="idx4").cpu()
    assert y.shape == (M, N)
    tiles = (0, (N // 128) // 2 + 1, N // 128 - 1)
    _check_rows(y, x, blob, lut, N, K, tiles)
    assert torch.equal(y, fx.qgemm_per_group_lut(x.to(DEV), bd, ld, bitwidth=4, group_size=128,
                                                 indices_layout="idx4").cpu())


@pytest.mark.parametrize("lut_dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,K", [(12288, 4096), (4096, 12288)])
def test_config1_decode_shapes_bf16_activations(N, K, lut_dtype):
    """BASELINE configs[1]: the two GEMV shapes of the MLP block with bf16 activations."""
    blob, lut = _full_weight(N, K, 50 + N // 1024, lut_dtype)
    x = make_x(1, K, seed=51, dtype=torch.bfloat16)
    y = fx.qgemm_gemv_splitk_stream(x.to(DEV), blob.to(DEV), lut.to(DEV), 4, 128).cpu()
    _check_rows(y, x, blob, lut, N, K, (0, 7, N // 128 - 1))


@pytest.mark.parametrize("N", [1024, 512])
@pytest.mark.parametrize("split", [0, 2, 4, 8])
def test_config2_narrow_shapes_every_split(N, split):
    """BASELINE configs[2]: K = 4096 -> N = 1024 and 512, the library's own choice
    (split 0) and the swept factors 2/4/8."""
    K = 4096
    blob, lut = _full_weight(N, K, 60 + N // 512, torch.float16)
    x = make_x(1, K, seed=61)
    y = fx.qgemm_gemv_splitk_stream(x.to(DEV), blob.to(DEV), lut.to(DEV), 4, 128,
                                    split=split).cpu()
    _check_rows(y, x, blob, lut, N, K, range(N // 128))


@pytest.mark.parametrize("M", [1, 8])
def test_config3_block128_rotation_fused(M):
    """BASELINE configs[3]: block-128 Walsh-Hadamard rotation of bf16 activations in front
    of the 4096 -> 12288 weight, M = 1 (fused GEMV prologue) and M = 8 (GEMM)."""
    N, K = 12288, 4096
    blob, lut = _full_weight(N, K, 70 + M, torch.float16)
    x = make_x(M, K, seed=71, dtype=torch.bfloat16)
    signs = torch.ones(K)
    xr = O.block_fht_reference(x, 128, signs)                      # rounded to bf16 like upstream's rotate
    bd, ld = blob.to(DEV), lut.to(DEV)
    if M == 1:
        y = fx.qgemm_gemv_splitk_stream(x.to(DEV), bd, ld, 4, 128, rot_signs=signs.to(DEV),
                                        rot_block=128).cpu()
    else:
        d = _lib.FluteLinear()
        sd, xd = signs.to(DEV), x.to(DEV)
        d.q1, d.lut1, d.q1_bytes = bd.data_ptr(), ld.data_ptr(), bd.numel()
        d.N, d.K, d.b1, d.group_size, d.lut_rows, d.lut_dtype = N, K, 4, 128, N // 128, _lib.F16
        d.signs, d.rot_block = sd.data_ptr(), 128
        C = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
        st = _lib.lib.flute_gemm(ctypes.byref(d), xd.data_ptr(), C.data_ptr(), M, K, N, _lib.BF16,
                                 torch.cuda.current_stream().cuda_stream)
        assert st == 0, _lib.last_error()
        y = C.cpu()
    _check_rows(y, xr, blob, lut, N, K, (0, 50, 95))
