"""Seeded random shapes and operand mixes through the M = 1 GEMV and the M > 1 GEMM, against the
oracle's fp64 closed form rounded once (relative L2 <= 1e-3 for float16 outputs, the benchmark's
tolerance).  The hand-picked cases of the other files cover the edges by name; this sweep covers
what nobody thought of: widths, second streams, group sizes, residual ranks, bias, rotation (the
descending power-of-two segments of K and equal blocks), explicit K splits and ragged M, drawn
together.  Every case prints its parameters first, so a failure names its case.
"""
import random

import pytest
import torch

import flute_extended as fx
import flute_oracle as O
from _util import make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-3


def _exact(w, x):
    return O.linear_exact(x, w["blob"].numpy(), w["lut"], w["N"], w["K"], w["gs"], w["bits"],
                          w["blob2"].numpy() if w["bits2"] else None, w["lut2"], w["bits2"],
                          w["resA"], w["resB"], w["bias"])


def _draw(rng, gemm):
    bits = rng.choice([4, 4, 4, 3, 2, 1])
    bits2 = rng.choice([0, 0, 0, 1, 3, 4]) if not gemm or rng.random() < 0.4 else 0
    if gemm and bits2 and (bits, bits2) not in fx.DUAL_STREAM_PAIRS:
        bits2 = 0
    gs = rng.choice([16, 32, 64, 128, 128, 128, 256, 512])
    N = 128 * rng.choice([1, 2, 3, 4, 6, 8, 12, 16])
    K = 64 * rng.choice([1, 2, 3, 4, 7, 8, 11, 16, 24, 32, 48, 64])
    rank = rng.choice([0, 0, 0, 1, 4, 16, 40])
    bias = rng.random() < 0.3
    return dict(N=N, K=K, bits=bits, bits2=bits2, gs=gs, rank=rank, bias=bias)


@pytest.mark.parametrize("seed", range(96))
def test_random_gemv(seed):
    rng = random.Random(1000 + seed)
    c = _draw(rng, gemm=False)
    K = c["K"]
    rot = rng.choice([None, None, "segments", "block"]) if K % 32 == 0 and K >= 32 else None
    block = 0
    if rot == "block":
        blocks = [b for b in (32, 64, 128, 256, 512) if K % b == 0]
        block = rng.choice(blocks)
    G = K // 64
    splits = [s for s in (1, 2, 4, 8) if G % s == 0 and (not block or (K // s) % block == 0)]
    split = rng.choice([0, 0] + splits)
    if rot == "segments" and split > 1:
        split = 0                                     # whole-row transform: the library's own choice
    print(f"case: gemv seed={seed} {c} rot={rot} block={block} split={split}", flush=True)
    w = make_weight(c["N"], K, c["bits"], c["gs"], seed=seed, bits2=c["bits2"], rank=c["rank"],
                    bias=c["bias"], device=DEV)
    x = make_x(1, K, seed=seed + 7)
    signs = O.rotation_signs(K, seed) if rot else None
    kw = dict(indices2=w.get("blob2_d"), lut2=w.get("lut2_d"), bitwidth2=c["bits2"],
              resB=w.get("resB_d"), resA=w.get("resA_d"), bias=w.get("bias_d"), split=split)
    if rot:
        kw.update(rot_signs=signs.to(DEV), rot_block=block)
    try:
        y = fx.qgemm_gemv_splitk_stream(x.to(DEV), w["blob_d"], w["lut_d"], c["bits"], c["gs"], **kw).cpu()
    except RuntimeError as err:
        # a shape the library declines must be declined for a stated reason, never served wrong
        assert any(s in str(err) for s in ("LDS", "split", "rotation", "segment")), err
        pytest.skip(f"declined: {str(err)[:100]}")
    xr = x if not rot else (O.block_fht_reference(x, block, signs) if block else O.fht_reference(x, signs)).half()
    assert rel_l2(y, _exact(w, xr).half()) <= TOL
    again = fx.qgemm_gemv_splitk_stream(x.to(DEV), w["blob_d"], w["lut_d"], c["bits"], c["gs"], **kw).cpu()
    assert torch.equal(y, again)


@pytest.mark.parametrize("seed", range(64))
def test_random_gemm(seed):
    rng = random.Random(5000 + seed)
    c = _draw(rng, gemm=True)
    M = rng.choice([2, 3, 8, 15, 16, 17, 31, 48, 64, 65, 100, 128, 200, 256, 300])
    print(f"case: gemm seed={seed} M={M} {c}", flush=True)
    w = make_weight(c["N"], c["K"], c["bits"], c["gs"], seed=100 + seed, bits2=c["bits2"],
                    rank=c["rank"], bias=c["bias"], device=DEV)
    x = make_x(M, c["K"], seed=seed + 11)
    y = fx.qgemm_dual_stream(x.to(DEV), w["blob_d"], w["lut_d"], c["bits"], c["gs"],
                             indices2=w.get("blob2_d"), lut2=w.get("lut2_d"), bitwidth2=c["bits2"],
                             resB=w.get("resB_d"), resA=w.get("resA_d"), bias=w.get("bias_d")).cpu()
    assert y.shape == (M, c["N"])
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    for m in (0, M // 2, M - 1):                      # row by row as well: no row hides behind the others
        assert rel_l2(y[m], _exact(w, x[m:m + 1]).half()[0]) <= 2 * TOL


@pytest.mark.parametrize("seed", range(32))
def test_random_lut_grouped_along_k(seed):
    """The LUT grouped along K (W[n, k] = lut[n, k // 128, idx[n, k]], no upstream form): random
    shapes the kernel serves (K a multiple of 512), splits, bias and rotation, against the closed form."""
    from flute_extended import idxN
    rng = random.Random(9000 + seed)
    N = 128 * rng.choice([1, 2, 3, 4, 8, 16, 24])
    K = 512 * rng.choice([1, 2, 3, 4, 6, 8, 16, 24])
    splits = [sp for sp in (1, 2, 4, 8) if (K // sp) % 512 == 0]
    split = rng.choice([0, 0] + splits)
    rot = rng.random() < 0.3 and split in (0, 1)
    bias = rng.random() < 0.3
    dtype = rng.choice([torch.float16, torch.float16, torch.bfloat16])
    print(f"case: kgroup seed={seed} N={N} K={K} split={split} rot={rot} bias={bias} {dtype}", flush=True)
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    lut = (torch.randn(N, K // 128, 16, generator=g) * 0.02).sort(dim=2).values.half()
    b = (torch.randn(N, generator=g) * 0.1).to(dtype) if bias else None
    blob = torch.from_numpy(idxN.pack_idxn(idx.numpy(), 4))
    x = make_x(1, K, seed=seed + 3, dtype=dtype)
    signs = O.rotation_signs(K, seed) if rot else None
    try:
        y = fx.qgemm_gemv_kgroup(x.to(DEV), blob.to(DEV), lut.to(DEV), bias=None if b is None else b.to(DEV),
                                 signs=None if signs is None else signs.to(DEV), split=split).cpu()
    except RuntimeError as err:
        assert any(s_ in str(err) for s_ in ("LDS", "split", "stages")), err
        pytest.skip(f"declined: {str(err)[:100]}")
    W = lut[torch.arange(N)[:, None], (torch.arange(K) // 128)[None, :], idx.long()].double()
    xr = (O.fht_reference(x, signs).to(dtype) if rot else x).double()
    want = xr @ W.t() + (0 if b is None else b.double())
    assert rel_l2(y, want.to(dtype)) <= (TOL if dtype == torch.float16 else 4e-3)
