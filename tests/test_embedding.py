"""PalettizedEmbedding: the row gather through the idxN layout.

CPU: the module's torch path against the oracle composition (dequant rows, 16-bit
stream add, fp32 residual, adjoint rotation).  GPU: the HIP gather through the C ABI.
Without a residual or a rotation the result is a pure gather plus one exactly rounded
add, so it must be bit-identical; with them the summation order differs and the
tolerance is relative L2 <= 1e-3.
"""
import ctypes

import pytest
import torch

import flute_oracle as O
import palettized_modules as pm
from _util import make_weight, rel_l2

DEV = "cuda:0"
CASES = [
    # bits, gs, bits2, rank, rot
    (4, 128, 0, 0, False),
    (3, 64, 0, 0, False),
    (2, 16, 0, 0, False),
    (1, 128, 0, 0, False),
    (4, 128, 2, 0, False),
    (3, 32, 3, 0, False),
    (4, 128, 0, 8, False),
    (4, 64, 1, 4, True),
    (4, 128, 0, 0, True),
]


def _module(w, rot, reference):
    kw = dict(rotation_seed=7, rotation_k=w["K"]) if rot else {}
    lut_res = lambda t: None if t is None else t.to(w["lut"].dtype)
    return pm.PalettizedEmbedding(w["blob"], w["lut"], w["bits"], w["gs"], w["N"], w["K"],
                                  indices2=w["blob2"], lut2=w["lut2"],
                                  bitwidth2=w["bits2"] or None, resA=lut_res(w["resA"]),
                                  resB=lut_res(w["resB"]), reference=reference, **kw)


def _oracle(w, ids, rot):
    return O.embedding_reference(ids, w["blob"].numpy(), w["lut"], w["N"], w["K"], w["gs"],
                                 w["bits"], w["blob2"].numpy() if w["bits2"] else None, w["lut2"],
                                 w["bits2"], w["resA"], w["resB"],
                                 O.rotation_signs(w["K"], 7) if rot else None)


@pytest.mark.parametrize("bits,gs,bits2,rank,rot", CASES)
def test_reference_path_matches_oracle(bits, gs, bits2, rank, rot):
    N, K = 384, 192
    w = make_weight(N, K, bits, gs, seed=bits + gs, bits2=bits2, rank=rank)
    ids = torch.tensor([[0, 1, 127, 128], [383, 200, 5, 5]])
    y = _module(w, rot, True)(ids)
    assert y.shape == (2, 4, K) and y.dtype == torch.float16
    ref = _oracle(w, ids, rot)
    if rank == 0 and not rot:
        assert torch.equal(y, ref)
    else:
        assert rel_l2(y, ref) <= 1e-3


def test_contract_errors():
    w = make_weight(256, 128, seed=1)
    m = _module(w, False, True)
    with pytest.raises(ValueError, match="integer"):
        m(torch.zeros(3))
    with pytest.raises(ValueError, match=r"\[0, 256\)"):
        m(torch.tensor([256]))
    with pytest.raises(ValueError, match=r"\[0, 256\)"):
        m(torch.tensor([-1]))
    with pytest.raises(ValueError, match="num_embeddings"):
        pm.PalettizedEmbedding(w["blob"], w["lut"], 4, 128, 256, 128, num_embeddings=100)
    with pytest.raises(ValueError, match="BOTH"):
        pm.PalettizedEmbedding(w["blob"], w["lut"], 4, 128, 256, 128, indices2=w["blob"])
    assert (m.num_embeddings, m.embedding_dim) == (256, 128)


@pytest.mark.gpu
@pytest.mark.parametrize("bits,gs,bits2,rank,rot", CASES)
def test_hip_gather_matches_oracle(bits, gs, bits2, rank, rot):
    N, K = 512, 4096 if rot else 1024
    w = make_weight(N, K, bits, gs, seed=bits * 3 + gs, bits2=bits2, rank=rank)
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, N, (3, 17), generator=g)
    ids[0, 0], ids[0, 1] = 0, N - 1
    m = _module(w, rot, False).to(DEV)
    pm.ROUTE_CENSUS.clear()
    y = m(ids.to(DEV))
    assert y.shape == (3, 17, K) and y.dtype == torch.float16
    assert pm.ROUTE_CENSUS.get("embedding_gather") == 1
    ref = _oracle(w, ids, rot)
    if rank == 0 and not rot:
        assert torch.equal(y.cpu(), ref)
    else:
        assert rel_l2(y.cpu(), ref) <= 1e-3
    assert torch.equal(m(ids.to(DEV)), y)                       # deterministic


@pytest.mark.gpu
def test_hip_gather_bf16_table_and_refusals():
    import flute_extended as fx
    N, K = 256, 512
    w = make_weight(N, K, 4, 128, seed=9, lut_dtype=torch.bfloat16, bits2=2)
    ids = torch.arange(0, N, 7)
    y = fx.embedding_gather(ids.to(DEV), w["blob"].to(DEV), w["lut"].to(DEV), N, K, 4, 128,
                            indices2=w["blob2"].to(DEV), lut2=w["lut2"].to(DEV), bitwidth2=2)
    ref = O.embedding_reference(ids, w["blob"].numpy(), w["lut"], N, K, 128, 4,
                                w["blob2"].numpy(), w["lut2"], 2)
    assert y.dtype == torch.bfloat16 and torch.equal(y.cpu(), ref)
    with pytest.raises(RuntimeError, match=r"\[0, 256\)"):
        fx.embedding_gather(torch.tensor([300], device=DEV), w["blob"].to(DEV), w["lut"].to(DEV),
                            N, K, 4, 128)
    with pytest.raises(RuntimeError, match="integer"):
        fx.embedding_gather(torch.zeros(2, device=DEV), w["blob"].to(DEV), w["lut"].to(DEV), N, K,
                            4, 128)
