"""load_quant_model / replace_linear_with_palettized on a small torch model and a synthetic
artifact directory (the upstream loader needs a hub model and real artifacts; the swap
logic is the same: scripts/loader.py:17-62, scripts/palettized_modules.py:2921-3026)."""
import json
import os

import pytest
import torch
from torch import nn

import artifacts
import flute_oracle as O
import loader
import palettized_modules as pm
from _util import make_weight, make_x, rel_l2
from test_artifacts import _write

H, I, V = 128, 256, 384


class _MLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.gate_proj, self.up_proj = nn.Linear(H, I, bias=False), nn.Linear(H, I, bias=False)
        self.down_proj = nn.Linear(I, H, bias=True)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


class _Layer(nn.Module):
    def __init__(self):
        super().__init__()
        self.mlp = _MLP()
        self.norm = nn.LayerNorm(H)

    def forward(self, x):
        return x + self.mlp(self.norm(x))


class _Text(nn.Module):
    def __init__(self, n):
        super().__init__()
        self.embed_tokens = nn.Embedding(V, H)
        self.layers = nn.ModuleList([_Layer() for _ in range(n)])


class _LM(nn.Module):
    def __init__(self, n=2):
        super().__init__()
        self.model = _Text(n)
        self.lm_head = nn.Linear(H, V, bias=False)

    def forward(self, ids):
        # a palettized embedding returns rows in its LUT's dtype: bring them to the model's
        x = self.model.embed_tokens(ids).to(self.model.layers[0].norm.weight.dtype)
        for layer in self.model.layers:
            x = layer(x)
        return self.lm_head(x)


def _artifact_dir(tmp, n=2, tied=False):
    tensors, weights = {}, {}
    seed = 100
    for i in range(n):
        for name, (N, K) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            seed += 1
            w = make_weight(N, K, bits=4, gs=128, seed=seed)
            key = f"model.layers.{i}.mlp.{name}.weight"
            tensors[key] = _write(tmp, key.replace(".", "_"), w)
            weights[key] = w
    w = make_weight(V, H, bits=4, gs=128, seed=seed + 1)
    weights["model.lm_head.weight"] = w
    tensors["model.lm_head.weight"] = _write(tmp, "lm_head", w)
    if tied:
        tensors["model.lm_head.weight"]["tied"] = True
    else:
        we = make_weight(V, H, bits=4, gs=128, seed=seed + 2)
        weights["model.embed_tokens.weight"] = we
        tensors["model.embed_tokens.weight"] = _write(tmp, "embed", we)
    with open(os.path.join(tmp, "metadata.json"), "w") as f:
        json.dump({"tensors": tensors}, f)
    return weights


def _oracle_forward(model, weights, ids, tied):
    """The same network evaluated with the oracle's reference forward per layer."""
    def lin(key, x, bias=None):
        w = weights[key]
        return O.linear_reference(x, w["blob"].numpy(), w["lut"], w["N"], w["K"], 128, 4, bias=bias)
    we = weights["model.lm_head.weight" if tied else "model.embed_tokens.weight"]
    x = O.embedding_reference(ids, we["blob"].numpy(), we["lut"], we["N"], we["K"], 128, 4)
    x = x.to(model.model.layers[0].norm.weight.dtype)
    for i, layer in enumerate(model.model.layers):
        h = layer.norm(x)
        g = lin(f"model.layers.{i}.mlp.gate_proj.weight", h)
        u = lin(f"model.layers.{i}.mlp.up_proj.weight", h)
        x = x + lin(f"model.layers.{i}.mlp.down_proj.weight", torch.nn.functional.silu(g) * u,
                    bias=layer.mlp.down_proj.bias)
    return lin("model.lm_head.weight", x)


@pytest.mark.parametrize("tied", [False, True])
def test_load_quant_model_reference_mode_equals_the_oracle(tmp_path, tied):
    torch.manual_seed(0)
    weights = _artifact_dir(str(tmp_path), tied=tied)
    model, meta = loader.load_quant_model(str(tmp_path), "tiny-test-model", "cpu",
                                          forward="reference", dtype=torch.float32, model=_LM())
    assert meta["model_name"] == "tiny-test-model" and "tensors" in meta
    assert isinstance(model.lm_head, pm.PalettizedLinear) and model.lm_head.reference
    assert isinstance(model.model.embed_tokens, pm.PalettizedEmbedding)
    for layer in model.model.layers:
        assert isinstance(layer.mlp, pm.FusedPalettizedMLP)          # wrapped for the merged launch
        assert isinstance(layer.mlp.down_proj, pm.PalettizedLinear) and layer.mlp.down_proj.bias is not None
    if tied:
        assert model.model.embed_tokens.indices.data_ptr() == model.lm_head.indices.data_ptr()
    ids = torch.tensor([[1, 5, 300], [7, 0, 383]])
    y = model(ids)
    ref = _oracle_forward(model, weights, ids, tied)
    assert y.shape == (2, 3, V)
    assert rel_l2(y, ref) <= 1e-5


def test_load_quant_model_contract(tmp_path):
    _artifact_dir(str(tmp_path))
    with pytest.raises(ValueError, match="model="):
        loader.load_quant_model(str(tmp_path), "Qwen/Qwen3.5-9B", "cpu", forward="reference")
    with pytest.raises(ValueError, match="forward"):
        loader.load_quant_model(str(tmp_path), "x", "cpu", forward="fast", model=_LM())
    with pytest.raises(TypeError):
        loader.load_quant_model(str(tmp_path), "x", "cpu", model=_LM(), bogus=1)
    # upstream's memory-attachment keywords are accepted
    loader.load_quant_model(str(tmp_path), "x", "cpu", forward="reference", model=_LM(),
                            use_m1m2=False, m1m2_mem_size=128)
    # a name that refers to nothing in the model
    meta = artifacts.load_metadata(str(tmp_path))
    meta["tensors"]["model.layers.0.mlp.nothing.weight"] = meta["tensors"]["model.lm_head.weight"]
    with pytest.raises(AttributeError):
        artifacts.replace_linear_with_palettized(_LM(), meta, str(tmp_path), reference=True)
    holder, leaf = artifacts.resolve_module(_LM(), "model.layers.1.mlp.up_proj.weight")
    assert leaf == "up_proj" and isinstance(getattr(holder, leaf), nn.Linear)


@pytest.mark.gpu
@torch.no_grad()
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_load_quant_model_kernel_mode_matches_reference_mode(tmp_path, dtype):
    torch.manual_seed(0)
    _artifact_dir(str(tmp_path))
    base = _LM()
    ref_model, _ = loader.load_quant_model(str(tmp_path), "tiny", "cpu", forward="reference",
                                           dtype=torch.float32, model=_LM())
    ref_model.load_state_dict(base.state_dict(), strict=False)      # same dense parameters
    ker_model, _ = loader.load_quant_model(str(tmp_path), "tiny", "cuda:0", forward="kernel",
                                           dtype=dtype, model=base)
    assert not ker_model.lm_head.reference
    pm.ROUTE_CENSUS.clear()
    ids = torch.tensor([[17]])                                       # one token: the decode routes
    y = ker_model(ids.to("cuda:0")).float().cpu()
    assert pm.ROUTE_CENSUS.get("gemv_mlp") == 2 and pm.ROUTE_CENSUS.get("embedding_gather") == 1
    ref = ref_model(ids)
    assert rel_l2(y, ref) <= (2e-3 if dtype == torch.float16 else 1.5e-2)   # 16-bit hidden states
    ids = torch.randint(0, V, (2, 9))                                # prefill: the GEMM routes
    y = ker_model(ids.to("cuda:0")).float().cpu()
    assert rel_l2(y, ref_model(ids)) <= (2e-3 if dtype == torch.float16 else 1.5e-2)
    # and back: the selector switches a loaded model in place
    loader.set_forward_mode(ker_model, "reference")
    assert rel_l2(ker_model(ids.to("cuda:0")).float().cpu(), ref_model(ids)) <= \
        (2e-3 if dtype == torch.float16 else 1.5e-2)
