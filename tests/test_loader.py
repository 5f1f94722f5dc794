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


# ---- norm-gain edits and the AWQ scales recovered from them ---------------------------------
# (scripts/palettized_modules.py:3029-3077, 3130-3262, 3378-3386 upstream)

def _sha_of(path):
    import hashlib
    with open(path, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def _awq_artifact_dir(tmp, pinned=False, legacy=False, stats_off=False):
    """The two-layer set above with a rotation on layer 0's gate/up, an AWQ scale folded into
    layer 0's norm gain the zero-centred way (w' = (1 + w)/s - 1) and the edit files that
    record it.  Returns (weights, model with the pristine gain, the scale)."""
    import numpy as np
    weights = _artifact_dir(tmp)
    meta = artifacts.load_metadata(tmp)
    g = torch.Generator().manual_seed(5)
    s = (torch.rand(H, generator=g) * 0.7 + 0.3).float()                # (0.3, 1]
    torch.manual_seed(1)
    model = _LM()
    with torch.no_grad():
        model.model.layers[0].norm.weight.copy_(torch.randn(H, generator=g) * 0.1)
    w0 = model.model.layers[0].norm.weight.detach().float()
    edited = (w0 / s) if legacy else ((1.0 + w0) / s - 1.0)
    if legacy:
        edited = edited - 2.0                                             # 1 + w' < 0: not a gain fold
    os.makedirs(os.path.join(tmp, "norm_edits"), exist_ok=True)
    np.save(os.path.join(tmp, "norm_edits", "l0.npy"), edited.numpy())
    # (a consumer is named by its key in metadata["tensors"], which is also its "var")
    consumers = ["model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight"]
    entry = {"file": "norm_edits/l0.npy", "sha256": _sha_of(os.path.join(tmp, "norm_edits", "l0.npy")),
             "alpha": 0.5, "consumers": consumers}
    if pinned:
        np.save(os.path.join(tmp, "norm_edits", "l0_scale.npy"), s.numpy())
        entry["awq_scale_file"] = "norm_edits/l0_scale.npy"
        entry["awq_scale_sha256"] = _sha_of(os.path.join(tmp, "norm_edits", "l0_scale.npy"))
    doc = {"edits": {"model.layers.0.norm.weight": entry,
                     "model.layers.1.norm.weight": {"file": "norm_edits/l0.npy", "alpha": 0.0,
                                                    "consumers": []}}}
    with open(os.path.join(tmp, "norm_gain_edits.json"), "w") as f:
        json.dump(doc, f)
    for key in ("model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight"):
        rec = meta["tensors"][key]
        rec["var"] = key
        rec["rotation"] = {"seed": 3, "k": H}
        off = 0.2 if stats_off else 0.0
        rec["awq"] = {"applied": True, "fold_order": "rotate_then_awq", "s_min": float(s.min()) + off,
                      "s_max": float(s.max()), "s_mean": float(s.mean())}
    with open(os.path.join(tmp, "metadata.json"), "w") as f:
        json.dump(meta, f)
    return weights, model, s


@pytest.mark.parametrize("pinned", [False, True])
def test_awq_scales_are_recovered_from_the_norm_edits(tmp_path, pinned):
    tmp = str(tmp_path)
    _, model, s = _awq_artifact_dir(tmp, pinned=pinned)
    meta, doc = artifacts.load_metadata(tmp), artifacts.read_norm_gain_doc(tmp)
    if pinned:
        # a gain trained further after the fold: the quotient would be wrong, the pinned file is not
        import numpy as np
        np.save(os.path.join(tmp, "norm_edits", "l0.npy"), np.zeros(H, dtype=np.float32))
        doc["edits"]["model.layers.0.norm.weight"]["sha256"] = None
    scales = artifacts.recover_awq_scales(model, tmp, meta, doc)
    assert set(scales) == {"model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight"}
    for got in scales.values():
        assert got.dtype == torch.float32 and got.shape == (H,)
        assert torch.allclose(got, s, rtol=(0 if pinned else 2e-6), atol=0)
    # alpha == 0 entries contribute nothing; no document, no scales
    assert artifacts.recover_awq_scales(model, tmp, meta, None) == {}
    assert artifacts.recover_awq_scales(model, tmp, meta, {"edits": {}}) == {}


def test_norm_edits_are_copied_into_the_model_once(tmp_path):
    import numpy as np
    tmp = str(tmp_path)
    _, model, s = _awq_artifact_dir(tmp)
    doc = artifacts.read_norm_gain_doc(tmp)
    del doc["edits"]["model.layers.1.norm.weight"]                   # (its file is layer 0's: shape ok too)
    before = model.model.layers[0].norm.weight.detach().clone()
    applied = artifacts.apply_norm_gain_edits(model, tmp)
    assert "model.layers.0.norm.weight" in applied
    want = torch.from_numpy(np.load(os.path.join(tmp, "norm_edits", "l0.npy")))
    assert torch.equal(model.model.layers[0].norm.weight.detach(), want)
    assert torch.allclose((1 + before) / (1 + want), s, rtol=1e-5)
    artifacts.apply_norm_gain_edits(model, tmp)                       # idempotent
    assert torch.equal(model.model.layers[0].norm.weight.detach(), want)
    assert artifacts.apply_norm_gain_edits(_LM(), str(tmp_path / "nothing_here")) == {}


def test_awq_recovery_refusals(tmp_path):
    import numpy as np
    tmp = str(tmp_path)
    # the legacy w/s fold: 1 + w' negative -> refused, not served approximately
    _, model, _ = _awq_artifact_dir(tmp, legacy=True)
    with pytest.raises(ValueError, match="zero-centred"):
        artifacts.recover_awq_scales(model, tmp, artifacts.load_metadata(tmp), artifacts.read_norm_gain_doc(tmp))
    # the tensors' own statistics disagree with the recovered scale
    _, model, _ = _awq_artifact_dir(tmp, stats_off=True)
    with pytest.raises(ValueError, match="s_min"):
        artifacts.recover_awq_scales(model, tmp, artifacts.load_metadata(tmp), artifacts.read_norm_gain_doc(tmp))
    _, model, s = _awq_artifact_dir(tmp)
    meta, doc = artifacts.load_metadata(tmp), artifacts.read_norm_gain_doc(tmp)
    # scales beyond (0, 1]: a model whose gain is not the one the edit was made from
    other = _LM()
    with torch.no_grad():
        other.model.layers[0].norm.weight.fill_(3.0)
    with pytest.raises(ValueError, match=r"\(0, 1\]"):
        artifacts.recover_awq_scales(other, tmp, meta, doc)
    # a parameter the model does not have; a corrupted edit file; a wrong shape
    doc2 = {"edits": {"model.layers.9.norm.weight": doc["edits"]["model.layers.0.norm.weight"]}}
    with pytest.raises(KeyError):
        artifacts.recover_awq_scales(model, tmp, meta, doc2)
    with open(os.path.join(tmp, "norm_gain_edits.json"), "w") as f:
        json.dump(doc2, f)
    with pytest.raises(KeyError):
        artifacts.apply_norm_gain_edits(model, tmp, strict=True)
    assert artifacts.apply_norm_gain_edits(model, tmp, strict=False) == {}
    np.save(os.path.join(tmp, "norm_edits", "l0.npy"), np.zeros(H, dtype=np.float32))
    with pytest.raises(ValueError, match="SHA256"):
        artifacts.recover_awq_scales(model, tmp, meta, doc)
    np.save(os.path.join(tmp, "norm_edits", "l0.npy"), np.zeros(H + 1, dtype=np.float32))
    with pytest.raises(ValueError, match="shape"):
        artifacts.recover_awq_scales(model, tmp, meta, doc, verify_sha=False)


@torch.no_grad()
def test_load_quant_model_recovers_and_applies_by_itself(tmp_path):
    """load_quant_model on an AWQ set: the scales come from the edits (recovered on the pristine
    gains), the gains are edited, and the rotated consumers carry the compensation: the same
    module values as when the caller hands the scale map over."""
    tmp = str(tmp_path)
    _, model, s = _awq_artifact_dir(tmp)
    state = {k: v.clone() for k, v in model.state_dict().items()}
    auto, _ = loader.load_quant_model(tmp, "tiny", "cpu", forward="reference", dtype=torch.float32,
                                      model=model)
    gate = auto.model.layers[0].mlp.gate_proj
    assert gate.awq_scale is not None and torch.allclose(gate.awq_scale.float(), s, rtol=2e-6)
    assert gate._compensated() and auto.model.layers[1].mlp.gate_proj.awq_scale is None
    edited = auto.model.layers[0].norm.weight
    assert torch.allclose((1 + state["model.layers.0.norm.weight"]) / (1 + edited), s, rtol=1e-5)
    # the caller's own map takes the recovered one's place; awq_compensation=False drops both
    manual = _LM()
    manual.load_state_dict(state)
    names = ["model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight"]
    manual, _ = loader.load_quant_model(tmp, "tiny", "cpu", forward="reference", dtype=torch.float32,
                                        model=manual, awq_scales={n: s for n in names})
    ids = torch.tensor([[3, 200, 77]])
    assert rel_l2(auto(ids), manual(ids)) <= 1e-5        # the recovered scale is s to a few ulps
    plain = _LM()
    plain.load_state_dict(state)
    plain, _ = loader.load_quant_model(tmp, "tiny", "cpu", forward="reference", dtype=torch.float32,
                                       model=plain, awq_compensation=False)
    assert plain.model.layers[0].mlp.gate_proj.awq_scale is None
    assert rel_l2(plain(ids), auto(ids)) > 1e-3
    # apply_norm_edits=False leaves the model's gains alone and recovers nothing
    raw = _LM()
    raw.load_state_dict(state)
    raw, _ = loader.load_quant_model(tmp, "tiny", "cpu", forward="reference", dtype=torch.float32,
                                     model=raw, apply_norm_edits=False)
    assert torch.equal(raw.model.layers[0].norm.weight, state["model.layers.0.norm.weight"])
    assert raw.model.layers[0].mlp.gate_proj.awq_scale is None


@pytest.mark.gpu
@torch.no_grad()
def test_kernel_mode_matches_reference_mode_with_awq_compensation(tmp_path):
    tmp = str(tmp_path)
    _, model, s = _awq_artifact_dir(tmp)
    state = {k: v.clone() for k, v in model.state_dict().items()}
    ref_model, _ = loader.load_quant_model(tmp, "tiny", "cpu", forward="reference",
                                           dtype=torch.float32, model=model)
    base = _LM()
    base.load_state_dict(state)
    ker_model, _ = loader.load_quant_model(tmp, "tiny", "cuda:0", forward="kernel",
                                           dtype=torch.float16, model=base)
    assert ker_model.model.layers[0].mlp.gate_proj.awq_scale is not None
    for ids in (torch.tensor([[17]]), torch.randint(0, V, (2, 9))):   # decode routes, prefill routes
        y = ker_model(ids.to("cuda:0")).float().cpu()
        assert rel_l2(y, ref_model(ids)) <= 2e-3
