"""Artifact reader (host logic, CPU): a directory of raw member files + a metadata
record -> PalettizedLinear / SplitQKV whose reference forward equals the oracle."""
import hashlib
import os

import numpy as np
import pytest
import torch

import artifacts
import flute_oracle as O
import palettized_modules as pm
from _util import make_weight, make_x, rel_l2


def _sha(path):
    return hashlib.sha256(open(path, "rb").read()).hexdigest()


def _write(tmp, san, w, stream2=False, residual=False, tag=""):
    """Member files of one tensor the way the upstream writer names them."""
    bits = w["bits"]
    idx_name, lut_name = f"{san}.idx{bits}{tag}", f"{san}.lut_scalar{tag}"
    w["blob"].numpy().tofile(os.path.join(tmp, idx_name))
    w["lut"].numpy().astype(np.float16).tofile(os.path.join(tmp, lut_name))
    meta = {"var": san, "index_file": idx_name, "lut_file": lut_name,
            "sha256_idx": _sha(os.path.join(tmp, idx_name)),
            "sha256_lut": _sha(os.path.join(tmp, lut_name)), "bitwidth": bits,
            "group_size": w["gs"], "indices_layout": f"idx{bits}", "dense_shape": [w["N"], w["K"]],
            "packed_len_bytes": w["blob"].numel()}
    if stream2:
        b2 = w["bits2"]
        n2, l2 = f"{san}.idx{b2}.2", f"{san}.lut_scalar.2"
        w["blob2"].numpy().tofile(os.path.join(tmp, n2))
        w["lut2"].numpy().astype(np.float16).tofile(os.path.join(tmp, l2))
        meta["streams"] = [{"file": idx_name},
                           {"file": n2, "sha256": _sha(os.path.join(tmp, n2)),
                            "sha256_lut": _sha(os.path.join(tmp, l2)), "bitwidth": b2,
                            "gs": w["gs"], "n_groups": w["lut2"].shape[0]}]
    if residual:
        w["resA"].numpy().tofile(os.path.join(tmp, f"{san}.resA"))
        w["resB"].numpy().tofile(os.path.join(tmp, f"{san}.resB"))
        meta["residual"] = {"resA_file": f"{san}.resA", "resB_file": f"{san}.resB",
                            "rank": w["resB"].shape[0],
                            "sha256_resA": _sha(os.path.join(tmp, f"{san}.resA")),
                            "sha256_resB": _sha(os.path.join(tmp, f"{san}.resB"))}
    return meta


def _exact(w, x, bias=None):
    return O.linear_exact(x, w["blob"].numpy(), w["lut"], w["N"], w["K"], w["gs"], w["bits"],
                          w["blob2"].numpy() if w["bits2"] else None, w["lut2"], w["bits2"],
                          w["resA"], w["resB"], bias)


def test_plain_tensor_round_trip(tmp_path):
    w = make_weight(256, 128, bits=4, gs=128, seed=1)
    meta = _write(str(tmp_path), "layers_0_mlp_up_proj", w)
    m = artifacts.load_palettized_weight(meta, str(tmp_path), reference=True)
    assert isinstance(m, pm.PalettizedLinear) and (m.N, m.K, m.bitwidth, m.group_size) == (256, 128, 4, 128)
    assert torch.equal(m.indices, w["blob"]) and torch.equal(m.lut, w["lut"])
    x = make_x(3, 128, seed=2)
    assert rel_l2(m(x), _exact(w, x).half()) <= 1e-3


def test_two_streams_residual_bias_and_rotation(tmp_path):
    w = make_weight(256, 128, bits=3, gs=64, seed=3, bits2=2, rank=4)
    meta = _write(str(tmp_path), "t", w, stream2=True, residual=True)
    meta["rotation"] = {"seed": 5, "k": 128}
    bias = torch.randn(256).half()
    m = artifacts.load_palettized_weight(meta, str(tmp_path), bias=bias, residual=True,
                                         reference=True)
    assert m.has_stream2 and m.bitwidth2 == 2 and m.has_residual() and m.rot_signs is not None
    x = make_x(2, 128, seed=4)
    xr = O.fht_reference(x, O.rotation_signs(128, 5))
    assert rel_l2(m(x), _exact(w, xr.half(), bias).half()) <= 2e-3
    # residual=False leaves the branch out even though the files exist
    m2 = artifacts.load_palettized_weight(meta, str(tmp_path), residual=False, reference=True)
    assert not m2.has_residual()


def test_group_size_recorded_or_derived(tmp_path):
    w = make_weight(384, 64, bits=4, gs=256, seed=6)        # ceil(384/256) = 2 LUT rows
    meta = _write(str(tmp_path), "g", w)
    m = artifacts.load_palettized_weight(meta, str(tmp_path), reference=True)
    assert m.group_size == 256                               # consistent: honoured
    artifacts.GS_MISMATCHES.clear()
    meta["group_size"] = 100                                 # stale: 2 rows != ceil(384/100)
    m = artifacts.load_palettized_weight(meta, str(tmp_path), reference=True)
    assert m.group_size == 192 and artifacts.GS_MISMATCHES == [("g", 100, 192)]


def test_refusals(tmp_path):
    tmp = str(tmp_path)
    w = make_weight(128, 64, bits=4, seed=7, bits2=1)
    meta = _write(tmp, "r", w, stream2=True)
    bad = dict(meta, sha256_idx="0" * 64)
    with pytest.raises(ValueError, match="SHA256 mismatch"):
        artifacts.load_palettized_weight(bad, tmp, reference=True)
    artifacts.load_palettized_weight(bad, tmp, reference=True, verify_sha=False)
    with pytest.raises(ValueError, match="indices_layout"):
        artifacts.load_palettized_weight(dict(meta, indices_layout="idx3"), tmp, reference=True)
    with pytest.raises(ValueError, match="not an idxN layout"):
        artifacts.load_palettized_weight(dict(meta, indices_layout="idx4.fd"), tmp, reference=True)
    with pytest.raises(ValueError, match="bitwidth"):
        artifacts.load_palettized_weight(dict(meta, bitwidth=3), tmp, reference=True)
    with pytest.raises(ValueError, match="expected"):
        artifacts.load_palettized_weight(dict(meta, dense_shape=[256, 64]), tmp, reference=True,
                                         verify_sha=False)
    wr = make_weight(128, 64, bits=4, seed=8, rank=4)
    mr = _write(tmp, "res", wr, residual=True)
    artifacts.load_palettized_weight(mr, tmp, residual=True, reference=True)
    short = dict(mr, residual=dict(mr["residual"], rank=8, sha256_resA=None, sha256_resB=None))
    with pytest.raises(ValueError, match=r"resA file res.resA holds 512 float16 values, expected "
                                         r"\[128, 8\]"):
        artifacts.load_palettized_weight(short, tmp, residual=True, reference=True)
    os.remove(os.path.join(tmp, "r.lut_scalar.2"))
    with pytest.raises(ValueError, match="missing"):
        artifacts.load_palettized_weight(meta, tmp, reference=True)
    with pytest.raises(ValueError, match="streams"):
        artifacts.load_palettized_weight(dict(meta, streams=[{"file": "r.idx4"}]), tmp,
                                         reference=True)


def test_name_rules():
    assert artifacts._lut_name_of("a.b.idx3.2") == "a.b.lut_scalar.2"
    assert artifacts._lut_name_of("a.idx4") == "a.lut_scalar"
    assert artifacts._bits_of_artifact_name("x.idx2.2") == 2
    assert not artifacts._is_idxn_artifact_name("x.idx5")
    assert not artifacts._is_idxn_artifact_name("d/x.idx4")
    assert not artifacts._is_idxn_artifact_name("x.idx4.a.b")


def test_qkv_components(tmp_path):
    tmp = str(tmp_path)
    K = 128
    ws = [make_weight(n, K, bits=b, gs=128, seed=10 + i)
          for i, (n, b) in enumerate([(256, 4), (128, 3), (128, 4)])]
    comps = {}
    for name, w in zip("QKV", ws):
        cm = _write(tmp, f"qkv_{name}", w)
        cm.pop("dense_shape")                               # components carry no shape of their own
        comps[name] = cm
    meta = {"var": "attn.qkv", "dense_shape": [512, K], "components": comps}
    bias = torch.randn(512).half()
    m = artifacts.load_palettized_weight(meta, tmp, bias=bias, reference=True)
    assert isinstance(m, pm.SplitQKV) and [c.N for c in (m.q_proj, m.k_proj, m.v_proj)] == [256, 128, 128]
    x = make_x(2, K, seed=20)
    ref = torch.cat([_exact(w, x, bias[o:o + w["N"]]).half()
                     for w, o in zip(ws, (0, 256, 384))], dim=-1)
    assert rel_l2(m(x), ref) <= 1e-3
    with pytest.raises(ValueError, match="bias length"):
        artifacts.load_palettized_weight(meta, tmp, bias=torch.zeros(500).half(), reference=True)


@pytest.mark.parametrize("where,order,compensated", [
    ("awq", "rotate_then_awq", True),          # the record's own awq.fold_order
    ("awq", "awq_then_rotate", False),
    ("rotation", "awq_then_rotate", False),    # only rotation.order records it
    ("rotation", "rotate_then_awq", True),
    (None, None, True),                        # no record: the legacy rotate-then-AWQ order
])
def test_awq_scale_map_with_tensor_values(tmp_path, where, order, compensated):
    """The scale map holds (K,) tensors (a truth test on one is an error), the fold order
    comes from awq.fold_order, else rotation.order, and decides whether the compensated
    rotation ((x * s) @ T) / s or the plain one runs."""
    w = make_weight(256, 128, bits=4, gs=128, seed=11)
    meta = _write(str(tmp_path), "layers_0_mlp_down_proj", w)
    meta["rotation"] = {"seed": 7, "k": 128}
    if where == "awq":
        meta["awq"] = {"fold_order": order}
    elif where == "rotation":
        meta["rotation"]["order"] = order
    s = torch.rand(128, generator=torch.Generator().manual_seed(3)) + 0.5
    scales = {"layers_0_mlp_down_proj": s, "someone_else": torch.ones(128)}
    m = artifacts.load_palettized_weight(meta, str(tmp_path), reference=True, awq_scales=scales)
    assert m.awq_scale is not None and torch.equal(m.awq_scale, s)
    assert m.fold_order == (order or "rotate_then_awq")
    assert m._compensated() is compensated
    x = make_x(2, 128, seed=5)
    signs = O.rotation_signs(128, 7)
    xr = O.fht_awq_reference(x, signs, s) if compensated else O.fht_reference(x, signs)
    assert rel_l2(m(x), _exact(w, xr).half()) <= 2e-3
    # a tensor the map does not name stays unscaled
    m0 = artifacts.load_palettized_weight(meta, str(tmp_path), reference=True,
                                          awq_scales={"other": s})
    assert m0.awq_scale is None
