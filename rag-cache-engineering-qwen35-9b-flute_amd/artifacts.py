"""Reader of palettized weight artifacts: one metadata record + the raw member
files of an artifact directory -> a PalettizedLinear, a SplitQKV or a
PalettizedEmbedding, and the swap of a built model's layers for them
(replace_linear_with_palettized, upstream :2921-3026).

Mirrors the upstream reader (src/scripts/palettized_modules.py:229-330 for the
name/layout rules, :2411-2483 `_read_indices_and_lut`, :2486-2500 `_read_residual`,
:2503-2590 `_read_stream2`, :2619-2724 `load_palettized_weight`): same metadata
keys, same validation order, same exceptions (ValueError naming the tensor and
the fix).  Member files are raw little-endian arrays without headers:

    <san>.idx{b}[.<tag>]       idxN blob, N*K*b/8 bytes
    <san>.lut_scalar[.<tag>]   float16 [n_groups, 2^b]
    resA_file / resB_file      float16 [N, rank] / [rank, K]

Nothing here touches the device; the modules are built on the CPU and moved by
the caller.
"""
from __future__ import annotations

import hashlib
import os
import re
from typing import Dict, Optional, Tuple

import numpy as np
import torch
from torch import nn

from palettized_modules import (PalettizedEmbedding, PalettizedLinear, SplitQKV,
                                install_fused_mlp)

__all__ = ["validate_indices_layout", "load_palettized_weight", "load_palettized_embedding",
           "load_tied_pair", "load_metadata", "get_layers", "resolve_module",
           "replace_linear_with_palettized", "LAYOUT_AUDIT", "GS_MISMATCHES"]

LAYOUT_AUDIT = {"idx4": 0, "idxN": 0}     # how many members of each kind were validated
GS_MISMATCHES = []                         # (ctx, recorded gs, derived gs): stale metadata seen

_NAME = re.compile(r"^(?P<base>.*)\.idx(?P<bits>[1-4])(?P<tag>\.[^.]+)?$")


def _bits_of_layout(layout) -> int:
    if isinstance(layout, str) and layout.startswith("idx") and layout[3:].isdigit() \
            and int(layout[3:]) in (1, 2, 3, 4):
        return int(layout[3:])
    raise ValueError(f"not an idxN layout name: {layout!r}")


def _is_idxn_artifact_name(name) -> bool:
    return isinstance(name, str) and "/" not in name and _NAME.match(name) is not None


def _bits_of_artifact_name(name) -> int:
    m = _NAME.match(str(name))
    if m is None:
        raise ValueError(f"not an idxN artifact name: {name!r}")
    return int(m.group("bits"))


def _lut_name_of(name) -> Optional[str]:
    """'<san>.idx{b}' -> '<san>.lut_scalar', '<san>.idx{b}.<tag>' -> '<san>.lut_scalar.<tag>'."""
    m = _NAME.match(str(name)) if name else None
    return None if m is None else m.group("base") + ".lut_scalar" + (m.group("tag") or "")


def validate_indices_layout(meta: Dict, ctx: str) -> None:
    """The layout string, the file name and the bitwidth field must agree on one
    idxN width; anything else is refused, because a blob read at the wrong width
    has the right byte count and decodes to garbage."""
    raw = meta.get("indices_layout") or meta.get("layout")
    try:
        layout_bits = _bits_of_layout(raw)
    except ValueError:
        raise ValueError(f"{ctx}: indices_layout={raw!r} is not an idxN layout ('idx1'..'idx4'); "
                         f"older artifact formats are not readable, re-run palettization")
    index_file = str(meta.get("index_file", ""))
    if not _is_idxn_artifact_name(index_file):
        raise ValueError(f"{ctx}: index file {index_file!r} is not an idxN artifact")
    if _bits_of_artifact_name(index_file) != layout_bits:
        raise ValueError(f"{ctx}: index file {index_file!r} declares "
                         f"idx{_bits_of_artifact_name(index_file)} but indices_layout={raw!r}")
    if meta.get("bitwidth") is not None and int(meta["bitwidth"]) != layout_bits:
        raise ValueError(f"{ctx}: metadata bitwidth {meta['bitwidth']} != the layout's "
                         f"{layout_bits} bits ({index_file!r})")
    LAYOUT_AUDIT["idx4" if layout_bits == 4 else "idxN"] += 1


def _check_sha(path: str, expected: Optional[str], ctx: str, verify: bool = True) -> None:
    if not verify or not expected:
        return
    h = hashlib.sha256()
    with open(path, "rb") as f:
        for chunk in iter(lambda: f.read(1 << 22), b""):
            h.update(chunk)
    if h.hexdigest() != expected:
        raise ValueError(f"{ctx}: SHA256 mismatch for {path} (metadata {expected[:16]}..., "
                         f"got {h.hexdigest()[:16]}...)")


def _read_indices_and_lut(meta: Dict, artifacts_dir: str, ctx: str, shape=None,
                          verify_sha: bool = True
                          ) -> Tuple[torch.Tensor, torch.Tensor, int, int, int, int]:
    """(indices blob, lut [n_groups, 2^b] fp16, bitwidth, group_size, N, K).  The recorded
    group_size is honoured when n_groups == ceil(N / group_size); otherwise the value
    derived from the LUT row count is used and the mismatch is noted."""
    idx_path = os.path.join(artifacts_dir, meta["index_file"])
    lut_path = os.path.join(artifacts_dir, meta["lut_file"])
    validate_indices_layout(meta, ctx)
    _check_sha(idx_path, meta.get("sha256_idx"), ctx, verify_sha)
    _check_sha(lut_path, meta.get("sha256_lut"), ctx, verify_sha)
    blob = np.fromfile(idx_path, dtype=np.uint8)
    lut_np = np.fromfile(lut_path, dtype=np.float16)
    bits = int(meta["bitwidth"])
    palette = 1 << bits
    if lut_np.size % palette:
        raise ValueError(f"{ctx}: LUT size {lut_np.size} not divisible by palette size {palette}")
    n_groups = lut_np.size // palette
    lut = torch.from_numpy(lut_np.copy()).view(n_groups, palette)
    N, K = shape if shape is not None else meta.get("dense_shape", [None, None])
    if N is None:
        raise ValueError(f"{ctx}: metadata missing dense_shape")
    N, K = int(N), int(K)
    meta_gs = int(meta["group_size"])
    if n_groups > 0:
        derived = (N + n_groups - 1) // n_groups
        if meta_gs > 0 and n_groups == (N + meta_gs - 1) // meta_gs:
            group_size = meta_gs
        else:
            group_size = derived
            if meta_gs > 0 and meta_gs != derived:
                GS_MISMATCHES.append((ctx, meta_gs, derived))
    else:
        group_size = meta_gs
    want = N * ((K * bits + 7) // 8)
    if blob.size != want:
        raise ValueError(f"{ctx}: index file {meta['index_file']} has {blob.size} B, expected "
                         f"N*K*b/8 = {want} B (N={N}, K={K}, bitwidth={bits})")
    return torch.from_numpy(blob.copy()), lut, bits, group_size, N, K


def _read_residual(meta: Dict, artifacts_dir: str, ctx: str, N: int, K: int):
    res = meta.get("residual")
    if not res:
        return None, None
    a_path = os.path.join(artifacts_dir, res["resA_file"])
    b_path = os.path.join(artifacts_dir, res["resB_file"])
    _check_sha(a_path, res.get("sha256_resA"), ctx)
    _check_sha(b_path, res.get("sha256_resB"), ctx)
    rank = int(res["rank"])
    factors = []
    for path, rows, cols, which in ((a_path, N, rank, "resA"), (b_path, rank, K, "resB")):
        flat = np.fromfile(path, dtype=np.float16)
        if rank <= 0 or flat.size != rows * cols:
            raise ValueError(f"{ctx}: {which} file {os.path.basename(path)} holds {flat.size} "
                             f"float16 values, expected [{rows}, {cols}] for rank {rank} "
                             f"(N={N}, K={K})")
        factors.append(torch.from_numpy(flat.copy()).view(rows, cols))
    return factors[0], factors[1]


def _read_stream2(meta: Dict, artifacts_dir: str, ctx: str, N: int, K: int, bitwidth: int,
                  group_size: int, verify_sha: bool = True):
    """The second member of a declared "streams" list -> (indices2, lut2, bitwidth2).
    A declared but missing member is an error, never a silent single-stream load."""
    streams = meta.get("streams")
    if not isinstance(streams, list) or len(streams) < 2:
        raise ValueError(f"{ctx}: metadata 'streams' must be a list with at least 2 entries, "
                         f"got {streams!r}")
    base = streams[0] if isinstance(streams[0], dict) else {}
    if base.get("file") != meta.get("index_file"):
        raise ValueError(f"{ctx}: streams[0] file {base.get('file')!r} != the meta's index_file "
                         f"{meta.get('index_file')!r}; the first entry must describe the base "
                         f"stream")
    entry = streams[1]
    if not isinstance(entry, dict) or "file" not in entry:
        raise ValueError(f"{ctx}: stream-2 entry must be a dict carrying 'file' (got {entry!r})")
    idx2 = str(entry["file"])
    if not _is_idxn_artifact_name(idx2):
        raise ValueError(f"{ctx}: stream-2 file {idx2!r} is not a (tagged) idxN artifact name")
    if entry.get("bitwidth") is not None:
        bits2 = int(entry["bitwidth"])
        if bits2 != _bits_of_artifact_name(idx2):
            raise ValueError(f"{ctx}: stream-2 entry bitwidth {bits2} != the file name's "
                             f"idx{_bits_of_artifact_name(idx2)} ({idx2!r})")
    else:
        bits2 = _bits_of_artifact_name(idx2)
    lut2 = _lut_name_of(idx2)
    for fname in (idx2, lut2):
        if not os.path.exists(os.path.join(artifacts_dir, fname)):
            raise ValueError(f"{ctx}: metadata declares {len(streams)} streams but stream-2 "
                             f"member {fname!r} is missing from {artifacts_dir}; the two-stream "
                             f"artifact set is incomplete")
    member = {"index_file": idx2, "lut_file": lut2, "sha256_idx": entry.get("sha256"),
              "sha256_lut": entry.get("sha256_lut"), "bitwidth": bits2,
              "group_size": int(entry.get("gs", group_size)), "indices_layout": f"idx{bits2}"}
    indices2, lut2_t, _, _, _, _ = _read_indices_and_lut(member, artifacts_dir, f"{ctx}:stream2",
                                                         shape=(N, K), verify_sha=verify_sha)
    if entry.get("n_groups") is not None and int(entry["n_groups"]) != lut2_t.shape[0]:
        raise ValueError(f"{ctx}: stream-2 n_groups {entry['n_groups']} != the LUT's "
                         f"{lut2_t.shape[0]} rows")
    return indices2, lut2_t, bits2


def _awq_for(meta: Dict, awq_scales: Optional[Dict]):
    """(scale tensor or None, fold order or None) for one tensor record
    (scripts/palettized_modules.py:2590-2615 upstream).  `awq_scales` maps consumer
    tensor names to (K,) tensors; a tensor without an entry is unscaled.  QKV components
    are resolved on the fused record (they share the module input and the one fold).
    The fold order is the record's awq.fold_order, else its rotation.order, else None
    (the constructor then assumes the legacy rotate-then-AWQ order)."""
    if not awq_scales:
        return None, None
    key = meta.get("var") or meta.get("name")
    s = awq_scales.get(key)
    if s is None:
        return None, None
    fold = (meta.get("awq") or {}).get("fold_order") or (meta.get("rotation") or {}).get("order")
    return s, fold


def _build(meta, artifacts_dir, ctx, shape, residual, reference, verify_sha, awq_s, fold, bias):
    indices, lut, bw, gs, N, K = _read_indices_and_lut(meta, artifacts_dir, ctx, shape, verify_sha)
    resA = resB = None
    if residual:
        resA, resB = _read_residual(meta, artifacts_dir, ctx, N, K)
    indices2 = lut2 = bw2 = None
    if meta.get("streams"):
        indices2, lut2, bw2 = _read_stream2(meta, artifacts_dir, ctx, N, K, bw, gs, verify_sha)
    rot = meta.get("rotation")
    return PalettizedLinear(indices, lut, bw, gs, N, K, bias=bias, resA=resA, resB=resB,
                            indices2=indices2, lut2=lut2, bitwidth2=bw2, reference=reference,
                            rotation_seed=rot["seed"] if rot else None,
                            rotation_k=rot["k"] if rot else None, awq_scale=awq_s,
                            fold_order=fold)


def load_palettized_weight(tensor_meta: Dict, artifacts_dir: str, bias=None,
                           residual: bool = False, reference: bool = False,
                           verify_sha: bool = True, awq_scales: Optional[Dict] = None):
    """PalettizedLinear for a plain record, SplitQKV for a record with "components"
    (Q, K, V members share K; each N comes from its packed_len_bytes; a bias is sliced
    per component)."""
    var = tensor_meta.get("var", "?")
    awq_s, fold = _awq_for(tensor_meta, awq_scales)
    if "components" not in tensor_meta:
        return _build(tensor_meta, artifacts_dir, var, None, residual, reference, verify_sha,
                      awq_s, fold, None if bias is None else bias.clone())
    K = int(tensor_meta["dense_shape"][1])
    comps = []
    for name in ("Q", "K", "V"):
        cm = tensor_meta["components"][name]
        n = int(cm["packed_len_bytes"]) * 8 // (K * int(cm["bitwidth"]))
        comps.append(_build(cm, artifacts_dir, f"{var}:{name}", (n, K), residual, reference,
                            verify_sha, awq_s, fold, None))
    if bias is not None:
        off = 0
        for m in comps:
            m.bias = nn.Parameter(bias[off:off + m.N].clone())
            off += m.N
        if off != bias.shape[0]:
            raise ValueError(f"{var}: bias length {bias.shape[0]} != sum of component N ({off})")
    return SplitQKV(*comps)


def load_palettized_embedding(tensor_meta: Dict, artifacts_dir: str, residual: bool = True,
                              verify_sha: bool = True, reference: bool = True):
    """PalettizedEmbedding for one record (scripts/palettized_modules.py:2731-2767 upstream):
    both declared streams, every member checked against its sha256, the residual pair when
    asked for and present, the rotation record of a tied head.  QKV components are refused:
    an embedding is a single matrix."""
    var = tensor_meta.get("var", "?")
    if "components" in tensor_meta:
        raise ValueError(f"{var}: an embedding record carries no QKV components")
    indices, lut, bw, gs, N, K = _read_indices_and_lut(tensor_meta, artifacts_dir, var, None,
                                                       verify_sha)
    resA = resB = None
    if residual:
        resA, resB = _read_residual(tensor_meta, artifacts_dir, var, N, K)
    indices2 = lut2 = bw2 = None
    if tensor_meta.get("streams"):
        indices2, lut2, bw2 = _read_stream2(tensor_meta, artifacts_dir, var, N, K, bw, gs,
                                            verify_sha)
    rot = tensor_meta.get("rotation")
    return PalettizedEmbedding(indices, lut, bw, gs, N, K, indices2=indices2, lut2=lut2,
                               bitwidth2=bw2, resA=resA, resB=resB,
                               rotation_seed=rot["seed"] if rot else None,
                               rotation_k=rot["k"] if rot else None, reference=reference)


def _member_rows(meta: Dict):
    """Every (member, file, digest) a record names: what two consumers of one tied artifact
    set must agree on."""
    rows = [("index_file", meta.get("index_file"), meta.get("sha256_idx")),
            ("lut_file", meta.get("lut_file"), meta.get("sha256_lut"))]
    for i, entry in enumerate(meta.get("streams") or []):
        rows += [(f"streams[{i}]", entry.get("file"), entry.get("sha256")),
                 (f"streams[{i}].lut", entry.get("file"), entry.get("sha256_lut"))]
    res = meta.get("residual") or {}
    if res:
        rows += [("resA", res.get("resA_file"), res.get("sha256_resA")),
                 ("resB", res.get("resB_file"), res.get("sha256_resB"))]
    return rows


def load_tied_pair(lm_head_meta: Dict, embed_meta: Optional[Dict], artifacts_dir: str,
                   residual: bool = True, reference: bool = False, verify_sha: bool = True,
                   awq_scales: Optional[Dict] = None):
    """(PalettizedLinear, PalettizedEmbedding) over ONE artifact set (upstream :2792-2863):
    the set is read once through the lm_head record, which must say "tied": true, and the
    embedding is built on the same tensors; it inherits the head's rotation record, so its
    gather un-rotates the rows.  When the embedding has a record of its own it must name
    the same members with the same digests."""
    var = str(lm_head_meta.get("var", "?"))
    if lm_head_meta.get("tied") is not True:
        raise ValueError(f"load_tied_pair({var}): the lm_head record is not marked \"tied\": true")
    if "components" in lm_head_meta:
        raise ValueError(f"load_tied_pair({var}): a tied head is a single matrix")
    if embed_meta is not None and _member_rows(embed_meta) != _member_rows(lm_head_meta):
        raise ValueError(f"load_tied_pair({var}, {embed_meta.get('var', '?')}): the two records "
                         f"describe different artifact sets")
    lm = load_palettized_weight(lm_head_meta, artifacts_dir, residual=residual,
                                reference=reference, verify_sha=verify_sha, awq_scales=awq_scales)
    rot = lm_head_meta.get("rotation")
    emb = PalettizedEmbedding(lm.indices, lm.lut, lm.bitwidth, lm.group_size, lm.N, lm.K,
                              indices2=lm.indices2, lut2=lm.lut2,
                              bitwidth2=lm.bitwidth2 if lm.has_stream2 else None,
                              resA=lm.resA, resB=lm.resB,
                              rotation_seed=rot["seed"] if rot else None,
                              rotation_k=rot["k"] if rot else None, reference=reference)
    return lm, emb


_HEADS = ("model.lm_head.weight", "model.embed_tokens.weight")


def read_norm_gain_doc(artifacts_dir: str) -> Optional[Dict]:
    """norm_gain_edits.json of an artifact directory, or None when the set has none
    (scripts/palettized_modules.py:3122-3129 upstream)."""
    import json
    path = os.path.join(artifacts_dir, "norm_gain_edits.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f)


def _load_vector(path: str, what: str) -> torch.Tensor:
    try:
        arr = np.load(path, allow_pickle=False)
    except Exception as exc:
        raise ValueError(f"{what}: cannot read {path!r} ({exc})") from exc
    return torch.from_numpy(np.ascontiguousarray(arr))


def recover_awq_scales(model, artifacts_dir: str, metadata: Dict, norm_doc: Optional[Dict],
                       verify_sha: bool = True) -> Dict:
    """Per-channel AWQ scales of every norm group with alpha > 0, keyed by consumer tensor
    name: what PalettizedLinear(awq_scale=...) needs to compensate sets whose rotation was
    folded before the AWQ scale (scripts/palettized_modules.py:3130-3262 upstream).

    Must run on the PRISTINE model, before apply_norm_gain_edits.  The producer folded the
    inverse scale into the zero-centred RMSNorm gain exactly, w' = (1 + w)/s - 1, and stored
    the complete edited parameter, so s = (1 + w_model) / (1 + w_edited) per channel.  An
    entry that pins the scale itself ("awq_scale_file", written by exports whose gain was
    trained further) is preferred over that quotient.

    Refused loudly, never served approximately:
      * an edited gain with 1 + w' < 0 anywhere (the legacy w/s fold, not a zero-centred one);
      * scales that are not finite or leave (0, 1 + 2e-3];
      * a consumer whose own metadata records AWQ statistics (s_min / s_max / s_mean) more
        than 2 % away from the recovered ones;
      * shapes that do not match the model's parameter; a parameter the model does not have.
    Returns {} when there are no edits or none with alpha > 0."""
    edits = (norm_doc or {}).get("edits") or {}
    if not edits:
        return {}
    params = dict(model.named_parameters())
    tensors_meta = metadata.get("tensors") or {}
    scales: Dict = {}
    for pname, entry in edits.items():
        try:
            alpha = float(entry.get("alpha") or 0.0)
        except (TypeError, ValueError):
            alpha = 0.0
        if alpha <= 0.0:
            continue
        what = f"awq_recover:{pname}"
        if pname not in params:
            raise KeyError(f"{what}: the model has no such parameter (norm edit with "
                           f"alpha={alpha}): artifact set and model disagree")
        w_model = params[pname].detach().float().cpu()
        pinned = entry.get("awq_scale_file")
        if pinned:
            path = os.path.join(artifacts_dir, str(pinned))
            _check_sha(path, entry.get("awq_scale_sha256"), what, verify_sha)
            s = _load_vector(path, what).float().reshape(-1)
            if s.numel() != w_model.numel():
                raise ValueError(f"{what}: pinned scale has {s.numel()} entries, the norm "
                                 f"parameter {w_model.numel()}")
        else:
            path = os.path.join(artifacts_dir, entry["file"])
            _check_sha(path, entry.get("sha256"), what, verify_sha)
            w_edit = _load_vector(path, what).float()
            if tuple(w_edit.shape) != tuple(w_model.shape):
                raise ValueError(f"{what}: edited gain has shape {tuple(w_edit.shape)}, the "
                                 f"model's parameter {tuple(w_model.shape)}")
            gain = 1.0 + w_edit
            if bool((gain < 0).any()):
                raise ValueError(f"{what}: 1 + w_edited is negative somewhere: not a fold into a "
                                 f"zero-centred RMSNorm gain (a legacy w/s producer?); no "
                                 f"compensation is derived from it")
            s = ((1.0 + w_model) / gain.clamp(min=1e-6)).reshape(-1)
        if not bool(torch.isfinite(s).all()) or bool((s <= 0).any()) or float(s.max()) > 1.0 + 2e-3:
            raise ValueError(f"{what}: recovered scales leave (0, 1]: min {float(s.min()):.4g}, "
                             f"max {float(s.max()):.4g}; norm edit and checkpoint disagree")
        stats = {"s_min": float(s.min()), "s_max": float(s.max()), "s_mean": float(s.mean())}
        for consumer in entry.get("consumers") or []:
            cname = str(consumer)
            recorded = (tensors_meta.get(cname) or {}).get("awq") or {}
            if recorded.get("applied"):
                for key, got in stats.items():
                    want = recorded.get(key)
                    if want is not None and abs(got - float(want)) > 0.02 * max(1.0, abs(float(want))):
                        raise ValueError(f"awq_recover:{cname}: recovered {key}={got:.4g}, the "
                                         f"tensor's metadata says {float(want):.4g} (> 2 %): the "
                                         f"norm edits and the tensor describe different scales")
            scales.setdefault(cname, s)
    return scales


def apply_norm_gain_edits(model, artifacts_dir: str, verify_sha: bool = True,
                          strict: bool = True) -> Dict:
    """Copies every edited RMSNorm gain of norm_gain_edits.json (norm_edits/*.npy, each the
    COMPLETE edited parameter) into the parameter it names, cast to that parameter's dtype;
    after constructing the model, before the module swap.  Idempotent.  Returns the entries
    applied (scripts/palettized_modules.py:3029-3077 upstream)."""
    doc = read_norm_gain_doc(artifacts_dir)
    if not doc:
        return {}
    params = dict(model.named_parameters())
    applied = {}
    for pname, entry in (doc.get("edits") or {}).items():
        if pname not in params:
            if strict:
                raise KeyError(f"apply_norm_gain_edits: parameter {pname!r} not found in model")
            continue
        path = os.path.join(artifacts_dir, entry["file"])
        _check_sha(path, entry.get("sha256"), f"norm_edit:{pname}", verify_sha)
        value = _load_vector(path, f"norm_edit:{pname}")
        target = params[pname]
        if tuple(value.shape) != tuple(target.shape):
            raise ValueError(f"norm_edit:{pname}: shape {tuple(value.shape)} != parameter shape "
                             f"{tuple(target.shape)}")
        with torch.no_grad():
            target.copy_(value.to(target.dtype))
        applied[pname] = entry
    return applied


def load_metadata(artifacts_dir: str) -> Dict:
    """metadata.json of an artifact directory (upstream :3114-3117)."""
    import json
    with open(os.path.join(artifacts_dir, "metadata.json")) as f:
        return json.load(f)


def get_layers(model):
    """The decoder layer list of a causal LM or of a multimodal wrapper (upstream :2866)."""
    inner = getattr(model, "model", None)
    if inner is not None and hasattr(inner, "layers"):
        return inner.layers
    if inner is not None and hasattr(inner, "language_model"):
        return inner.language_model.layers
    raise AttributeError("Cannot find decoder layers in model structure")


def resolve_module(model, tensor_name: str):
    """(holder module, attribute name) of the module a metadata tensor name refers to
    (upstream :2874-2918): `model.layers.<i>.<path>.weight` inside the layer list,
    `model.lm_head.weight` / `model.embed_tokens.weight` on the wrapper or on its text model
    (two different modules of that name are refused)."""
    parts = tensor_name.split(".")
    if len(parts) == 3 and parts[0] == "model" and parts[2] == "weight" and \
            parts[1] in ("lm_head", "embed_tokens"):
        name = parts[1]
        holders = [h for h in (model, getattr(model, "model", model)) if hasattr(h, name)]
        if not holders:
            raise ValueError(f"resolve_module({tensor_name}): the model has no {name!r}")
        if any(getattr(h, name) is not getattr(holders[0], name) for h in holders[1:]):
            raise ValueError(f"resolve_module({tensor_name}): ambiguous, the wrapper and the "
                             f"text model hold different {name!r} modules")
        return holders[0], name
    if len(parts) < 5 or parts[0] != "model" or parts[1] != "layers" or parts[-1] != "weight":
        raise ValueError(f"resolve_module({tensor_name}): expected model.layers.<i>.<path>.weight")
    parent = get_layers(model)[int(parts[2])]
    for attr in parts[3:-2]:
        parent = getattr(parent, attr)
    return parent, parts[-2]


def replace_linear_with_palettized(model, metadata: Dict, artifacts_dir: str,
                                   residual: bool = False, reference: bool = False,
                                   verify_sha: bool = True, awq_scales: Optional[Dict] = None,
                                   heads_dir: Optional[str] = None):
    """Swap every module that metadata["tensors"] names for its palettized counterpart
    (upstream :2921-3026): linear layers (a fused QKV record becomes a SplitQKV), the
    embedding, a tied head pair from one artifact set; with heads_dir the two head records
    come from that directory's metadata instead.  A bias of the replaced layer is kept.
    Afterwards every gated MLP whose gate and up are palettized is wrapped for the merged
    decode launch (FLUTE_NO_MERGE=1 skips that).  Returns the model."""
    tensors = dict(metadata["tensors"])
    if heads_dir is not None:
        heads = load_metadata(heads_dir)["tensors"]
        for key in _HEADS:
            tensors.pop(key, None)
            if key in heads:
                tensors[key] = heads[key]
    compensated = 0
    for name, meta in tensors.items():
        src = heads_dir if (heads_dir is not None and name in _HEADS) else artifacts_dir
        if name == "model.lm_head.weight" and meta.get("tied") is True:
            lm, emb = load_tied_pair(meta, None, src, residual=residual, reference=reference,
                                     verify_sha=verify_sha, awq_scales=awq_scales)
            holder, leaf = resolve_module(model, name)
            setattr(holder, leaf, lm)
            holder, leaf = resolve_module(model, "model.embed_tokens.weight")
            setattr(holder, leaf, emb)
            compensated += lm._compensated()
            continue
        holder, leaf = resolve_module(model, name)
        old = getattr(holder, leaf)
        if name == "model.embed_tokens.weight":
            new = load_palettized_embedding(meta, src, residual=residual, verify_sha=verify_sha,
                                            reference=reference)
        else:
            bias = getattr(old, "bias", None)
            new = load_palettized_weight(meta, src, bias=None if bias is None else bias.data,
                                         residual=residual, reference=reference,
                                         verify_sha=verify_sha, awq_scales=awq_scales)
            members = (new.q_proj, new.k_proj, new.v_proj) if isinstance(new, SplitQKV) else (new,)
            compensated += sum(m._compensated() for m in members)
        setattr(holder, leaf, new)
    if compensated:
        print(f"  [ROT] rotate-then-AWQ fold order compensated on {compensated} tensor group(s)",
              flush=True)
    fused = install_fused_mlp(model)
    if fused:
        print(f"  [merge] FusedPalettizedMLP installed on {fused} MLP group(s) "
              f"(FLUTE_NO_MERGE=1 disables)", flush=True)
    return model
