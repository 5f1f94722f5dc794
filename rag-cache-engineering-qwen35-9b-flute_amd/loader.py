"""load_quant_model: the quantised-model loader (src/scripts/loader.py:17-62 upstream).

Upstream builds a Hugging Face model by hub name and swaps its layers from an artifact
directory.  Fetching a model by name is outside this package; everything after that is
here: the caller hands over a constructed torch model (anything with the
`model.layers[i].<path>` / `lm_head` / `embed_tokens` structure the artifact names refer
to), and load_quant_model swaps every tensor that metadata.json lists for its palettized
module, wraps the gated MLPs for the merged decode launch, moves the result to the device
and applies the selector upstream exposes: forward = "kernel" (the HIP kernels) or
"reference" (torch arithmetic, the only CPU-legal route).
"""
from __future__ import annotations

from palettized_modules import FusedPalettizedMLP, PalettizedEmbedding, PalettizedLinear, \
    SplitQKV, install_fused_mlp

__all__ = ["set_forward_mode", "load_quant_model"]


def set_forward_mode(model, forward: str = "kernel", fuse_mlp: bool = True):
    """Switch every palettized module of `model` to the HIP kernels ("kernel") or to the
    torch arithmetic ("reference"); with "kernel", gated MLPs are wrapped for the merged
    decode launch unless fuse_mlp is False."""
    if forward not in ("kernel", "reference"):
        raise ValueError(f"forward must be 'kernel' or 'reference', got {forward!r}")
    for m in model.modules():
        if isinstance(m, PalettizedLinear):
            if forward == "kernel" and (m.N % 128 or m.K % 64):
                raise ValueError(f"idxN layout requires N%128==0 and K%64==0, got N={m.N}, K={m.K}")
            m.reference = forward == "reference"
        if isinstance(m, PalettizedEmbedding):
            m.reference = forward == "reference"
        if isinstance(m, (FusedPalettizedMLP, SplitQKV)):
            m._merge_state = None
    if forward == "kernel" and fuse_mlp:
        install_fused_mlp(model)
    return model


def load_quant_model(artifacts_dir, model_name, device, residual=False, dtype=None,
                     forward="kernel", awq_compensation=True, heads_dir=None, model=None,
                     awq_scales=None, verify_sha=True, apply_norm_edits=True, **unused):
    """Returns (model, metadata), like upstream's loader.

    model: the constructed torch model whose layers are to be swapped.  Required: without
    it upstream would fetch `model_name` from the hub, which this package does not do (a
    ValueError says so).  model_name is kept for the signature and recorded in the
    metadata returned.
    forward: "kernel" or "reference".  residual: attach the low-rank residual pairs.
    dtype: dtype of the modules that stay dense (default float16); palettized buffers keep
    their own types.  With apply_norm_edits (default), the artifact set's norm_gain_edits.json is
    honoured as upstream does (scripts/palettized_modules.py:3378-3386): while the model is
    still pristine the AWQ scales of every alpha > 0 norm group are recovered from the edits
    (artifacts.recover_awq_scales), then the edited gains are copied into the model
    (artifacts.apply_norm_gain_edits), then the layers are swapped with those scales.
    awq_scales: a consumer name -> (K,) scale map of the caller's own takes the place of the
    recovered one; awq_compensation=False drops the compensation (differential debugging:
    the rotate-then-scale sets then serve wrong values on purpose).  heads_dir: separate artifact directory of the
    embedding and lm_head records.  Keyword arguments of upstream's memory attachments
    (use_m1m2, m1m2_mem_size, m1m2_gates_path) are accepted and ignored: those modules are
    not part of this package."""
    import torch
    import artifacts
    if forward not in ("kernel", "reference"):
        raise ValueError(f"forward must be 'kernel' or 'reference', got {forward!r}")
    if model is None:
        raise ValueError(
            f"load_quant_model: pass the constructed model as model=...; building "
            f"{model_name!r} from the hub is outside this package")
    known = {"use_m1m2", "m1m2_mem_size", "m1m2_gates_path"}
    extra = set(unused) - known
    if extra:
        raise TypeError(f"load_quant_model: unexpected arguments {sorted(extra)}")
    metadata = artifacts.load_metadata(artifacts_dir)
    model = model.to(dtype if dtype is not None else torch.float16)
    if apply_norm_edits:
        norm_doc = artifacts.read_norm_gain_doc(artifacts_dir)
        if norm_doc and awq_compensation and awq_scales is None:
            # on the pristine gains: the recovery divides them by the edited ones
            awq_scales = artifacts.recover_awq_scales(model, artifacts_dir, metadata, norm_doc,
                                                      verify_sha=verify_sha)
        artifacts.apply_norm_gain_edits(model, artifacts_dir, verify_sha=verify_sha)
    artifacts.replace_linear_with_palettized(
        model, metadata, artifacts_dir, residual=residual, reference=(forward == "reference"),
        verify_sha=verify_sha, awq_scales=awq_scales if awq_compensation else None,
        heads_dir=heads_dir)
    model = model.to(device)
    set_forward_mode(model, forward)
    metadata = dict(metadata)
    metadata["model_name"] = model_name
    return model, metadata
