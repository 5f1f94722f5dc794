"""load_quant_model: the upstream entry (src/scripts/loader.py:17-62) builds a
Hugging Face model by name and swaps its linear layers from an artifact
directory.  Model construction is outside this package; what this module keeps is
the selector that upstream exposes there, `forward="kernel" | "reference"`, applied
to modules the caller already built (artifacts.load_palettized_weight reads one
tensor's members from an artifact directory into such a module).
"""
from __future__ import annotations

from palettized_modules import FusedPalettizedMLP, PalettizedLinear, SplitQKV, install_fused_mlp

__all__ = ["set_forward_mode", "load_quant_model"]


def set_forward_mode(model, forward: str = "kernel", fuse_mlp: bool = True):
    """Switch every PalettizedLinear of `model` to the HIP kernels ("kernel") or
    to the torch arithmetic ("reference"); with "kernel", gated MLPs are wrapped
    for the merged decode launch unless fuse_mlp is False."""
    if forward not in ("kernel", "reference"):
        raise ValueError(f"forward must be 'kernel' or 'reference', got {forward!r}")
    for m in model.modules():
        if isinstance(m, PalettizedLinear):
            if forward == "kernel" and (m.N % 128 or m.K % 64):
                raise ValueError(f"idxN layout requires N%128==0 and K%64==0, got N={m.N}, K={m.K}")
            m.reference = forward == "reference"
        if isinstance(m, (FusedPalettizedMLP, SplitQKV)):
            m._merge_state = None
    if forward == "kernel" and fuse_mlp:
        install_fused_mlp(model)
    return model


def load_quant_model(*args, **kwargs):
    raise NotImplementedError(
        "load_quant_model needs the upstream model code and an artifact directory, neither of "
        "which is part of this package; build the modules and call set_forward_mode(model, "
        "forward='kernel' | 'reference')")
