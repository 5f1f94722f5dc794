"""Seeded synthetic weights shaped like the benchmark configurations: uniform
b-bit indices, per-group LUT ~ N(0, 0.02) sorted ascending, activations ~ N(0, 1)."""
import numpy as np
import torch

from flute_extended import idxN


def make_weight(N, K, bits=4, gs=128, seed=0, lut_dtype=torch.float16, bits2=0, rank=0,
                bias=False, act_dtype=torch.float16, device="cpu"):
    g = torch.Generator().manual_seed(seed)
    w = {"N": N, "K": K, "bits": bits, "gs": gs, "bits2": bits2}
    rows = (N + gs - 1) // gs

    def stream(b):
        idx = torch.randint(0, 1 << b, (N, K), generator=g, dtype=torch.uint8)
        lut = (torch.randn(rows, 1 << b, generator=g) * 0.02).sort(dim=1).values.to(lut_dtype)
        blob = torch.from_numpy(idxN.pack_idxn(idx.numpy(), b))
        return idx, lut, blob

    w["idx"], w["lut"], w["blob"] = stream(bits)
    if bits2:
        w["idx2"], w["lut2"], w["blob2"] = stream(bits2)
    else:
        w["idx2"] = w["lut2"] = w["blob2"] = None
    if rank:
        w["resB"] = (torch.randn(rank, K, generator=g) * 0.05).to(act_dtype)
        w["resA"] = (torch.randn(N, rank, generator=g) * 0.05).to(act_dtype)
    else:
        w["resB"] = w["resA"] = None
    w["bias"] = (torch.randn(N, generator=g) * 0.1).to(act_dtype) if bias else None
    if device != "cpu":
        for k, v in list(w.items()):
            if torch.is_tensor(v) and k not in ("idx", "idx2"):
                w[k + "_d"] = v.to(device)
    return w


def make_x(M, K, seed=1, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(M, K, generator=g).to(dtype)


def rel_l2(a, b):
    a, b = a.detach().double().flatten(), b.detach().double().flatten()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))
