"""Module layer of the idxN LUT-palettized linear layer.

Host-side counterpart of upstream src/scripts/palettized_modules.py for the hot
path only: `reference_dequant`, `PalettizedLinear` (constructor contract, the
torch "reference" forward and the kernel route chain), `FusedPalettizedMLP` and
`install_fused_mlp`.  Artifact discovery, the model loader and the training
helpers of the upstream file are outside this package.

Two execution modes, chosen explicitly at construction (`reference=`), never by
fallback:

  reference=True   the torch arithmetic of upstream's forward="reference"
                   (palettized_modules.py:1235-1251 upstream): unpack, gather,
                   fp32 matmul.  Runs anywhere.
  reference=False  the HIP kernels through flute_extended.  A missing library
                   or a CPU tensor raises; nothing is recomputed in torch.

Route order of the kernel mode (upstream :1228-1359): rotation fused into the
M = 1 GEMV -> explicit rotation -> M = 1 GEMV -> small-M fused GEMM (M <= 16)
-> per-stream GEMM (+ stream add) -> residual and bias post-adds for whatever
the chosen kernel did not fuse.  The environment switches keep upstream's names:
FLUTE_NO_FHT_FUSE, FLUTE_NO_SPLITK, FLUTE_NO_WIDE_PREF, FLUTE_NO_MERGE,
FLUTE_ROTATION (auto | fht | reference | matmul), FLUTE_MERGE_DEBUG.
"""
from __future__ import annotations

import importlib.util
import os
import sys
from typing import Optional

import numpy as np
import torch
import torch.nn as nn

_HERE = os.path.dirname(os.path.abspath(__file__))
_TRUE = ("1", "true", "True")

ROUTE_CENSUS: dict = {}      # route name -> number of forwards that took it


def _count(route: str) -> None:
    ROUTE_CENSUS[route] = ROUTE_CENSUS.get(route, 0) + 1


def _load_by_path(name: str, path: str):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_idxn = None
_fht = None


def _get_idxn():
    """idxN.py loaded standalone (numpy only), so the reference mode works
    without the compiled library."""
    global _idxn
    if _idxn is None:
        _idxn = _load_by_path("flute_idxn_standalone",
                              os.path.join(_HERE, "flute_extended", "idxN.py"))
    return _idxn


def _get_fht():
    global _fht
    if _fht is None:
        _fht = _load_by_path("flute_fht_standalone", os.path.join(_HERE, "fht.py"))
    return _fht


def _flute():
    """The kernel package; importing it loads libflute_hip.so or raises."""
    if _HERE not in sys.path:
        sys.path.insert(0, _HERE)
    import flute_extended
    return flute_extended


def _env_on(name: str) -> bool:
    return os.environ.get(name, "").strip() in _TRUE


def reference_dequant(indices_blob, lut, N: int, K: int, group_size: int,
                      bitwidth: int = 4) -> torch.Tensor:
    """W[n, k] = LUT[n // group_size, idx[n, k]] as an (N, K) fp32 tensor on the
    LUT's device (upstream :125-162).  The unpack runs on the host."""
    if bitwidth not in (1, 2, 3, 4):
        raise ValueError(f"reference_dequant supports bitwidths 1-4, got {bitwidth}")
    blob = indices_blob.detach().cpu().numpy() if torch.is_tensor(indices_blob) else indices_blob
    idx = _get_idxn().unpack_idxn(np.ascontiguousarray(blob, dtype=np.uint8).reshape(-1),
                                  N, K, int(bitwidth))
    lut_t = lut if torch.is_tensor(lut) else torch.from_numpy(np.asarray(lut))
    if lut_t.dim() != 2:
        lut_t = lut_t.view(-1, 1 << bitwidth)
    groups = torch.div(torch.arange(N, device=lut_t.device), int(group_size),
                       rounding_mode="floor").clamp_(max=lut_t.shape[0] - 1)
    idx_t = torch.from_numpy(idx.astype(np.int64)).to(lut_t.device)
    return lut_t[groups].float().gather(1, idx_t)


class PalettizedLinear(nn.Module):
    """y = x W1^T (+ x W2^T) + (x resB^T) resA^T + bias with W = LUT[n // gs, idx].

    Constructor arguments and validation follow upstream :413-542.  Buffers are
    non-persistent so that .to(device) moves them without entering state_dict.
    """

    def __init__(self, indices, lut, bitwidth, group_size, N, K, bias=None, resA=None,
                 resB=None, indices2=None, lut2=None, bitwidth2=None, reference: bool = False,
                 rotation_seed: int = None, rotation_k: int = None, awq_scale=None,
                 fold_order: str = None):
        super().__init__()
        self.bitwidth = int(bitwidth)
        self.bitwidth2 = int(bitwidth2) if bitwidth2 is not None else self.bitwidth
        self.group_size = int(group_size)
        self.N, self.K = int(N), int(K)
        self.reference = bool(reference)
        if (self.N % 128 or self.K % 64) and not self.reference:
            raise ValueError(f"idxN layout requires N%128==0 and K%64==0, got N={self.N}, "
                             f"K={self.K}")
        for which, b in (("stream-1", self.bitwidth), ("stream-2", self.bitwidth2)):
            if b not in (1, 2, 3, 4):
                raise ValueError(f"PalettizedLinear: {which} bitwidth must be 1-4, got {b}")
        want = self.N * self.K * self.bitwidth // 8
        if indices.numel() != want:
            raise ValueError(f"idx{self.bitwidth} blob numel {indices.numel()} != "
                             f"N*K*{self.bitwidth}/8 {want} (N={self.N}, K={self.K})")
        self.register_buffer("indices", indices, persistent=False)
        self.register_buffer("lut", lut, persistent=False)

        if resA is not None and resB is not None:
            if tuple(resA.shape) != (self.N, resB.shape[0]) or resB.shape[1] != self.K:
                raise ValueError(f"residual factors shape mismatch: A {tuple(resA.shape)}, "
                                 f"B {tuple(resB.shape)} for N={self.N}, K={self.K}")
            self.register_buffer("resA", resA, persistent=False)
            self.register_buffer("resB", resB, persistent=False)
        else:
            self.resA = self.resB = None

        if indices2 is None and lut2 is None:
            self.indices2 = self.lut2 = None
        elif indices2 is None or lut2 is None:
            raise ValueError("PalettizedLinear: a second stream needs BOTH indices2 and lut2")
        else:
            want2 = self.N * self.K * self.bitwidth2 // 8
            if indices2.numel() != want2:
                raise ValueError(f"idx{self.bitwidth2} stream-2 blob numel {indices2.numel()} "
                                 f"!= N*K*{self.bitwidth2}/8 {want2}")
            l1 = lut.view(-1, 1 << self.bitwidth) if lut.dim() != 2 else lut
            l2 = lut2.view(-1, 1 << self.bitwidth2) if lut2.dim() != 2 else lut2
            if l2.shape[1] != (1 << self.bitwidth2):
                raise ValueError(f"stream-2 LUT palette width {l2.shape[1]} != 2**bitwidth2")
            if l2.shape[0] != l1.shape[0]:
                raise ValueError(f"stream-2 LUT groups {l2.shape[0]} != stream-1 {l1.shape[0]}")
            self.register_buffer("indices2", indices2, persistent=False)
            self.register_buffer("lut2", lut2, persistent=False)

        if bias is not None:
            self.bias = nn.Parameter(bias)
        else:
            self.register_parameter("bias", None)

        self.rotation_seed = int(rotation_seed) if rotation_seed is not None else None
        self.rotation_k = int(rotation_k) if rotation_k is not None else None
        self.fold_order = fold_order if fold_order in ("awq_then_rotate",
                                                       "rotate_then_awq") else None
        self.rot_signs = None
        self.awq_scale = None
        self._dev_cache = {}
        self._idx_logical = self._idx_logical2 = None
        if self.rotation_seed is not None and self.rotation_k is not None:
            if self.rotation_k != self.K:
                raise ValueError(f"PalettizedLinear: rotation_k {self.rotation_k} != the input "
                                 f"dim K {self.K}")
            self.rot_signs = _get_fht().rotation_signs(self.rotation_k, self.rotation_seed)
            if awq_scale is not None:
                st = torch.as_tensor(awq_scale, dtype=torch.float32).detach().cpu()
                if st.dim() != 1 or st.numel() != self.K:
                    raise ValueError(f"PalettizedLinear: awq_scale must be a (K,) vector for "
                                     f"K={self.K}, got {tuple(st.shape)}")
                if not torch.isfinite(st).all() or bool((st <= 0).any()):
                    raise ValueError("PalettizedLinear: awq_scale must be finite and > 0")
                self.awq_scale = st
                if self.fold_order is None:
                    self.fold_order = "rotate_then_awq"
        elif awq_scale is not None:
            raise ValueError("PalettizedLinear: awq_scale passed without rotation metadata")

    # -- small accessors ----------------------------------------------------------
    @property
    def has_stream2(self) -> bool:
        return self.indices2 is not None and self.lut2 is not None

    def has_residual(self) -> bool:
        return self.resA is not None and self.resB is not None

    def _on(self, key: str, t: torch.Tensor, device) -> torch.Tensor:
        k = (key, str(device))
        if k not in self._dev_cache:
            self._dev_cache[k] = t.to(device)
        return self._dev_cache[k]

    def _signs_on(self, device):
        return self._on("signs", self.rot_signs, device)

    def _awq_scale_on(self, device):
        return None if self.awq_scale is None else self._on("awq", self.awq_scale, device)

    def _compensated(self) -> bool:
        return self.awq_scale is not None and self.fold_order == "rotate_then_awq"

    def _rotation_backend(self) -> str:
        choice = os.environ.get("FLUTE_ROTATION", "auto").strip().lower()
        if choice in ("", "auto", "fht"):
            return "auto"
        if choice in ("reference", "matmul"):
            return choice
        raise ValueError(f"FLUTE_ROTATION={choice!r} is not one of auto/fht/reference/matmul")

    def _rotate_input(self, x: torch.Tensor) -> torch.Tensor:
        """x @ T, or ((x*s) @ T)/s for rotate-then-AWQ artifacts (upstream :594-636)."""
        fht = _get_fht()
        backend = self._rotation_backend()
        signs = self._signs_on(x.device)
        if self._compensated():
            return fht.fht_apply_awq(x, signs, self._awq_scale_on(x.device), backend=backend)
        return fht.fht_apply(x, signs, backend=backend)

    # -- reference arithmetic -----------------------------------------------------
    @torch.no_grad()
    def _cache_logical_indices(self) -> "PalettizedLinear":
        """Keep the unpacked int64 indices so that reference forwards skip the
        per-call unpack (upstream :668-705)."""
        idxn = _get_idxn()
        if self._idx_logical is None:
            a = idxn.unpack_idxn(self.indices.detach().cpu().numpy(), self.N, self.K, self.bitwidth)
            self._idx_logical = torch.from_numpy(a.astype(np.int64)).to(self.lut.device)
        if self.has_stream2 and self._idx_logical2 is None:
            a = idxn.unpack_idxn(self.indices2.detach().cpu().numpy(), self.N, self.K,
                                 self.bitwidth2)
            self._idx_logical2 = torch.from_numpy(a.astype(np.int64)).to(self.lut2.device)
        return self

    def _weight_stream(self, blob, lut, cached, bits) -> torch.Tensor:
        if cached is not None:
            rows = torch.div(torch.arange(self.N, device=lut.device), self.group_size,
                             rounding_mode="floor").clamp_(max=lut.shape[0] - 1)
            return lut[rows].float().gather(1, cached)
        return reference_dequant(blob, lut, self.N, self.K, self.group_size, bits)

    def _forward_reference(self, x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        y = xf @ self._weight_stream(self.indices, self.lut, self._idx_logical, self.bitwidth).t()
        if self.has_stream2:
            y = y + xf @ self._weight_stream(self.indices2, self.lut2, self._idx_logical2,
                                             self.bitwidth2).t()
        return y.to(x.dtype)

    # -- kernel routes ------------------------------------------------------------
    def _stream_kwargs(self):
        b2 = self.bitwidth2 if self.has_stream2 else 0
        return dict(indices2=self.indices2 if self.has_stream2 else None,
                    lut2=self.lut2 if self.has_stream2 else None, bitwidth2=b2), b2

    def _cast_on(self, key: str, t: torch.Tensor, device, dtype) -> torch.Tensor:
        """t on `device` in `dtype`, contiguous; converted once and kept (artifact readers
        hand over float16 residual factors whatever the activation dtype is)."""
        k = (key, str(device), str(dtype), t.data_ptr())
        if k not in self._dev_cache:
            self._dev_cache[k] = t.detach().to(device=device, dtype=dtype).contiguous()
        return self._dev_cache[k]

    def _fusable(self, x, max_rank, device=None):
        """(resB, resA, bias) the fused kernels can take: in the activation dtype, contiguous,
        on the device of x; None when the rank is beyond the kernels' limit.  Operands in
        another floating dtype are converted once per (device, dtype) and cached."""
        device = x.device if device is None else device
        resB = resA = None
        if self.has_residual():
            if self.resB.shape[0] > max_rank:
                return None
            resB = self._cast_on("resB", self.resB, device, x.dtype)
            resA = self._cast_on("resA", self.resA, device, x.dtype)
        bias = self.bias
        if bias is not None:
            bias = self._cast_on("bias", bias, device, x.dtype)
        return resB, resA, bias

    def _gemv_route(self, x, rotated_in_kernel: bool):
        """One GEMV launch for M == 1 (upstream :870-1137).  Returns the output or
        None when the shape is outside the GEMV contract (a routing decision,
        not an error)."""
        fx = _flute()
        if x.shape[0] != 1 or x.dtype not in (torch.float16, torch.bfloat16) \
                or not x.is_contiguous() or x.requires_grad:
            return None
        if self.lut.dtype not in (torch.float16, torch.bfloat16):
            return None
        if self.lut.dtype == torch.bfloat16 and x.dtype != torch.bfloat16:
            return None                     # the kernels refuse this pair: a routing decision here
        kw, b2 = self._stream_kwargs()
        rot = {}
        if rotated_in_kernel:
            if _env_on("FLUTE_NO_FHT_FUSE") or self._rotation_backend() != "auto":
                return None
            rot = dict(rot_signs=self._signs_on(x.device),
                       awq_scale=self._awq_scale_on(x.device) if self._compensated() else None)
        wide = self.N // 128 >= 160 and not _env_on("FLUTE_NO_WIDE_PREF") and \
            fx.gemv_stream_supported(self.bitwidth, b2, self.group_size, self.N, self.K, 1)
        gate = fx.gemv_splitk_fht_supported if rotated_in_kernel else fx.gemv_splitk_supported
        if not wide and not _env_on("FLUTE_NO_SPLITK"):
            fused = self._fusable(x, fx.GEMV_SPLITK_MAX_RESIDUAL_RANK)
            rank = int(self.resB.shape[0]) if self.has_residual() else 0
            if fused is not None and gate(self.bitwidth, b2, self.group_size, self.N, self.K, 1,
                                          rank):
                _count("gemv_splitk_fht" if rotated_in_kernel else "gemv_splitk")
                return fx.qgemm_gemv_splitk_stream(x, self.indices, self.lut, self.bitwidth,
                                                   self.group_size, resB=fused[0], resA=fused[1],
                                                   bias=fused[2], **kw, **rot)
        gate = fx.gemv_fht_stream_supported if rotated_in_kernel else fx.gemv_stream_supported
        fused = self._fusable(x, 16)
        if fused is not None and gate(self.bitwidth, b2, self.group_size, self.N, self.K, 1):
            _count("gemv_fht" if rotated_in_kernel else "gemv")
            return fx.qgemm_gemv_stream(x, self.indices, self.lut, self.bitwidth,
                                        self.group_size, resB=fused[0], resA=fused[1],
                                        bias=fused[2], **kw, **rot)
        return None

    def _forward_kernel(self, x: torch.Tensor) -> torch.Tensor:
        fx = _flute()
        if isinstance(self.lut, nn.Parameter) and self.lut.requires_grad:
            raise ValueError("PalettizedLinear(kernel path): trainable LUT - the kernels need a "
                             "frozen 16-bit LUT; use reference=True for training")
        if self.lut.dtype not in (torch.float16, torch.bfloat16):
            raise ValueError(f"PalettizedLinear(kernel path): LUT dtype must be float16 or "
                             f"bfloat16, got {self.lut.dtype}")
        out_dtype = x.dtype
        if self.rot_signs is not None:
            y = self._gemv_route(x, rotated_in_kernel=True)
            if y is not None:
                return y
            x = self._rotate_input(x)
        xk = x if x.dtype in (torch.float16, torch.bfloat16) else x.half()
        if self.lut.dtype == torch.bfloat16 and xk.dtype != torch.bfloat16:
            xk = xk.to(torch.bfloat16)
        xk = xk.contiguous()
        y = self._gemv_route(xk, rotated_in_kernel=False)
        if y is not None:
            return y.to(out_dtype)
        kw, b2 = self._stream_kwargs()
        if xk.shape[0] <= fx.DUAL_STREAM_MAX_M and \
                fx.dual_stream_supported(self.bitwidth, b2, self.group_size, self.N, self.K):
            fused = self._fusable(xk, 16)
            if fused is not None:
                _count("dual_stream")
                return fx.qgemm_dual_stream(xk, self.indices, self.lut, self.bitwidth,
                                            self.group_size, resB=fused[0], resA=fused[1],
                                            bias=fused[2], **kw).to(out_dtype)
        _count("per_group_lut")
        y = fx.qgemm_per_group_lut(xk, self.indices, self.lut, bitwidth=self.bitwidth,
                                   group_size=self.group_size,
                                   indices_layout=f"idx{self.bitwidth}")
        if self.has_stream2:
            y = y + fx.qgemm_per_group_lut(xk, self.indices2, self.lut2, bitwidth=self.bitwidth2,
                                           group_size=self.group_size,
                                           indices_layout=f"idx{self.bitwidth2}")
        y = y.to(out_dtype)
        if self.has_residual():
            y = y + ((xk @ self.resB.to(xk.dtype).t()) @ self.resA.to(xk.dtype).t()).to(y.dtype)
        if self.bias is not None:
            y = y + self.bias
        return y

    def forward(self, x):
        shape = x.shape
        if x.dim() != 2:
            x = x.reshape(-1, shape[-1])
        if self.reference:
            if self.rot_signs is not None:
                x = self._rotate_input(x)
            y = self._forward_reference(x)
            if self.has_residual():
                xr = x.to(self.resA.dtype)
                y = y + ((xr @ self.resB.t()) @ self.resA.t()).to(y.dtype)
            if self.bias is not None:
                y = y + self.bias
        else:
            y = self._forward_kernel(x)
        return y.reshape(*shape[:-1], self.N)


def _operand_problem(m, device) -> Optional[str]:
    """Why a member's blobs and LUTs cannot be handed to a kernel by address, or None
    (upstream's _build_state makes the same checks, :1740-1790): uint8 blobs, LUTs of
    one 16-bit dtype, all contiguous, all on the device of the activations."""
    def bad(t, dtype):
        return t is None or not t.is_cuda or t.device != device or not t.is_contiguous() \
            or t.dtype != dtype
    if bad(m.indices, torch.uint8):
        return "indices are not a contiguous uint8 tensor on the input's device"
    if bad(m.lut, m.lut.dtype) or m.lut.dtype not in (torch.float16, torch.bfloat16):
        return "lut is not a contiguous 16-bit tensor on the input's device"
    if m.has_stream2:
        if bad(m.indices2, torch.uint8):
            return "stream-2 indices are not a contiguous uint8 tensor on the input's device"
        if bad(m.lut2, m.lut.dtype):
            return "stream-2 lut does not match the first lut's dtype and device"
    return None


def _operand_ptrs(members) -> tuple:
    """Addresses a cached segment table was built from: a table is stale once any of them
    changes (a module moved to another device and back, a buffer replaced)."""
    out = []
    for m in members:
        for name in ("indices", "lut", "indices2", "lut2", "resA", "resB", "bias"):
            t = getattr(m, name, None)
            out.append(t.data_ptr() if torch.is_tensor(t) else 0)
    return tuple(out)


class FusedPalettizedMLP(nn.Module):
    """down(act(gate(x)) * up(x)) with the decode shape (one token) collapsed
    into one merged gate+up+SiLU*mul launch followed by the down GEMV
    (upstream :1643-1908).  Every other shape takes the per-module chain."""

    def __init__(self, gate_proj, up_proj, down_proj, act_fn):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj, self.act_fn = \
            gate_proj, up_proj, down_proj, act_fn
        self._merge_state = None

    def forward(self, x):
        h = self._fused_gate_up(x)
        if h is not None:
            out = self.down_proj(h)
            return out.view(*x.shape[:-1], out.shape[-1]) if x.dim() == 3 else out
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))

    def _fused_gate_up(self, x):
        if _env_on("FLUTE_NO_MERGE"):
            return None
        lead = None
        if x.dim() == 3:
            if x.shape[0] * x.shape[1] != 1:
                return None
            lead = (x.shape[0], x.shape[1])
            x = x.reshape(1, x.shape[2])
        if x.dim() != 2 or x.shape[0] != 1 or not x.is_cuda or not x.is_contiguous() \
                or x.requires_grad or x.dtype not in (torch.float16, torch.bfloat16):
            return None
        state = self._merge_state
        if state is None or state["device"] != x.device or state["dtype"] != x.dtype or \
                state.get("ptrs") != _operand_ptrs((self.gate_proj, self.up_proj)):
            state = self._merge_state = self._build_state(x.device, x.dtype)
        if not state["ok"]:
            return None
        fx = _flute()
        _count("gemv_mlp")
        y = fx.qgemm_gemv_mlp(x, state["seg_table"], state["out"],
                              lut_dtype=self.gate_proj.lut.dtype)
        return y.view(lead[0], lead[1], y.shape[1]) if lead is not None else y

    def _build_state(self, device, dtype):
        """Fusion verdict, persistent output and the CPU segment table, once per
        (device, dtype).  `reason` says why a pair is not fused."""
        g, u = self.gate_proj, self.up_proj
        state = {"ok": False, "device": device, "dtype": dtype, "ptrs": _operand_ptrs((g, u))}

        def refuse(why):
            state["reason"] = why
            return state

        if not (isinstance(g, PalettizedLinear) and isinstance(u, PalettizedLinear)):
            return refuse("non-PalettizedLinear member")
        if g.reference or u.reference:
            return refuse("reference member")
        if act_name(self.act_fn) not in ("silu", "swish"):
            return refuse("activation is not SiLU")
        if g.K != u.K or g.N != u.N or g.N % 128:
            return refuse("K/N mismatch (not MLP twins)")
        if (g.rot_signs is None) != (u.rot_signs is None):
            return refuse("mixed rotation presence")
        if g.lut.dtype != u.lut.dtype or g.lut.dtype not in (torch.float16, torch.bfloat16):
            return refuse("lut dtype")
        if g.lut.dtype == torch.bfloat16 and dtype != torch.bfloat16:
            return refuse("bfloat16 lut needs bfloat16 activations")
        fx = _flute()
        rows, keep, specs, ranks = [], [], [], []
        for m in (g, u):
            why = _operand_problem(m, device)
            if why is not None:
                return refuse(why)
            fused = m._fusable(torch.empty(0, dtype=dtype), fx.GEMV_SPLITK_MAX_RESIDUAL_RANK,
                               device=device)
            if fused is None:
                return refuse("residual/bias contract")
            resB, resA, bias = fused
            signs = awq = None
            if m.rot_signs is not None:
                if m._rotation_backend() != "auto":
                    return refuse("pinned rotation backend")
                signs = m._signs_on(device).contiguous()
                awq = m._awq_scale_on(device) if m._compensated() else None
            b2 = m.bitwidth2 if m.has_stream2 else 0
            ptr = lambda t: 0 if t is None else t.data_ptr()
            rows.append([ptr(m.indices), ptr(m.lut), ptr(m.indices2) if b2 else 0,
                         ptr(m.lut2) if b2 else 0, ptr(resB), ptr(resA), ptr(bias), 0, m.N,
                         0 if resB is None else int(resB.shape[0]), m.bitwidth, b2,
                         m.group_size, ptr(signs), ptr(awq)])
            keep.append((signs, awq, resB, resA, bias))
            specs.append((m.bitwidth, b2, m.group_size))
            ranks.append(0 if resB is None else int(resB.shape[0]))
        if not fx.gemv_mlp_supported(g.K, g.N, specs, ranks[0], ranks[1],
                                     g.rot_signs is not None, False):
            return refuse("extension/gate: mlp")
        state.update(ok=True, seg_table=torch.tensor(rows, dtype=torch.int64),
                     out=torch.zeros(1, g.N, dtype=dtype, device=device), keepalive=keep,
                     specs=specs)
        if _env_on("FLUTE_MERGE_DEBUG"):
            print(f"  [merge] FusedPalettizedMLP ON: N={g.N}, K={g.K}, specs {specs}", flush=True)
        return state


class SplitQKV(nn.Module):
    """Three palettized projections that share their input, concatenated along the
    output axis (upstream :1390-1641).  One token takes one grouped launch that
    writes the three outputs side by side into a persistent [1, Nq+Nk+Nv] row; every
    other shape is the per-module chain plus torch.cat."""

    def __init__(self, q_proj, k_proj, v_proj):
        super().__init__()
        self.q_proj, self.k_proj, self.v_proj = q_proj, k_proj, v_proj
        self._merge_state = None

    def forward(self, x):
        y = self._gemv_multi_decode(x)
        if y is not None:
            return y
        return torch.cat([self.q_proj(x), self.k_proj(x), self.v_proj(x)], dim=-1)

    def _gemv_multi_decode(self, x):
        if _env_on("FLUTE_NO_MERGE"):
            return None
        lead = None
        if x.dim() == 3:
            if x.shape[0] * x.shape[1] != 1:
                return None
            lead = (x.shape[0], x.shape[1])
            x = x.reshape(1, x.shape[2])
        if x.dim() != 2 or x.shape[0] != 1 or not x.is_cuda or not x.is_contiguous() \
                or x.requires_grad or x.dtype not in (torch.float16, torch.bfloat16):
            return None
        state = self._merge_state
        if state is None or state["device"] != x.device or state["dtype"] != x.dtype or \
                state.get("ptrs") != _operand_ptrs((self.q_proj, self.k_proj, self.v_proj)):
            state = self._merge_state = self._build_state(x.device, x.dtype)
        if not state["ok"]:
            return None
        _count("gemv_multi")
        _flute().qgemm_gemv_multi(x, state["seg_table"], lut_dtype=self.q_proj.lut.dtype)
        y = state["out"]
        return y.view(lead[0], lead[1], y.shape[1]) if lead is not None else y

    def _build_state(self, device, dtype):
        members = (self.q_proj, self.k_proj, self.v_proj)
        state = {"ok": False, "device": device, "dtype": dtype, "ptrs": _operand_ptrs(members)}

        def refuse(why):
            state["reason"] = why
            return state

        if not all(isinstance(m, PalettizedLinear) for m in members):
            return refuse("non-PalettizedLinear member")
        if any(m.reference for m in members):
            return refuse("reference member")
        if len({m.K for m in members}) != 1 or any(m.N % 128 for m in members):
            return refuse("K mismatch or ragged N")
        if len({m.lut.dtype for m in members}) != 1 or \
                members[0].lut.dtype not in (torch.float16, torch.bfloat16):
            return refuse("lut dtype")
        if members[0].lut.dtype == torch.bfloat16 and dtype != torch.bfloat16:
            return refuse("bfloat16 lut needs bfloat16 activations")
        rot = [m.rot_signs is not None for m in members]
        if any(rot) and not all(rot):
            return refuse("mixed rotation presence")
        for m in members:
            why = _operand_problem(m, device)
            if why is not None:
                return refuse(why)
        fx = _flute()
        total = sum(m.N for m in members)
        out = torch.zeros(1, total, dtype=dtype, device=device)
        rows, keep, specs, off = [], [], [], 0
        esize = out.element_size()
        for m in members:
            fused = m._fusable(torch.empty(0, dtype=dtype), fx.GEMV_SPLITK_MAX_RESIDUAL_RANK,
                               device=device)
            if fused is None:
                return refuse("residual/bias contract")
            resB, resA, bias = fused
            signs = awq = None
            if m.rot_signs is not None:
                if m._rotation_backend() != "auto":
                    return refuse("pinned rotation backend")
                signs = m._signs_on(device).contiguous()
                awq = m._awq_scale_on(device) if m._compensated() else None
            b2 = m.bitwidth2 if m.has_stream2 else 0
            ptr = lambda t: 0 if t is None else t.data_ptr()
            rank = 0 if resB is None else int(resB.shape[0])
            keep.append((resB, resA, bias))
            rows.append([ptr(m.indices), ptr(m.lut), ptr(m.indices2) if b2 else 0,
                         ptr(m.lut2) if b2 else 0, ptr(resB), ptr(resA), ptr(bias),
                         out.data_ptr() + off * esize, m.N, rank, m.bitwidth, b2, m.group_size,
                         ptr(signs), ptr(awq)])
            keep.append((signs, awq))
            specs.append((m.bitwidth, b2, m.group_size, m.N, rank))
            off += m.N
        if (out.data_ptr() % 16) or any((r[7] % 16) for r in rows):
            return refuse("output slices are not 16-byte aligned")
        if not fx.gemv_multi_supported(members[0].K, total // 128,
                                       [(b1, b2, gs) for b1, b2, gs, _, _ in specs],
                                       sum(r for _, _, _, _, r in specs), all(rot)):
            return refuse("extension/gate: multi")
        state.update(ok=True, seg_table=torch.tensor(rows, dtype=torch.int64), out=out,
                     keepalive=keep, specs=specs)
        return state


class PalettizedEmbedding(nn.Module):
    """Embedding whose table is a palettized weight: a row gather through the idxN
    layout (upstream :1979-2335).  Dtype ladder of the module: the two streams are
    added in the LUT's 16-bit type (stream 1 first), the residual resA[ids] @ resB is
    added in fp32, a rotated (tied) table is un-rotated with the adjoint transform, and
    the row is rounded once to the LUT's dtype.  No bias.

    reference=True: torch gathers on any device (upstream's only path).
    reference=False: one HIP gather launch (flute_embedding) for ids on the GPU."""

    def __init__(self, indices, lut, bitwidth, group_size, N, K, indices2=None, lut2=None,
                 bitwidth2=None, resA=None, resB=None, num_embeddings=None, embedding_dim=None,
                 rotation_seed: int = None, rotation_k: int = None, reference: bool = True):
        super().__init__()
        self.bitwidth = int(bitwidth)
        self.bitwidth2 = int(bitwidth2) if bitwidth2 is not None else self.bitwidth
        for b in (self.bitwidth, self.bitwidth2):
            if b not in (1, 2, 3, 4):
                raise ValueError(f"PalettizedEmbedding: bitwidth {b} not in 1..4")
        self.group_size, self.N, self.K = int(group_size), int(N), int(K)
        self.reference = bool(reference)
        if num_embeddings is not None and int(num_embeddings) != self.N:
            raise ValueError(f"PalettizedEmbedding: num_embeddings {num_embeddings} != N {self.N}")
        if embedding_dim is not None and int(embedding_dim) != self.K:
            raise ValueError(f"PalettizedEmbedding: embedding_dim {embedding_dim} != K {self.K}")
        if self.N % 128 or self.K % 64:
            raise ValueError(f"idxN layout requires N%128==0 and K%64==0, got N={self.N}, "
                             f"K={self.K}")
        if indices.numel() != self.N * self.K * self.bitwidth // 8:
            raise ValueError(f"idx{self.bitwidth} blob numel {indices.numel()} != "
                             f"N*K*{self.bitwidth}/8 (N={self.N}, K={self.K})")
        lut = lut if lut.dim() == 2 else lut.view(-1, 1 << self.bitwidth)
        if lut.shape[1] != 1 << self.bitwidth:
            raise ValueError(f"PalettizedEmbedding: LUT palette width {lut.shape[1]} != "
                             f"2**bitwidth {1 << self.bitwidth}")
        self.register_buffer("indices", indices, persistent=False)
        self.register_buffer("lut", lut, persistent=False)
        if (indices2 is None) != (lut2 is None):
            raise ValueError("PalettizedEmbedding: a second stream needs BOTH indices2 and lut2")
        self.has_stream2 = indices2 is not None
        if self.has_stream2:
            if indices2.numel() != self.N * self.K * self.bitwidth2 // 8:
                raise ValueError(f"idx{self.bitwidth2} stream-2 blob numel {indices2.numel()} != "
                                 f"N*K*{self.bitwidth2}/8")
            lut2 = lut2 if lut2.dim() == 2 else lut2.view(-1, 1 << self.bitwidth2)
            if lut2.shape[1] != 1 << self.bitwidth2 or lut2.shape[0] != lut.shape[0]:
                raise ValueError("PalettizedEmbedding: stream-2 LUT must be "
                                 f"[{lut.shape[0]}, {1 << self.bitwidth2}], got {tuple(lut2.shape)}")
            self.register_buffer("indices2", indices2, persistent=False)
            self.register_buffer("lut2", lut2, persistent=False)
        else:
            self.indices2 = self.lut2 = None
        if resA is not None and resB is not None:
            if resA.shape != (self.N, resB.shape[0]) or resB.shape[1] != self.K:
                raise ValueError(f"residual factors shape mismatch: A {tuple(resA.shape)}, B "
                                 f"{tuple(resB.shape)} for N={self.N}, K={self.K}")
            self.register_buffer("resA", resA, persistent=False)
            self.register_buffer("resB", resB, persistent=False)
        else:
            self.resA = self.resB = None
        self.rot_signs = None
        if rotation_seed is not None and rotation_k is not None:
            if int(rotation_k) != self.K:
                raise ValueError(f"PalettizedEmbedding: rotation_k {rotation_k} != K {self.K}")
            self.rot_signs = _get_fht().rotation_signs(self.K, int(rotation_seed))
        self._logical = {}

    num_embeddings = property(lambda self: self.N)
    embedding_dim = property(lambda self: self.K)

    def _logical_indices(self, which):
        key = (which, self.indices.device)
        if key not in self._logical:
            blob = self.indices if which == 1 else self.indices2
            bits = self.bitwidth if which == 1 else self.bitwidth2
            idx = _get_idxn().unpack_idxn(blob.cpu().numpy(), self.N, self.K, bits)
            self._logical[key] = torch.from_numpy(idx).to(blob.device)
        return self._logical[key]

    def _gather_stream(self, ids, lut, which):
        rows = lut[torch.clamp(ids // self.group_size, max=lut.shape[0] - 1)]
        return rows.gather(-1, self._logical_indices(which)[ids].long())

    def forward(self, ids):
        if not torch.is_tensor(ids):
            ids = torch.as_tensor(ids)
        if ids.dtype not in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8):
            raise ValueError(f"PalettizedEmbedding.forward: ids must be an integer tensor, got "
                             f"dtype {ids.dtype}")
        ids = ids.long()
        capturing = ids.is_cuda and torch.cuda.is_current_stream_capturing()
        # one reduction and one host read; skipped under graph capture, where no value can
        # reach the host (the kernel writes a row of zeros for an id outside the table)
        if ids.numel() and not capturing and bool(((ids < 0) | (ids >= self.N)).any()):
            raise ValueError(f"PalettizedEmbedding.forward: ids must lie in [0, {self.N})")
        if not self.reference and ids.is_cuda:
            _count("embedding_gather")
            signs = None if self.rot_signs is None else self.rot_signs.to(ids.device)
            return _flute().embedding_gather(
                ids, self.indices, self.lut, self.N, self.K, self.bitwidth, self.group_size,
                indices2=self.indices2, lut2=self.lut2,
                bitwidth2=self.bitwidth2 if self.has_stream2 else 0,
                resB=self.resB, resA=self.resA, signs=signs, check_ids=False)
        w = self._gather_stream(ids, self.lut, 1)
        if self.has_stream2:
            w = w + self._gather_stream(ids, self.lut2, 2)
        w = w.float()
        if self.resA is not None:
            w = w + self.resA[ids].float() @ self.resB.float()
        if self.rot_signs is not None:
            w = _get_fht().fht_adjoint(w, self.rot_signs.to(w.device), backend="reference")
        return w.to(self.lut.dtype)


def act_name(fn) -> str:
    name = getattr(fn, "__name__", None) or type(fn).__name__
    return name.lower().replace("activation", "")


def install_fused_mlp(model) -> int:
    """Wrap every child named like the dense gated MLP (gate_proj/up_proj/
    down_proj/act_fn with palettized gate and up) in a FusedPalettizedMLP
    (upstream _install_fused_mlp, :1910-1942)."""
    if _env_on("FLUTE_NO_MERGE"):
        return 0
    targets = []
    for parent in model.modules():
        for name, child in parent.named_children():
            if isinstance(child, FusedPalettizedMLP):
                continue
            gate, up = getattr(child, "gate_proj", None), getattr(child, "up_proj", None)
            down, act = getattr(child, "down_proj", None), getattr(child, "act_fn", None)
            if isinstance(gate, PalettizedLinear) and isinstance(up, PalettizedLinear) \
                    and down is not None and act is not None:
                targets.append((parent, name, gate, up, down, act))
    for parent, name, gate, up, down, act in targets:
        setattr(parent, name, FusedPalettizedMLP(gate, up, down, act))
    return len(targets)
