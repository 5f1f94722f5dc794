"""Walsh-Hadamard boundary-fold rotation: x @ T in O(K log K).

Same public surface as the upstream module of this name
(src/flute_extended/fht.py): rotation_signs, segments, hadamard_matrix,
build_rotation_matrix, fht_apply, fht_apply_awq, fht_adjoint, fht_apply_,
kernel_available, and the backend names "auto" | "kernel" | "reference" |
"matmul".  Like upstream it lives NEXT TO the flute_extended package, imports it
lazily, and stays importable on a machine without the compiled library.

Conventions (upstream fht.py:19-44):

    T = blockdiag_b( H_b diag(s_b) / sqrt(b) )   over the descending
                                                 power-of-two segments of K
    x @ T   = ((x @ H) * s) / sqrt(b)            signs on the output
    y @ T^T = ((y * s) @ H) / sqrt(b)            signs on the input
    s       = randint(0, 2, (K,), manual_seed(seed + 4242)) * 2 - 1

Backends: "kernel" is the HIP kernel (flute_extended._C.fht_*), refused loudly
when the library or a GPU tensor is missing; "auto" picks it for GPU tensors
whose K the kernel serves and the torch butterfly otherwise; "reference" is the
torch butterfly (fp32, any device); "matmul" builds the explicit matrix.
The kernel and the torch butterfly run the same stage order, so for fp32 I/O
they agree bit for bit.
"""
from __future__ import annotations

import math
import os
import sys
from typing import List, Optional, Tuple

import torch

__all__ = [
    "rotation_signs", "segments", "build_rotation_matrix", "hadamard_matrix",
    "fht_apply", "fht_apply_awq", "fht_adjoint", "fht_apply_", "FhtBackend",
    "kernel_available",
]

FhtBackend = str
_BACKENDS = ("auto", "kernel", "reference", "matmul")
_HERE = os.path.dirname(os.path.abspath(__file__))
_MAX_SEGMENT = 16384          # columns one workgroup transforms in LDS


# ---------------------------------------------------------------------------
# signs, segments, explicit matrices
# ---------------------------------------------------------------------------

def rotation_signs(K: int, seed: int) -> torch.Tensor:
    """(K,) float32 vector of +-1, deterministic in (K, seed)."""
    gen = torch.Generator().manual_seed(int(seed) + 4242)
    return torch.randint(0, 2, (int(K),), generator=gen).float().mul(2).sub(1)


def segments(K: int) -> List[Tuple[int, int]]:
    """[(offset, size)] of the descending power-of-two blocks of K
    (12288 -> [(0, 8192), (8192, 4096)])."""
    K = int(K)
    if K < 1:
        raise ValueError("segments: K must be >= 1")
    out, off = [], 0
    while off < K:
        b = 1 << ((K - off).bit_length() - 1)
        out.append((off, b))
        off += b
    return out


def hadamard_matrix(K: int) -> torch.Tensor:
    """Sylvester H_K (entries +-1, symmetric, H @ H = K I): H[i, j] = (-1)^popcount(i & j)."""
    K = int(K)
    if K < 1 or K & (K - 1):
        raise ValueError("hadamard_matrix needs a power-of-two K")
    idx = torch.arange(K)
    both = idx[:, None] & idx[None, :]
    parity = torch.zeros_like(both)
    while bool(both.any()):
        parity ^= both & 1
        both = both >> 1
    return (1 - 2 * parity).to(torch.float32)


def _matrix_from_signs(signs: torch.Tensor) -> torch.Tensor:
    K = int(signs.numel())
    s = signs.detach().float().cpu()
    T = torch.zeros(K, K, dtype=torch.float32)
    for off, b in segments(K):
        T[off:off + b, off:off + b] = hadamard_matrix(b) * s[off:off + b].view(1, b) / math.sqrt(b)
    return T


def build_rotation_matrix(K: int, seed: int, device=None) -> torch.Tensor:
    """Explicit (K, K) T; ground truth for tests and the "matmul" backend."""
    T = _matrix_from_signs(rotation_signs(K, seed))
    return T.to(device) if device is not None else T


def build_rotation_matrix_from_signs(signs: torch.Tensor, K: int, device=None) -> torch.Tensor:
    if int(signs.numel()) != int(K):
        raise ValueError("signs must have K entries")
    T = _matrix_from_signs(signs)
    return T.to(device) if device is not None else T


# ---------------------------------------------------------------------------
# torch butterfly
# ---------------------------------------------------------------------------

def _butterfly(v: torch.Tensor) -> torch.Tensor:
    """v @ H_b on the last axis of an (R, b) fp32 tensor, stage length doubling:
    each pair (i, i + len) of a 2*len group becomes (a + c, a - c)."""
    R, b = v.shape
    ln = 1
    while ln < b:
        pairs = v.view(R, b // (2 * ln), 2, ln)
        lo, hi = pairs[:, :, 0, :], pairs[:, :, 1, :]
        v = torch.stack((lo + hi, lo - hi), dim=2).reshape(R, b)
        ln *= 2
    return v


def _check(x: torch.Tensor, signs: torch.Tensor) -> Tuple[int, int]:
    """(rows, K) of x seen as a matrix over its last axis; refuses what upstream refuses
    (fht.py:195-203 upstream), with its exception types."""
    K = int(x.shape[-1]) if x.dim() > 0 else 0
    if not x.is_floating_point():
        raise TypeError(f"fht: x must be floating point, got {x.dtype}")
    if K < 1:
        raise ValueError("fht: x's last dim must be >= 1")
    if tuple(signs.shape) != (K,):
        raise ValueError(f"fht: signs must be a (K,) vector matching x's last dim "
                         f"(got signs {tuple(signs.shape)}, x {tuple(x.shape)})")
    return x.numel() // K, K


def _per_segment(x: torch.Tensor, signs: torch.Tensor, signs_first: bool) -> torch.Tensor:
    """The torch transform both directions share: every segment of the last axis goes through
    the butterfly in fp32 and is scaled by 1/sqrt(its width); the signs multiply the output
    (forward, x @ T) or the input (adjoint, v @ T^T).  fht.py:206-238 upstream."""
    rows, K = _check(x, signs)
    widths = [b for _, b in segments(K)]
    flat = x.reshape(rows, K).to(torch.float32)
    sgn = signs.to(device=flat.device, dtype=torch.float32)
    pieces = []
    for part, sg in zip(torch.split(flat, widths, dim=1), torch.split(sgn, widths)):
        part = part * sg if signs_first else part
        part = _butterfly(part.contiguous())
        part = part if signs_first else part * sg
        pieces.append(part * (1.0 / math.sqrt(part.shape[1])))
    return torch.cat(pieces, dim=1).reshape(x.shape).to(x.dtype)


def fht_reference(x: torch.Tensor, signs: torch.Tensor) -> torch.Tensor:
    """((x @ H) * s) * (1/sqrt(b)) per segment, fp32, returned in x's dtype."""
    return _per_segment(x, signs, signs_first=False)


def fht_reference_adjoint(v: torch.Tensor, signs: torch.Tensor) -> torch.Tensor:
    """((v * s) @ H) * (1/sqrt(b)) per segment."""
    return _per_segment(v, signs, signs_first=True)


def fht_matmul(x: torch.Tensor, signs: torch.Tensor, K: Optional[int] = None,
               seed: Optional[int] = None) -> torch.Tensor:
    """Explicit x @ T (builds the K x K matrix)."""
    M, Kdim = _check(x, signs)
    s = rotation_signs(K if K is not None else Kdim, seed) if seed is not None else signs
    T = _matrix_from_signs(s).to(x.device)
    return (x.reshape(M, Kdim).float() @ T).reshape(x.shape).to(x.dtype)


# ---------------------------------------------------------------------------
# kernel dispatch
# ---------------------------------------------------------------------------

_C = None
_C_tried = False


def _load_kernel():
    """flute_extended._C, or None when the package (its compiled library) is absent."""
    global _C, _C_tried
    if not _C_tried:
        _C_tried = True
        if _HERE not in sys.path:
            sys.path.insert(0, _HERE)
        try:
            import flute_extended._C as mod
            _C = mod
        except Exception:
            _C = None
    return _C


def kernel_available(x: Optional[torch.Tensor] = None) -> bool:
    if _load_kernel() is None:
        return False
    return True if x is None else bool(x.is_cuda)


def _kernel_eligible(K: int) -> bool:
    """K % 32 == 0, 32 <= K <= 65504 and every segment fits one LDS tile."""
    if K < 32 or K % 32 != 0 or K > 65504:
        return False
    return segments(K)[0][1] <= _MAX_SEGMENT


def _resolve(backend: str, x: torch.Tensor) -> str:
    if backend not in _BACKENDS:
        raise ValueError(f"fht: unknown backend {backend!r} (expected one of {_BACKENDS})")
    if backend in ("reference", "matmul"):
        return backend
    usable = _load_kernel() is not None and x.is_cuda
    if backend == "kernel":
        if not usable:
            raise RuntimeError("fht(backend='kernel'): the HIP library is unavailable or the "
                               "input is not on the GPU. Build it with `make -C csrc`, or use "
                               "backend='auto'/'reference'. Never a silent fallback.")
        if not _kernel_eligible(int(x.shape[-1])):
            raise RuntimeError(f"fht(backend='kernel'): K={int(x.shape[-1])} is outside the "
                               "kernel contract (K % 32 == 0, 32 <= K <= 65504, every segment "
                               "<= 16384)")
        return "kernel"
    return "kernel" if usable and _kernel_eligible(int(x.shape[-1])) else "reference"


def _signs_for_kernel(signs: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    if signs.device != x.device or signs.dtype != torch.float32 or not signs.is_contiguous():
        signs = signs.detach().to(x.device, torch.float32).contiguous()
    return signs


def _run(x2d: torch.Tensor, signs: torch.Tensor, transpose: bool, backend: str) -> torch.Tensor:
    if backend == "kernel":
        C = _load_kernel()
        sf = _signs_for_kernel(signs, x2d)
        return C.fht_backward(x2d, sf) if transpose else C.fht_forward(x2d, sf)
    if backend == "matmul":
        T = _matrix_from_signs(signs).to(x2d.device)
        return (x2d.float() @ (T.t() if transpose else T)).to(x2d.dtype)
    return fht_reference_adjoint(x2d, signs) if transpose else fht_reference(x2d, signs)


class _FhtFn(torch.autograd.Function):
    """y = x @ T (transpose=False) or x @ T^T; the backward is the other one
    because T is orthogonal."""

    @staticmethod
    def forward(ctx, x2d, signs, transpose, backend):
        ctx.save_for_backward(signs)
        ctx.transpose = bool(transpose)
        ctx.backend = backend
        return _run(x2d, signs, transpose, backend)

    @staticmethod
    def backward(ctx, grad_out):
        (signs,) = ctx.saved_tensors
        return (_FhtFn.apply(grad_out.contiguous(), signs, not ctx.transpose, ctx.backend),
                None, None, None)


def _apply(x: torch.Tensor, signs: torch.Tensor, transpose: bool, backend: str) -> torch.Tensor:
    M, K = _check(x, signs)
    resolved = _resolve(backend, x)
    x2d = x.reshape(M, K)
    if not x2d.is_contiguous():
        x2d = x2d.contiguous()
    signs = signs.detach()
    if signs.device != x2d.device:
        signs = signs.to(x2d.device)
    if x2d.requires_grad:
        out = _FhtFn.apply(x2d, signs, transpose, resolved)
    else:
        out = _run(x2d, signs, transpose, resolved)
    return out.reshape(x.shape)


def fht_apply(x: torch.Tensor, signs: torch.Tensor, backend: FhtBackend = "auto") -> torch.Tensor:
    """out = x @ T for x of shape (..., K); fp16/bf16/fp32 in and out, fp32 inside."""
    return _apply(x, signs, False, backend)


def fht_adjoint(v: torch.Tensor, signs: torch.Tensor, backend: FhtBackend = "auto") -> torch.Tensor:
    """out = v @ T^T (weight-space un-rotation, gradient adjoint)."""
    return _apply(v, signs, True, backend)


def fht_apply_awq(x: torch.Tensor, signs: torch.Tensor, s: torch.Tensor,
                  backend: FhtBackend = "auto") -> torch.Tensor:
    """out = ((x * s) @ T) / s in fp32 with a true division, cast to x's dtype:
    the compensated rotation of rotate-then-AWQ artifacts."""
    M, K = _check(x, signs)
    if s.dim() != 1 or s.numel() != K:
        raise ValueError(f"fht_awq: s must be a (K,) vector matching x's last dim "
                         f"(got {tuple(s.shape)}, K={K})")
    if not torch.is_floating_point(s):
        raise TypeError(f"fht_awq: s must be floating point, got {s.dtype}")
    if backend not in _BACKENDS:
        raise ValueError(f"fht_awq: unknown backend {backend!r}")
    x2d = x.reshape(M, K)
    if not x2d.is_contiguous():
        x2d = x2d.contiguous()
    signs = signs.detach().to(x2d.device)
    s = s.detach().to(x2d.device, torch.float32).contiguous()
    C = _load_kernel()
    use_kernel = (backend in ("auto", "kernel") and C is not None and x2d.is_cuda
                  and _kernel_eligible(K) and not x2d.requires_grad)
    if backend == "kernel" and not use_kernel:
        raise RuntimeError("fht_apply_awq(backend='kernel'): the compensated-rotation kernel is "
                           "unavailable (library missing, CPU input, grad required, or K outside "
                           "the contract). Never a silent fallback.")
    if use_kernel:
        out = C.fht_forward_awq(x2d, _signs_for_kernel(signs, x2d), s)
    elif backend == "matmul":
        T = _matrix_from_signs(signs).to(x2d.device)
        out = ((x2d.float() * s) @ T / s).to(x2d.dtype)
    else:
        out = (fht_reference(x2d.float() * s, signs).float() / s).to(x2d.dtype)
    return out.reshape(x.shape)


def fht_apply_(x: torch.Tensor, signs: torch.Tensor, backend: FhtBackend = "auto") -> torch.Tensor:
    """In place x <- x @ T.  Refuses tensors that require grad."""
    if x.requires_grad:
        raise RuntimeError("fht_apply_: in-place rotation of a tensor that requires grad - use "
                           "fht_apply")
    M, K = _check(x, signs)
    x2d = x.reshape(M, K)
    aliases = x2d.data_ptr() == x.data_ptr() and x2d.is_contiguous()
    resolved = _resolve(backend, x)
    if resolved == "kernel" and aliases:
        _load_kernel().fht_inplace_(x2d, _signs_for_kernel(signs.detach(), x2d))
        return x
    x.copy_(fht_apply(x, signs, backend=resolved))
    return x


def _selfcheck() -> int:
    torch.manual_seed(0)
    ok = True
    for K in (64, 256, 4096, 12288):
        signs = rotation_signs(K, seed=K)
        x = torch.randn(3, 7, K)
        T = build_rotation_matrix(K, seed=K)
        fwd = (fht_reference(x, signs) - x @ T).abs().max().item()
        adj = (fht_reference_adjoint(x, signs) - x @ T.t()).abs().max().item()
        xa = torch.randn(5, K, requires_grad=True)
        ga = torch.randn(5, K)
        fht_apply(xa, signs, backend="reference").backward(ga)
        grad = (xa.grad - fht_reference_adjoint(ga, signs)).abs().max().item()
        line = fwd < 1e-4 and adj < 1e-4 and grad < 1e-4
        ok &= line
        print(f"K={K:6d}: fwd {fwd:.2e} adj {adj:.2e} grad {grad:.2e} {'OK' if line else 'FAIL'}")
    print("selfcheck:", "PASS" if ok else "FAIL")
    return 0 if ok else 1


if __name__ == "__main__":
    raise SystemExit(_selfcheck())
