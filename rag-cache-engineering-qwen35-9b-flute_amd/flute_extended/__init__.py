"""flute_extended for AMD Instinct MI355X (gfx950): LUT-palettized linear-layer ops.

Drop-in for the upstream package of the same name
(src/flute_extended/flute_extended/__init__.py): the same public callables,
keyword names, tables and `*_available` / `*_supported` gate functions, backed by
hand-written HIP kernels behind a C ABI (libflute_hip.so) instead of a CUDA
extension.  Put the directory that CONTAINS this package on sys.path, exactly as
upstream's callers do.

Ops (all weights in the idxN blob layout, see idxN.py):

    qgemm_per_group_lut(A, indices, lut, bitwidth=, group_size=, indices_layout=)
        C[M,N] = A @ W^T                                  MFMA GEMM, any M
    qgemm_dual_stream(...)      both streams + residual + bias, small M
    qgemm_gemv_stream(...)      M = 1 GEMV (optionally with the fused rotation)
    qgemm_gemv_splitk_stream(...)   the same op; upstream's split-K entry
    qgemm_gemv_multi(A, seg_table)  2-4 weights sharing x, one launch
    qgemm_gemv_mlp(A, seg_table, C) silu(gate(x)) * up(x), one launch

Differences from upstream that a caller can observe: activations (and outputs)
may be bfloat16 as well as float16; a bfloat16 LUT is accepted with bfloat16
activations; the GEMV entries share one kernel whose K split is chosen for 256
CUs, so `qgemm_gemv_stream` and `qgemm_gemv_splitk_stream` differ only in the
contract they enforce (pair table, group sizes, residual rank).  There is no
silent fallback anywhere: a missing library fails the import, a shape outside
the contract raises.
"""
from __future__ import annotations

from typing import Literal, Optional

import functools

import torch

from . import _C
from ._C import (qgemm_per_group_lut as _qgemm_per_group_lut,
                 qgemm_debug_simple,
                 qgemm_cutlass_dense,
                 qgemm_cutlass_streaming)
from ._C import qgemm_dual_stream as _qgemm_dual_stream
from ._C import qgemm_gemv_stream as _qgemm_gemv_stream
from ._C import qgemm_gemv_fht_stream as _qgemm_gemv_fht_stream
from ._C import qgemm_gemv_splitk_stream as _qgemm_gemv_splitk_stream
from ._C import qgemm_gemv_splitk_fht_stream as _qgemm_gemv_splitk_fht_stream
from ._C import qgemm_gemv_multi as _qgemm_gemv_multi
from ._C import qgemm_gemv_mlp as _qgemm_gemv_mlp
from ._C import dequant_idxn
from ._C import embedding_gather
from ._C import qgemm_gemv_kgroup, dequant_kgroup

Backend = Literal["debug_simple", "cutlass_dense", "cutlass_streaming", "auto"]
IndicesLayout = Literal["idx1", "idx2", "idx3", "idx4"]

_LAYOUT_BITS = {"idx1": 1, "idx2": 2, "idx3": 3, "idx4": 4}

# LDS of one MI355X compute unit; the gates below admit a shape when one GEMV
# workgroup fits (upstream's constant is the 99 KB of an A10G block).
LDS_BYTES_PER_CU = 160 * 1024


_EMPTY = {}


def _empty(device, dtype):
    """One zero-element tensor per (device, dtype): the placeholders carry no data, so
    every call can share them instead of allocating three new ones."""
    key = (device, dtype)
    t = _EMPTY.get(key)
    if t is None:
        t = _EMPTY[key] = torch.empty(0, dtype=dtype, device=device)
    return t


def _none_to_empty(A: torch.Tensor, indices2, lut2, resB, resA, bias, lut_dtype=None):
    """The `_C` convention: an absent operand is an empty tensor
    (upstream __init__.py:321-334)."""
    e8 = _empty(A.device, torch.uint8)
    e16 = _empty(A.device, A.dtype)
    el = _empty(A.device, lut_dtype or A.dtype)
    return (indices2 if indices2 is not None else e8,
            lut2 if lut2 is not None else el,
            resB if resB is not None else e16,
            resA if resA is not None else e16,
            bias if bias is not None else e16)


# ---------------------------------------------------------------------------
# GEMM                                             (upstream __init__.py:138-219)
# ---------------------------------------------------------------------------

def qgemm_per_group_lut(A: torch.Tensor, indices: torch.Tensor, lut: torch.Tensor,
                        bitwidth: int = 4, group_size: int = 32, backend: Backend = "auto",
                        indices_layout: IndicesLayout = "idx4") -> torch.Tensor:
    """Y = A @ W^T for a palettized W.  indices_layout must name the idxN width
    and agree with bitwidth; N % 128 == 0 and K % 64 == 0 are required."""
    if backend == "auto":
        backend = "cutlass_streaming"
    if indices_layout not in _LAYOUT_BITS:
        raise ValueError(f"indices_layout={indices_layout!r} is not supported; the supported "
                         f"layouts are {sorted(_LAYOUT_BITS)}")
    if int(bitwidth) != _LAYOUT_BITS[indices_layout]:
        raise ValueError(f"indices_layout={indices_layout!r} implies bitwidth="
                         f"{_LAYOUT_BITS[indices_layout]}, but bitwidth={bitwidth} was passed")
    W_empty = torch.empty(0, dtype=A.dtype, device=A.device)
    return _qgemm_per_group_lut(A, indices, lut, W_empty, int(bitwidth), int(group_size),
                                backend, 1)


def qgemm_dense(A: torch.Tensor, W_dense: torch.Tensor, group_size: int = 32,
                backend: Backend = "cutlass_dense") -> torch.Tensor:
    """Dense baseline entry; refused here as it is upstream without CUTLASS."""
    if backend != "cutlass_dense":
        raise ValueError("qgemm_dense only supports backend='cutlass_dense'")
    e8 = torch.empty(0, dtype=torch.uint8, device=A.device)
    e16 = torch.empty(0, dtype=A.dtype, device=A.device)
    return _qgemm_per_group_lut(A, e8, e16, W_dense, 4, int(group_size), backend)


# ---------------------------------------------------------------------------
# small-M fused GEMM                               (upstream __init__.py:226-334)
# ---------------------------------------------------------------------------

# Every (bitwidth, bitwidth2) pair is served; the upstream table listed only the
# pairs its artifacts contained.
DUAL_STREAM_PAIRS = frozenset((b1, b2) for b1 in range(1, 5) for b2 in range(0, 5))
DUAL_STREAM_GROUP_SIZES = frozenset({16, 32, 64, 128, 256, 512, 1024, 2048})
DUAL_STREAM_MAX_M = 16


def dual_stream_available() -> bool:
    return True


def dual_stream_supported(bitwidth: int, bitwidth2: int, group_size: int, N: int, K: int) -> bool:
    b2 = int(bitwidth2) if bitwidth2 else 0
    return ((int(bitwidth), b2) in DUAL_STREAM_PAIRS
            and int(group_size) in DUAL_STREAM_GROUP_SIZES
            and int(N) % 128 == 0 and int(K) % 64 == 0)


def qgemm_dual_stream(A, indices, lut, bitwidth: int, group_size: int,
                      indices2: Optional[torch.Tensor] = None,
                      lut2: Optional[torch.Tensor] = None, bitwidth2: int = 0,
                      resB: Optional[torch.Tensor] = None, resA: Optional[torch.Tensor] = None,
                      bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """C = A W1^T (+ A W2^T) + (A resB^T) resA^T + bias, fp32 accumulate, one
    rounding (the reference forward's association)."""
    i2, l2, rb, ra, bi = _none_to_empty(A, indices2, lut2, resB, resA, bias, lut.dtype)
    return _qgemm_dual_stream(A, indices, lut, int(bitwidth), i2, l2, int(bitwidth2), rb, ra, bi,
                              int(group_size))


# ---------------------------------------------------------------------------
# M = 1 GEMV                                       (upstream __init__.py:341-589)
# ---------------------------------------------------------------------------

GEMV_STREAM_PAIRS = frozenset({(1, 4), (4, 1), (2, 3), (2, 4), (3, 3), (3, 0), (4, 0)})
GEMV_STREAM_GROUP_SIZES = frozenset({64, 128, 256, 512, 1024, 2048})


def gemv_stream_available() -> bool:
    return True


@functools.lru_cache(maxsize=4096)
def _lds_need(N: int, K: int, b1: int, b2: int, gs: int, fht: bool, rank: int) -> int:
    return _C.gemv_lds_bytes(N, K, b1, b2, gs, fht=fht, residual_rank=rank)


def _lds_ok(N, K, b1, b2, gs, fht, rank=0) -> bool:
    # pure host arithmetic of the shape: asked once per shape, not once per call
    need = _lds_need(int(N), int(K), int(b1), int(b2), int(gs), bool(fht), int(rank))
    return 0 < need <= LDS_BYTES_PER_CU


def gemv_stream_supported(bitwidth: int, bitwidth2: int, group_size: int, N: int, K: int,
                          M: int) -> bool:
    b1, b2 = int(bitwidth), int(bitwidth2) if bitwidth2 else 0
    return (int(M) == 1 and (b1, b2) in GEMV_STREAM_PAIRS
            and int(group_size) in GEMV_STREAM_GROUP_SIZES
            and int(N) % 128 == 0 and int(K) % 64 == 0
            and _lds_ok(N, K, b1, b2, group_size, False))


def gemv_fht_stream_available() -> bool:
    return True


def _fht_k_ok(K: int) -> bool:
    K = int(K)
    return K % 32 == 0 and 32 <= K <= 65504 and (1 << (K.bit_length() - 1)) <= 16384


def gemv_fht_stream_supported(bitwidth: int, bitwidth2: int, group_size: int, N: int, K: int,
                              M: int) -> bool:
    b1, b2 = int(bitwidth), int(bitwidth2) if bitwidth2 else 0
    return (int(M) == 1 and (b1, b2) in GEMV_STREAM_PAIRS
            and int(group_size) in GEMV_STREAM_GROUP_SIZES
            and int(N) % 128 == 0 and int(K) % 64 == 0 and _fht_k_ok(K)
            and _lds_ok(N, K, b1, b2, group_size, True))


def _coerce_vec(name: str, who: str, v: torch.Tensor, A: torch.Tensor) -> torch.Tensor:
    K = int(A.shape[1])
    if v.dim() != 1 or int(v.numel()) != K:
        raise ValueError(f"{who}: {name} must be a (K,) vector matching A's last dim "
                         f"(got {tuple(v.shape)}, K={K})")
    v = v.detach()
    if v.device != A.device or v.dtype != torch.float32 or not v.is_contiguous():
        v = v.to(A.device, torch.float32).contiguous()
    return v


def _gemv_entry(who, plain, fused, A, indices, lut, bitwidth, group_size, indices2, lut2,
                bitwidth2, resB, resA, bias, rot_signs, awq_scale, **extra):
    if rot_signs is None and awq_scale is not None:
        raise ValueError(f"{who}: awq_scale only exists as a companion to rot_signs - pass "
                         "rot_signs too, or drop awq_scale")
    i2, l2, rb, ra, bi = _none_to_empty(A, indices2, lut2, resB, resA, bias, lut.dtype)
    if rot_signs is None:
        return plain(A, indices, lut, int(bitwidth), i2, l2, int(bitwidth2), rb, ra, bi,
                     int(group_size), **{k: v for k, v in extra.items() if k == "split"})
    signs = _coerce_vec("rot_signs", who, rot_signs, A)
    s = torch.empty(0, dtype=torch.float32, device=A.device)
    if awq_scale is not None:
        s = _coerce_vec("awq_scale", who, awq_scale, A)
    return fused(A, indices, lut, int(bitwidth), i2, l2, int(bitwidth2), rb, ra, bi,
                 int(group_size), signs, s, **extra)


def qgemm_gemv_stream(A, indices, lut, bitwidth: int, group_size: int,
                      indices2: Optional[torch.Tensor] = None,
                      lut2: Optional[torch.Tensor] = None, bitwidth2: int = 0,
                      resB: Optional[torch.Tensor] = None, resA: Optional[torch.Tensor] = None,
                      bias: Optional[torch.Tensor] = None,
                      rot_signs: Optional[torch.Tensor] = None,
                      awq_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Decode GEMV, M must be 1:  C = A W1^T (+ A W2^T) + (A resB^T) resA^T + bias,
    everything accumulated in fp32 and rounded once.  With rot_signs, A is the
    UNROTATED row and x @ T (or ((x*s) @ T)/s with awq_scale) runs as the kernel
    prologue, bit-identical to rotating first with fht_apply."""
    return _gemv_entry("qgemm_gemv_stream", _qgemm_gemv_stream, _qgemm_gemv_fht_stream, A,
                       indices, lut, bitwidth, group_size, indices2, lut2, bitwidth2, resB, resA,
                       bias, rot_signs, awq_scale)


# ---------------------------------------------------------------------------
# split-K GEMV                                     (upstream __init__.py:597-862)
# ---------------------------------------------------------------------------

GEMV_SPLITK_PAIRS = frozenset((b1, b2) for b1 in range(1, 5) for b2 in range(0, 5))
GEMV_SPLITK_GROUP_SIZES = frozenset({16, 32, 64, 128, 256, 512, 1024, 2048})
GEMV_SPLITK_MAX_RESIDUAL_RANK = 256


def gemv_split_hint(N: int, K: int) -> int:
    """The K split the library picks for an (N, K) single-stream GEMV on this
    device.  Upstream's policy targets 160 workgroups on 80 SMs
    (src/gemv_host.cpp:29-38).  On the MI355X the unsplit launch measured fastest up to
    K = 24576 for every N (N = 1024, K = 4096: 4.5 us against 5.9 / 10.4 / 11.4 us split
    2 / 4 / 8 ways: the exchange of partial sums costs three memory round trips), so the
    answer is 1 there; from K = 32768 it is 4 for N <= 512 and 2 for N <= 1024 (N = 512,
    K = 32768: 7.5 us against 9.0 us unsplit).  An explicit split passed to the split-K
    entry points is always honoured."""
    return _C.pick_split(int(N), int(K))


def gemv_splitk_available() -> bool:
    return True


def gemv_splitk_fht_available() -> bool:
    return True


def _splitk_gate(bitwidth, bitwidth2, group_size, N, K, M, residual_rank, fht) -> bool:
    b1, b2 = int(bitwidth), int(bitwidth2) if bitwidth2 else 0
    if int(M) != 1 or (b1, b2) not in GEMV_SPLITK_PAIRS:
        return False
    if int(group_size) not in GEMV_SPLITK_GROUP_SIZES:
        return False
    if int(N) % 128 != 0 or int(K) % 64 != 0:
        return False
    if int(residual_rank) > GEMV_SPLITK_MAX_RESIDUAL_RANK:
        return False
    if fht and not _fht_k_ok(K):
        return False
    return _lds_ok(N, K, b1, b2, group_size, fht, int(residual_rank))


def gemv_splitk_supported(bitwidth: int, bitwidth2: int, group_size: int, N: int, K: int,
                          M: int, residual_rank: int = 0) -> bool:
    return _splitk_gate(bitwidth, bitwidth2, group_size, N, K, M, residual_rank, False)


def gemv_splitk_fht_supported(bitwidth: int, bitwidth2: int, group_size: int, N: int, K: int,
                              M: int, residual_rank: int = 0) -> bool:
    return _splitk_gate(bitwidth, bitwidth2, group_size, N, K, M, residual_rank, True)


def qgemm_gemv_splitk_stream(A, indices, lut, bitwidth: int, group_size: int,
                             indices2: Optional[torch.Tensor] = None,
                             lut2: Optional[torch.Tensor] = None, bitwidth2: int = 0,
                             resB: Optional[torch.Tensor] = None,
                             resA: Optional[torch.Tensor] = None,
                             bias: Optional[torch.Tensor] = None,
                             rot_signs: Optional[torch.Tensor] = None,
                             awq_scale: Optional[torch.Tensor] = None,
                             split: int = 0, rot_block: int = 0) -> torch.Tensor:
    """The decode GEMV with the wide contract: every width pair, group sizes
    16..2048, residual rank up to 256.  `split` (0 = policy) and `rot_block`
    (0 = upstream's power-of-two segments) are extensions."""
    extra = {"split": int(split)}
    if rot_signs is not None:
        extra["rot_block"] = int(rot_block)
    return _gemv_entry("qgemm_gemv_splitk_stream", _qgemm_gemv_splitk_stream,
                       _qgemm_gemv_splitk_fht_stream, A, indices, lut, bitwidth, group_size,
                       indices2, lut2, bitwidth2, resB, resA, bias, rot_signs, awq_scale, **extra)


# ---------------------------------------------------------------------------
# grouped launches                                 (upstream __init__.py:877-1109)
# ---------------------------------------------------------------------------

def gemv_multi_available() -> bool:
    return True


def _specs_ok(specs) -> bool:
    return all((int(b1), int(b2)) in GEMV_SPLITK_PAIRS and int(gs) in GEMV_SPLITK_GROUP_SIZES
               for b1, b2, gs in specs)


def gemv_multi_supported(K: int, tiles_total: int, specs, residual_rank_total: int = 0,
                         fht: bool = False) -> bool:
    """specs = [(b1, b2, gs), ...] per segment, 2-4 rows."""
    if int(K) % 64 != 0 or not 2 <= len(specs) <= 4 or not _specs_ok(specs):
        return False
    if int(residual_rank_total) > 4 * GEMV_SPLITK_MAX_RESIDUAL_RANK:
        return False
    if fht and not _fht_k_ok(K):
        return False
    return all(_lds_ok(128, K, b1, b2, gs, fht) for b1, b2, gs in specs)


def qgemm_gemv_multi(A: torch.Tensor, seg_table: torch.Tensor,
                     lut_dtype: Optional[torch.dtype] = None) -> None:
    """2-4 weights sharing one input row in one launch.  seg_table: CPU int64
    [count, 15] of raw data_ptr() values, columns
    [q1, lut1, q2, lut2, resB, resA, bias, C, N, R, b1, b2, gs, signs, s]."""
    if not (A.dim() == 2 and A.shape[0] == 1 and A.is_contiguous()
            and A.dtype in (torch.float16, torch.bfloat16)):
        raise ValueError("qgemm_gemv_multi: A must be a contiguous [1, K] float16/bfloat16 tensor")
    if not (seg_table.device.type == "cpu" and seg_table.dtype == torch.int64
            and seg_table.dim() == 2 and seg_table.size(1) == 15):
        raise ValueError("qgemm_gemv_multi: seg_table must be a CPU int64 [count, 15] tensor")
    _qgemm_gemv_multi(A, seg_table, lut_dtype)


def gemv_mlp_available() -> bool:
    return True


def gemv_mlp_supported(K: int, N: int, specs, residual_rank_g: int = 0, residual_rank_u: int = 0,
                       fht: bool = False, folds_differ: bool = False) -> bool:
    """specs = [(b1g, b2g, gsg), (b1u, b2u, gsu)].  folds_differ costs nothing
    here: every workgroup rotates its own copy of the row."""
    if int(K) % 64 != 0 or int(N) % 128 != 0 or len(specs) != 2 or not _specs_ok(specs):
        return False
    if max(int(residual_rank_g), int(residual_rank_u)) > GEMV_SPLITK_MAX_RESIDUAL_RANK:
        return False
    if fht and not _fht_k_ok(K):
        return False
    return all(_lds_ok(N, K, b1, b2, gs, fht) for b1, b2, gs in specs)


def qgemm_gemv_mlp(A: torch.Tensor, seg_table: torch.Tensor, C: torch.Tensor,
                   lut_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """C = silu(gate(A)) * up(A) in one launch; seg_table row 0 = gate, row 1 = up.
    The table holds raw pointers: LUTs are float16 unless lut_dtype says bfloat16."""
    if not (A.dim() == 2 and A.shape[0] == 1 and A.is_contiguous()
            and A.dtype in (torch.float16, torch.bfloat16)):
        raise ValueError("qgemm_gemv_mlp: A must be a contiguous [1, K] float16/bfloat16 tensor")
    if not (seg_table.device.type == "cpu" and seg_table.dtype == torch.int64
            and seg_table.dim() == 2 and seg_table.size(0) == 2 and seg_table.size(1) == 15):
        raise ValueError("qgemm_gemv_mlp: seg_table must be a CPU int64 [2, 15] tensor")
    if not (C.dtype == A.dtype and C.is_contiguous()):
        raise ValueError("qgemm_gemv_mlp: C must be a contiguous output buffer of A's dtype")
    return _qgemm_gemv_mlp(A, seg_table, C, lut_dtype)


__all__ = [
    "qgemm_per_group_lut", "qgemm_dense", "qgemm_debug_simple", "qgemm_cutlass_dense",
    "qgemm_cutlass_streaming", "qgemm_dual_stream", "dual_stream_available",
    "dual_stream_supported", "DUAL_STREAM_PAIRS", "DUAL_STREAM_GROUP_SIZES",
    "DUAL_STREAM_MAX_M", "qgemm_gemv_stream", "gemv_stream_available",
    "gemv_stream_supported", "GEMV_STREAM_PAIRS", "GEMV_STREAM_GROUP_SIZES",
    "gemv_fht_stream_available", "gemv_fht_stream_supported", "qgemm_gemv_splitk_stream",
    "gemv_splitk_available", "gemv_splitk_supported", "gemv_splitk_fht_available",
    "gemv_splitk_fht_supported", "qgemm_gemv_multi", "gemv_multi_available",
    "gemv_multi_supported", "qgemm_gemv_mlp", "gemv_mlp_available", "gemv_mlp_supported",
    "gemv_split_hint", "GEMV_SPLITK_PAIRS", "GEMV_SPLITK_GROUP_SIZES",
    "GEMV_SPLITK_MAX_RESIDUAL_RANK", "dequant_idxn", "embedding_gather",
    "qgemm_gemv_kgroup", "dequant_kgroup",
]
