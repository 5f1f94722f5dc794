"""Tensor-level entry points over the C ABI: the module upstream builds as the
pybind11 extension `flute_extended._C` (src/flute_extended/src/bindings.cpp:230-546).

Same callable names, positional signatures and conventions:

  * "absent" operands are EMPTY tensors, never None; bitwidth2 == 0 means a
    single stream (flute_extended/__init__.py:321-334 upstream);
  * N is derived from the blob byte count, N = numel / (K*b/8)
    (src/kernel_gemv.cu:379-388);
  * every contract violation raises RuntimeError (upstream: TORCH_CHECK);
  * outputs are fresh tensors, except qgemm_gemv_mlp (caller's C) and
    qgemm_gemv_multi (pointers inside the segment table);
  * launches go to the current stream of the input's device, no host sync.

What differs from upstream, on purpose: activations may be bfloat16 as well as
float16 (outputs follow the activation dtype), LUTs may be bfloat16 when the
activations are, and the K split is chosen for 256 CUs.  Shape and dtype
checks run before the device check, so the refusal paths can be exercised with
CPU tensors on a machine without a GPU; a CPU tensor that passes them is
refused as "must be a CUDA tensor".
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import FluteLinear, check, lib

_ACT = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}
_ANY = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}

_GS_ALL = (16, 32, 64, 128, 256, 512, 1024, 2048)


def _fail(msg: str):
    raise RuntimeError(msg)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None or t.numel() == 0 else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_of(t: torch.Tensor) -> int:
    """Handle of torch's current stream on t's device (the raw query where this torch has
    it: it skips building a Stream object on every call)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None
                           else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _on_device_of:
    """Device guard for a launch: a no-op when t's device is already current."""

    def __init__(self, t: torch.Tensor):
        idx = t.device.index
        self._guard = None if idx is None or idx == torch.cuda.current_device() \
            else torch.cuda.device(t.device)

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            self._guard.__exit__(*exc)
        return False


def _aligned16(t: torch.Tensor) -> torch.Tensor:
    # fresh allocations are 256-byte aligned; views and slices may not be
    return t if t.data_ptr() % 16 == 0 else t.clone()


_DTYPE_CODE = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32,
               torch.uint8: _lib.U8}
_DTYPE_NAME = {}


def _record(rec: "_lib.FluteTensor", t: Optional[torch.Tensor]) -> None:
    """Fill one flute_tensor record from a tensor (None: the operand was not passed)."""
    if t is None:
        rec.present = 0
        return
    rec.present = 1
    n = t.numel()
    if n == 0:
        # upstream's "absent operand": only the emptiness is looked at, unless the entry's own
        # arguments (a second bit width) say the operand is needed, and then it fails on its size
        rec.ndim = t.dim()
        if rec.ndim > 1:
            for i, v in enumerate(t.shape[:4]):
                rec.size[i] = v
        rec.dtype = _DTYPE_CODE.get(t.dtype, -1)
        rec.contiguous = 1
        rec.device = -1
        return
    rec.numel = n
    rec.ndim = t.dim()
    for i, n in enumerate(t.shape[:4]):
        rec.size[i] = n
    code = _DTYPE_CODE.get(t.dtype, -1)
    rec.dtype = code
    if code < 0:
        name = _DTYPE_NAME.get(t.dtype)
        if name is None:
            name = _DTYPE_NAME[t.dtype] = str(t.dtype).encode()
        rec.dtype_name = name
    rec.contiguous = 1 if t.is_contiguous() else 0
    rec.device = (t.device.index if t.device.index is not None else torch.cuda.current_device()) \
        if t.is_cuda else -1
    rec.data = t.data_ptr()


def _check_2d_input(who: str, A: torch.Tensor, need_m1: bool) -> tuple:
    """The checks of the input matrix (flute_check_input in the library: one copy for this mirror
    and the compiled binding)."""
    rec = _lib.FluteTensor()
    _record(rec, A)
    if lib.flute_check_input(who.encode(), ctypes.byref(rec), 1 if need_m1 else 0) != _lib.FLUTE_OK:
        _fail(_lib.last_error())
    return int(A.shape[0]), int(A.shape[1])


def _gs_mask(sizes: Sequence[int]) -> int:
    mask = 0
    for g in sizes:
        mask |= 1 << (int(g).bit_length() - 1)
    return mask


_GS_MASKS = {}


def _describe(who: str, A: torch.Tensor, K: int, indices, lut, bitwidth, indices2, lut2,
              bitwidth2, resB, resA, bias, group_size, signs=None, awq=None,
              rot_block: int = 0, gs_allowed: Sequence[int] = _GS_ALL,
              max_rank: int = 256):
    """Validate one weight's tensors and return (FluteLinear, N, keepalive).  The checks
    themselves are flute_describe_linear's: this function only records what it was given."""
    indices = _aligned16(indices) if indices.is_cuda else indices
    if int(bitwidth2) > 0 and indices2 is not None and indices2.is_cuda:
        indices2 = _aligned16(indices2)
    ops = _lib.FluteOperands()
    _record(ops.A, A)
    _record(ops.indices, indices)
    _record(ops.lut, lut)
    _record(ops.indices2, indices2)
    _record(ops.lut2, lut2)
    _record(ops.resB, resB)
    _record(ops.resA, resA)
    _record(ops.bias, bias)
    _record(ops.signs, signs)
    _record(ops.awq, awq)
    ops.K, ops.b1, ops.b2 = int(K), int(bitwidth), int(bitwidth2)
    gs = int(group_size)
    ops.group_size = gs if -2 ** 31 <= gs < 2 ** 31 else -1
    ops.rot_block, ops.max_rank = int(rot_block), int(max_rank)
    key = tuple(gs_allowed)
    mask = _GS_MASKS.get(key)
    if mask is None:
        mask = _GS_MASKS[key] = _gs_mask(key)
    ops.gs_allowed = mask
    w = FluteLinear()
    n = ctypes.c_int64(0)
    if lib.flute_describe_linear(who.encode(), ctypes.byref(ops), ctypes.byref(w),
                                 ctypes.byref(n)) != _lib.FLUTE_OK:
        _fail(_lib.last_error())
    return w, int(n.value), (indices, indices2)


def _gemv(who, A, indices, lut, bitwidth, indices2, lut2, bitwidth2, resB, resA, bias,
          group_size, signs=None, s=None, split: int = 0, rot_block: int = 0,
          gs_allowed=_GS_ALL, max_rank=256):
    M, K = _check_2d_input(who, A, need_m1=True)
    if K == 0 or indices.numel() == 0:
        # degenerate shapes never reach the device (src/kernel_gemv.cu:456-461 upstream)
        N = int(lut.shape[0]) * int(group_size) if (K == 0 and lut.dim() == 2) else 0
        return torch.zeros((1, N), dtype=A.dtype, device=A.device)
    w, N, keep = _describe(who, A, K, indices, lut, bitwidth, indices2, lut2, bitwidth2,
                           resB, resA, bias, group_size, signs, s, rot_block, gs_allowed,
                           max_rank)
    A = _aligned16(A)
    with _on_device_of(A):
        C = torch.empty((1, N), dtype=A.dtype, device=A.device)
        check(lib.flute_gemv(ctypes.byref(w), A.data_ptr(), C.data_ptr(), _ACT[A.dtype],
                             int(split), _stream_of(A)))
    del keep
    return C


# ---------------------------------------------------------------------------
# M = 1 GEMV family                         (src/bindings.cpp:277-354 upstream)
# ---------------------------------------------------------------------------

_GS_PLAIN = (64, 128, 256, 512, 1024, 2048)


def qgemm_gemv_stream(A, indices, lut, bitwidth, indices2, lut2, bitwidth2, resB, resA, bias,
                      group_size):
    """Plain decode GEMV, A already rotated (src/kernel_gemv.cu:322-510 upstream)."""
    return _gemv("qgemm_gemv_stream", A, indices, lut, bitwidth, indices2, lut2, bitwidth2,
                 resB, resA, bias, group_size, gs_allowed=_GS_PLAIN, max_rank=16)


def qgemm_gemv_fht_stream(A, indices, lut, bitwidth, indices2, lut2, bitwidth2, resB, resA,
                          bias, group_size, signs, s):
    """Decode GEMV with the rotation fused into the prologue
    (src/kernel_gemv.cu:579-776 upstream)."""
    return _gemv("qgemm_gemv_fht_stream", A, indices, lut, bitwidth, indices2, lut2, bitwidth2,
                 resB, resA, bias, group_size, signs, s, gs_allowed=_GS_PLAIN, max_rank=16)


def qgemm_gemv_splitk_stream(A, indices, lut, bitwidth, indices2, lut2, bitwidth2, resB, resA,
                             bias, group_size, split: int = 0):
    """Split-K decode GEMV (src/kernel_gemv_splitk.cu:813-830 upstream).  `split` is an
    extension: 0 lets the library choose."""
    return _gemv("qgemm_gemv_splitk_stream", A, indices, lut, bitwidth, indices2, lut2,
                 bitwidth2, resB, resA, bias, group_size, split=split)


def qgemm_gemv_splitk_fht_stream(A, indices, lut, bitwidth, indices2, lut2, bitwidth2, resB,
                                 resA, bias, group_size, signs, s, split: int = 0,
                                 rot_block: int = 0):
    """Split-K decode GEMV with the fused rotation.  `rot_block` > 0 selects equal
    rotation blocks (an extension; upstream rotates over the descending
    power-of-two segments of K)."""
    return _gemv("qgemm_gemv_splitk_fht_stream", A, indices, lut, bitwidth, indices2, lut2,
                 bitwidth2, resB, resA, bias, group_size, signs, s, split=split,
                 rot_block=rot_block)


# ---------------------------------------------------------------------------
# segment-table entries                     (src/bindings.cpp:368-384 upstream)
# ---------------------------------------------------------------------------

_SEG_COLS = 15   # q1 lut1 q2 lut2 resB resA bias C N R b1 b2 gs signs s


def _check_seg_inputs(who: str, A: torch.Tensor, seg_table: torch.Tensor, rows: Optional[int]):
    if A.dim() != 2 or A.shape[0] != 1 or A.dtype not in _ACT or not A.is_contiguous():
        _fail(f"{who}: A must be a contiguous [1, K] float16/bfloat16 tensor")
    if seg_table.device.type != "cpu" or seg_table.dtype != torch.int64 \
            or seg_table.dim() != 2 or seg_table.shape[1] != _SEG_COLS:
        _fail(f"{who}: seg_table must be a CPU int64 [count, 15] tensor")
    count = int(seg_table.shape[0])
    if rows is not None and count != rows:
        _fail(f"{who}: seg_table must have {rows} rows (got {count})")
    if rows is None and not 1 <= count <= 4:
        _fail(f"{who}: 1..4 segments per launch (got {count})")
    return count


def _seg_descs(who: str, A: torch.Tensor, seg_table: torch.Tensor, lut_dtype: int):
    K = int(A.shape[1])
    table = seg_table.tolist()
    descs = (FluteLinear * len(table))()
    outs = []
    for i, row in enumerate(table):
        q1, l1, q2, l2, rB, rA, bi, C, N, R, b1, b2, gs, sg, sc = (int(v) for v in row)
        for name, ptr in (("q1", q1), ("q2", q2), ("resB", rB), ("resA", rA), ("signs", sg),
                          ("s", sc)):
            if ptr % 16 != 0:
                _fail(f"{who}: segment {i} pointer {name} must be 16-byte aligned")
        if q1 == 0 or l1 == 0:
            _fail(f"{who}: segment {i} has no stream-1 indices/lut")
        if gs <= 0:
            _fail(f"{who}: segment {i} group_size must be positive")
        w = descs[i]
        w.q1, w.lut1 = q1, l1
        w.q2, w.lut2 = (q2 or None), (l2 or None)
        w.resB, w.resA, w.bias = (rB or None), (rA or None), (bi or None)
        w.signs, w.awq = (sg or None), (sc or None)
        w.N, w.K, w.R, w.b1, w.b2, w.group_size = N, K, R, b1, b2, gs
        w.q1_bytes = N * K * b1 // 8
        w.q2_bytes = N * K * b2 // 8
        w.lut_rows = (N + gs - 1) // gs
        w.lut_dtype = lut_dtype
        outs.append(C)
    return descs, outs


def qgemm_gemv_multi(A, seg_table, lut_dtype: Optional[torch.dtype] = None, split: int = 0):
    """2-4 weights sharing one input row, one launch; outputs land in the C
    pointers of the table (src/kernel_gemv_multi.cu upstream).  The table holds
    raw pointers, so dtypes follow A: residual/bias/outputs in A's dtype, LUTs
    float16 unless lut_dtype says bfloat16."""
    who = "qgemm_gemv_multi"
    _check_seg_inputs(who, A, seg_table, None)
    if not A.is_cuda:
        _fail(f"{who}: A must be a CUDA (HIP) tensor")
    descs, outs = _seg_descs(who, A, seg_table, _ACT[lut_dtype or torch.float16])
    for i, c in enumerate(outs):
        if c == 0:
            _fail(f"{who}: segment {i} has no output pointer")
    arr = (ctypes.c_void_p * len(outs))(*outs)
    A = _aligned16(A)
    with _on_device_of(A):
        check(lib.flute_gemv_multi(descs, len(outs), A.data_ptr(), arr, _ACT[A.dtype],
                                   int(split), _stream_of(A)))
    return None


def qgemm_gemv_mlp(A, seg_table, C, lut_dtype: Optional[torch.dtype] = None, split: int = 0):
    """C = silu(gate(A)) * up(A), rows 0/1 of the table = gate/up
    (src/kernel_gemv_mlp.cu:536-691 upstream)."""
    who = "qgemm_gemv_mlp"
    _check_seg_inputs(who, A, seg_table, 2)
    if C.dtype != A.dtype or not C.is_contiguous():
        _fail(f"{who}: C must be a contiguous {A.dtype} output buffer")
    N = int(seg_table[0, 8])
    if int(seg_table[1, 8]) != N or C.numel() != N:
        _fail(f"{who}: gate/up/C must agree in N")
    if not (A.is_cuda and C.is_cuda):
        _fail(f"{who}: A and C must be CUDA (HIP) tensors")
    if C.device != A.device:
        _fail(f"{who}: C must live on A's device {A.device}")
    descs, _ = _seg_descs(who, A, seg_table, _ACT[lut_dtype or torch.float16])
    A = _aligned16(A)
    with _on_device_of(A):
        check(lib.flute_gemv_mlp(ctypes.byref(descs[0]), ctypes.byref(descs[1]), A.data_ptr(),
                                 C.data_ptr(), _ACT[A.dtype], int(split), _stream_of(A)))
    return C


# ---------------------------------------------------------------------------
# GEMM family                               (src/bindings.cpp:231-270 upstream)
# ---------------------------------------------------------------------------

def _gemm(who, A, indices, lut, bitwidth, indices2, lut2, bitwidth2, resB, resA, bias,
          group_size, gs_allowed=_GS_ALL, max_rank=256):
    M, K = _check_2d_input(who, A, need_m1=False)
    if K == 0 or M == 0 or indices.numel() == 0:
        N = 0 if K == 0 else indices.numel() // max(1, (K * int(bitwidth)) // 8)
        return torch.zeros((M, N), dtype=A.dtype, device=A.device)
    w, N, keep = _describe(who, A, K, indices, lut, bitwidth, indices2, lut2, bitwidth2,
                           resB, resA, bias, group_size, None, None, 0, gs_allowed, max_rank)
    A = _aligned16(A)
    with _on_device_of(A):
        C = torch.empty((M, N), dtype=A.dtype, device=A.device)
        check(lib.flute_gemm(ctypes.byref(w), A.data_ptr(), C.data_ptr(), M, K, N,
                             _ACT[A.dtype], _stream_of(A)))
    del keep
    return C


def _empty_like_u8(A):
    return torch.empty(0, dtype=torch.uint8, device=A.device)


def qgemm_cutlass_streaming(A, indices, lut, bitwidth, group_size, q_layout: int = 1):
    """C[M, N] = A @ W^T on the idxN blob (src/kernel_streaming.cu:2297-2443 upstream).
    The name is kept for drop-in compatibility; the kernel is an MFMA kernel."""
    if int(q_layout) != 1:
        _fail("qgemm_cutlass_streaming: only q_layout=1 (the idxN blob) is served")
    e8, e16 = _empty_like_u8(A), torch.empty(0, dtype=A.dtype, device=A.device)
    return _gemm("qgemm_cutlass_streaming", A, indices, lut, bitwidth, e8, e16, 0, e16, e16,
                 e16, group_size)


def qgemm_per_group_lut(A, indices, lut, W_dense, bitwidth, group_size, backend: str = "auto",
                        q_layout: int = 1):
    """Backend-string dispatcher (src/bindings.cpp:202-228 upstream)."""
    if backend in ("auto", "cutlass_streaming"):
        return qgemm_cutlass_streaming(A, indices, lut, bitwidth, group_size, q_layout)
    if backend == "debug_simple":
        return qgemm_debug_simple(A, indices, lut, bitwidth, group_size)
    if backend == "cutlass_dense":
        return qgemm_cutlass_dense(A, W_dense, bitwidth, group_size)
    _fail(f"qgemm_per_group_lut: unknown backend {backend!r}")


def qgemm_dual_stream(A, indices, lut, bitwidth, indices2, lut2, bitwidth2, resB, resA, bias,
                      group_size: int = 512):
    """Both streams + residual + bias in one launch at small M
    (src/kernel_streaming.cu:2113-2294 upstream)."""
    return _gemm("qgemm_dual_stream", A, indices, lut, bitwidth, indices2, lut2, bitwidth2,
                 resB, resA, bias, group_size)


def qgemm_debug_simple(A, indices, lut, bitwidth, group_size, q_layout: int = 0):
    """Scalar differential twin of the GEMM (src/kernel_debug_simple.cu:94-267 upstream):
    one thread per output, no matrix cores, no LDS.  Like upstream's twin it consumes the
    LOGICAL packed layout, indices [N, K*bitwidth/8] uint8, LSB-first along K; q_layout=1
    (an extension) reads the idxN blob instead, so that the twin and the fast kernel can be
    run on the same bytes."""
    who = "qgemm_debug_simple"
    M, K = _check_2d_input(who, A, need_m1=False)
    b, gs = int(bitwidth), int(group_size)
    if not 1 <= b <= 4:
        _fail(f"{who}: bitwidth must be 1, 2, 3 or 4 (got {b})")
    if indices.dtype != torch.uint8 or not indices.is_contiguous() or not indices.is_cuda:
        _fail(f"{who}: indices must be a contiguous uint8 tensor on the GPU")
    if not A.is_cuda or indices.device != A.device:
        _fail(f"{who}: A and indices must live on the same GPU")
    if lut.dtype not in _ACT or lut.dim() != 2 or lut.shape[1] != (1 << b) or \
            not lut.is_contiguous() or lut.device != A.device:
        _fail(f"{who}: lut must be a contiguous [groups, 2^bitwidth] float16/bfloat16 tensor on "
              f"the device of A")
    if K == 0 or (K * b) % 8:
        _fail(f"{who}: K*bitwidth must be a positive whole number of bytes (K = {K})")
    row_bytes = K * b // 8
    N = indices.numel() // row_bytes
    if N <= 0 or N * row_bytes != indices.numel():
        _fail(f"{who}: {indices.numel()} index bytes are not N*(K*{b}/8) for any N (K = {K})")
    if int(q_layout) == 0 and indices.dim() == 2 and tuple(indices.shape) != (N, row_bytes):
        _fail(f"{who}: logical indices must be [N, K*bitwidth/8] = [{N}, {row_bytes}]")
    A = A if A.stride(-1) == 1 else A.contiguous()
    with _on_device_of(A):
        C = torch.empty((M, N), dtype=A.dtype, device=A.device)
        check(lib.flute_gemm_debug_simple(indices.data_ptr(), indices.numel(), int(q_layout),
                                          lut.data_ptr(), lut.shape[0], _ACT[lut.dtype], b, gs, N,
                                          K, A.data_ptr(), C.data_ptr(), M, A.stride(0) if M else K,
                                          N, _ACT[A.dtype], _stream_of(A)))
    return C


def qgemm_cutlass_dense(A, W_dense, bitwidth, group_size):
    """Dense baseline: upstream compiles this to a refusal without CUTLASS
    (src/kernel_cutlass_dense.cu:238-254); the dense comparator on this
    hardware is torch.matmul."""
    _fail("qgemm_cutlass_dense: not built (use torch.matmul as the dense comparator)")


def dequant_idxn(indices, lut, N: int, K: int, bitwidth: int, group_size: int):
    """Dense [N, K] dump of one stream in the LUT's dtype (bit exact)."""
    who = "dequant_idxn"
    A = torch.empty((1, K), dtype=lut.dtype, device=lut.device)
    e8, e16 = _empty_like_u8(A), torch.empty(0, dtype=A.dtype, device=A.device)
    w, N2, keep = _describe(who, A, int(K), indices, lut, bitwidth, e8, e16, 0, e16, e16, e16,
                            group_size)
    if N2 != int(N):
        _fail(f"{who}: blob holds N={N2}, not {N}")
    with _on_device_of(A):
        W = torch.empty((N2, int(K)), dtype=lut.dtype, device=lut.device)
        check(lib.flute_dequant(ctypes.byref(w), 1, W.data_ptr(), _stream_of(A)))
    del keep
    return W


# ---------------------------------------------------------------------------
# LUT grouped along K (no upstream counterpart: no upstream kernel or artifact has this
# form; one 16-entry row per (output row, 128-wide K group))
# ---------------------------------------------------------------------------

K_GROUP = 128


def _describe_kgroup(who: str, A: torch.Tensor, K: int, indices, lut, bias=None, signs=None,
                     awq=None, rot_block: int = 0):
    """Descriptor of a weight whose LUT is [N, K/128, 16]: W[n, k] = lut[n, k // 128, idx[n, k]],
    indices the 4-bit idxN blob.  The checks of _describe where they apply, then the form's own."""
    if lut.dim() != 3 or lut.shape[2] != 16:
        _fail(f"{who}: a LUT grouped along K must be [N, K/{K_GROUP}, 16] (got {tuple(lut.shape)})")
    if K % K_GROUP != 0:
        _fail(f"{who}: a LUT grouped along K needs K % {K_GROUP} == 0 (got K={K})")
    N = int(lut.shape[0])
    if lut.shape[1] != K // K_GROUP:
        _fail(f"{who}: a LUT grouped along K must be [N, K/{K_GROUP}, 16] = "
              f"[{N}, {K // K_GROUP}, 16] (got {tuple(lut.shape)})")
    e8 = torch.empty(0, dtype=torch.uint8, device=A.device)
    e16 = torch.empty(0, dtype=A.dtype, device=A.device)
    # the shared checks see a stand-in LUT of the N-grouped shape for the same N
    n_blob = indices.numel() // max(K // 2, 1)
    if n_blob != N:
        _fail(f"{who}: the blob holds N={n_blob} rows, the LUT {N}")
    stand_in = lut.reshape(-1, 16)[: (N + 127) // 128]
    w, N2, keep = _describe(who, A, K, indices, stand_in, 4, e8, e16, 0, e16, e16,
                            bias if bias is not None else e16, 128, signs, awq, rot_block)
    if N2 != N:
        _fail(f"{who}: the blob holds N={N2} rows, the LUT {N}")
    if not lut.is_contiguous():
        _fail(f"{who}: the LUT must be contiguous")
    lut = _aligned16(lut)
    w.lut1 = lut.data_ptr()
    w.lut_rows = N * (K // K_GROUP)
    w.k_group = K_GROUP
    return w, N, (keep, lut)


def qgemm_gemv_kgroup(A, indices, lut, bias=None, signs=None, s=None, split: int = 0,
                      rot_block: int = 0):
    """Decode GEMV over a weight whose LUT is grouped along K: y[1, N] = A[1, K] . W^T with
    W[n, k] = lut[n, k // 128, idx[n, k]] (lut [N, K/128, 16], indices the 4-bit idxN blob).
    signs (and s) select the fused rotation of A as in qgemm_gemv_fht_stream."""
    who = "qgemm_gemv_kgroup"
    M, K = _check_2d_input(who, A, need_m1=True)
    w, N, keep = _describe_kgroup(who, A, K, indices, lut, bias, signs, s, rot_block)
    A = _aligned16(A)
    with _on_device_of(A):
        C = torch.empty((1, N), dtype=A.dtype, device=A.device)
        check(lib.flute_gemv(ctypes.byref(w), A.data_ptr(), C.data_ptr(), _ACT[A.dtype],
                             int(split), _stream_of(A)))
    del keep
    return C


def dequant_kgroup(indices, lut, K: int):
    """Dense [N, K] dump of a weight whose LUT is grouped along K, in the LUT's dtype (bit exact)."""
    who = "dequant_kgroup"
    A = torch.empty((1, int(K)), dtype=lut.dtype, device=lut.device)
    w, N, keep = _describe_kgroup(who, A, int(K), indices, lut)
    with _on_device_of(A):
        W = torch.empty((N, int(K)), dtype=lut.dtype, device=lut.device)
        check(lib.flute_dequant(ctypes.byref(w), 1, W.data_ptr(), _stream_of(A)))
    del keep
    return W


# ---------------------------------------------------------------------------
# rotation                                  (src/bindings.cpp:386-399 upstream)
# ---------------------------------------------------------------------------

def _fht(who, x, signs, awq, out, adjoint, block=0):
    if x.dim() != 2:
        _fail(f"{who}: x must be 2-D (M, K)")
    if x.dtype not in _ANY:
        _fail(f"{who}: x must be float16, bfloat16 or float32 (got {x.dtype})")
    M, K = int(x.shape[0]), int(x.shape[1])
    if K < 32 or K % 32 != 0 or K > 65504:
        _fail(f"{who}: K must be a multiple of 32 in [32, 65504] (got {K})")
    if signs.dtype != torch.float32 or signs.dim() != 1 or signs.numel() != K \
            or not signs.is_contiguous():
        _fail(f"{who}: signs must be a contiguous (K,) float32 vector")
    if awq is not None and (awq.dtype != torch.float32 or awq.dim() != 1 or awq.numel() != K
                            or not awq.is_contiguous()):
        _fail(f"{who}: s must be a contiguous (K,) float32 vector")
    if not x.is_contiguous():
        _fail(f"{who}: x must be contiguous")
    if not (x.is_cuda and signs.is_cuda and (awq is None or awq.is_cuda)):
        _fail(f"{who}: all tensors must be CUDA (HIP) tensors")
    if signs.device != x.device or (awq is not None and awq.device != x.device):
        _fail(f"{who}: all tensors must live on x's device {x.device}")
    with _on_device_of(x):
        if out is None:
            out = torch.empty_like(x)
        check(lib.flute_fht(x.data_ptr(), signs.data_ptr(), _ptr(awq), out.data_ptr(), M, K,
                            _ANY[x.dtype], int(adjoint), int(block), _stream_of(x)))
    return out


def fht_forward(x, signs, block: int = 0):
    return _fht("fht_forward", x, signs, None, None, 0, block)


def fht_backward(x, signs, block: int = 0):
    return _fht("fht_backward", x, signs, None, None, 1, block)


def fht_inplace_(x, signs, block: int = 0):
    return _fht("fht_inplace_", x, signs, None, x, 0, block)


def fht_forward_awq(x, signs, s):
    return _fht("fht_forward_awq", x, signs, s, None, 0, 0)


# ---------------------------------------------------------------------------
# host-side queries
# ---------------------------------------------------------------------------

def pick_split(N: int, K: int) -> int:
    return int(lib.flute_pick_split(int(N), int(K)))


def gemv_lds_bytes(N: int, K: int, bitwidth: int, bitwidth2: int, group_size: int,
                   fht: bool = False, residual_rank: int = 0, split: int = 0) -> int:
    """LDS bytes of one GEMV workgroup for this shape, 0 if the library refuses
    it.  Pure host arithmetic (dummy non-NULL pointers, no device access)."""
    w = FluteLinear()
    dummy = 4096
    w.q1 = w.lut1 = dummy
    b2 = int(bitwidth2)
    if b2 > 0:
        w.q2 = w.lut2 = dummy
    if residual_rank > 0:
        w.resA = w.resB = dummy
    if fht:
        w.signs = dummy
    w.N, w.K, w.R = int(N), int(K), int(residual_rank)
    w.b1, w.b2, w.group_size = int(bitwidth), b2, int(group_size)
    w.q1_bytes = w.N * w.K * w.b1 // 8
    w.q2_bytes = w.N * w.K * b2 // 8
    w.lut_rows = (w.N + w.group_size - 1) // w.group_size if w.group_size > 0 else 0
    w.lut_dtype = _lib.F16
    return int(lib.flute_gemv_lds_bytes(ctypes.byref(w), int(split)))


def embedding_gather(ids, indices, lut, N: int, K: int, bitwidth: int, group_size: int,
                     indices2=None, lut2=None, bitwidth2: int = 0, resB=None, resA=None,
                     signs=None, rot_block: int = 0, check_ids: bool = True):
    """Rows `ids` of a palettized table in the LUT's dtype (PalettizedEmbedding.forward,
    scripts/palettized_modules.py:2298-2335 upstream).  ids: any integer tensor on the
    table's device; ids outside [0, N) raise, as upstream's range check does
    (check_ids=False skips that host read for a caller that has checked already or
    is capturing a graph: the kernel then writes a row of zeros for such an id)."""
    who = "embedding_gather"
    if ids.dtype not in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8):
        _fail(f"{who}: ids must be an integer tensor, got dtype {ids.dtype}")
    if ids.device != lut.device:
        _fail(f"{who}: ids are on {ids.device}, the table on {lut.device}")
    A = torch.empty((1, int(K)), dtype=lut.dtype, device=lut.device)
    e8 = _empty_like_u8(A)
    e16 = torch.empty(0, dtype=A.dtype, device=A.device)
    w, N2, keep = _describe(who, A, int(K), indices, lut, bitwidth,
                            indices2 if indices2 is not None else e8,
                            lut2 if lut2 is not None else e16, bitwidth2,
                            resB if resB is not None else e16, resA if resA is not None else e16,
                            e16, group_size, signs, None, rot_block)
    if N2 != int(N):
        _fail(f"{who}: blob holds N={N2}, not {N}")
    flat = ids.reshape(-1).long().contiguous()
    if check_ids and flat.numel() and bool(((flat < 0) | (flat >= N2)).any()):
        _fail(f"{who}: ids must lie in [0, {N2})")
    with _on_device_of(A):
        out = torch.empty((flat.numel(), int(K)), dtype=lut.dtype, device=lut.device)
        check(lib.flute_embedding(ctypes.byref(w), flat.data_ptr(), flat.numel(), out.data_ptr(),
                                  _stream_of(A)))
    del keep
    return out.reshape(*ids.shape, int(K))


# ---------------------------------------------------------------------------
# compiled binding
# ---------------------------------------------------------------------------
# flute_extended/_C_native (csrc/torch_binding.cpp, built by csrc/build_torch_binding.py) is
# the compiled PyTorch-ROCm counterpart of upstream's pybind module for the entries a decode
# loop calls per token.  When it is built and speaks this library's ABI it takes those names
# over (same signatures, checks and messages; about a third of the host time per call); the
# Python forms above stay reachable as PYTHON_BINDING[name], serve everything else, and serve
# all of it when the module is absent or FLUTE_PYTHON_BINDING is set.  Either way the
# kernels are the ones in libflute_hip.so: there is no other implementation to fall back to.

NATIVE_NAMES = ("qgemm_gemv_stream", "qgemm_gemv_fht_stream", "qgemm_gemv_splitk_stream",
                "qgemm_gemv_splitk_fht_stream", "qgemm_gemv_multi", "qgemm_gemv_mlp",
                "qgemm_cutlass_streaming", "qgemm_dual_stream")
PYTHON_BINDING = {name: globals()[name] for name in NATIVE_NAMES}
native = None


def _load_native():
    import os
    if os.environ.get("FLUTE_PYTHON_BINDING"):
        return None
    try:
        from . import _C_native
    except ImportError:
        return None
    if _C_native.abi_version() != lib.flute_abi_version():
        return None
    return _C_native


native = _load_native()
if native is not None:
    for _name in NATIVE_NAMES:
        globals()[_name] = getattr(native, _name)
    del _name
