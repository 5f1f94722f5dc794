"""CPU oracle for the idxN LUT-palettized linear layer.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this file;
only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
call it, and only as the checker.

It restates, in plain numpy/torch-CPU, the algorithm of the upstream
`forward="reference"` path.  Every function cites the upstream file:line it
follows (paths relative to the upstream tree).

How each function is pinned (none of them by re-typing its own formula):

  pair_coords / pack_idxn / unpack_idxn
      * three independent statements must agree byte for byte: the scalar
        closed-form walk here (pack_idxn_scalar), the vectorised map here
        (pack_idxn), and the C restatement (flute_oracle.c);
      * at b=4 chunk byte p equals the logical packed byte q[n, kp],
        kp = kt*8 + (lane&3) + 4*s2  (flute_extended/flute_extended/idxN.py:52-55);
      * the bit-field statement used by the upstream GEMV decode
        (include/flute/gemv.cuh:66-96) is checked as a separate reading of the
        same bit positions (tests/test_oracle_idxn.py);
      * round trip, blob size N*K*b/8, width confusion refused
        (idxN.py:311-329).
  dequant
      pure gather, bit exact by definition (docs/QUANTIZATION.md:28-38,161-171).
  linear_reference / mlp_reference
      checked against an fp64 evaluation of the closed form
      y = x W1^T + x W2^T + (x resB^T) resA^T + bias, and against hand-built
      cases (one-hot x selects a weight column; constant LUT gives sum(x)*c).
  fht_reference / fht_adjoint
      checked against the explicit Sylvester matrix x @ T, H H = b I,
      adjoint(forward(x)) == x, norm preservation, per-segment independence
      (fht.py:19-35,137-167,740-771).
  rotation_signs
      values pinned: upstream's recipe (fht.py:105-115) is randint(0, 2) on a CPU
      generator seeded seed + 4242, i.e. the low bit of each word of the textbook
      MT19937 stream; checked against numpy's MT19937 at K = 64, 4096, 12288 and
      against the generator written out in the test (tests/test_oracle_math.py).
  pick_split
      the worked examples printed in src/kernel_gemv_splitk.cu:54-59.
"""
from __future__ import annotations

import math
from typing import List, Optional, Tuple

import numpy as np
import torch

ROWS_PER_TILE = 128      # idxN.py:85
K_PER_TILE = 64          # idxN.py:86
CHUNKS_PER_TILE = 64     # idxN.py:89
PAIRS_PER_CHUNK = 64     # idxN.py:87


# --------------------------------------------------------------------------
# idxN blob layout                      (idxN.py:37-55, QUANTIZATION.md:79-101)
# --------------------------------------------------------------------------

def check_shape(N: int, K: int, bits: int) -> None:
    """idxN.py:95-108 — widths 1..4, N % 128 == 0, K % 64 == 0, else ValueError."""
    if int(bits) not in (1, 2, 3, 4):
        raise ValueError(f"bits must be 1..4, got {bits}")
    if N % ROWS_PER_TILE != 0:
        raise ValueError(f"N % 128 != 0 (N={N})")
    if K % K_PER_TILE != 0:
        raise ValueError(f"K % 64 != 0 (K={K})")


def pair_coords(th: int, p: int) -> Tuple[int, int]:
    """Tile-local (row, k) of the FIRST element of pair p of chunk th.

    idxN.py:46-51: p = kt*16 + v*4 + d*2 + s2;
    row = wx*64 + v*16 + d*8 + (lane >> 2);  k = kt*16 + 2*(lane & 3) + 8*s2.
    The second element of the pair is (row, k+1).
    """
    wx, lane = th >> 5, th & 31
    kt, v, d, s2 = p >> 4, (p >> 2) & 3, (p >> 1) & 1, p & 1
    return wx * 64 + v * 16 + d * 8 + (lane >> 2), kt * 16 + 2 * (lane & 3) + 8 * s2


def pack_idxn_scalar(idx: np.ndarray, bits: int) -> np.ndarray:
    """Scalar walk of the normative layout (small shapes only).

    Writes field f = 2p+j (j = 0 for k, 1 for k+1) of chunk th at bit offset
    b*f of the chunk, LSB first (idxN.py:46-47, 158-192), chunk th at byte
    th*16*b of the tile, tile (t,g) at byte ((t*K/64)+g)*1024*b (idxN.py:39-44).
    """
    N, K = idx.shape
    check_shape(N, K, bits)
    b = int(bits)
    G = K // K_PER_TILE
    blob = np.zeros(N * K * b // 8, dtype=np.uint8)
    for t in range(N // ROWS_PER_TILE):
        for g in range(G):
            tile0 = (t * G + g) * 1024 * b
            for th in range(CHUNKS_PER_TILE):
                chunk0 = tile0 + th * 16 * b
                for p in range(PAIRS_PER_CHUNK):
                    r, k = pair_coords(th, p)
                    for j in range(2):
                        val = int(idx[t * 128 + r, g * 64 + k + j])
                        bit = b * (2 * p + j)
                        for q in range(b):
                            if (val >> q) & 1:
                                pos = bit + q
                                blob[chunk0 + (pos >> 3)] |= np.uint8(1 << (pos & 7))
    return blob


def _maps() -> Tuple[np.ndarray, np.ndarray]:
    """(row, k) of every field of every chunk: two [64, 128] arrays
    (idxN.py:124-155)."""
    rows = np.empty((CHUNKS_PER_TILE, 128), dtype=np.int64)
    cols = np.empty((CHUNKS_PER_TILE, 128), dtype=np.int64)
    for th in range(CHUNKS_PER_TILE):
        for p in range(PAIRS_PER_CHUNK):
            r, k = pair_coords(th, p)
            rows[th, 2 * p] = rows[th, 2 * p + 1] = r
            cols[th, 2 * p] = k
            cols[th, 2 * p + 1] = k + 1
    return rows, cols


def _fields_to_bytes(fields: np.ndarray, b: int) -> np.ndarray:
    """(..., 128) b-bit fields -> (..., 16*b) bytes, LSB first (idxN.py:158-192).

    Done through an explicit bit matrix so that all four widths share one
    statement (the upstream packer special-cases each width)."""
    bitsel = (fields[..., :, None].astype(np.uint8) >> np.arange(b, dtype=np.uint8)) & 1
    flat = bitsel.reshape(*fields.shape[:-1], 128 * b)
    return np.packbits(flat, axis=-1, bitorder="little")


def _bytes_to_fields(chunk_bytes: np.ndarray, b: int) -> np.ndarray:
    """Inverse of _fields_to_bytes (idxN.py:195-232)."""
    flat = np.unpackbits(chunk_bytes, axis=-1, bitorder="little")
    bitsel = flat.reshape(*chunk_bytes.shape[:-1], 128, b)
    weights = (1 << np.arange(b)).astype(np.uint8)
    return (bitsel * weights).sum(axis=-1).astype(np.uint8)


def pack_idxn(idx: np.ndarray, bits: int) -> np.ndarray:
    """Logical [N, K] indices -> idxN blob (idxN.py:235-264)."""
    idx = np.ascontiguousarray(idx, dtype=np.uint8)
    if idx.ndim != 2:
        raise ValueError("expected [N, K]")
    N, K = idx.shape
    check_shape(N, K, bits)
    b = int(bits)
    if idx.size and int(idx.max()) >= (1 << b):
        raise ValueError(f"index >= 2**{b}")
    rows, cols = _maps()
    T, G = N // 128, K // 64
    rr = rows[None, None] + (np.arange(T) * 128)[:, None, None, None]
    cc = cols[None, None] + (np.arange(G) * 64)[None, :, None, None]
    fields = idx[rr, cc]                                  # [T, G, 64, 128]
    return np.ascontiguousarray(_fields_to_bytes(fields, b).reshape(-1))


def unpack_idxn(blob: np.ndarray, N: int, K: int, bits: int) -> np.ndarray:
    """idxN blob -> logical [N, K] indices (idxN.py:267-291)."""
    check_shape(N, K, bits)
    b = int(bits)
    blob = np.ascontiguousarray(blob, dtype=np.uint8).reshape(-1)
    if blob.size != N * K * b // 8:
        raise ValueError(f"blob has {blob.size} bytes, expected {N * K * b // 8}")
    rows, cols = _maps()
    T, G = N // 128, K // 64
    fields = _bytes_to_fields(blob.reshape(T, G, 64, 16 * b), b)
    rr = rows[None, None] + (np.arange(T) * 128)[:, None, None, None]
    cc = cols[None, None] + (np.arange(G) * 64)[None, :, None, None]
    out = np.empty((N, K), dtype=np.uint8)
    out[rr, cc] = fields
    return out


def logical_packed_rows(idx: np.ndarray, bits: int) -> np.ndarray:
    """[N, K] indices -> [N, K*b/8] LSB-first row stream (QUANTIZATION.md:40-51)."""
    N, K = idx.shape
    b = int(bits)
    bitsel = (idx[..., None].astype(np.uint8) >> np.arange(b, dtype=np.uint8)) & 1
    return np.packbits(bitsel.reshape(N, K * b), axis=-1, bitorder="little")


# --------------------------------------------------------------------------
# dequantisation and the reference forward
# --------------------------------------------------------------------------

def dequant(blob, lut: torch.Tensor, N: int, K: int, group_size: int,
            bits: int = 4) -> torch.Tensor:
    """W[n, k] = LUT[n // gs, idx[n, k]] as fp32 (palettized_modules.py:125-162)."""
    if torch.is_tensor(blob):
        blob = blob.detach().cpu().numpy()
    idx = unpack_idxn(blob, N, K, bits)
    lut2 = lut.reshape(-1, 1 << int(bits))
    groups = (torch.arange(N) // int(group_size)).clamp_(max=lut2.shape[0] - 1)
    return lut2[groups].float().gather(1, torch.from_numpy(idx.astype(np.int64)))


def linear_reference(x: torch.Tensor, blob, lut, N: int, K: int, group_size: int,
                     bits: int = 4, blob2=None, lut2=None, bits2: int = 0,
                     resA=None, resB=None, bias=None, signs=None,
                     awq_scale=None) -> torch.Tensor:
    """The upstream reference forward, step for step
    (palettized_modules.py:1204-1211, 1235-1251, 1360-1369):

    rotate (if signs) -> x.float() @ W1^T (+ x.float() @ W2^T, one fp32 add)
    -> cast to x.dtype -> + ((x @ resB^T) @ resA^T) computed in resA's dtype,
    cast to the output dtype -> + bias.
    """
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    if signs is not None:
        if awq_scale is not None:
            x2 = fht_awq_reference(x2, signs, awq_scale)
        else:
            x2 = fht_reference(x2, signs)
    xf = x2.float()
    y = xf @ dequant(blob, lut, N, K, group_size, bits).t()
    if blob2 is not None:
        y = y + xf @ dequant(blob2, lut2, N, K, group_size, bits2).t()
    out = y.to(x2.dtype)
    if resA is not None and resB is not None:
        xr = x2.to(resA.dtype)
        out = out + ((xr @ resB.t()) @ resA.t()).to(out.dtype)
    if bias is not None:
        out = out + bias
    return out.reshape(*shape[:-1], N)


def linear_exact(x: torch.Tensor, blob, lut, N, K, group_size, bits=4, blob2=None,
                 lut2=None, bits2=0, resA=None, resB=None, bias=None) -> torch.Tensor:
    """fp64 evaluation of y = x W1^T + x W2^T + (x resB^T) resA^T + bias
    (QUANTIZATION.md:30-34) with NO intermediate rounding.  x is taken as
    given (already rotated).  Bounds both the reference forward and the fused
    kernels, which round once at the end (kernel_gemv.cu:238-252)."""
    xd = x.reshape(-1, K).double()
    y = xd @ dequant(blob, lut, N, K, group_size, bits).double().t()
    if blob2 is not None:
        y = y + xd @ dequant(blob2, lut2, N, K, group_size, bits2).double().t()
    if resA is not None and resB is not None:
        y = y + (xd @ resB.double().t()) @ resA.double().t()
    if bias is not None:
        y = y + bias.double()
    return y


def silu_mul_exact(yg: torch.Tensor, yu: torch.Tensor) -> torch.Tensor:
    """silu(yg) * yu = yg / (1 + exp(-yg)) * yu  (kernel_gemv_mlp.cu:382-383),
    evaluated in the dtype given (pass fp64 for a bound)."""
    return yg / (1.0 + torch.exp(-yg)) * yu


def mlp_reference(x, gate: dict, up: dict, down: dict) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)) through the reference forward of each module
    (palettized_modules.py:1673-1682; modeling.py:989-1003).  Each dict holds
    the keyword arguments of linear_reference."""
    g = linear_reference(x, **gate)
    u = linear_reference(x, **up)
    h = torch.nn.functional.silu(g) * u
    return linear_reference(h, **down)


# --------------------------------------------------------------------------
# Walsh-Hadamard rotation                           (fht.py:105-260, 583-652)
# --------------------------------------------------------------------------

def rotation_signs(K: int, seed: int) -> torch.Tensor:
    """fht.py:105-115 — randint(0,2,(K,)) * 2 - 1 from manual_seed(seed+4242)."""
    g = torch.Generator().manual_seed(int(seed) + 4242)
    return torch.randint(0, 2, (int(K),), generator=g).float().mul(2).sub(1)


def segments(K: int) -> List[Tuple[int, int]]:
    """fht.py:118-134 — descending power-of-two blocks [(offset, size)]."""
    out, off, rem = [], 0, int(K)
    while rem > 0:
        b = 1 << (rem.bit_length() - 1)
        out.append((off, b))
        off += b
        rem -= b
    return out


def hadamard(b: int) -> np.ndarray:
    """Sylvester H_b by its closed form H[i, j] = (-1)^popcount(i & j)
    (equals the recursive doubling of fht.py:137-148)."""
    i = np.arange(b)
    parity = np.zeros((b, b), dtype=np.int64)
    anded = i[:, None] & i[None, :]
    while anded.any():
        parity ^= anded & 1
        anded >>= 1
    return (1 - 2 * parity).astype(np.float64)


def rotation_matrix(signs: torch.Tensor) -> np.ndarray:
    """Explicit T (fp64): blockdiag of H_b * s[None, :] / sqrt(b)
    (fht.py:151-167)."""
    K = signs.numel()
    s = signs.double().numpy()
    T = np.zeros((K, K), dtype=np.float64)
    for off, b in segments(K):
        T[off:off + b, off:off + b] = hadamard(b) * s[None, off:off + b] / math.sqrt(b)
    return T


def _butterfly_np(v: np.ndarray) -> np.ndarray:
    """Stage-doubling WHT on the last axis in fp32: for len = 1, 2, 4, ...
    every pair (i, i+len) inside a 2*len group becomes (a+b, a-b)
    (fht.py:174-192; include/flute/fht.cuh stage definition)."""
    v = v.astype(np.float32).copy()
    b = v.shape[-1]
    ln = 1
    while ln < b:
        w = v.reshape(*v.shape[:-1], b // (2 * ln), 2, ln)
        lo = w[..., 0, :] + w[..., 1, :]
        hi = w[..., 0, :] - w[..., 1, :]
        v = np.stack([lo, hi], axis=-2).reshape(*v.shape[:-1], b)
        ln *= 2
    return v


def fht_reference(x: torch.Tensor, signs: torch.Tensor) -> torch.Tensor:
    """x @ T = ((x @ H) * s) * (1/sqrt(b)) per segment, fp32, cast back
    (fht.py:206-222)."""
    K = x.shape[-1]
    v = x.reshape(-1, K).float().numpy()
    s = signs.float().numpy()
    out = np.empty_like(v)
    for off, b in segments(K):
        seg = _butterfly_np(v[:, off:off + b])
        out[:, off:off + b] = (seg * s[None, off:off + b]) * np.float32(1.0 / math.sqrt(b))
    return torch.from_numpy(out).reshape(x.shape).to(x.dtype)


def fht_adjoint_reference(v: torch.Tensor, signs: torch.Tensor) -> torch.Tensor:
    """v @ T^T = ((v * s) @ H) * (1/sqrt(b)) per segment (fht.py:225-238)."""
    K = v.shape[-1]
    g = v.reshape(-1, K).float().numpy()
    s = signs.float().numpy()
    out = np.empty_like(g)
    for off, b in segments(K):
        seg = _butterfly_np(g[:, off:off + b] * s[None, off:off + b])
        out[:, off:off + b] = seg * np.float32(1.0 / math.sqrt(b))
    return torch.from_numpy(out).reshape(v.shape).to(v.dtype)


def fht_awq_reference(x: torch.Tensor, signs: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    """((x * s) @ T) / s in fp32 with a true division, cast back
    (fht.py:646-651)."""
    out = fht_reference(x.float() * s.float(), signs).float() / s.float()
    return out.to(x.dtype)


def block_fht_reference(x: torch.Tensor, block: int, signs: Optional[torch.Tensor] = None
                        ) -> torch.Tensor:
    """Block-diagonal transform with equal blocks of `block` columns, each
    normalised by 1/sqrt(block): the reference butterfly applied to the rows
    reshaped to (-1, block).  With signs it is the blockdiag of the same.
    This is the variant the benchmark configuration names (block 128); the
    upstream code has no such mode, so it is defined by this closed form."""
    K = x.shape[-1]
    assert K % block == 0 and block & (block - 1) == 0
    v = x.reshape(-1, block).float().numpy()
    seg = _butterfly_np(v).reshape(-1, K)
    if signs is not None:
        seg = seg * signs.float().numpy()[None, :]
    seg = seg * np.float32(1.0 / math.sqrt(block))
    return torch.from_numpy(seg.astype(np.float32)).reshape(x.shape).to(x.dtype)


# --------------------------------------------------------------------------
# split policy                                         (gemv_host.cpp:29-38)
# --------------------------------------------------------------------------

def pick_split_upstream(tiles: int, G: int) -> int:
    """The upstream A10G policy: largest power of two <= 16 with
    G % (4*s) == 0, stopping once tiles*s >= 160; 1 when tiles >= 160."""
    if tiles >= 160:
        return 1
    best, s = 1, 2
    while s <= 16:
        if G < 4 * s or G % (4 * s) != 0:
            break
        best = s
        if tiles * s >= 160:
            break
        s <<= 1
    return best


def embedding_reference(ids, blob, lut, N, K, group_size, bits, blob2=None, lut2=None, bits2=0,
                        resA=None, resB=None, signs=None):
    """Rows `ids` of a palettized embedding table, in the dtype ladder of
    PalettizedEmbedding.forward (scripts/palettized_modules.py:1998-2015, 2298-2335):
    16-bit add of the two streams (stream 1 first), fp32 residual resA[ids] @ resB,
    adjoint rotation of the sum for a rotated table, one cast to the LUT's dtype.
    A composition of dequant and fht_adjoint_reference, which carry the pins."""
    ids = torch.as_tensor(ids).long()
    w = dequant(blob, lut, N, K, group_size, bits).to(lut.dtype)[ids]
    if bits2:
        w = w + dequant(blob2, lut2, N, K, group_size, bits2).to(lut.dtype)[ids]
    w = w.float()
    if resA is not None:
        w = w + resA[ids].float() @ resB.float()
    if signs is not None:
        flat = fht_adjoint_reference(w.reshape(-1, K), signs)
        w = flat.reshape(w.shape)
    return w.to(lut.dtype)
