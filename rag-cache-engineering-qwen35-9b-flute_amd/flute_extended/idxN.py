"""idxN blob packer / unpacker (bit widths 1..4), numpy only.

Same contract as the upstream module of this name
(src/flute_extended/flute_extended/idxN.py): `pack_idxn`, `unpack_idxn`,
`pack_idxn_from_packed`, `blob_bytes`, `packed_row_bytes`, `check_bits`,
`check_eligible`, `self_test`, and the tile constants.  Importing it needs no
GPU and no compiled library.

Layout (upstream idxN.py:37-55).  The blob is a permutation of the logical
index matrix I[N, K] (N % 128 == 0, K % 64 == 0):

  * one tile of 1024*b bytes per (t = n // 128, g = k // 64) at byte
    ((t * K//64) + g) * 1024*b;
  * inside a tile, chunk th = wx*32 + lane (wx < 2, lane < 32) is the 16*b
    bytes at th*16*b and holds 64 k-pairs; pair p = kt*16 + v*4 + d*2 + s2 sits
    at bit 2*b*p (LSB first) and covers
        n = t*128 + wx*64 + v*16 + d*8 + (lane >> 2)
        k = g*64  + kt*16 + 2*(lane & 3) + 8*s2      and k + 1.

Implementation.  Both index axes factor exactly along those digits,

    n = (t, wx, v, d, lane>>2)        k = (g, kt, s2, lane&3, j)

so the permutation is one reshape + transpose of a 10-axis view; no gather
tables are needed.  The b-bit fields of a chunk are then packed with integer
shifts on uint64 words.
"""
from __future__ import annotations

import numpy as np

ROWS_PER_TILE = 128
K_PER_GROUP = 64
PAIRS_PER_CHUNK = 64
CHUNK_BYTES_PER_BIT = 2
TILE_THREADS = 64
TILE_BYTES_PER_BIT = 1024

BITS_SUPPORTED = (1, 2, 3, 4)

# axes of the 10-d view of I[N, K]: (t, wx, v, d, r8 | g, kt, s2, i, j)
_TO_BLOB = (0, 5, 1, 4, 8, 6, 2, 3, 7, 9)      # -> (t, g, wx, r8, i | kt, v, d, s2, j)
_FROM_BLOB = tuple(int(a) for a in np.argsort(_TO_BLOB))


def check_bits(bits: int) -> int:
    b = int(bits)
    if b not in BITS_SUPPORTED:
        raise ValueError(f"idxN supports bit widths {BITS_SUPPORTED}, got bits={bits}")
    return b


def check_eligible(N: int, K: int) -> None:
    if int(N) % ROWS_PER_TILE != 0:
        raise ValueError(f"idxN layout requires N % 128 == 0, got N={N}")
    if int(K) % K_PER_GROUP != 0:
        raise ValueError(f"idxN layout requires K % 64 == 0, got K={K}")


def blob_bytes(N: int, K: int, bits: int) -> int:
    return (int(N) * int(K) * check_bits(bits)) // 8


def packed_row_bytes(K: int, bits: int) -> int:
    return (int(K) * check_bits(bits)) // 8


def _pack_fields(fields: np.ndarray, b: int) -> np.ndarray:
    """(..., 8*m) b-bit values -> (..., b*m) bytes, LSB first.

    Eight consecutive fields always fill exactly b bytes, so they are combined
    into one little-endian uint64 word and its low b bytes are kept.
    """
    lead = fields.shape[:-1]
    oct_ = fields.reshape(*lead, -1, 8).astype(np.uint64)
    word = np.zeros(oct_.shape[:-1], dtype=np.uint64)
    for j in range(8):
        word |= oct_[..., j] << np.uint64(b * j)
    # the bytes of a little-endian uint64, in ascending significance
    as_bytes = np.ascontiguousarray(word).astype("<u8").view(np.uint8).reshape(*word.shape, 8)
    return np.ascontiguousarray(as_bytes[..., :b]).reshape(*lead, -1)


def _unpack_fields(data: np.ndarray, b: int) -> np.ndarray:
    """Inverse of _pack_fields: (..., b*m) bytes -> (..., 8*m) values."""
    lead = data.shape[:-1]
    grp = data.reshape(*lead, -1, b)
    padded = np.zeros(grp.shape[:-1] + (8,), dtype=np.uint8)
    padded[..., :b] = grp
    word = padded.view("<u8")[..., 0]
    mask = np.uint64((1 << b) - 1)
    out = np.empty(word.shape + (8,), dtype=np.uint8)
    for j in range(8):
        out[..., j] = ((word >> np.uint64(b * j)) & mask).astype(np.uint8)
    return out.reshape(*lead, -1)


def pack_idxn(indices: np.ndarray, bits: int) -> np.ndarray:
    """Logical b-bit indices [N, K] -> flat uint8 idxN blob of N*K*b/8 bytes."""
    b = check_bits(bits)
    idx = np.ascontiguousarray(indices, dtype=np.uint8)
    if idx.ndim != 2:
        raise ValueError(f"expected a 2-D index matrix, got shape {idx.shape}")
    N, K = idx.shape
    check_eligible(N, K)
    if idx.size and int(idx.max()) >= (1 << b):
        raise ValueError(f"idx{b} indices must be < {1 << b}, got max {int(idx.max())}")
    T, G = N // ROWS_PER_TILE, K // K_PER_GROUP
    view = idx.reshape(T, 2, 4, 2, 8, G, 4, 2, 4, 2)
    chunks = np.ascontiguousarray(view.transpose(_TO_BLOB)).reshape(T, G, TILE_THREADS, 128)
    return np.ascontiguousarray(_pack_fields(chunks, b).reshape(-1))


def unpack_idxn(blob: np.ndarray, N: int, K: int, bits: int) -> np.ndarray:
    """Flat idxN blob -> logical indices [N, K] (uint8)."""
    b = check_bits(bits)
    check_eligible(N, K)
    flat = np.ascontiguousarray(blob, dtype=np.uint8).reshape(-1)
    want = blob_bytes(N, K, b)
    if flat.size != want:
        raise ValueError(
            f"idx{b} blob has {flat.size} bytes, expected N*K*{b}/8 = {want} (N={N}, K={K})")
    T, G = N // ROWS_PER_TILE, K // K_PER_GROUP
    fields = _unpack_fields(flat.reshape(T, G, TILE_THREADS, 16 * b), b)
    view = fields.reshape(T, G, 2, 8, 4, 4, 4, 2, 2, 2)
    return np.ascontiguousarray(view.transpose(_FROM_BLOB)).reshape(N, K)


def pack_idxn_from_packed(q: np.ndarray, bits: int) -> np.ndarray:
    """Logical packed rows [N, K*b/8] (LSB first along K) -> idxN blob."""
    b = check_bits(bits)
    q = np.ascontiguousarray(q, dtype=np.uint8)
    if q.ndim != 2:
        raise ValueError(f"expected a 2-D packed matrix, got shape {q.shape}")
    if q.shape[1] % b != 0:
        raise ValueError(f"row byte count {q.shape[1]} is not a multiple of {b}")
    return pack_idxn(_unpack_fields(q, b), b)


def self_test(shapes=((128, 64), (256, 128), (384, 192), (1024, 512)),
              bits_all=BITS_SUPPORTED) -> bool:
    """Round trip at every width; a blob read at the wrong width must be refused."""
    rng = np.random.default_rng(0)
    for b in bits_all:
        for N, K in shapes:
            idx = rng.integers(0, 1 << b, size=(N, K), dtype=np.uint8)
            blob = pack_idxn(idx, b)
            assert blob.size == blob_bytes(N, K, b)
            assert np.array_equal(unpack_idxn(blob, N, K, b), idx), (b, N, K)
            try:
                unpack_idxn(blob, N, K, 2 if b == 4 else 4)
            except ValueError:
                pass
            else:
                raise AssertionError("width confusion not caught")
            # the logical row stream re-packs to the same blob
            rows = _pack_fields(idx, b)
            assert np.array_equal(pack_idxn_from_packed(rows, b), blob), (b, N, K)
    return True


if __name__ == "__main__":
    print("idxN self_test:", "PASS" if self_test() else "FAIL")
