"""The idxN layout: three independent statements of the upstream map must agree
(scalar walk and vectorised map in oracle/flute_oracle.py, the C restatement,
and the product packer), plus the identities upstream states about the layout
(flute_extended/idxN.py:37-55, 311-329; include/flute/gemv.cuh:66-96)."""
import ctypes
import os

import numpy as np
import pytest

import flute_oracle as O
from flute_extended import idxN as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def clib():
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        pytest.skip("oracle/liboracle.so not built (run __graft_entry__.build())")
    return ctypes.CDLL(path)


def _c_pack(clib, idx, b):
    N, K = idx.shape
    out = np.zeros(N * K * b // 8, dtype=np.uint8)
    assert clib.oracle_pack_idxn(idx.ctypes.data_as(ctypes.c_void_p), N, K, b,
                                 out.ctypes.data_as(ctypes.c_void_p)) == 0
    return out


@pytest.mark.parametrize("b", [1, 2, 3, 4])
def test_three_statements_agree_on_one_tile(b, clib):
    rng = np.random.default_rng(10 + b)
    idx = rng.integers(0, 1 << b, size=(128, 64), dtype=np.uint8)
    scalar = O.pack_idxn_scalar(idx, b)
    assert np.array_equal(scalar, O.pack_idxn(idx, b))
    assert np.array_equal(scalar, P.pack_idxn(idx, b))
    assert np.array_equal(scalar, _c_pack(clib, idx, b))


@pytest.mark.parametrize("b", [1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(256, 128), (384, 192), (1024, 512)])
def test_pack_unpack_agree_and_round_trip(b, shape, clib):
    rng = np.random.default_rng(b * 100 + shape[0])
    idx = rng.integers(0, 1 << b, size=shape, dtype=np.uint8)
    blob = P.pack_idxn(idx, b)
    assert blob.size == shape[0] * shape[1] * b // 8 == P.blob_bytes(*shape, b)
    assert np.array_equal(blob, O.pack_idxn(idx, b))
    assert np.array_equal(blob, _c_pack(clib, idx, b))
    assert np.array_equal(P.unpack_idxn(blob, *shape, b), idx)
    assert np.array_equal(O.unpack_idxn(blob, *shape, b), idx)
    back = np.zeros_like(idx)
    assert clib.oracle_unpack_idxn(blob.ctypes.data_as(ctypes.c_void_p), shape[0], shape[1], b,
                                   back.ctypes.data_as(ctypes.c_void_p)) == 0
    assert np.array_equal(back, idx)


def test_b4_chunk_byte_is_the_logical_packed_byte():
    """idxN.py:52-55 upstream: at b = 4, byte p of chunk (wx, lane) of tile (t, g)
    equals q[n, kp], kp = g*32 + kt*8 + (lane & 3) + 4*s2, with q the LSB-first
    nibble rows (even k in the low nibble)."""
    rng = np.random.default_rng(3)
    N, K = 256, 192
    idx = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    q = (idx[:, 0::2] | (idx[:, 1::2] << 4)).astype(np.uint8)
    assert np.array_equal(q, O.logical_packed_rows(idx, 4))
    blob = P.pack_idxn(idx, 4).reshape(N // 128, K // 64, 64, 64)
    for t in range(N // 128):
        for g in range(K // 64):
            for th in (0, 5, 31, 32, 47, 63):
                wx, lane = th >> 5, th & 31
                for p in range(64):
                    kt, v, d, s2 = p >> 4, (p >> 2) & 3, (p >> 1) & 1, p & 1
                    n = t * 128 + wx * 64 + v * 16 + d * 8 + (lane >> 2)
                    kp = g * 32 + kt * 8 + (lane & 3) + 4 * s2
                    assert blob[t, g, th, p] == q[n, kp]


@pytest.mark.parametrize("b", [1, 2, 3])
def test_sub4_pair_codes_as_the_gemv_decode_reads_them(b):
    """include/flute/gemv.cuh:66-96 upstream: the two codes of pair p come from
    b = 2: byte p>>1, bits 4*(p&1) and +2;  b = 1: byte p>>2, bits 2*(p&3) and +1;
    b = 3: 24-bit little-endian group 3*(p>>2), 6-bit field 6*(p&3)."""
    rng = np.random.default_rng(20 + b)
    idx = rng.integers(0, 1 << b, size=(128, 64), dtype=np.uint8)
    blob = P.pack_idxn(idx, b).reshape(64, 16 * b)
    for th in (0, 9, 33, 63):
        chunk = blob[th]
        for p in range(64):
            if b == 2:
                byte = int(chunk[p >> 1]); sh = 4 * (p & 1)
                c0, c1 = (byte >> sh) & 3, (byte >> (sh + 2)) & 3
            elif b == 1:
                byte = int(chunk[p >> 2]); sh = 2 * (p & 3)
                c0, c1 = (byte >> sh) & 1, (byte >> (sh + 1)) & 1
            else:
                o = 3 * (p >> 2)
                val = int(chunk[o]) | int(chunk[o + 1]) << 8 | int(chunk[o + 2]) << 16
                c0, c1 = (val >> (6 * (p & 3))) & 7, (val >> (6 * (p & 3) + 3)) & 7
            r, k = O.pair_coords(th, p)
            assert (c0, c1) == (idx[r, k], idx[r, k + 1])


def test_tile_offsets_and_sizes():
    """Tile (t, g) sits at byte ((t*K/64)+g)*1024*b (idxN.py:39-41 upstream):
    changing one index changes bytes of exactly that tile."""
    N, K, b = 384, 256, 3
    base = np.zeros((N, K), dtype=np.uint8)
    ref = P.pack_idxn(base, b)
    for (n, k) in ((0, 0), (130, 70), (383, 255), (200, 64)):
        idx = base.copy(); idx[n, k] = 7
        diff = np.nonzero(P.pack_idxn(idx, b) != ref)[0]
        t, g = n // 128, k // 64
        lo = ((t * (K // 64)) + g) * 1024 * b
        assert diff.size > 0 and diff.min() >= lo and diff.max() < lo + 1024 * b


def test_refusals():
    idx = np.zeros((128, 64), dtype=np.uint8)
    for mod in (P, O):
        with pytest.raises(ValueError):
            mod.pack_idxn(np.zeros((100, 64), dtype=np.uint8), 4)     # N % 128
        with pytest.raises(ValueError):
            mod.pack_idxn(np.zeros((128, 32), dtype=np.uint8), 4)     # K % 64
        with pytest.raises(ValueError):
            mod.pack_idxn(idx, 5)                                     # width
        with pytest.raises(ValueError):
            mod.pack_idxn(idx + 4, 2)                                 # value >= 2**b
        blob = mod.pack_idxn(idx, 2)
        with pytest.raises(ValueError):
            mod.unpack_idxn(blob, 128, 64, 4)                         # width confusion
        with pytest.raises(ValueError):
            mod.unpack_idxn(blob[:-1], 128, 64, 2)                    # truncated blob
    assert P.self_test(shapes=((128, 64), (256, 128)))


def test_from_packed_rows():
    rng = np.random.default_rng(5)
    for b in (1, 2, 3, 4):
        idx = rng.integers(0, 1 << b, size=(128, 128), dtype=np.uint8)
        rows = O.logical_packed_rows(idx, b)
        assert rows.shape == (128, P.packed_row_bytes(128, b))
        assert np.array_equal(P.pack_idxn_from_packed(rows, b), O.pack_idxn(idx, b))
