"""Pins of the floating-point half of the oracle: dequantisation, the reference
forward, SiLU*mul, the rotation and the split policy, each against something
the mathematics fixes rather than against its own formula."""
import ctypes
import math
import json
import os

import numpy as np
import pytest
import torch

import flute_oracle as O
from _util import make_weight, make_x, rel_l2

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_dequant_is_a_gather():
    w = make_weight(256, 128, bits=3, gs=64, seed=2)
    W = O.dequant(w["blob"], w["lut"], 256, 128, 64, 3)
    idx = w["idx"].long()
    for n, k in ((0, 0), (63, 5), (64, 5), (255, 127), (130, 77)):
        assert W[n, k].item() == w["lut"][n // 64, idx[n, k]].float().item()
    assert W.dtype == torch.float32 and W.shape == (256, 128)


def test_dequant_c_matches_numpy():
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        pytest.skip("oracle/liboracle.so not built")
    lib = ctypes.CDLL(path)
    for b, dt in ((4, torch.float16), (2, torch.bfloat16)):
        w = make_weight(256, 128, bits=b, gs=128, seed=b, lut_dtype=dt)
        W = np.zeros((256, 128), dtype=np.float32)
        blob = w["blob"].numpy()
        lut = w["lut"].view(torch.int16).numpy()
        assert lib.oracle_dequant(blob.ctypes.data_as(ctypes.c_void_p),
                                  lut.ctypes.data_as(ctypes.c_void_p), int(dt == torch.bfloat16),
                                  256, 128, 128, b, W.ctypes.data_as(ctypes.c_void_p)) == 0
        assert np.array_equal(W, O.dequant(w["blob"], w["lut"], 256, 128, 128, b).numpy())


def test_linear_special_cases():
    N, K = 128, 64
    w = make_weight(N, K, bits=4, gs=128, seed=4)
    W = O.dequant(w["blob"], w["lut"], N, K, 128, 4)
    # a one-hot x selects column k of W
    x = torch.zeros(1, K, dtype=torch.float16); x[0, 17] = 1.0
    y = O.linear_reference(x, w["blob"], w["lut"], N, K, 128, 4)
    assert torch.equal(y[0], W[:, 17].half())
    # a constant LUT makes every output c * sum(x)
    lut = torch.full_like(w["lut"], 0.5)
    x = make_x(1, K, seed=3)
    y = O.linear_exact(x, w["blob"], lut, N, K, 128, 4)
    assert torch.allclose(y, torch.full_like(y, 0.5 * x.double().sum().item()), rtol=0, atol=1e-12)


def test_reference_forward_against_fp64_closed_form():
    N, K = 256, 192
    w = make_weight(N, K, bits=4, gs=64, seed=6, bits2=2, rank=8, bias=True,
                    act_dtype=torch.float32)
    x = make_x(3, K, seed=8, dtype=torch.float32)
    y = O.linear_reference(x, w["blob"], w["lut"], N, K, 64, 4, w["blob2"], w["lut2"], 2,
                           w["resA"], w["resB"], w["bias"])
    W1 = O.dequant(w["blob"], w["lut"], N, K, 64, 4).double()
    W2 = O.dequant(w["blob2"], w["lut2"], N, K, 64, 2).double()
    xd = x.double()
    exact = xd @ (W1 + W2).t() + (xd @ w["resB"].double().t()) @ w["resA"].double().t() \
        + w["bias"].double()
    assert rel_l2(y, exact) < 1e-6
    assert rel_l2(O.linear_exact(x, w["blob"], w["lut"], N, K, 64, 4, w["blob2"], w["lut2"], 2,
                                 w["resA"], w["resB"], w["bias"]), exact) < 1e-14


def test_silu_mul():
    g = torch.linspace(-8, 8, 41, dtype=torch.float64)
    u = torch.linspace(2, -2, 41, dtype=torch.float64)
    assert torch.allclose(O.silu_mul_exact(g, u), torch.nn.functional.silu(g) * u, atol=1e-15)
    assert O.silu_mul_exact(torch.tensor([0.0]), torch.tensor([3.0])).item() == 0.0


@pytest.mark.parametrize("K", [32, 64, 96, 256, 4096, 12288])
def test_fht_against_explicit_matrix(K):
    signs = O.rotation_signs(K, seed=K)
    assert set(signs.tolist()) <= {-1.0, 1.0} and signs.dtype == torch.float32
    x = make_x(3, K, seed=K, dtype=torch.float32)
    T = O.rotation_matrix(signs)
    fwd = O.fht_reference(x, signs).double().numpy()
    adj = O.fht_adjoint_reference(x, signs).double().numpy()
    assert np.abs(fwd - x.double().numpy() @ T).max() < 1e-4
    assert np.abs(adj - x.double().numpy() @ T.T).max() < 1e-4
    # T is orthogonal: adjoint(forward(x)) == x, norms are preserved
    back = O.fht_adjoint_reference(O.fht_reference(x, signs), signs)
    assert (back - x).abs().max().item() < 1e-5
    assert abs(np.linalg.norm(fwd) - x.double().norm().item()) < 1e-3


def test_hadamard_identities_and_segments():
    for b in (2, 8, 64):
        H = O.hadamard(b)
        assert np.array_equal(H @ H, b * np.eye(b)) and np.array_equal(H, H.T)
    H2 = O.hadamard(2)
    assert np.array_equal(O.hadamard(4), np.kron(H2, H2))          # Sylvester doubling
    assert O.segments(12288) == [(0, 8192), (8192, 4096)]
    assert O.segments(4096) == [(0, 4096)]
    assert O.segments(6144) == [(0, 4096), (4096, 2048)]
    assert O.segments(96) == [(0, 64), (64, 32)]
    # segments are independent: changing x in one segment leaves the other's output alone
    signs = O.rotation_signs(96, 1)
    x = make_x(1, 96, dtype=torch.float32)
    x2 = x.clone(); x2[0, 70] += 1.0
    a, b_ = O.fht_reference(x, signs), O.fht_reference(x2, signs)
    assert torch.equal(a[:, :64], b_[:, :64]) and not torch.equal(a[:, 64:], b_[:, 64:])


def _mt19937_words(seed, count):
    """The textbook MT19937 (Matsumoto & Nishimura 1998, init_genrand + genrand_int32),
    written out so that the sign pin below does not rest on a library's word for it."""
    mt = [0] * 624
    mt[0] = seed & 0xFFFFFFFF
    for i in range(1, 624):
        mt[i] = (1812433253 * (mt[i - 1] ^ (mt[i - 1] >> 30)) + i) & 0xFFFFFFFF
    out, idx = [], 624
    while len(out) < count:
        if idx >= 624:
            for k in range(624):
                y = (mt[k] & 0x80000000) | (mt[(k + 1) % 624] & 0x7FFFFFFF)
                mt[k] = mt[(k + 397) % 624] ^ (y >> 1) ^ (0x9908B0DF if y & 1 else 0)
            idx = 0
        y = mt[idx]; idx += 1
        y ^= y >> 11
        y ^= (y << 7) & 0x9D2C5680
        y ^= (y << 15) & 0xEFC60000
        y ^= y >> 18
        out.append(y)
    return out


@pytest.mark.parametrize("K", [64, 4096, 12288])
@pytest.mark.parametrize("seed", [0, 7, 42])
def test_rotation_sign_values_are_the_mt19937_low_bits(K, seed):
    """Pins the VALUES of the sign vector.  Upstream draws
    randint(0, 2, (K,)) * 2 - 1 from a CPU generator seeded seed + 4242
    (fht.py:105-115); torch's CPU generator is MT19937 and randint(0, 2) keeps the low
    bit of each 32-bit word, so sign k = 2 * (word_k & 1) - 1 of the textbook stream.
    Checked against numpy's MT19937 at every size and against the generator written
    out above on the first 700 words (past one state refill)."""
    signs = O.rotation_signs(K, seed)
    assert signs.dtype == torch.float32 and signs.shape == (K,)
    bits = ((signs + 1) / 2).numpy().astype(np.int64)
    words = np.random.RandomState(seed + 4242)._bit_generator.random_raw(K)
    assert np.array_equal(bits, words & 1)
    head = min(K, 700)
    assert bits[:head].tolist() == [w & 1 for w in _mt19937_words(seed + 4242, head)]
    # the product's own draw is the same vector
    import fht
    assert torch.equal(fht.rotation_signs(K, seed), signs)


def test_mt19937_known_answer():
    """genrand_int32 after init_genrand(5489) starts 3499211612, 581869302 (the
    reference output of mt19937ar.c, also the C++11 default-seeded mt19937)."""
    assert _mt19937_words(5489, 2) == [3499211612, 581869302]
    assert _mt19937_words(5489, 10000)[-1] == 4123659995      # C++11 [rand.predef] 10000th value


def test_fht_c_matches_numpy_bit_for_bit():
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        pytest.skip("oracle/liboracle.so not built")
    lib = ctypes.CDLL(path)
    for K in (96, 4096, 12288):
        signs = O.rotation_signs(K, 9)
        x = make_x(2, K, seed=K, dtype=torch.float32)
        for adj in (0, 1):
            out = np.zeros((2, K), dtype=np.float32)
            xn, sn = x.numpy().copy(), signs.numpy().copy()
            lib.oracle_fht(xn.ctypes.data_as(ctypes.c_void_p), sn.ctypes.data_as(ctypes.c_void_p),
                           2, K, adj, out.ctypes.data_as(ctypes.c_void_p))
            ref = (O.fht_adjoint_reference if adj else O.fht_reference)(x, signs).numpy()
            assert np.array_equal(out, ref)


def test_block_fht_and_awq():
    K = 512
    x = make_x(2, K, seed=2, dtype=torch.float32)
    y = O.block_fht_reference(x, 128)
    H = O.hadamard(128) / math.sqrt(128)
    exp = (x.double().numpy().reshape(-1, 128) @ H).reshape(2, K)
    assert np.abs(y.double().numpy() - exp).max() < 1e-5
    signs = O.rotation_signs(K, 3)
    s = torch.rand(K) + 0.5
    T = O.rotation_matrix(signs)
    exp = (x.double().numpy() * s.double().numpy()) @ T / s.double().numpy()
    assert np.abs(O.fht_awq_reference(x, signs, s).double().numpy() - exp).max() < 1e-4


def _golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_stated_examples.json")) as f:
        return json.load(f)


def test_upstream_split_policy_examples():
    """(tiles, K) -> split and workgroup count: the worked examples upstream states in
    src/kernel_gemv_splitk.cu:54-59, held as data in tests/golden."""
    lib = None
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if os.path.exists(path):
        lib = ctypes.CDLL(path)
    cases = _golden()["split_policy"]["cases"]
    assert len(cases) >= 7
    for tiles, K, want, wgs in cases:
        assert O.pick_split_upstream(tiles, K // 64) == want
        assert tiles * want == wgs
        if lib is not None:
            assert lib.oracle_pick_split_upstream(tiles, K // 64) == want


def test_upstream_segment_examples():
    """The decompositions upstream lists in the docstring of segments (fht.py:118-124)."""
    for K, want in _golden()["segments"]["cases"].items():
        assert O.segments(int(K)) == [tuple(p) for p in want]
        assert sum(b for _, b in O.segments(int(K))) == int(K)


def test_blob_geometry_constants():
    g = _golden()["blob_geometry"]
    assert (O.ROWS_PER_TILE, O.K_PER_TILE, O.CHUNKS_PER_TILE, O.PAIRS_PER_CHUNK) == \
        (g["tile_rows"], g["tile_k"], g["chunks_per_tile"], g["pairs_per_chunk"])
