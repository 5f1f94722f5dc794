"""GPU parity of the rotation kernel and of the dequantisation dump: both are
bit-exact against the oracle (fp32 butterfly in the same stage order; a pure
gather)."""
import pytest
import torch

import fht
import flute_extended as fx
import flute_oracle as O
from _util import make_weight, make_x

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("K", [32, 96, 128, 1536, 4096, 12288, 16384, 24576])
@pytest.mark.parametrize("M", [1, 8])
def test_fht_fp32_bit_exact(K, M):
    signs = O.rotation_signs(K, K + 1)
    x = make_x(M, K, seed=K, dtype=torch.float32)
    y = fht.fht_apply(x.to(DEV), signs.to(DEV), backend="kernel").cpu()
    assert torch.equal(y, O.fht_reference(x, signs))
    ya = fht.fht_adjoint(x.to(DEV), signs.to(DEV), backend="kernel").cpu()
    assert torch.equal(ya, O.fht_adjoint_reference(x, signs))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fht_16bit_io(dtype):
    K = 4096
    signs = O.rotation_signs(K, 3)
    x = make_x(8, K, seed=1, dtype=dtype)
    y = fht.fht_apply(x.to(DEV), signs.to(DEV), backend="kernel").cpu()
    assert y.dtype == dtype and torch.equal(y, O.fht_reference(x, signs))
    z = x.clone().to(DEV)
    fht.fht_apply_(z, signs.to(DEV), backend="kernel")
    assert torch.equal(z.cpu(), y)
    s = torch.rand(K, generator=torch.Generator().manual_seed(2)) + 0.5
    ya = fht.fht_apply_awq(x.to(DEV), signs.to(DEV), s.to(DEV), backend="kernel").cpu()
    assert torch.equal(ya, O.fht_awq_reference(x, signs, s))


def test_fht_block_mode_and_round_trip():
    K = 4096
    x = make_x(8, K, seed=4, dtype=torch.float32)
    signs = O.rotation_signs(K, 5)
    y = fx._C.fht_forward(x.to(DEV), signs.to(DEV), block=128).cpu()
    assert torch.equal(y, O.block_fht_reference(x, 128, signs))
    fwd = fht.fht_apply(x.to(DEV), signs.to(DEV), backend="kernel")
    back = fht.fht_adjoint(fwd, signs.to(DEV), backend="kernel").cpu()
    assert (back - x).abs().max().item() < 1e-5
    # norm preservation at the benchmark width, leading dims flattened
    x3 = make_x(6, K, seed=6, dtype=torch.float32).reshape(2, 3, K)
    y3 = fht.fht_apply(x3.to(DEV), signs.to(DEV)).cpu()
    assert y3.shape == x3.shape
    assert torch.allclose(y3.norm(dim=-1), x3.norm(dim=-1), rtol=1e-5)
    with pytest.raises(RuntimeError):
        fx._C.fht_forward(make_x(1, 100, dtype=torch.float32).to(DEV), torch.ones(100).to(DEV))


@pytest.mark.parametrize("steps", ["0", "2", "4"])
@pytest.mark.parametrize("K", [1536, 4096, 12288, 24576])
def test_fht_every_kernel_variant_bit_exact(tuning_env, steps, K):
    """Segments are transformed through the LDS buffer, or up to 4096 / 8192 columns in
    registers with one LDS pass; the library picks by K and the number of rows.  Each
    variant forced in turn (FLUTE_FHT_STEPS) must give the reference's bits."""
    tuning_env("FLUTE_FHT_STEPS", steps)
    signs = O.rotation_signs(K, 7)
    for dtype in (torch.float32, torch.bfloat16):
        x = make_x(3, K, seed=K, dtype=dtype)
        y = fht.fht_apply(x.to(DEV), signs.to(DEV), backend="kernel").cpu()
        assert torch.equal(y, O.fht_reference(x, signs))
        ya = fht.fht_adjoint(x.to(DEV), signs.to(DEV), backend="kernel").cpu()
        assert torch.equal(ya, O.fht_adjoint_reference(x, signs))


@pytest.mark.parametrize("block", [32, 64, 128, 256, 512, 2048])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_fht_every_block_size_bit_exact(block, dtype):
    """Blocks up to 256 columns are transformed in registers, larger ones in LDS: both
    must give the reference butterfly's bits, forward and adjoint, also in place and on
    rows that do not start on a 16-byte boundary."""
    K, M = 6144, 5
    signs = O.rotation_signs(K, block)
    x = make_x(M, K, seed=block, dtype=dtype)
    xd, sd = x.to(DEV), signs.to(DEV)
    y = fx._C.fht_forward(xd, sd, block=block).cpu()
    assert y.dtype == dtype and torch.equal(y, O.block_fht_reference(x, block, signs))
    ya = fx._C.fht_backward(xd, sd, block=block).cpu()
    xs = (x.float() * signs).to(torch.float32)
    assert torch.equal(ya, O.block_fht_reference(xs, block).to(dtype))
    z = xd.clone()
    fx._C.fht_inplace_(z, sd, block=block)
    assert torch.equal(z.cpu(), y)
    # a view whose rows start 2 (or 4) bytes into a 16-byte line
    off = torch.zeros(M * K + 1, dtype=dtype, device=DEV)
    off[1:] = xd.reshape(-1)
    yo = fx._C.fht_forward(off[1:].reshape(M, K), sd, block=block).cpu()
    assert torch.equal(yo, y)


@pytest.mark.parametrize("bits", [1, 2, 3, 4])
@pytest.mark.parametrize("gs", [16, 128, 512])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_dequant_bit_exact(bits, gs, dtype):
    N, K = 384, 256
    w = make_weight(N, K, bits, gs, seed=bits + gs, lut_dtype=dtype, device=DEV)
    W = fx.dequant_idxn(w["blob_d"], w["lut_d"], N, K, bits, gs).cpu()
    assert W.dtype == dtype
    assert torch.equal(W.float(), O.dequant(w["blob"], w["lut"], N, K, gs, bits))


def test_dequant_benchmark_size_checksum():
    N, K = 12288, 4096
    w = make_weight(N, K, 4, 128, seed=11, device=DEV)
    W = fx.dequant_idxn(w["blob_d"], w["lut_d"], N, K, 4, 128)
    rows = (torch.arange(N) // 128)
    ref = w["lut"][rows].gather(1, w["idx"].long())
    assert torch.equal(W.cpu(), ref)
