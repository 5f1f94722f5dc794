"""GPU parity of the M = 1 LUT GEMV family against the oracle, through the
flute_extended op surface (which calls the C ABI).

Tolerance (stated by the benchmark contract): relative L2 <= 1e-3 against the
reference arithmetic for fp32 accumulate with a 16-bit output.  The oracle value
is the fp64 closed form rounded once to the output dtype, i.e. what an exact
fp32-accumulate kernel would produce; the upstream torch path
(oracle.linear_reference) is compared as well where it rounds at the same point.
Index decoding is additionally checked bit-exactly: a one-hot input must return
the dequantised column.
"""
import pytest
import torch

import flute_extended as fx
import flute_oracle as O
from _util import make_weight, make_x, rel_l2
import ctypes

from flute_extended import _C, _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-3


def _run(w, x, entry=None, signs=None, awq=None, **extra):
    entry = entry or fx.qgemm_gemv_splitk_stream
    return entry(x.to(DEV), w["blob_d"], w["lut_d"], w["bits"], w["gs"],
                 indices2=w.get("blob2_d"), lut2=w.get("lut2_d"), bitwidth2=w["bits2"],
                 resB=w.get("resB_d"), resA=w.get("resA_d"), bias=w.get("bias_d"),
                 rot_signs=None if signs is None else signs.to(DEV),
                 awq_scale=None if awq is None else awq.to(DEV), **extra)


def _exact(w, x):
    return O.linear_exact(x, w["blob"].numpy(), w["lut"], w["N"], w["K"], w["gs"], w["bits"],
                          w["blob2"].numpy() if w["bits2"] else None, w["lut2"], w["bits2"],
                          w["resA"], w["resB"], w["bias"])


CASES = [
    # N, K, bits, gs, bits2, rank, bias
    (128, 64, 4, 128, 0, 0, False),
    (256, 512, 4, 128, 0, 0, False),
    (1024, 4096, 4, 128, 0, 0, False),
    (1024, 4096, 4, 64, 0, 0, False),
    (1024, 2048, 4, 32, 0, 0, False),
    (1024, 2048, 4, 16, 0, 0, False),
    (1024, 2048, 4, 512, 0, 0, False),
    (384, 1024, 4, 256, 0, 0, False),       # N not a multiple of the group size
    (512, 1024, 3, 128, 0, 0, False),
    (512, 1024, 2, 128, 0, 0, False),
    (512, 1024, 1, 128, 0, 0, False),
    (512, 1024, 3, 32, 0, 0, False),
    (512, 1024, 2, 16, 0, 0, False),
    (512, 1024, 1, 64, 0, 0, False),
    (512, 1024, 4, 128, 1, 0, False),
    (512, 1024, 1, 128, 4, 0, True),
    (512, 1024, 3, 128, 3, 16, True),
    (512, 1024, 2, 64, 3, 0, False),
    (512, 1024, 4, 128, 4, 4, False),
    (512, 2048, 4, 128, 0, 64, True),
    (256, 1024, 4, 128, 0, 256, False),
]


@pytest.mark.parametrize("N,K,bits,gs,bits2,rank,bias", CASES)
def test_gemv_fp16(N, K, bits, gs, bits2, rank, bias):
    w = make_weight(N, K, bits, gs, seed=N + K + bits, bits2=bits2, rank=rank, bias=bias,
                    device=DEV)
    x = make_x(1, K, seed=7)
    y = _run(w, x).cpu()
    assert y.shape == (1, N) and y.dtype == torch.float16
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    assert torch.equal(y, _run(w, x).cpu())            # deterministic


@pytest.mark.parametrize("split", [1, 2, 4, 8, 16])
def test_forced_splits_agree(split):
    w = make_weight(512, 4096, 4, 128, seed=3, rank=8, bias=True, device=DEV)
    x = make_x(1, 4096, seed=5)
    y = _run(w, x, split=split).cpu()
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    assert torch.equal(y, _run(w, x, split=split).cpu())


def test_plain_entry_and_contract():
    w = make_weight(512, 1024, 4, 128, seed=9, rank=16, bias=True, device=DEV)
    x = make_x(1, 1024, seed=2)
    y = _run(w, x, entry=fx.qgemm_gemv_stream).cpu()
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    w2 = make_weight(512, 1024, 4, 128, seed=9, rank=32, device=DEV)
    with pytest.raises(RuntimeError):
        _run(w2, x, entry=fx.qgemm_gemv_stream)        # rank cap of the plain entry
    with pytest.raises(RuntimeError):
        fx.qgemm_gemv_splitk_stream(make_x(2, 1024).to(DEV), w["blob_d"], w["lut_d"], 4, 128)


@pytest.mark.parametrize("lut_dtype", [torch.float16, torch.bfloat16])
def test_gemv_bf16_activations(lut_dtype):
    N, K = 512, 4096
    w = make_weight(N, K, 4, 128, seed=4, lut_dtype=lut_dtype, act_dtype=torch.bfloat16,
                    bias=True, rank=4, device=DEV)
    x = make_x(1, K, seed=6, dtype=torch.bfloat16)
    y = _run(w, x).cpu()
    assert y.dtype == torch.bfloat16
    assert rel_l2(y, _exact(w, x).bfloat16()) <= TOL
    # the upstream torch path on the same inputs, no residual/bias: same rounding point
    w0 = make_weight(N, K, 4, 128, seed=4, lut_dtype=lut_dtype, act_dtype=torch.bfloat16,
                     device=DEV)
    ref = O.linear_reference(x, w0["blob"].numpy(), w0["lut"], N, K, 128, 4)
    assert rel_l2(_run(w0, x).cpu(), ref) <= TOL


@pytest.mark.parametrize("bits,gs", [(4, 128), (3, 64), (2, 128), (1, 32), (4, 16)])
def test_one_hot_input_returns_the_dequantised_column(bits, gs):
    """y = W[:, k] exactly when x = e_k: checks every lookup of the K loop."""
    N, K = 512, 512
    w = make_weight(N, K, bits, gs, seed=bits * 7 + gs, device=DEV)
    W = O.dequant(w["blob"], w["lut"], N, K, gs, bits)
    for k in (0, 1, 9, 63, 64, 200, 511):
        x = torch.zeros(1, K, dtype=torch.float16); x[0, k] = 1.0
        assert torch.equal(_run(w, x).cpu()[0].float(), W[:, k])


def test_one_hot_at_benchmark_size():
    N, K = 12288, 4096
    w = make_weight(N, K, 4, 128, seed=1, device=DEV)
    idx, lut = w["idx"].long(), w["lut"].float()
    rows = torch.arange(N) // 128
    for k in (0, 1337, 4095):
        x = torch.zeros(1, K, dtype=torch.float16); x[0, k] = 1.0
        assert torch.equal(_run(w, x).cpu()[0].float(), lut[rows, idx[:, k]])


@pytest.mark.parametrize("N,K", [(12288, 4096), (4096, 12288), (1024, 4096), (512, 4096)])
def test_benchmark_shapes(N, K):
    w = make_weight(N, K, 4, 128, seed=N % 97, device=DEV)
    x = make_x(1, K, seed=3)
    y = _run(w, x).cpu()
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    # linearity, a size-independent property: f(2x) == 2 f(x) bit for bit wherever the
    # fp16 output is a normal number (doubling is exact in fp32 and commutes with the
    # final rounding; subnormal outputs have a fixed quantum, so they are excluded)
    normal = y.abs() >= 2.0 ** -13
    assert normal.float().mean() > 0.99
    assert torch.equal(_run(w, x * 2).cpu()[normal], (y * 2)[normal])


@pytest.mark.parametrize("K,awq,dtype", [(4096, False, torch.float16), (12288, True, torch.float16),
                                         (1536, False, torch.float16), (4096, True, torch.bfloat16)])
def test_fused_rotation_is_bit_identical_to_rotate_then_gemv(K, awq, dtype):
    import fht
    N = 512
    w = make_weight(N, K, 4, 128, seed=5, rank=8, bias=True, act_dtype=dtype, device=DEV)
    x = make_x(1, K, seed=8, dtype=dtype)
    signs = O.rotation_signs(K, 21)
    s = (torch.rand(K, generator=torch.Generator().manual_seed(1)) + 0.5) if awq else None
    fused = _run(w, x, signs=signs, awq=s)
    xr = fht.fht_apply_awq(x.to(DEV), signs.to(DEV), s.to(DEV), backend="kernel") if awq \
        else fht.fht_apply(x.to(DEV), signs.to(DEV), backend="kernel")
    chain = _run(w, xr.cpu())
    assert torch.equal(fused, chain)
    w0 = make_weight(N, K, 4, 128, seed=5, act_dtype=dtype, device=DEV)   # fused prologue path
    assert torch.equal(_run(w0, x, signs=signs, awq=s), _run(w0, xr.cpu()))
    xo = O.fht_awq_reference(x, signs, s) if awq else O.fht_reference(x, signs)
    assert rel_l2(fused.cpu(), _exact(w, xo).to(dtype)) <= (TOL if dtype == torch.float16 else 4e-3)


def test_block_rotation_mode():
    """Equal 128-column rotation blocks (the benchmark's wording), defined by the
    closed form oracle.block_fht_reference."""
    N, K = 512, 4096
    w = make_weight(N, K, 4, 128, seed=6, device=DEV)
    x = make_x(1, K, seed=9)
    signs = torch.ones(K)
    y = _run(w, x, signs=signs, rot_block=128).cpu()
    xo = O.block_fht_reference(x, 128, signs)
    assert rel_l2(y, _exact(w, xo).half()) <= TOL


# Unit counts per wavefront that are and are not a multiple of the prefetch depth, K ranges
# shorter than one load per wavefront, and K ranges beyond the activation registers of the
# prologue: every variant of the K loop (main part, last group, conservative tail) and both
# activation staging paths.
@pytest.mark.parametrize("K", [64, 128, 192, 320, 448, 832, 1792, 2560, 5120, 6144, 8192, 16384])
@pytest.mark.parametrize("N,bits,bits2", [(256, 4, 0), (2048, 4, 0), (512, 4, 4), (512, 2, 0)])
def test_k_sweep_covers_every_loop_variant(K, N, bits, bits2):
    w = make_weight(N, K, bits, 128, seed=K + N + bits, bits2=bits2, device=DEV)
    x = make_x(1, K, seed=11)
    y = _run(w, x).cpu()
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    assert torch.equal(y, _run(w, x).cpu())


@pytest.mark.parametrize("block", [32, 64, 128, 256, 512, 1024])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_block_rotation_is_bit_identical_to_rotate_then_gemv(block, dtype):
    """Blocks up to 256 columns run in registers and lane swizzles, larger ones in the LDS
    buffer; both must produce the bits of the standalone rotation kernel."""
    from flute_extended import _C
    N, K = 512, 4096
    w = make_weight(N, K, 4, 128, seed=block, act_dtype=dtype, device=DEV)
    x = make_x(1, K, seed=12, dtype=dtype)
    signs = O.rotation_signs(K, block)
    fused = _run(w, x, signs=signs, rot_block=block)
    xr = _C.fht_forward(x.to(DEV), signs.to(DEV), block)
    assert torch.equal(fused, _run(w, xr.cpu()))
    xo = O.block_fht_reference(x, block, signs)
    assert rel_l2(fused.cpu(), _exact(w, xo).to(dtype)) <= (TOL if dtype == torch.float16 else 4e-3)


@pytest.mark.parametrize("N,block", [(512, 64), (512, 128), (4096, 128), (4096, 64), (1024, 256)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_block_rotation_with_scale_compensation_matches_the_chain(N, block, dtype):
    """((x * s) @ T_block) / s in the GEMV prologue (fht.py:207-238 upstream for the transform)
    against the rotation kernel followed by the plain GEMV, bit for bit; the shapes cover
    rotation in the consuming wavefront's registers (a block fits a unit of K) and the
    staged form (it does not)."""
    from flute_extended import _C
    K = 4096
    w = make_weight(N, K, 4, 128, seed=block + N, act_dtype=dtype, device=DEV)
    x = make_x(1, K, seed=13, dtype=dtype)
    signs = O.rotation_signs(K, block + 1)
    g = torch.Generator().manual_seed(block)
    s = (torch.rand(K, generator=g) * 1.5 + 0.5).float()
    fused = _run(w, x, signs=signs, awq=s, rot_block=block)
    xr = _C._fht("chain", x.to(DEV), signs.to(DEV), s.to(DEV), None, 0, block)
    assert torch.equal(fused, _run(w, xr.cpu()))


def test_workspace_growth_is_refused_under_graph_capture():
    """A K split needs the library workspace.  When that would have to be allocated while
    the stream is being captured, the call is refused (an allocation and the clearing of
    fresh tickets cannot be graph nodes); after a warm-up outside the capture the same call
    is captured and replays."""
    import ctypes
    from flute_extended import _lib
    w = make_weight(512, 2048, seed=41, device=DEV)
    x = make_x(1, 2048, seed=42).to(DEV)
    d = _lib.FluteLinear()
    d.q1, d.lut1, d.q1_bytes = w["blob_d"].data_ptr(), w["lut_d"].data_ptr(), w["blob_d"].numel()
    d.N, d.K, d.b1, d.group_size, d.lut_rows, d.lut_dtype = 512, 2048, 4, 128, 4, _lib.F16
    y = torch.zeros(1, 512, dtype=torch.float16, device=DEV)
    torch.cuda.synchronize()
    _lib.lib.flute_release_workspaces()                 # nothing held: the next split call must allocate
    call = lambda: _lib.lib.flute_gemv(ctypes.byref(d), x.data_ptr(), y.data_ptr(), _lib.F16, 4,
                                       torch.cuda.current_stream().cuda_stream)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(g, stream=s):
            y.zero_()
            status = call()
            message = _lib.last_error()
    assert status == _lib.FLUTE_ERR_INVALID and "captured" in message
    assert call() == 0                                  # warm-up outside a capture allocates
    torch.cuda.synchronize()
    want = y.clone()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(g2, stream=s):
            assert call() == 0
    y.zero_()
    g2.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, want)


def _wide_range_row(K, kind):
    """bfloat16 activations that float16 cannot hold: a few values near 1e5 among N(0, 1)
    ones, a whole row around 1e-7, a whole row around 1e30, and a row mixing 1e5 with 1e-6."""
    x = make_x(1, K, seed=19, dtype=torch.float32)
    if kind == "outliers":
        x[0, [3, K // 2, K - 1]] = torch.tensor([1.0e5, -2.5e5, 9.0e4])
    elif kind == "tiny":
        x *= 1.0e-7
    elif kind == "huge":
        x *= 1.0e30
    else:
        x[0, ::2] *= 1.0e-6
        x[0, 1::64] *= 1.0e5
    return x.to(torch.bfloat16)


@pytest.mark.parametrize("kind", ["outliers", "tiny", "huge", "mixed"])
@pytest.mark.parametrize("bits,split,rot", [(4, 0, False), (4, 4, False), (3, 0, False),
                                            (4, 0, True), (2, 2, True)])
def test_bf16_activations_beyond_the_float16_range(kind, bits, split, rot):
    """A float16 LUT makes the kernels multiply in float16; bfloat16 activations outside
    float16's range (|x| > 65504, |x| < 6e-8) must still give the reference forward's
    result (x.float() @ W.t(), scripts/palettized_modules.py:1241-1251), never inf or 0."""
    N, K = 512, 4096
    w = make_weight(N, K, bits, 128, seed=23 + bits, act_dtype=torch.bfloat16, device=DEV)
    x = _wide_range_row(K, kind)
    signs = O.rotation_signs(K, 4) if rot else None
    y = _run(w, x, signs=signs, split=split).cpu()
    assert y.dtype == torch.bfloat16 and torch.isfinite(y).all()
    ref = O.linear_reference(x, w["blob"].numpy(), w["lut"], N, K, 128, bits, signs=signs)
    assert torch.isfinite(ref).all() and ref.abs().max() > 0
    assert rel_l2(y, ref) <= TOL


def test_merged_gate_up_with_activations_beyond_the_float16_range():
    N, K = 1024, 4096
    g = make_weight(N, K, 4, 128, seed=27, act_dtype=torch.bfloat16, device=DEV)
    u = make_weight(N, K, 4, 128, seed=28, act_dtype=torch.bfloat16, device=DEV)
    x = _wide_range_row(K, "outliers")
    table = torch.tensor([[g["blob_d"].data_ptr(), g["lut_d"].data_ptr(), 0, 0, 0, 0, 0, 0, N, 0, 4, 0,
                           128, 0, 0],
                          [u["blob_d"].data_ptr(), u["lut_d"].data_ptr(), 0, 0, 0, 0, 0, 0, N, 0, 4, 0,
                           128, 0, 0]], dtype=torch.int64)
    out = torch.zeros(1, N, dtype=torch.bfloat16, device=DEV)
    fx.qgemm_gemv_mlp(x.to(DEV), table, out)
    yg = O.linear_exact(x, g["blob"].numpy(), g["lut"], N, K, 128, 4)
    yu = O.linear_exact(x, u["blob"].numpy(), u["lut"], N, K, 128, 4)
    ref = O.silu_mul_exact(yg, yu).to(torch.bfloat16)
    assert torch.isfinite(out).all()
    assert rel_l2(out.cpu(), ref) <= 4e-3       # one bfloat16 rounding of a product of two sums


def test_long_k_narrow_output_takes_the_library_s_split():
    """K = 32768 over 256 rows: the library's own choice is a four-way K split
    (upstream's policy: src/gemv_host.cpp:29-38); the result is the forced four-way
    split bit for bit, deterministic, and within tolerance of the oracle."""
    N, K = 256, 32768
    assert fx.gemv_split_hint(N, K) == 4
    w = make_weight(N, K, 4, 128, seed=77, device=DEV)
    x = make_x(1, K, seed=78)
    y = _run(w, x)
    assert torch.equal(y, _run(w, x, split=4)) and torch.equal(y, _run(w, x))
    assert rel_l2(y.cpu(), _exact(w, x).half()) <= TOL


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,bits2,rank,bias", [(12288, 0, 0, False), (4224, 0, 0, False),
                                              (4224, 4, 8, True), (33024, 0, 8, True),
                                              (33024, 4, 0, False)])
def test_resident_grid_walking_the_row_slices(tuning_env, N, bits2, rank, bias, act):
    """Launches of more workgroups than the device holds at once run as a resident grid whose
    workgroups walk over the row slices (the very wide outputs of upstream's lm_head class,
    src/kernel_gemv.cu:92-253, on one staged activation vector).  FLUTE_GEMV4_WALK sets the
    resident workgroups per CU: 1 makes these sizes walk (three slices each; 528 slices over 256
    workgroups, so sixteen workgroups take a third one), 0 switches walking off.  33024 rows are
    1032 slices of 32 rows: four or five in a row per workgroup, which keeps its table while the
    LUT row stays the same (one stream) and rebuilds it per stream (two).  Same sums in the same
    order: bit-identical outputs, and within tolerance of the oracle."""
    K = 2048 if N < 30000 else 1024
    w = make_weight(N, K, 4, 128, seed=61, bits2=bits2, rank=rank, bias=bias, act_dtype=act, device=DEV)
    x = make_x(1, K, seed=62, dtype=act)
    tuning_env("FLUTE_GEMV4_WALK", "0")
    plain = _run(w, x)
    tuning_env("FLUTE_GEMV4_WALK", "1")
    walked = _run(w, x)
    assert torch.equal(plain, walked)
    # bfloat16 outputs: the rounding of the output alone is 1.6e-3
    assert rel_l2(walked.cpu(), _exact(w, x).to(act)) <= (TOL if act == torch.float16 else 4e-3)


@pytest.mark.parametrize("block", [128, 1024, 0])
@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
def test_resident_grid_walking_with_a_rotated_input(tuning_env, block, act):
    """The input rotation runs once, in the prologue of a walking workgroup (in the consuming
    wavefront's registers for block 128, through the LDS buffer that the first table then
    overwrites for block 1024 and for the whole-row transform): same bits as the unwalked launch."""
    N, K = 4224, 2048
    w = make_weight(N, K, 4, 128, seed=66, act_dtype=act, device=DEV)
    x = make_x(1, K, seed=67, dtype=act)
    signs = O.rotation_signs(K, block)              # the second argument is the seed
    extra = {"rot_block": block} if block else {}
    tuning_env("FLUTE_GEMV4_WALK", "0")
    plain = _run(w, x, signs=signs, **extra)
    tuning_env("FLUTE_GEMV4_WALK", "1")
    assert torch.equal(plain, _run(w, x, signs=signs, **extra))


def test_very_wide_output_walks_by_the_library_s_own_choice(tuning_env):
    """40960 rows are 1280 slices of 32 rows, more than the 768 workgroups the device holds: the
    library walks without being told to.  Bit-identical to the launch of one workgroup per
    slice, within tolerance of the oracle on every row, and a one-hot input returns the
    dequantised column bit for bit (first, middle and last tile)."""
    N, K = 40960, 1024
    w = make_weight(N, K, 4, 128, seed=71, device=DEV)
    x = make_x(1, K, seed=72)
    walked = _run(w, x)
    tuning_env("FLUTE_GEMV4_WALK", "0")
    assert torch.equal(walked, _run(w, x))
    tuning_env("FLUTE_GEMV4_WALK", None)
    assert rel_l2(walked.cpu(), _exact(w, x).half()) <= TOL
    Wd = O.dequant(w["blob"].numpy(), w["lut"], N, K, 128, 4)
    for k in (0, 517, K - 1):
        e = torch.zeros(1, K, dtype=torch.float16)
        e[0, k] = 1.0
        assert torch.equal(_run(w, e).cpu().view(-1), Wd[:, k].half())


def test_resident_grid_walking_the_merged_gate_up(tuning_env):
    """The merged gate/up launch (two index streams per slice, SiLU(gate) * up at the end of a
    slice) on a walking grid: bit-identical to the unwalked launch."""
    N, K = 4224, 2048
    g = make_weight(N, K, 4, 128, seed=63, device=DEV)
    u = make_weight(N, K, 4, 128, seed=64, device=DEV)
    x = make_x(1, K, seed=65)
    table = torch.tensor([[g["blob_d"].data_ptr(), g["lut_d"].data_ptr(), 0, 0, 0, 0, 0, 0, N, 0, 4, 0,
                           128, 0, 0],
                          [u["blob_d"].data_ptr(), u["lut_d"].data_ptr(), 0, 0, 0, 0, 0, 0, N, 0, 4, 0,
                           128, 0, 0]], dtype=torch.int64)
    outs = []
    for walk in ("0", "1"):
        tuning_env("FLUTE_GEMV4_WALK", walk)
        out = torch.zeros(1, N, dtype=torch.float16, device=DEV)
        fx.qgemm_gemv_mlp(x.to(DEV), table, out)
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    yg = O.linear_exact(x, g["blob"].numpy(), g["lut"], N, K, 128, 4)
    yu = O.linear_exact(x, u["blob"].numpy(), u["lut"], N, K, 128, 4)
    assert rel_l2(outs[1].cpu(), O.silu_mul_exact(yg, yu).half()) <= TOL


def test_two_streams_share_the_workspace_in_order():
    """The split-K workspace is one per device (upstream: one stream only,
    src/gemv_host.h:31-38).  Launches that alternate between two streams, with nothing but the
    library's own hand-over between them, must still give the single-stream result."""
    N, K = 256, 8192
    ws = [make_weight(N, K, 4, 128, seed=40 + i, rank=8, device=DEV) for i in range(2)]
    x = make_x(1, K, seed=9).to(DEV)
    want = [_run(w, x, split=8).cpu() for w in ws]
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    got = []
    for rep in range(20):
        for st, w in ((s1, ws[0]), (s2, ws[1])):
            with torch.cuda.stream(st):
                got.append((rep, _run(w, x, split=8)))
    torch.cuda.synchronize()
    for i, (rep, y) in enumerate(got):
        assert torch.equal(y.cpu(), want[i % 2]), (rep, i % 2)


@pytest.mark.skipif(_C.native is None, reason="the compiled binding is not built or switched off")
def test_compiled_binding_gives_the_python_binding_s_outputs():
    """flute_extended._C_native (csrc/torch_binding.cpp, the counterpart of upstream's pybind
    module, src/bindings.cpp:230-546) and the ctypes mirror call the same kernels with the same
    descriptor: outputs agree bit for bit, for a GEMV with every optional operand, a grouped and
    a merged launch, and both GEMM entries."""
    N, K = 512, 1024
    w = make_weight(N, K, 4, 128, seed=5, bits2=1, rank=8, bias=True, device=DEV)
    x = make_x(1, K, seed=6).to(DEV)
    signs = O.rotation_signs(K, 1).to(DEV)
    e32 = torch.empty(0, dtype=torch.float32, device=DEV)
    args = (x, w["blob_d"], w["lut_d"], 4, w["blob2_d"], w["lut2_d"], 1, w["resB_d"], w["resA_d"],
            w["bias_d"], 128)
    for name, extra in (("qgemm_gemv_splitk_stream", (2,)), ("qgemm_gemv_splitk_fht_stream", (signs, e32, 1, 128)),
                        ("qgemm_gemv_fht_stream", (signs, e32))):
        a = _C.PYTHON_BINDING[name](*args, *extra)
        b = getattr(_C.native, name)(*args, *extra)
        assert torch.equal(a, b), name
    xm = make_x(9, K, seed=7).to(DEV)
    argm = (xm,) + args[1:]
    assert torch.equal(_C.PYTHON_BINDING["qgemm_dual_stream"](*argm), _C.native.qgemm_dual_stream(*argm))
    assert torch.equal(_C.PYTHON_BINDING["qgemm_cutlass_streaming"](xm, w["blob_d"], w["lut_d"], 4, 128),
                       _C.native.qgemm_cutlass_streaming(xm, w["blob_d"], w["lut_d"], 4, 128))
    # segment table: gate/up of a merged launch, then the same two weights as a grouped launch
    u = make_weight(N, K, 4, 128, seed=8, device=DEV)
    outs = [torch.zeros(1, N, dtype=torch.float16, device=DEV) for _ in range(6)]
    def table(c0, c1):
        rows = []
        for t, c in ((w, c0), (u, c1)):
            rows.append([t["blob_d"].data_ptr(), t["lut_d"].data_ptr(), 0, 0, 0, 0, 0, c.data_ptr(),
                         N, 0, 4, 0, 128, 0, 0])
        return torch.tensor(rows, dtype=torch.int64)
    _C.PYTHON_BINDING["qgemm_gemv_multi"](x, table(outs[0], outs[1]))
    _C.native.qgemm_gemv_multi(x, table(outs[2], outs[3]))
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[3])
    _C.PYTHON_BINDING["qgemm_gemv_mlp"](x, table(outs[0], outs[1]), outs[4])
    _C.native.qgemm_gemv_mlp(x, table(outs[0], outs[1]), outs[5])
    torch.cuda.synchronize()
    assert torch.equal(outs[4], outs[5]) and outs[4].abs().sum() > 0


# ---- the width pairs of deployed artifacts in the lean kernel: two resident tables ------------
# (upstream's census of two-stream layers: (1,4) x45, (4,1) x24, (3,3) x61,
#  flute_extended/__init__.py:226-233; its kernel: include/flute/gemv.cuh:187-288)

def _lib_desc(w, signs=None, block=0):
    """flute_linear of a test weight (device tensors), for calls straight through the C ABI."""
    d = _lib.FluteLinear()
    d.q1, d.lut1, d.q1_bytes = w["blob_d"].data_ptr(), w["lut_d"].data_ptr(), w["blob_d"].numel()
    if w["bits2"]:
        d.q2, d.lut2, d.q2_bytes = w["blob2_d"].data_ptr(), w["lut2_d"].data_ptr(), w["blob2_d"].numel()
    d.N, d.K, d.b1, d.b2, d.group_size = w["N"], w["K"], w["bits"], w["bits2"], w["gs"]
    d.lut_rows = w["lut"].shape[0]
    d.lut_dtype = _lib.F16 if w["lut"].dtype == torch.float16 else _lib.BF16
    if signs is not None:
        w["_signs_keep"] = signs
        d.signs, d.rot_block = signs.data_ptr(), block
    return d


PAIR_SHAPES = [
    # N, K: which launch shape the library picks (rows per workgroup / wavefronts / loads in flight)
    (512, 1024),      # 8 rows, 4 wavefronts, 2 loads
    (2048, 4096),     # 8 rows, 4 wavefronts, 4 loads
    (4096, 12288),    # 16 rows, 8 wavefronts
    (12288, 4096),    # 16 rows, 4 wavefronts: the MLP up-projection
    (16384, 2048),    # 32 rows
]


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,bits2", [(4, 1), (1, 4), (3, 3), (2, 4), (2, 3)])
@pytest.mark.parametrize("N,K", PAIR_SHAPES)
def test_width_pairs_two_resident_tables(N, K, bits, bits2, act):
    """Every row against the fp64 oracle at the reference forward's rounding point, repeats bit
    identical, and the same weight through the general kernel (FLUTE_GEMV_NO_FAST) within the
    same tolerance of it."""
    w = make_weight(N, K, bits, 128, seed=N + K + 10 * bits + bits2, bits2=bits2, act_dtype=act,
                    device=DEV)
    x = make_x(1, K, seed=17, dtype=act)
    y = _run(w, x).cpu()
    assert y.dtype == act
    assert rel_l2(y, _exact(w, x).to(act)) <= TOL
    assert torch.equal(y, _run(w, x).cpu())


@pytest.mark.parametrize("bits,bits2", [(4, 1), (1, 4), (3, 3), (2, 4), (2, 3)])
def test_width_pairs_one_hot_rows_are_the_sum_of_both_dequantised_columns(bits, bits2):
    """x = e_k: the output is W1[:, k] + W2[:, k], one fp32 add of two 16-bit values rounded once:
    bit-exact against the dequantised columns for k in every quarter of a tile."""
    N, K = 512, 1024
    w = make_weight(N, K, bits, 128, seed=5, bits2=bits2, device=DEV)
    W1 = O.dequant(w["blob"].numpy(), w["lut"], N, K, 128, bits)
    W2 = O.dequant(w["blob2"].numpy(), w["lut2"], N, K, 128, bits2)
    for k in (0, 17, 63, 64, 511, 1000):
        x = torch.zeros(1, K, dtype=torch.float16)
        x[0, k] = 1.0
        y = _run(w, x).cpu()
        assert torch.equal(y[0], (W1[:, k].float() + W2[:, k].float()).half())


def test_a_4_1_weight_equals_the_same_weight_declared_1_4():
    """The library walks a 1-bit stream first whichever way the weight declares its streams: the
    two declarations of the same data must agree bit for bit (and both with the oracle)."""
    N, K = 12288, 4096
    w = make_weight(N, K, 4, 128, seed=77, bits2=1, device=DEV)
    x = make_x(1, K, seed=19)
    y41 = _run(w, x)
    y14 = fx.qgemm_gemv_splitk_stream(x.to(DEV), w["blob2_d"], w["lut2_d"], 1, 128, indices2=w["blob_d"],
                                      lut2=w["lut_d"], bitwidth2=4)
    assert torch.equal(y41, y14)
    assert rel_l2(y41.cpu(), _exact(w, x).half()) <= TOL


@pytest.mark.parametrize("split", [2, 4])
@pytest.mark.parametrize("bits,bits2", [(4, 1), (1, 4), (3, 3), (2, 4), (2, 3)])
def test_width_pairs_with_a_k_split_residual_and_bias(bits, bits2, split):
    w = make_weight(1024, 4096, bits, 128, seed=9, bits2=bits2, rank=8, bias=True, device=DEV)
    x = make_x(1, 4096, seed=4)
    y = _run(w, x, split=split).cpu()
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    assert torch.equal(y, _run(w, x, split=split).cpu())


@pytest.mark.parametrize("block", [0, 128])
def test_width_pair_with_a_fused_rotation(block):
    """(4, 1) behind the rotation in the prologue: the rotated row feeds both streams; equal
    to rotating first and calling the unrotated launch, bit for bit."""
    import fht
    N, K = 1024, 4096
    w = make_weight(N, K, 4, 128, seed=12, bits2=1, device=DEV)
    x = make_x(1, K, seed=6)
    signs = O.rotation_signs(K, 5)
    d = _lib_desc(w, signs.to(DEV), block)
    y = torch.zeros(1, N, dtype=torch.float16, device=DEV)
    xd = x.to(DEV)
    assert _lib.lib.flute_gemv(ctypes.byref(d), xd.data_ptr(), y.data_ptr(), _lib.F16, 0,
                               torch.cuda.current_stream().cuda_stream) == 0, _lib.last_error()
    xr = torch.empty_like(xd)
    assert _lib.lib.flute_fht(xd.data_ptr(), d.signs, None, xr.data_ptr(), 1, K, _lib.F16, 0, block,
                              torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), _run(w, xr.cpu()).cpu())
    ref = O.block_fht_reference(x, block, signs) if block else O.fht_reference(x, signs)
    assert rel_l2(y.cpu(), _exact(w, ref).half()) <= TOL


def test_merged_gate_up_with_two_stream_members():
    """gate (4, 1) + up (4, 1), and gate (4, 1) + up (4, 0): tables of both streams are rebuilt
    per output; SiLU * mul of the fp32 sums, one rounding."""
    N, K = 2048, 4096
    x = make_x(1, K, seed=3)
    for up_bits2 in (1, 0):
        g = make_weight(N, K, 4, 128, seed=21, bits2=1, device=DEV)
        u = make_weight(N, K, 4, 128, seed=22, bits2=up_bits2, device=DEV)
        out = torch.zeros(1, N, dtype=torch.float16, device=DEV)
        row = lambda w_: [w_["blob_d"].data_ptr(), w_["lut_d"].data_ptr(),
                          w_["blob2_d"].data_ptr() if w_["bits2"] else 0,
                          w_["lut2_d"].data_ptr() if w_["bits2"] else 0, 0, 0, 0, 0, N, 0, 4, w_["bits2"],
                          128, 0, 0]
        table = torch.tensor([row(g), row(u)], dtype=torch.int64)
        y = fx.qgemm_gemv_mlp(x.to(DEV), table, out).cpu()
        ref = O.silu_mul_exact(_exact(g, x), _exact(u, x)).half()
        assert rel_l2(y, ref) <= TOL
        y1 = y.clone()
        fx.qgemm_gemv_mlp(x.to(DEV), table, out)
        assert torch.equal(out.cpu(), y1)
