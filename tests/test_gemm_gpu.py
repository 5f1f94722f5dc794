"""GPU parity of the M > 1 LUT GEMM (MFMA) against the oracle, through the
flute_extended op surface (which calls the C ABI).

Tolerance: relative L2 <= 1e-3 for fp16 outputs (the benchmark contract's figure
for fp32 accumulate + one 16-bit rounding), <= 4e-3 for bf16 outputs, whose final
rounding alone is 2^-9.  The oracle is the fp64 closed form.  Index decoding is
checked bit-exactly: with A = identity rows (one-hot in k) the GEMM must return
the dequantised columns exactly, because a single product with 1.0 and a sum of
zeros involves no rounding.
"""
import pytest
import torch

import flute_extended as fx
import flute_oracle as O
from _util import make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-3
TOL_BF16 = 4e-3


def _exact(w, x):
    return O.linear_exact(x, w["blob"].numpy(), w["lut"], w["N"], w["K"], w["gs"], w["bits"],
                          w["blob2"].numpy() if w["bits2"] else None, w["lut2"], w["bits2"],
                          w["resA"], w["resB"], w["bias"])


def _dual(w, x):
    return fx.qgemm_dual_stream(x.to(DEV), w["blob_d"], w["lut_d"], w["bits"], w["gs"],
                                indices2=w.get("blob2_d"), lut2=w.get("lut2_d"),
                                bitwidth2=w["bits2"], resB=w.get("resB_d"), resA=w.get("resA_d"),
                                bias=w.get("bias_d"))


SINGLE = [
    # M, N, K, bits, gs
    (2, 128, 64, 4, 128),
    (16, 256, 512, 4, 128),
    (17, 256, 512, 4, 128),
    (33, 384, 1024, 4, 256),           # N not a multiple of the group size
    (64, 512, 1024, 4, 128),
    (100, 512, 1024, 4, 64),
    (128, 256, 2048, 4, 32),
    (130, 256, 1024, 4, 16),
    (256, 1024, 4096, 4, 128),
    (300, 256, 704, 4, 128),           # K/64 = 11: ragged over the k ways
    (8, 512, 1024, 3, 128),
    (48, 512, 1024, 3, 32),
    (8, 512, 1024, 2, 128),
    (200, 256, 1024, 2, 16),
    (8, 512, 1024, 1, 64),
    (96, 256, 1024, 1, 128),
]


@pytest.mark.parametrize("M,N,K,bits,gs", SINGLE)
def test_gemm_single_stream_fp16(M, N, K, bits, gs):
    w = make_weight(N, K, bits, gs, seed=M + N + K + bits, device=DEV)
    x = make_x(M, K, seed=11)
    y = fx.qgemm_per_group_lut(x.to(DEV), w["blob_d"], w["lut_d"], bitwidth=bits, group_size=gs,
                               indices_layout=f"idx{bits}").cpu()
    assert y.shape == (M, N) and y.dtype == torch.float16
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    y2 = fx.qgemm_per_group_lut(x.to(DEV), w["blob_d"], w["lut_d"], bitwidth=bits, group_size=gs,
                                indices_layout=f"idx{bits}").cpu()
    assert torch.equal(y, y2)                           # deterministic


@pytest.mark.parametrize("rows", ["16", "32", "64", "128"])
@pytest.mark.parametrize("M,N,K,bits,gs", [c for c in SINGLE if c[0] > 16])
def test_gemm_every_workgroup_shape(tuning_env, rows, M, N, K, bits, gs):
    """The library picks the rows of A per workgroup (16, 32, 64 or 128) from M, N and K; at
    the small N of these cases it would always pick 16, so each shape is forced in turn
    (FLUTE_GEMM_ROWS) and must give the oracle's result."""
    tuning_env("FLUTE_GEMM_ROWS", rows)
    w = make_weight(N, K, bits, gs, seed=M + N + K + bits, device=DEV)
    x = make_x(M, K, seed=11)
    y = fx.qgemm_per_group_lut(x.to(DEV), w["blob_d"], w["lut_d"], bitwidth=bits, group_size=gs,
                               indices_layout=f"idx{bits}").cpu()
    assert rel_l2(y, _exact(w, x).half()) <= TOL


@pytest.mark.parametrize("rows", ["16", "32", "64", "128"])
def test_gemm_two_streams_residual_bias_every_workgroup_shape(tuning_env, rows):
    tuning_env("FLUTE_GEMM_ROWS", rows)
    M, N, K = 40, 256, 1024
    for lut_dtype, act_dtype in ((torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16)):
        w = make_weight(N, K, 4, 128, seed=7, bits2=2, rank=8, bias=True, lut_dtype=lut_dtype,
                        act_dtype=act_dtype, device=DEV)
        x = make_x(M, K, seed=13, dtype=act_dtype)
        y = _dual(w, x).cpu()
        ref = _exact(w, x).to(act_dtype)
        assert rel_l2(y, ref) <= (TOL if act_dtype == torch.float16 else TOL_BF16)


@pytest.mark.parametrize("M,N,K,gs", [(5, 256, 512, 128), (16, 512, 1024, 64), (33, 384, 1024, 256),
                                      (130, 256, 2048, 128)])
@pytest.mark.parametrize("act,lut", [(torch.float16, torch.float16), (torch.bfloat16, torch.float16),
                                     (torch.bfloat16, torch.bfloat16)])
def test_gemm_direct_activations_match_the_pre_pass(tuning_env, M, N, K, gs, act, lut):
    """With one 16-row block per wavefront the kernel reads A itself and transposes the
    pieces in registers; FLUTE_GEMM_NO_DIRECT=1 sends the same call through the activation
    pre-pass.  Both present identical operands, so the outputs are bit-identical; rows that
    are not 16-byte aligned take the pre-pass by themselves."""
    w = make_weight(N, K, 4, gs, seed=M + N, lut_dtype=lut, act_dtype=act, bias=True, device=DEV)
    x = make_x(M, K, seed=17, dtype=act)
    xd = x.to(DEV)
    y = _dual(w, xd)
    assert rel_l2(y.cpu(), _exact(w, x).to(act)) <= (TOL if act == torch.float16 else TOL_BF16)
    tuning_env("FLUTE_GEMM_NO_DIRECT", "1")
    assert torch.equal(_dual(w, xd), y)
    tuning_env("FLUTE_GEMM_NO_DIRECT", None)
    shifted = torch.zeros(M * K + 1, dtype=act, device=DEV)
    shifted[1:] = xd.reshape(-1)
    assert torch.equal(_dual(w, shifted[1:].reshape(M, K)), y)


DUAL = [
    # M, N, K, bits, gs, bits2, rank, bias
    (8, 512, 1024, 4, 128, 1, 0, False),
    (16, 512, 1024, 1, 128, 4, 0, True),
    (16, 512, 1024, 3, 128, 3, 16, True),
    (4, 512, 1024, 2, 64, 3, 0, False),
    (12, 512, 1024, 4, 128, 4, 4, False),
    (16, 256, 2048, 4, 512, 0, 64, True),
    (5, 256, 1024, 4, 16, 2, 256, False),
    (40, 256, 1024, 4, 128, 2, 8, True),               # beyond upstream's M <= 16
]


@pytest.mark.parametrize("M,N,K,bits,gs,bits2,rank,bias", DUAL)
def test_gemm_dual_stream_fp16(M, N, K, bits, gs, bits2, rank, bias):
    w = make_weight(N, K, bits, gs, seed=M + N + bits2, bits2=bits2, rank=rank, bias=bias,
                    device=DEV)
    x = make_x(M, K, seed=13)
    y = _dual(w, x).cpu()
    assert y.shape == (M, N)
    assert rel_l2(y, _exact(w, x).half()) <= TOL
    assert torch.equal(y, _dual(w, x).cpu())


@pytest.mark.parametrize("lut_dtype,act_dtype", [(torch.bfloat16, torch.bfloat16),
                                                 (torch.float16, torch.bfloat16)])
def test_gemm_dtype_mixes(lut_dtype, act_dtype):
    M, N, K = 48, 512, 2048
    w = make_weight(N, K, 4, 128, seed=5, lut_dtype=lut_dtype, act_dtype=act_dtype, bias=True,
                    device=DEV)
    x = make_x(M, K, seed=3, dtype=act_dtype)
    y = _dual(w, x).cpu()
    assert y.dtype == act_dtype
    ref = _exact(w, x).to(act_dtype)                   # the reference forward uses x.float()
    tol = TOL if act_dtype == torch.float16 else TOL_BF16
    assert rel_l2(y, ref) <= tol


@pytest.mark.parametrize("bits,gs", [(4, 128), (3, 64), (2, 16), (1, 128), (4, 32)])
def test_gemm_one_hot_rows_return_dequantised_columns(bits, gs):
    N, K = 256, 128
    w = make_weight(N, K, bits, gs, seed=bits * 7 + gs, device=DEV)
    eye = torch.eye(K, dtype=torch.float16)             # M = K = 128 one-hot rows
    y = fx.qgemm_per_group_lut(eye.to(DEV), w["blob_d"], w["lut_d"], bitwidth=bits,
                               group_size=gs, indices_layout=f"idx{bits}").cpu()
    W = O.dequant(w["blob"].numpy(), w["lut"], N, K, gs, bits)       # [N, K] fp32 of fp16 values
    assert torch.equal(y, W.t().half())


def test_gemm_matches_gemv_rows():
    """Row m of the GEMM equals the M = 1 kernel on that row up to summation order."""
    N, K = 512, 4096
    w = make_weight(N, K, 4, 128, seed=21, device=DEV)
    x = make_x(8, K, seed=2)
    y = _dual(w, x).cpu()
    for m in (0, 7):
        ym = fx.qgemm_gemv_splitk_stream(x[m:m + 1].to(DEV), w["blob_d"], w["lut_d"], 4, 128).cpu()
        assert rel_l2(y[m:m + 1], ym) <= TOL


def test_gemm_strided_views_and_empty():
    N, K = 256, 512
    w = make_weight(N, K, 4, 128, seed=9, device=DEV)
    x = make_x(24, K, seed=4)
    y = _dual(w, x).cpu()
    assert torch.equal(_dual(w, x[:0]).cpu(), torch.zeros(0, N, dtype=torch.float16))
    assert torch.equal(_dual(w, x[3:19]).cpu(), _dual(w, x[3:19].clone()).cpu())
    assert rel_l2(_dual(w, x[3:19]).cpu(), y[3:19]) <= TOL   # same rows through another shape


def test_gemm_full_size_linearity():
    """At the benchmark's full shape the oracle is too slow; use linearity instead:
    gemm(a*x1 + x2) == a*gemm(x1) + gemm(x2) within rounding, and row consistency
    between M = 256 and M = 16 launches (different shapes of the same kernel)."""
    N, K = 12288, 4096
    gen = torch.Generator(device=DEV).manual_seed(0)
    blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, device=DEV, generator=gen)
    lut = (torch.randn(N // 128, 16, device=DEV, generator=gen) * 0.02).sort(dim=1).values.half()
    x = torch.randn(256, K, device=DEV, generator=gen).half()
    run = lambda a: fx.qgemm_per_group_lut(a, blob, lut, bitwidth=4, group_size=128,
                                           indices_layout="idx4")
    y = run(x)
    y16 = run(x[32:48])
    assert rel_l2(y[32:48], y16) <= TOL
    y1 = fx.qgemm_gemv_splitk_stream(x[5:6], blob, lut, 4, 128)
    assert rel_l2(y[5:6], y1) <= TOL
    z = run((2.0 * x[:64].float() + x[64:128].float()).half())
    assert rel_l2(z, 2.0 * y[:64].float() + y[64:128].float()) <= 3e-3


@pytest.mark.parametrize("N,K,M,lut_dtype", [(12288, 4096, 256, torch.bfloat16), (4096, 12288, 256, torch.bfloat16),
                                             (12288, 4096, 1024, torch.float16), (1024, 4096, 200, torch.bfloat16)])
def test_lean_loop_is_bit_identical_to_the_scheduled_loop(tuning_env, N, K, M, lut_dtype):
    """Four-block workgroups run the loop with hand-written loads and waits by default and the
    compiler-scheduled loop under FLUTE_GEMM_NO_LEAN=1: same sums in the same order, so the
    outputs must be equal bit for bit.  Full benchmark shapes: the blobs are large enough for tile
    addresses with bit 31 set to occur."""
    gen = torch.Generator(device=DEV).manual_seed(N + K + M)
    blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, device=DEV, generator=gen)
    lut = (torch.randn(N // 128, 16, device=DEV, generator=gen) * 0.02).sort(dim=1).values.to(lut_dtype)
    x = torch.randn(M, K, device=DEV, generator=gen).bfloat16()
    run = lambda: fx.qgemm_per_group_lut(x, blob, lut, bitwidth=4, group_size=128, indices_layout="idx4")
    lean = run()
    tuning_env("FLUTE_GEMM_NO_LEAN", "1")
    scheduled = run()
    tuning_env("FLUTE_GEMM_NO_LEAN", None)
    assert torch.equal(lean, scheduled)
    y1 = fx.qgemm_gemv_splitk_stream(x[7:8], blob, lut, 4, 128)        # and against the M = 1 kernel
    assert rel_l2(lean[7:8], y1) <= 4e-3                               # (bf16 outputs: one rounding each)


@pytest.mark.parametrize("N,K,M,rot", [(12288, 4096, 256, False), (4096, 12288, 256, False), (4096, 12288, 200, True),
                                       (12288, 4096, 1000, True), (1024, 4096, 300, True)])
def test_hand_overs_between_the_k_ways_equal_the_tree(tuning_env, N, K, M, rot):
    """Workgroups of four-block wavefronts end with hand-overs between their k ways (the activation
    image is written with the blocks in the order those expect) and, under FLUTE_GEMM_NO_HANDOVER=1,
    with the reduction tree over the image in plain order: the same additions, so equal bit for
    bit, whether the image comes from the pre-pass or from the rotation that writes it itself,
    with ragged M, four k ways (K = 4096) and eight (K = 12288)."""
    import ctypes
    from flute_extended import _lib
    import fht
    gen = torch.Generator(device=DEV).manual_seed(N + K + M)
    blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, device=DEV, generator=gen)
    lut = (torch.randn(N // 128, 16, device=DEV, generator=gen) * 0.02).sort(dim=1).values.bfloat16().contiguous()
    x = torch.randn(M, K, device=DEV, generator=gen).bfloat16()
    signs = O.rotation_signs(K, 3).to(DEV) if rot else None
    if N == 1024:
        tuning_env("FLUTE_GEMM_ROWS", "128")
    d = _lib.FluteLinear()
    d.q1, d.lut1, d.q1_bytes = blob.data_ptr(), lut.data_ptr(), blob.numel()
    d.N, d.K, d.b1, d.group_size, d.lut_rows, d.lut_dtype = N, K, 4, 128, N // 128, _lib.BF16
    if rot:
        d.signs = signs.data_ptr()

    def run():
        C = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
        st = _lib.lib.flute_gemm(ctypes.byref(d), x.data_ptr(), C.data_ptr(), M, K, N, _lib.BF16,
                                 torch.cuda.current_stream().cuda_stream)
        assert st == 0, _lib.last_error()
        return C

    handed = run()
    tuning_env("FLUTE_GEMM_NO_HANDOVER", "1")
    tree = run()
    tuning_env("FLUTE_GEMM_NO_HANDOVER", None)
    assert torch.equal(handed, tree)
    xr = fht.fht_apply(x, signs, backend="kernel") if rot else x
    y1 = fx.qgemm_gemv_splitk_stream(xr[M - 1:M], blob, lut, 4, 128)   # and against the M = 1 kernel
    assert rel_l2(handed[M - 1:M], y1) <= 4e-3


@pytest.mark.parametrize("kind", ["outliers", "tiny", "huge", "mixed"])
@pytest.mark.parametrize("M,rows", [(8, None), (40, None), (130, "64"), (300, "128")])
def test_gemm_bf16_activations_beyond_the_float16_range(tuning_env, kind, M, rows):
    """bfloat16 rows that float16 cannot hold (|x| > 65504 or < 6e-8) in front of a float16
    LUT: every row is scaled by its own power of two before it meets the matrix cores and
    scaled back afterwards, so the result is the reference forward's (x.float() @ W.t()),
    never inf or 0.  Rows of very different magnitude share a launch."""
    if rows:
        tuning_env("FLUTE_GEMM_ROWS", rows)
    N, K = 256, 1024
    w = make_weight(N, K, 4, 128, seed=29, act_dtype=torch.bfloat16, device=DEV)
    x = make_x(M, K, seed=31, dtype=torch.float32)
    if kind == "outliers":
        x[::3, 5] = 1.0e5
        x[1, K - 1] = -3.0e5
    elif kind == "tiny":
        x *= 1.0e-7
    elif kind == "huge":
        x[: M // 2] *= 1.0e30
    else:
        x[::2] *= 1.0e-6
        x[1::2, ::64] *= 1.0e5
    x = x.to(torch.bfloat16)
    y = _dual(w, x).cpu()
    assert torch.isfinite(y).all()
    ref = O.linear_reference(x, w["blob"].numpy(), w["lut"], N, K, 128, 4)   # same rounding point
    assert torch.isfinite(ref).all()
    # row by row: a launch-wide norm would let the large rows hide the small ones
    for m in range(M):
        assert rel_l2(y[m], ref[m]) <= TOL, f"row {m}"


@pytest.mark.parametrize("bits,gs", [(1, 128), (2, 64), (3, 128), (4, 128), (4, 16), (3, 32)])
def test_scalar_twin_differential_chain(bits, gs):
    """Upstream's differential chain (test_flute.py:172-223): the fast kernel on the idxN
    blob, the scalar twin on the LOGICAL packed rows and the twin on the blob.  The twin
    shares no code with the fast path (one thread per output, bit-position decode, LUT in
    global memory), so agreement means both read the format the same way: the two twin
    layouts must agree bit for bit (same sums in the same order), twin and fast kernel
    within fp32 reassociation, and all three exactly on one-hot rows."""
    M, K, N = 64, 512, 256
    w = make_weight(N, K, bits, gs, seed=43 + bits, device=DEV)
    logical = torch.from_numpy(O.logical_packed_rows(w["idx"].numpy(), bits)).to(DEV)
    assert logical.shape == (N, K * bits // 8)
    x = make_x(M, K, seed=44).to(DEV)
    fast = fx.qgemm_per_group_lut(x, w["blob_d"], w["lut_d"], bitwidth=bits, group_size=gs,
                                  indices_layout=f"idx{bits}")
    twin = fx.qgemm_per_group_lut(x, logical, w["lut_d"], bitwidth=bits, group_size=gs,
                                  backend="debug_simple", indices_layout=f"idx{bits}")
    twin_blob = fx.qgemm_debug_simple(x, w["blob_d"], w["lut_d"], bits, gs, q_layout=1)
    assert torch.equal(twin, twin_blob)
    assert rel_l2(fast.cpu(), twin.cpu()) <= 5e-4
    assert rel_l2(twin.cpu(), _exact(w, x.cpu()).half()) <= TOL
    eye = torch.eye(K, dtype=torch.float16, device=DEV)
    W = O.dequant(w["blob"].numpy(), w["lut"], N, K, gs, bits).t().half()
    assert torch.equal(fx.qgemm_debug_simple(eye, logical, w["lut_d"], bits, gs).cpu(), W)
    assert torch.equal(fx.qgemm_debug_simple(eye, w["blob_d"], w["lut_d"], bits, gs, q_layout=1).cpu(), W)
    assert torch.equal(fx.qgemm_per_group_lut(eye, w["blob_d"], w["lut_d"], bitwidth=bits,
                                              group_size=gs, indices_layout=f"idx{bits}").cpu(), W)


def test_scalar_twin_refusals_and_bf16():
    w = make_weight(256, 128, 4, 128, seed=47, lut_dtype=torch.bfloat16, device=DEV)
    x = make_x(3, 128, seed=48, dtype=torch.bfloat16).to(DEV)
    y = fx.qgemm_debug_simple(x, w["blob_d"], w["lut_d"], 4, 128, q_layout=1)
    assert y.dtype == torch.bfloat16
    assert rel_l2(y.cpu(), _exact(w, x.cpu()).bfloat16()) <= TOL
    with pytest.raises(RuntimeError):
        fx.qgemm_debug_simple(x, w["blob_d"][:-1], w["lut_d"], 4, 128)        # truncated
    with pytest.raises(RuntimeError):
        fx.qgemm_debug_simple(x, w["blob_d"], w["lut_d"][:, :8], 4, 128)      # wrong LUT width
    with pytest.raises(RuntimeError):
        fx.qgemm_debug_simple(x, w["blob_d"], w["lut_d"], 5, 128)
