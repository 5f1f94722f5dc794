"""GPU parity of the merged gate/up launch, the grouped launch, the MLP block
and the module layer's kernel mode against the oracle / the reference mode."""
import ctypes

import pytest
import torch

import flute_extended as fx
import flute_oracle as O
import palettized_modules as pm
from flute_extended import _lib
from _util import make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-3


def _row(w, out=None, signs=None, awq=None):
    p = lambda t: 0 if t is None else t.data_ptr()
    return [p(w["blob_d"]), p(w["lut_d"]), p(w.get("blob2_d")), p(w.get("lut2_d")),
            p(w.get("resB_d")), p(w.get("resA_d")), p(w.get("bias_d")), p(out), w["N"],
            0 if w["resB"] is None else w["resB"].shape[0], w["bits"], w["bits2"], w["gs"],
            p(signs), p(awq)]


def _exact(w, x):
    return O.linear_exact(x, w["blob"].numpy(), w["lut"], w["N"], w["K"], w["gs"], w["bits"],
                          w["blob2"].numpy() if w["bits2"] else None, w["lut2"], w["bits2"],
                          w["resA"], w["resB"], w["bias"])


@pytest.mark.parametrize("gspec,uspec", [
    (dict(bits=4), dict(bits=4)),
    (dict(bits=4, bits2=1, gs=64), dict(bits=1, bits2=4, rank=8, bias=True)),
    (dict(bits=3, gs=32), dict(bits=2, rank=4)),
])
def test_merged_gate_up_silu(gspec, uspec):
    N, K = 1024, 2048
    g = make_weight(N, K, seed=1, device=DEV, **gspec)
    u = make_weight(N, K, seed=2, device=DEV, **uspec)
    x = make_x(1, K, seed=3)
    out = torch.zeros(1, N, dtype=torch.float16, device=DEV)
    table = torch.tensor([_row(g), _row(u)], dtype=torch.int64)
    y = fx.qgemm_gemv_mlp(x.to(DEV), table, out)
    assert y.data_ptr() == out.data_ptr()
    ref = O.silu_mul_exact(_exact(g, x), _exact(u, x)).half()
    assert rel_l2(y.cpu(), ref) <= TOL
    y1 = y.clone()
    fx.qgemm_gemv_mlp(x.to(DEV), table, out)
    assert torch.equal(out, y1)


def test_merged_gate_up_with_different_rotations():
    N, K = 512, 4096
    g = make_weight(N, K, seed=1, device=DEV)
    u = make_weight(N, K, seed=2, device=DEV)
    x = make_x(1, K, seed=3)
    sg, su = O.rotation_signs(K, 1).to(DEV), O.rotation_signs(K, 2).to(DEV)
    out = torch.zeros(1, N, dtype=torch.float16, device=DEV)
    table = torch.tensor([_row(g, signs=sg), _row(u, signs=su)], dtype=torch.int64)
    y = fx.qgemm_gemv_mlp(x.to(DEV), table, out).cpu()
    ref = O.silu_mul_exact(_exact(g, O.fht_reference(x, sg.cpu())),
                           _exact(u, O.fht_reference(x, su.cpu()))).half()
    assert rel_l2(y, ref) <= TOL


@pytest.mark.parametrize("rank", [0, 8])
def test_merged_gate_up_different_rotations_bfloat16_rows_float16_lut(rank):
    """bfloat16 activations in front of float16 LUTs are scaled per staged row, and a member with
    its own signs makes the launch stage the row a second time while the first output's partial
    row sums still wait in LDS: the scaling's scratch words must not be those sums.  Every gate
    row is checked (the first rows of each slice were the ones at risk), with magnitudes beyond
    float16's range so the scaling is exercised."""
    N, K = 512, 4096
    bf = torch.bfloat16
    g = make_weight(N, K, seed=11, rank=rank, act_dtype=bf, device=DEV)
    u = make_weight(N, K, seed=12, rank=rank, act_dtype=bf, device=DEV)
    x = (make_x(1, K, seed=13).float() * 3.0e5).to(bf)
    sg, su = O.rotation_signs(K, 1).to(DEV), O.rotation_signs(K, 2).to(DEV)
    out = torch.zeros(1, N, dtype=bf, device=DEV)
    table = torch.tensor([_row(g, signs=sg), _row(u, signs=su)], dtype=torch.int64)
    y = fx.qgemm_gemv_mlp(x.to(DEV), table, out).cpu()
    yg = _exact(g, O.fht_reference(x, sg.cpu()))
    yu = _exact(u, O.fht_reference(x, su.cpu()))
    ref = O.silu_mul_exact(yg, yu)
    assert torch.isfinite(y).all()
    assert rel_l2(y, ref.to(bf)) <= TOL           # same rounding point as the reference forward
    # row by row: one bfloat16 rounding (2^-9) of a value whose factors are exact to ~1e-6
    # (values far below bfloat16's normal range, where SiLU of a large negative sum underflows,
    # are left to the norm above)
    big = ref.double().abs() > 1e-30
    err = (y.double() - ref.double()).abs()[big] / ref.double().abs()[big]
    assert int(big.sum()) > N // 4 and float(err.max()) <= 2.0 ** -8
    # each member alone through the single-weight entry gives the same sums
    yg1 = fx.qgemm_gemv_stream(x.to(DEV), g["blob_d"], g["lut_d"], 4, 128, rot_signs=sg,
                               **({"resA": g["resA_d"], "resB": g["resB_d"]} if rank else {})).cpu()
    assert rel_l2(yg1, yg.to(bf)) <= TOL


def test_grouped_launch():
    K = 2048
    ws = [make_weight(512, K, seed=1, device=DEV),
          make_weight(256, K, bits=3, gs=64, bits2=3, rank=8, seed=2, device=DEV),
          make_weight(128, K, bits=2, gs=32, bias=True, seed=3, device=DEV)]
    outs = [torch.zeros(1, w["N"], dtype=torch.float16, device=DEV) for w in ws]
    x = make_x(1, K, seed=4)
    table = torch.tensor([_row(w, o) for w, o in zip(ws, outs)], dtype=torch.int64)
    assert fx.qgemm_gemv_multi(x.to(DEV), table) is None
    for w, o in zip(ws, outs):
        assert rel_l2(o.cpu(), _exact(w, x).half()) <= TOL


def _desc(w):
    d = _lib.FluteLinear()
    d.q1, d.lut1 = w["blob_d"].data_ptr(), w["lut_d"].data_ptr()
    d.q1_bytes = w["blob_d"].numel()
    d.N, d.K, d.b1, d.group_size = w["N"], w["K"], w["bits"], w["gs"]
    d.lut_rows = w["lut"].shape[0]
    d.lut_dtype = _lib.F16 if w["lut"].dtype == torch.float16 else _lib.BF16
    return d


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mlp_block_through_the_c_abi(dtype):
    """Benchmark configuration 2 at full size: gate/up 4096 -> 12288, SiLU*mul,
    down 12288 -> 4096, called straight through flute_mlp_block."""
    H, I = 4096, 12288
    g = make_weight(I, H, seed=1, device=DEV)
    u = make_weight(I, H, seed=2, device=DEV)
    d = make_weight(H, I, seed=3, device=DEV)
    x = make_x(1, H, seed=4, dtype=dtype)
    xd = x.to(DEV)
    h = torch.zeros(1, I, dtype=dtype, device=DEV)
    y = torch.zeros(1, H, dtype=dtype, device=DEV)
    dg, du, dd = _desc(g), _desc(u), _desc(d)
    act = _lib.F16 if dtype == torch.float16 else _lib.BF16
    st = _lib.lib.flute_mlp_block(ctypes.byref(dg), ctypes.byref(du), ctypes.byref(dd),
                                  xd.data_ptr(), h.data_ptr(), y.data_ptr(), act,
                                  torch.cuda.current_stream().cuda_stream)
    assert st == 0, _lib.last_error()
    torch.cuda.synchronize()
    h_ref = O.silu_mul_exact(_exact(g, x), _exact(u, x)).to(dtype)
    tol = TOL if dtype == torch.float16 else 4e-3      # bf16: the output rounding alone is 2^-9
    assert rel_l2(h.cpu(), h_ref) <= tol
    assert rel_l2(y.cpu(), _exact(d, h.cpu()).to(dtype)) <= tol


def _modules(w, **kw):
    args = dict(bias=w["bias"], resA=w["resA"], resB=w["resB"], indices2=w["blob2"],
                lut2=w["lut2"], bitwidth2=w["bits2"] or None)
    args.update(kw)
    ref = pm.PalettizedLinear(w["blob"], w["lut"], w["bits"], w["gs"], w["N"], w["K"],
                              reference=True, **args)
    ker = pm.PalettizedLinear(w["blob"], w["lut"], w["bits"], w["gs"], w["N"], w["K"],
                              reference=False, **args).to(DEV)
    return ref, ker


@pytest.mark.parametrize("spec", [dict(), dict(bits2=2, rank=8, bias=True), dict(bits=3, gs=32)])
@pytest.mark.parametrize("rot", [False, True])
def test_module_kernel_mode_matches_reference_mode_m1(spec, rot):
    N, K = 512, 1024
    w = make_weight(N, K, seed=5, **spec)
    kw = dict(rotation_seed=9, rotation_k=K) if rot else {}
    ref, ker = _modules(w, **kw)
    x = make_x(1, K, seed=6)
    pm.ROUTE_CENSUS.clear()
    y = ker(x.to(DEV).reshape(1, 1, K))
    assert y.shape == (1, 1, N)
    assert rel_l2(y.cpu().reshape(1, N), ref(x)) <= TOL
    assert list(pm.ROUTE_CENSUS) == ["gemv_splitk_fht" if rot else "gemv_splitk"]


def test_fused_mlp_module():
    H, I = 1024, 2048
    wg, wu, wd = (make_weight(I, H, seed=1), make_weight(I, H, seed=2, bits2=1),
                  make_weight(H, I, seed=3))
    refs, kers = zip(*[_modules(w) for w in (wg, wu, wd)])
    act = torch.nn.functional.silu
    mref = pm.FusedPalettizedMLP(*refs, act)
    mker = pm.FusedPalettizedMLP(*kers, act)
    x = make_x(1, H, seed=7)
    pm.ROUTE_CENSUS.clear()
    y = mker(x.to(DEV))
    assert pm.ROUTE_CENSUS.get("gemv_mlp") == 1 and mker._merge_state["ok"]
    assert rel_l2(y.cpu(), mref(x)) <= 2e-3       # two 16-bit roundings (h, then y) on each side


def test_merged_tables_follow_moved_and_converted_members():
    """The cached segment table holds raw addresses.  A member moved to the CPU and back has
    new buffers: the table is rebuilt (stale addresses would be a memory fault).  Residual
    factors kept in float16 are converted once for bfloat16 activations, so the merged
    launch still serves them."""
    H, I = 512, 1024
    wg, wu, wd = (make_weight(I, H, seed=1, rank=8), make_weight(I, H, seed=2, rank=8),
                  make_weight(H, I, seed=3))
    refs, kers = zip(*[_modules(w) for w in (wg, wu, wd)])
    act = torch.nn.functional.silu
    mref, mker = pm.FusedPalettizedMLP(*refs, act), pm.FusedPalettizedMLP(*kers, act)
    x = make_x(1, H, seed=7)
    y0 = mker(x.to(DEV))
    first = mker._merge_state
    assert first["ok"]
    mker.gate_proj.to("cpu")
    mker.gate_proj.to(DEV)
    y1 = mker(x.to(DEV))
    assert mker._merge_state is not first and mker._merge_state["ok"]
    assert torch.equal(y0, y1)
    # bfloat16 activations against float16 residual factors: merged launch, not the fallback
    xb = make_x(1, H, seed=8, dtype=torch.bfloat16)
    pm.ROUTE_CENSUS.clear()
    yb = mker(xb.to(DEV))
    assert pm.ROUTE_CENSUS.get("gemv_mlp") == 1
    assert rel_l2(yb.cpu(), mref(xb)) <= 8e-3     # bf16 h and y, residual factors rounded to bf16


def test_fused_mlp_module_replays_from_a_graph():
    """The module layer is host-bound in eager mode (tens of microseconds of Python per
    call against ~20 us of kernels), so decode loops capture it in a HIP graph.  Every
    replay, with eager work and synchronisations in between, must reproduce the eager
    result bit for bit, also after the input buffer's contents change."""
    H, I = 1024, 2048
    wg, wu, wd = make_weight(I, H, seed=1), make_weight(I, H, seed=2), make_weight(H, I, seed=3)
    kers = [_modules(w)[1] for w in (wg, wu, wd)]
    mker = pm.FusedPalettizedMLP(*kers, torch.nn.functional.silu)
    x = make_x(1, H, seed=7).to(DEV)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):                        # warm-up: workspaces, merge state
        for _ in range(3):
            mker(x)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = mker(x)
    for seed in (7, 8, 9):
        x.copy_(make_x(1, H, seed=seed).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        want = mker(x)                                   # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, want)


@pytest.mark.parametrize("M,spec,route", [
    (8, dict(), "dual_stream"),
    (16, dict(bits2=2, rank=8, bias=True), "dual_stream"),
    (40, dict(bits2=2, rank=8, bias=True), "per_group_lut"),
    (130, dict(bits=3, gs=32), "per_group_lut"),
])
@pytest.mark.parametrize("rot", [False, True])
def test_module_kernel_mode_matches_reference_mode_prefill(M, spec, route, rot):
    """M > 1 goes to the MFMA GEMM: the fused small-M entry up to 16 rows, the plain
    entry (second stream, residual and bias added by the module) above."""
    N, K = 512, 1024
    w = make_weight(N, K, seed=5, **spec)
    kw = dict(rotation_seed=9, rotation_k=K) if rot else {}
    ref, ker = _modules(w, **kw)
    x = make_x(M, K, seed=6)
    pm.ROUTE_CENSUS.clear()
    y = ker(x.to(DEV))
    assert y.shape == (M, N)
    assert rel_l2(y.cpu(), ref(x)) <= (TOL if M <= 16 else 2e-3)   # module-side adds round twice
    assert list(pm.ROUTE_CENSUS) == [route]


@pytest.mark.parametrize("M,lda_pad,act,lut,rank", [
    (8, 0, torch.bfloat16, torch.float16, 0),       # the rotated-input configuration
    (8, 0, torch.float16, torch.float16, 0),
    (40, 0, torch.bfloat16, torch.bfloat16, 0),     # several 16-row blocks, padded rows
    (24, 64, torch.bfloat16, torch.float16, 0),     # rows of A further apart than K
    (100, 0, torch.float16, torch.float16, 0),      # 64-row workgroups
    (8, 0, torch.float16, torch.float16, 4),        # residual: rotated rows are kept as rows
    (24, 64, torch.float16, torch.float16, 4),
])
def test_gemm_with_rotation_through_the_c_abi(M, lda_pad, act, lut, rank):
    """flute_gemm rotates its input itself when the descriptor carries signs (block-128
    form and the full-K form).  Without a residual the rotation writes the activations
    straight in the order the matrix cores read them; with one, as rows first."""
    N, K = 512, 4096
    w = make_weight(N, K, seed=11, lut_dtype=lut, act_dtype=act, rank=rank, device=DEV)
    x = make_x(M, K, seed=12, dtype=act)
    lda = K + lda_pad
    xd = torch.zeros(M, lda, dtype=act, device=DEV)
    xd[:, :K] = x.to(DEV)
    for block in (128, 0):
        signs = O.rotation_signs(K, 3)
        sd = signs.to(DEV)
        d = _desc(w)
        d.signs, d.rot_block = sd.data_ptr(), block
        if rank:
            d.resA, d.resB, d.R = w["resA_d"].data_ptr(), w["resB_d"].data_ptr(), rank
        C = torch.zeros(M, N, dtype=act, device=DEV)
        st = _lib.lib.flute_gemm(ctypes.byref(d), xd.data_ptr(), C.data_ptr(), M, lda, N,
                                 _lib.F16 if act == torch.float16 else _lib.BF16,
                                 torch.cuda.current_stream().cuda_stream)
        assert st == 0, _lib.last_error()
        xr = O.block_fht_reference(x, 128, signs) if block else O.fht_reference(x, signs)
        # the rotated activations are rounded to the activation type before the GEMM
        xr = xr.to(act)
        ref = O.linear_exact(xr, w["blob"].numpy(), w["lut"], N, K, w["gs"], w["bits"],
                             None, None, 0, None, None, None).double()
        if rank:
            ref = ref + (xr.double() @ w["resB"].double().t()) @ w["resA"].double().t()
        tol = 1.5e-3 if act == torch.float16 else 4e-3
        assert rel_l2(C.cpu(), ref.to(act)) <= tol


@pytest.mark.parametrize("rot", [False, True])
def test_split_qkv_module(rot):
    """One token: one grouped launch writes Q|K|V side by side; several tokens: the
    per-module chain and a concatenation.  Both against the reference-mode modules."""
    K = 1024
    ws = [make_weight(512, K, seed=1), make_weight(256, K, bits=3, gs=64, bits2=3, rank=8, seed=2),
          make_weight(256, K, bits=4, gs=128, bias=True, seed=3)]
    kw = dict(rotation_seed=4, rotation_k=K) if rot else {}
    pairs = [_modules(w, **kw) for w in ws]
    ref = pm.SplitQKV(*[p[0] for p in pairs])
    ker = pm.SplitQKV(*[p[1] for p in pairs])
    x = make_x(1, K, seed=5)
    pm.ROUTE_CENSUS.clear()
    y = ker(x.to(DEV).reshape(1, 1, K))
    assert y.shape == (1, 1, 1024)
    assert pm.ROUTE_CENSUS.get("gemv_multi") == 1 and ker._merge_state["ok"], ker._merge_state
    assert rel_l2(y.cpu().reshape(1, -1), ref(x)) <= TOL
    y2 = ker(x.to(DEV))                                  # persistent output, same values
    assert torch.equal(y2.cpu(), y.cpu().reshape(1, -1))
    xs = make_x(5, K, seed=6)
    assert rel_l2(ker(xs.to(DEV)).cpu(), ref(xs)) <= 2e-3
