"""Host-side contract, no GPU needed: the C ABI library loads and exports every
symbol include/flute_hip.h declares; every refusal upstream lists
(test_flute.py:226-262, src/kernel_gemv.cu:338-454) raises the same exception
type here; the gate mirrors and the module layer behave as documented."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import flute_extended as fx
from flute_extended import _C, _lib
import palettized_modules as pm
import fht
import flute_oracle as O
from _util import make_weight, make_x

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "flute_hip.h")).read()
    body = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(flute_[a-z0-9_]+)\s*\(", body))
    assert declared == set(_lib.SYMBOLS), declared ^ set(_lib.SYMBOLS)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.flute_abi_version() == 2
    assert _lib.lib.flute_target_arch() == b"gfx950"


@pytest.mark.parametrize("addr", [0x00007F3A80001000, 0x00007F3AFFFFF000, 0x0000800012345678,
                                  0x00007FFF7FFFFFF0, 0xFFFFFFFE80000010, 0x0000000080000000, 0])
def test_address_halves_rejoin_for_every_bit_pattern(addr):
    """The kernels move wavefront-uniform 64-bit pointers into scalar registers half by half
    through a builtin that returns a signed int.  Converting such a half straight to 64 bits
    sign-extends it: a low half with bit 31 set then fills the upper half with ones (an address
    outside every allocation, which small test buffers below 2 GiB of an aperture never showed).
    The library's helper takes both halves as unsigned first; checked here on addresses with bit
    31 set, bit 47 set, and both."""
    as_i32 = lambda v: ctypes.c_int32(v & 0xFFFFFFFF).value        # what the builtin hands back
    lo, hi = as_i32(addr), as_i32(addr >> 32)
    assert _lib.lib.flute_join_address_halves(lo, hi) == addr
    # the sign-extending form this replaces is wrong exactly when bit 31 of the low half is set
    naive = ((lo & 0xFFFFFFFFFFFFFFFF) | ((hi & 0xFFFFFFFF) << 32)) & 0xFFFFFFFFFFFFFFFF
    assert (naive == addr) == (lo >= 0)


def test_loaded_library_is_the_tree_s_build():
    """flute_build_id() is the hash of the sources the library was compiled from; a stale
    library on disk (sources edited, `make` not run) shows up here and in any harness that
    compares the two before timing."""
    assert re.fullmatch(r"[0-9a-f]{16}", _lib.build_id())
    assert _lib.build_id() == _lib.tree_build_id(), "lib/libflute_hip.so is older than csrc/: run make"


def test_struct_layout_matches_header():
    # 9 pointers, 2 int64, 10 int32 -> 8*9 + 16 + 40 = 128 (k_group took the tail padding)
    assert ctypes.sizeof(_lib.FluteLinear) == 128
    assert _lib.FluteLinear.q1_bytes.offset == 72 and _lib.FluteLinear.lut_rows.offset == 88
    assert _lib.FluteLinear.rot_block.offset == 120 and _lib.FluteLinear.k_group.offset == 124


def _desc(N=256, K=128, b1=4, b2=0, gs=128, R=0, **over):
    w = _lib.FluteLinear()
    w.q1 = w.lut1 = 4096
    if b2:
        w.q2 = w.lut2 = 4096
    if R:
        w.resA = w.resB = 4096
    w.N, w.K, w.R, w.b1, w.b2, w.group_size = N, K, R, b1, b2, gs
    w.q1_bytes, w.q2_bytes = N * K * b1 // 8, N * K * b2 // 8
    w.lut_rows = (N + gs - 1) // gs
    w.lut_dtype = _lib.F16
    for k, v in over.items():
        setattr(w, k, v)
    return w


@pytest.mark.parametrize("over,code", [
    ({}, _lib.FLUTE_OK),
    ({"b1": 5}, _lib.FLUTE_ERR_INVALID),
    ({"b2": 7}, _lib.FLUTE_ERR_INVALID),
    ({"K": 96}, _lib.FLUTE_ERR_INVALID),
    ({"N": 200}, _lib.FLUTE_ERR_INVALID),
    ({"group_size": 48}, _lib.FLUTE_ERR_INVALID),
    ({"group_size": 8}, _lib.FLUTE_ERR_INVALID),
    ({"q1_bytes": 100}, _lib.FLUTE_ERR_INVALID),          # truncated blob
    ({"lut_rows": 7}, _lib.FLUTE_ERR_INVALID),            # wrong LUT geometry
    ({"q1": 4097}, _lib.FLUTE_ERR_INVALID),               # misaligned indices
    ({"q1": None}, _lib.FLUTE_ERR_INVALID),
    ({"R": 300, "resA": 4096, "resB": 4096}, _lib.FLUTE_ERR_INVALID),
    ({"resA": 4096}, _lib.FLUTE_ERR_INVALID),             # resA without resB
    ({"awq": 4096}, _lib.FLUTE_ERR_INVALID),              # awq without signs
    ({"lut_dtype": 2}, _lib.FLUTE_ERR_INVALID),
    # operands off their element boundary: one case per pointer the kernels read
    ({"lut1": 4097}, _lib.FLUTE_ERR_INVALID),
    ({"b2": 2, "lut2": 4097}, _lib.FLUTE_ERR_INVALID),
    ({"b2": 2, "q2": 4104}, _lib.FLUTE_ERR_INVALID),      # stream-2 indices 8- but not 16-byte aligned
    ({"R": 8, "resA": 4097, "resB": 4096}, _lib.FLUTE_ERR_INVALID),
    ({"R": 8, "resA": 4096, "resB": 4099}, _lib.FLUTE_ERR_INVALID),
    ({"bias": 4097}, _lib.FLUTE_ERR_INVALID),
    ({"signs": 4098}, _lib.FLUTE_ERR_INVALID),
    ({"signs": 4096, "awq": 4102}, _lib.FLUTE_ERR_INVALID),
    ({"signs": 4096, "awq": 4100, "bias": 4098, "R": 8, "resA": 4098, "resB": 4102}, _lib.FLUTE_OK),
])
def test_c_validation(over, code):
    w = _desc(**over)
    assert _lib.lib.flute_validate(ctypes.byref(w), 0) == code
    if code != _lib.FLUTE_OK:
        assert _lib.last_error()


def _kdesc(N=256, K=512, **over):
    """A weight whose LUT is grouped along K: [N, K/128, 16]."""
    over = dict({"k_group": 128, "lut_rows": N * (K // 128)}, **over)
    return _desc(N=N, K=K, **over)


@pytest.mark.parametrize("over,mode,code", [
    ({}, 0, _lib.FLUTE_OK),
    ({}, 1, _lib.FLUTE_ERR_UNSUPPORTED),                  # the GEMM does not serve the form
    ({"k_group": 64}, 0, _lib.FLUTE_ERR_INVALID),
    ({"k_group": 256}, 0, _lib.FLUTE_ERR_INVALID),
    ({"lut_rows": 2}, 0, _lib.FLUTE_ERR_INVALID),         # the N-grouped row count
    ({"b1": 3}, 0, _lib.FLUTE_ERR_UNSUPPORTED),
    ({"b2": 1, "q2": 4096, "lut2": 4096}, 0, _lib.FLUTE_ERR_UNSUPPORTED),
    ({"K": 192, "lut_rows": 256}, 0, _lib.FLUTE_ERR_INVALID),      # K not whole groups
    ({"lut1": 4096 + 8}, 0, _lib.FLUTE_ERR_INVALID),      # read 16 bytes at a time
    ({"group_size": 64}, 0, _lib.FLUTE_OK),               # not read
])
def test_c_validation_of_a_lut_grouped_along_k(over, mode, code):
    w = _kdesc(**over)
    assert _lib.lib.flute_validate(ctypes.byref(w), mode) == code
    if code != _lib.FLUTE_OK:
        assert _lib.last_error()


def test_lut_grouped_along_k_is_refused_outside_the_single_gemv():
    w = _kdesc()
    assert _lib.lib.flute_gemm(ctypes.byref(w), 4096, 4096, 4, 512, 256, 0, None) == _lib.FLUTE_ERR_UNSUPPORTED
    assert "grouped along K" in _lib.last_error()
    assert _lib.lib.flute_embedding(ctypes.byref(w), 4096, 1, 4096, None) == _lib.FLUTE_ERR_UNSUPPORTED
    g, u = _kdesc(), _kdesc()
    assert _lib.lib.flute_gemv_mlp(ctypes.byref(g), ctypes.byref(u), 4096, 4096, 0, 0, None) \
        == _lib.FLUTE_ERR_UNSUPPORTED
    # the single GEMV plans it: LDS = LUT rows of a workgroup + activations + sums
    assert _lib.lib.flute_gemv_lds_bytes(ctypes.byref(w), 0) > 0
    # a split that cuts a K group in two is refused (K = 512: split 8 leaves 64 columns)
    assert _lib.lib.flute_gemv_lds_bytes(ctypes.byref(w), 8) == 0


def test_c_entry_points_refuse_before_touching_the_device():
    w = _desc()
    assert _lib.lib.flute_gemv(ctypes.byref(w), None, 4096, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_gemv(ctypes.byref(w), 4096, 4096, 7, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_gemv(ctypes.byref(w), 4096, 4096, 0, 3, None) == _lib.FLUTE_ERR_INVALID  # split !| K/64
    w2 = _desc(lut_dtype=_lib.BF16)
    assert _lib.lib.flute_gemv(ctypes.byref(w2), 4096, 4096, _lib.F16, 0, None) \
        == _lib.FLUTE_ERR_UNSUPPORTED
    assert _lib.lib.flute_fht(4096, 4096, None, 4096, 1, 100, 0, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_fht(4096, 4096, 4096, 4096, 1, 128, 0, 1, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_fht(4096, 4096, None, 4096, 1, 32768, 0, 0, 0, None) \
        == _lib.FLUTE_ERR_UNSUPPORTED
    # operands of the calls themselves: x is read 16 bytes at a time, outputs are 16-bit stores,
    # the rotation's rows sit on element boundaries, the dense output takes 4-byte stores
    assert _lib.lib.flute_gemv(ctypes.byref(w), 4096 + 8, 4096, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert "16-byte" in _lib.last_error()
    assert _lib.lib.flute_gemv(ctypes.byref(w), 4096, 4097, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_gemv_noalloc(ctypes.byref(w), 4096 + 2, 4096, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_fht(4097, 4096, None, 4096, 1, 128, 0, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_fht(4096, 4098, None, 4096, 1, 128, 0, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_fht(4098, 4096, None, 4096, 1, 128, _lib.F32, 0, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_dequant(ctypes.byref(w), 1, 4098, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_gemm(ctypes.byref(w), 4097, 4096, 4, 128, 256, 0, None) == _lib.FLUTE_ERR_INVALID
    assert _lib.lib.flute_embedding(ctypes.byref(w), 4100, 1, 4096, None) == _lib.FLUTE_ERR_INVALID
    g, u = _desc(), _desc(N=384)
    assert _lib.lib.flute_gemv_mlp(ctypes.byref(g), ctypes.byref(u), 4096, 4096, 0, 0, None) \
        == _lib.FLUTE_ERR_INVALID


def _cpu_args(N=256, K=128, b=4, gs=128, dtype=torch.float16):
    w = make_weight(N, K, b, gs, seed=1, act_dtype=dtype)
    return make_x(1, K, dtype=dtype), w


def test_tensor_level_refusals_raise_runtimeerror():
    x, w = _cpu_args()
    call = lambda **kw: fx.qgemm_gemv_splitk_stream(
        kw.pop("A", x), kw.pop("indices", w["blob"]), kw.pop("lut", w["lut"]),
        kw.pop("bitwidth", 4), kw.pop("group_size", 128), **kw)
    with pytest.raises(RuntimeError, match="CUDA"):
        call()                                                     # valid shapes, CPU tensors
    with pytest.raises(RuntimeError, match="M == 1"):
        call(A=make_x(2, 128))
    with pytest.raises(RuntimeError, match="byte count"):
        call(indices=w["blob"][:-7])                                # truncated blob
    with pytest.raises(RuntimeError, match="lut must be"):
        call(lut=w["lut"][:, :8].contiguous())                      # wrong LUT width
    with pytest.raises(RuntimeError, match="group_size"):
        call(group_size=48)
    with pytest.raises(RuntimeError, match="bitwidth"):
        call(bitwidth=5)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        call(A=make_x(1, 96))
    with pytest.raises(RuntimeError, match="float16"):
        call(A=make_x(1, 128, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="together"):
        call(resB=torch.zeros(4, 128, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="rank"):
        call(resB=torch.zeros(300, 128, dtype=torch.float16),
             resA=torch.zeros(256, 300, dtype=torch.float16))
    with pytest.raises(ValueError, match="awq_scale"):
        call(awq_scale=torch.ones(128))                             # awq without signs
    with pytest.raises(ValueError, match="rot_signs"):
        call(rot_signs=torch.ones(64))
    with pytest.raises(RuntimeError, match="group_size"):
        fx.qgemm_gemv_stream(x, w["blob"], w["lut"], 4, 32)         # plain entry: gs >= 64 only


def _rec(rec, shape, dtype, device=0, data=4096, present=1, name=None, contiguous=1):
    rec.present, rec.ndim, rec.dtype, rec.device, rec.contiguous = present, len(shape), dtype, device, contiguous
    n = 1
    for i, v in enumerate(shape):
        rec.size[i] = v
        n *= v
    rec.numel = n if shape else 0
    rec.data = data if n else None
    if name:
        rec.dtype_name = name


def _operands(N=256, K=128, b1=4, gs=128, **over):
    ops = _lib.FluteOperands()
    _rec(ops.A, (1, K), _lib.F16)
    _rec(ops.indices, (N * K * b1 // 8,), _lib.U8)
    _rec(ops.lut, ((N + gs - 1) // gs, 1 << b1), _lib.F16)
    for name in ("indices2", "lut2", "resB", "resA", "bias"):
        _rec(getattr(ops, name), (0,), _lib.F16)
    ops.signs.present = ops.awq.present = 0
    ops.K, ops.b1, ops.b2, ops.group_size, ops.max_rank = K, b1, 0, gs, 256
    ops.gs_allowed = sum(1 << i for i in range(4, 12))
    for k, v in over.items():
        v(ops) if callable(v) else setattr(ops, k, v)
    return ops


def test_the_library_s_own_argument_checks_fill_the_descriptor():
    """flute_describe_linear from plain records, no tensor library involved: the descriptor it
    returns, and one refusal of each kind with upstream's message."""
    def run(ops):
        w, n = _lib.FluteLinear(), ctypes.c_int64(0)
        st = _lib.lib.flute_describe_linear(b"entry", ctypes.byref(ops), ctypes.byref(w), ctypes.byref(n))
        return st, w, n.value, _lib.last_error()
    st, w, n, _ = run(_operands())
    assert st == _lib.FLUTE_OK and n == 256
    assert (w.N, w.K, w.b1, w.b2, w.R, w.group_size, w.lut_rows, w.q1_bytes) == (256, 128, 4, 0, 0, 128, 2, 16384)
    assert w.q1 == 4096 and w.lut1 == 4096 and not w.q2 and not w.resA and not w.signs and w.k_group == 0
    assert _lib.lib.flute_validate(ctypes.byref(w), 0) == _lib.FLUTE_OK
    cases = [
        (dict(b1=5), "entry: bitwidth must be 1, 2, 3 or 4 (got 5)"),
        (dict(group_size=48), "entry: group_size must be one of 16/32/64/128/256/512/1024/2048 (got 48)"),
        (dict(gs_allowed=sum(1 << i for i in range(6, 12)), group_size=32),
         "entry: group_size must be one of 64/128/256/512/1024/2048 (got 32)"),
        (dict(x=lambda o: _rec(o.indices, (16377,), _lib.U8)),
         "entry: stream-1 byte count 16377 is not N*(K*4/8) for any N (K = 128)"),
        (dict(x=lambda o: _rec(o.lut, (2, 8), _lib.F16)),
         "entry: stream-1 lut must be [ceil(N/group_size), 2^bitwidth] = [2, 16] (got (2, 8))"),
        (dict(x=lambda o: _rec(o.lut, (2, 16), _lib.BF16)), "entry: a bfloat16 lut needs bfloat16 activations"),
        (dict(x=lambda o: _rec(o.resB, (4, 128), _lib.F16)),
         "entry: resB and resA must be supplied together (both empty or both populated)"),
        (dict(x=lambda o: _rec(o.bias, (7,), _lib.F16)),
         "entry: bias must be a contiguous (N,) torch.float16 tensor (N=256)"),
        (dict(x=lambda o: _rec(o.signs, (64,), _lib.F32)),
         "entry: signs must be a contiguous (K,) float32 vector (K=128)"),
        (dict(x=lambda o: _rec(o.awq, (128,), _lib.F32)), "entry: awq scale without rotation signs"),
        (dict(x=lambda o: _rec(o.lut, (2, 16), _lib.F16, device=-1)), "entry: all tensors must be CUDA (HIP) tensors"),
        (dict(x=lambda o: _rec(o.lut, (2, 16), _lib.F16, device=1)),
         "entry: all tensors must live on A's device cuda:0"),
    ]
    for over, msg in cases:
        st, _, _, err = run(_operands(**over))
        assert st == _lib.FLUTE_ERR_INVALID and err == msg, (over, err)
    a = _lib.FluteTensor()
    _rec(a, (1, 128), -1, name=b"torch.float64")
    assert _lib.lib.flute_check_input(b"entry", ctypes.byref(a), 1) == _lib.FLUTE_ERR_INVALID
    assert _lib.last_error() == "entry: A must be float16 or bfloat16 (got torch.float64)"
    _rec(a, (3, 128), _lib.BF16)
    assert _lib.lib.flute_check_input(b"entry", ctypes.byref(a), 0) == _lib.FLUTE_OK
    assert _lib.lib.flute_check_input(b"entry", ctypes.byref(a), 1) == _lib.FLUTE_ERR_INVALID
    assert "M == 1 (got M=3)" in _lib.last_error()


def _first_line(fn):
    with pytest.raises(RuntimeError) as err:
        fn()
    return str(err.value).splitlines()[0]


@pytest.mark.skipif(_C.native is None, reason="the compiled binding is not built or switched off")
def test_compiled_binding_refuses_with_the_python_binding_s_words():
    """csrc/torch_binding.cpp and flute_extended/_C.py hand their tensors to the same checks in
    the library (upstream: the TORCH_CHECKs of src/kernel_gemv.cu:338-454): same order, same
    first line, whichever binding recorded the tensors."""
    x, w = _cpu_args()
    e8 = torch.empty(0, dtype=torch.uint8)
    e16 = torch.empty(0, dtype=torch.float16)
    base = dict(A=x, indices=w["blob"], lut=w["lut"], b1=4, i2=e8, l2=e16, b2=0, rb=e16, ra=e16,
                bi=e16, gs=128)
    cases = [dict(), dict(A=make_x(2, 128)), dict(A=make_x(1, 96)), dict(A=make_x(1, 128, dtype=torch.float32)),
             dict(indices=w["blob"][:-7]), dict(lut=w["lut"][:, :8].contiguous()), dict(gs=48),
             dict(b1=5), dict(b2=7), dict(rb=torch.zeros(4, 128, dtype=torch.float16)),
             dict(rb=torch.zeros(300, 128, dtype=torch.float16), ra=torch.zeros(256, 300, dtype=torch.float16)),
             dict(bi=torch.zeros(7, dtype=torch.float16)),
             dict(b2=1, i2=torch.zeros(3, dtype=torch.uint8), l2=torch.zeros(2, 2, dtype=torch.float16)),
             dict(lut=w["lut"].bfloat16())]
    for name in ("qgemm_gemv_splitk_stream", "qgemm_dual_stream"):
        for over in cases:
            a = dict(base, **over)
            args = (a["A"], a["indices"], a["lut"], a["b1"], a["i2"], a["l2"], a["b2"], a["rb"],
                    a["ra"], a["bi"], a["gs"])
            if name == "qgemm_dual_stream" and "A" in over and over["A"].shape[0] == 2:
                continue                                   # M = 2 is fine for the GEMM
            py = _first_line(lambda: _C.PYTHON_BINDING[name](*args))
            cc = _first_line(lambda: getattr(_C.native, name)(*args))
            assert py == cc, (name, over.keys(), py, cc)
    seg = torch.zeros(2, 15, dtype=torch.int64)
    for args in ((x, seg[:, :14].contiguous(), e16), (make_x(2, 128), seg, e16),
                 (x, seg, torch.zeros(5, dtype=torch.float32))):
        py = _first_line(lambda: _C.PYTHON_BINDING["qgemm_gemv_mlp"](*args))
        cc = _first_line(lambda: _C.native.qgemm_gemv_mlp(*args))
        assert py == cc


def test_layout_string_guards():
    x, w = _cpu_args()
    with pytest.raises(ValueError):
        fx.qgemm_per_group_lut(x, w["blob"], w["lut"], 4, 128, indices_layout="idx9")
    with pytest.raises(ValueError):
        fx.qgemm_per_group_lut(x, w["blob"], w["lut"], 2, 128, indices_layout="idx4")
    with pytest.raises(RuntimeError):
        fx.qgemm_debug_simple(x, w["blob"], w["lut"], 4, 128)
    with pytest.raises(RuntimeError):
        fx.qgemm_dense(x, torch.zeros(256, 128, dtype=torch.float16))
    with pytest.raises(ValueError):
        fx.qgemm_gemv_mlp(x, torch.zeros(3, 15, dtype=torch.int64), torch.zeros(1, 256).half())
    with pytest.raises(ValueError):
        fx.qgemm_gemv_multi(x, torch.zeros(2, 14, dtype=torch.int64))


def test_gates_and_tables():
    assert fx.gemv_stream_available() and fx.gemv_splitk_available() and fx.gemv_mlp_available()
    assert fx.gemv_multi_available() and fx.dual_stream_available()
    assert fx.gemv_splitk_fht_available() and fx.gemv_fht_stream_available()
    assert len(fx.GEMV_SPLITK_PAIRS) == 20 and (4, 0) in fx.GEMV_STREAM_PAIRS
    assert fx.GEMV_SPLITK_MAX_RESIDUAL_RANK == 256 and fx.DUAL_STREAM_MAX_M == 16
    assert fx.gemv_splitk_supported(4, 0, 128, 12288, 4096, 1)
    assert fx.gemv_splitk_supported(1, 4, 16, 4096, 12288, 1, 256)
    assert not fx.gemv_splitk_supported(4, 0, 128, 12288, 4096, 2)          # M != 1
    assert not fx.gemv_splitk_supported(4, 0, 128, 12288, 4096, 1, 300)     # rank cap
    assert not fx.gemv_splitk_supported(4, 0, 48, 12288, 4096, 1)
    assert not fx.gemv_splitk_supported(4, 0, 128, 12200, 4096, 1)
    assert not fx.gemv_stream_supported(4, 4, 128, 4096, 4096, 1)           # pair table
    assert not fx.gemv_stream_supported(4, 0, 32, 4096, 4096, 1)            # gs table
    assert fx.gemv_splitk_fht_supported(4, 0, 128, 4096, 12288, 1)
    assert not fx.gemv_splitk_fht_supported(4, 0, 128, 4096, 32768, 1)      # segment > 16384
    assert fx.gemv_mlp_supported(4096, 12288, [(4, 0, 128), (4, 1, 128)])
    assert not fx.gemv_mlp_supported(4096, 12288, [(4, 0, 128)])
    assert fx.gemv_multi_supported(4096, 48, [(4, 0, 128), (3, 3, 64)])
    assert fx.dual_stream_supported(4, 0, 128, 4096, 4096)
    assert not fx.dual_stream_supported(4, 0, 128, 4000, 4096)
    # the split policy of this library (upstream's: src/gemv_host.cpp:29-38, other numbers): a
    # hint always divides K/64; the unsplit launch measured fastest up to K = 24576, from
    # K = 32768 narrow outputs split four ways (N <= 512) or two ways (N <= 1024)
    assert fx.gemv_split_hint(12288, 4096) == 1 and fx.gemv_split_hint(248320, 4096) == 1
    for N in (1024, 512, 128):
        s = fx.gemv_split_hint(N, 4096)
        assert s >= 1 and 64 % s == 0
        assert fx.gemv_split_hint(N, 24576) == 1
    assert fx.gemv_split_hint(512, 32768) == 4 and fx.gemv_split_hint(128, 65536) == 4
    assert fx.gemv_split_hint(1024, 32768) == 2 and fx.gemv_split_hint(2048, 32768) == 1
    assert fx.gemv_split_hint(512, 32768 + 64) == 1          # 513 tiles: neither 4 nor 2 divides
    assert 0 < _C.gemv_lds_bytes(12288, 4096, 4, 0, 128) <= fx.LDS_BYTES_PER_CU


def test_fht_module_surface():
    assert fht.segments(12288) == [(0, 8192), (8192, 4096)]
    signs = fht.rotation_signs(256, 11)
    assert torch.equal(signs, O.rotation_signs(256, 11))
    x = make_x(4, 256, dtype=torch.float32)
    assert torch.equal(fht.fht_apply(x, signs, backend="reference"), O.fht_reference(x, signs))
    assert torch.equal(fht.fht_adjoint(x, signs, backend="reference"),
                       O.fht_adjoint_reference(x, signs))
    T = fht.build_rotation_matrix(256, 11)
    assert np.allclose(T.double().numpy(), O.rotation_matrix(signs), atol=1e-7)
    assert (fht.fht_apply(x, signs, backend="matmul") - x @ T).abs().max() < 1e-5
    s = torch.rand(256) + 0.5
    assert torch.equal(fht.fht_apply_awq(x, signs, s, backend="reference"),
                       O.fht_awq_reference(x, signs, s))
    with pytest.raises(RuntimeError):
        fht.fht_apply(x, signs, backend="kernel")                   # CPU tensor
    with pytest.raises(ValueError):
        fht.fht_apply(x, signs, backend="nope")
    with pytest.raises(ValueError):
        fht.fht_apply(x, signs[:-1])
    y = x.clone()
    fht.fht_apply_(y, signs, backend="reference")
    assert torch.equal(y, O.fht_reference(x, signs))
    xa = x.clone().requires_grad_(True)
    g = make_x(4, 256, seed=9, dtype=torch.float32)
    fht.fht_apply(xa, signs, backend="reference").backward(g)
    assert torch.equal(xa.grad, O.fht_adjoint_reference(g, signs))


def test_module_layer_reference_mode_matches_oracle():
    N, K = 256, 128
    w = make_weight(N, K, 4, 64, seed=3, bits2=2, rank=8, bias=True, act_dtype=torch.float32)
    m = pm.PalettizedLinear(w["blob"], w["lut"], 4, 64, N, K, bias=w["bias"], resA=w["resA"],
                            resB=w["resB"], indices2=w["blob2"], lut2=w["lut2"], bitwidth2=2,
                            reference=True, rotation_seed=5, rotation_k=K)
    x = make_x(2, K, dtype=torch.float32).reshape(1, 2, K)
    ref = O.linear_reference(x, w["blob"], w["lut"], N, K, 64, 4, w["blob2"], w["lut2"], 2,
                             w["resA"], w["resB"], w["bias"], signs=O.rotation_signs(K, 5))
    assert torch.equal(m(x), ref) and m(x).shape == (1, 2, N)
    m._cache_logical_indices()
    assert torch.equal(m(x), ref)                                  # cached-index gather
    assert torch.equal(pm.reference_dequant(w["blob"], w["lut"], N, K, 64, 4),
                       O.dequant(w["blob"], w["lut"], N, K, 64, 4))


def test_module_layer_constructor_contract():
    w = make_weight(256, 128, 4, 128, seed=3)
    mk = lambda **kw: pm.PalettizedLinear(kw.pop("indices", w["blob"]), w["lut"],
                                          kw.pop("bitwidth", 4), 128, kw.pop("N", 256),
                                          kw.pop("K", 128), **kw)
    mk()
    with pytest.raises(ValueError):
        mk(N=200, indices=torch.zeros(200 * 64, dtype=torch.uint8))   # kernel mode needs N%128
    mk(N=200, indices=torch.zeros(200 * 64, dtype=torch.uint8), reference=True)
    with pytest.raises(ValueError):
        mk(indices=w["blob"][:-1])
    with pytest.raises(ValueError):
        mk(bitwidth=5)
    with pytest.raises(ValueError):
        mk(indices2=w["blob"])                                        # half a second stream
    with pytest.raises(ValueError):
        mk(awq_scale=torch.ones(128))                                 # awq without rotation
    with pytest.raises(ValueError):
        mk(rotation_seed=1, rotation_k=64)
    with pytest.raises(ValueError):
        mk(rotation_seed=1, rotation_k=128, awq_scale=-torch.ones(128))
    with pytest.raises(ValueError):
        mk(resA=torch.zeros(256, 4), resB=torch.zeros(5, 128))
    m = mk(rotation_seed=1, rotation_k=128, awq_scale=torch.ones(128))
    assert m.fold_order == "rotate_then_awq"
    # kernel mode on CPU tensors fails loudly instead of computing in torch
    with pytest.raises(RuntimeError):
        mk()(make_x(1, 128))


def test_fused_mlp_falls_through_on_unfusable_inputs():
    wg, wu = make_weight(256, 128, seed=1), make_weight(256, 128, seed=2)
    wd = make_weight(128, 256, seed=3)
    g = pm.PalettizedLinear(wg["blob"], wg["lut"], 4, 128, 256, 128, reference=True)
    u = pm.PalettizedLinear(wu["blob"], wu["lut"], 4, 128, 256, 128, reference=True)
    d = pm.PalettizedLinear(wd["blob"], wd["lut"], 4, 128, 128, 256, reference=True)
    mlp = pm.FusedPalettizedMLP(g, u, d, torch.nn.functional.silu)
    x = make_x(1, 128, dtype=torch.float32)
    y = mlp(x)
    ref = O.mlp_reference(x, *[dict(blob=w["blob"], lut=w["lut"], N=w["N"], K=w["K"],
                                    group_size=128, bits=4) for w in (wg, wu, wd)])
    assert torch.equal(y, ref)
    assert mlp._merge_state is None                                 # fp32 input: never built
    assert mlp._build_state(torch.device("cpu"), torch.float16)["reason"] == "reference member"


def test_workspace_decision_refuses_growth_under_capture():
    """The branch get_workspace takes: enough room -> nothing happens (capturing or not);
    too little -> grow outside a capture, refuse inside one."""
    from flute_extended import _lib
    dec = _lib.lib.flute_workspace_decision
    assert dec(1 << 20, 1000, 1 << 14, 10, 0) == 0
    assert dec(1 << 20, 1000, 1 << 14, 10, 1) == 0
    assert dec(1 << 20, (1 << 20) + 1, 1 << 14, 10, 0) == 1
    assert dec(1 << 20, (1 << 20) + 1, 1 << 14, 10, 1) == 2
    assert dec(0, 0, 0, 1, 1) == 2 and dec(0, 0, 0, 0, 1) == 0


def test_tuning_is_read_once_and_on_reload(monkeypatch):
    """Tuning variables do not reach the library until flute_reload_tuning(): the split
    policy (pure host arithmetic) shows which value is in force."""
    from flute_extended import _lib
    before = _lib.lib.flute_gemv_lds_bytes
    w = _lib.FluteLinear()
    w.q1 = w.lut1 = 16
    w.N, w.K, w.b1, w.group_size, w.lut_rows, w.lut_dtype = 1024, 4096, 4, 128, 8, _lib.F16
    w.q1_bytes = 1024 * 4096 // 2
    base = before(w, 1)
    monkeypatch.setenv("FLUTE_GEMV_TABLE_LOG2", "13")
    assert before(w, 1) == base                         # not re-read per call
    _lib.lib.flute_reload_tuning()
    try:
        assert before(w, 1) != base
    finally:
        monkeypatch.undo()
        _lib.lib.flute_reload_tuning()
    assert before(w, 1) == base


def test_merged_modules_refuse_operands_they_cannot_pass_by_address():
    """The merged launches read raw addresses out of a table: members left on the CPU, a
    stream-2 LUT of another dtype, or a non-contiguous blob must end in the per-module chain
    (a refusal with a reason), never in a kernel launch."""
    wg, wu = make_weight(256, 128, seed=1, bits2=2), make_weight(256, 128, seed=2, bits2=2)

    def member(w, **over):
        args = dict(indices2=w["blob2"], lut2=w["lut2"], bitwidth2=2, reference=False)
        args.update(over)
        return pm.PalettizedLinear(w["blob"], w["lut"], 4, 128, 256, 128, **args)

    silu = torch.nn.functional.silu
    cpu = torch.device("cpu")
    mlp = pm.FusedPalettizedMLP(member(wg), member(wu), member(wg), silu)
    assert "device" in mlp._build_state(cpu, torch.float16)["reason"]      # CPU members
    assert mlp._fused_gate_up(make_x(1, 128)) is None                      # and a CPU input
    qkv = pm.SplitQKV(member(wg), member(wu), member(wg))
    assert "device" in qkv._build_state(cpu, torch.float16)["reason"]
    # the verdict names the first problem it meets; each is a refusal of its own
    m = member(wg)
    assert "indices" in pm._operand_problem(m, cpu)
    m.lut2 = m.lut2.float()
    assert pm._operand_problem(m, cpu) is not None
    # pointer tuple: replacing a buffer changes it, so a cached table would be rebuilt
    before = pm._operand_ptrs((m,))
    m.indices = m.indices.clone()
    assert pm._operand_ptrs((m,)) != before
    # members that are not palettized at all (a dense layer left in place) have no blobs: the
    # tuple is still defined, and the verdict is a refusal that carries it
    dense = torch.nn.Linear(128, 256)
    assert pm._operand_ptrs((dense,))[:4] == (0, 0, 0, 0)
    for wrapper in (pm.FusedPalettizedMLP(dense, member(wu), member(wg), silu),
                    pm.SplitQKV(dense, member(wu), member(wg))):
        state = wrapper._build_state(cpu, torch.float16)
        assert state["reason"] == "non-PalettizedLinear member" and "ptrs" in state
