// flute_extended._C_native: the decode and prefill entry points of the operator surface as a
// compiled PyTorch-ROCm extension over the C ABI (include/flute_hip.h).  Upstream builds its
// kernels into a pybind11 module `flute_extended._C` (src/bindings.cpp:230-546); this file is
// that module's counterpart for the entries an eager decode loop calls per token:
//
//   qgemm_gemv_stream, qgemm_gemv_fht_stream, qgemm_gemv_splitk_stream,
//   qgemm_gemv_splitk_fht_stream            (src/bindings.cpp:277-354)
//   qgemm_gemv_multi, qgemm_gemv_mlp        (src/bindings.cpp:368-384)
//   qgemm_cutlass_streaming, qgemm_dual_stream   (src/bindings.cpp:245-270)
//
// Same positional signatures, same conventions (empty tensor = absent operand, N from the
// blob's byte count, RuntimeError on every contract violation, fresh outputs, launches on the
// current stream of the input's device) and the same checks, in the same order and with the
// same messages, as the ctypes mirror in flute_extended/_C.py, which stays the binding for
// everything else and the fallback when this module is not built.  Host code only: nothing
// here runs on the device, the kernels are in libflute_hip.so.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <sstream>
#include <string>
#include <vector>

#include "flute_hip.h"

namespace {

using torch::Tensor;

int act_code(const Tensor &t) { return t.scalar_type() == at::kBFloat16 ? FLUTE_BF16 : FLUTE_F16; }
bool is_act(const Tensor &t) {
    return t.scalar_type() == at::kHalf || t.scalar_type() == at::kBFloat16;
}
// the name Python prints for a dtype
const char *dtype_name(const Tensor &t) {
    switch (t.scalar_type()) {
        case at::kBFloat16: return "torch.bfloat16";
        case at::kHalf: return "torch.float16";
        case at::kFloat: return "torch.float32";
        case at::kDouble: return "torch.float64";
        case at::kByte: return "torch.uint8";
        case at::kChar: return "torch.int8";
        case at::kShort: return "torch.int16";
        case at::kInt: return "torch.int32";
        case at::kLong: return "torch.int64";
        case at::kBool: return "torch.bool";
        default: return c10::toString(t.scalar_type());
    }
}

void *stream_of(const Tensor &t) {
    return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}
Tensor aligned16(const Tensor &t) {
    // fresh allocations are 256-byte aligned; views and slices may not be
    return ((uintptr_t)t.data_ptr() % 16 == 0) ? t : t.clone();
}
void check_status(flute_status st) {
    TORCH_CHECK(st == FLUTE_OK, flute_last_error());
}

struct Shape2 {
    int64_t M, K;
};

// What the library's argument checks need to know about a tensor (flute_tensor): no tensor
// type crosses the C ABI.  `name` keeps the printed dtype alive for the duration of the call.
struct Record {
    flute_tensor t = {};
    std::string name;
};
void record(Record &r, const Tensor *t) {
    if (t == nullptr || !t->defined()) {
        r.t.present = 0;
        return;
    }
    r.t.present = 1;
    r.t.numel = t->numel();
    r.t.ndim = (int32_t)t->dim();
    for (int64_t i = 0; i < t->dim() && i < 4; ++i) r.t.size[i] = t->size(i);
    switch (t->scalar_type()) {
        case at::kHalf: r.t.dtype = FLUTE_F16; break;
        case at::kBFloat16: r.t.dtype = FLUTE_BF16; break;
        case at::kFloat: r.t.dtype = FLUTE_F32; break;
        case at::kByte: r.t.dtype = FLUTE_U8; break;
        default:
            r.t.dtype = -1;
            r.name = dtype_name(*t);
            r.t.dtype_name = r.name.c_str();
    }
    r.t.contiguous = t->is_contiguous() ? 1 : 0;
    r.t.device = t->is_cuda() ? (int32_t)t->device().index() : -1;
    r.t.data = t->numel() ? t->data_ptr() : nullptr;
}

// The checks of the input matrix: flute_check_input (one copy for this binding and the ctypes
// mirror).
Shape2 check_2d_input(const char *who, const Tensor &A, bool need_m1) {
    Record r;
    record(r, &A);
    check_status(flute_check_input(who, &r.t, need_m1 ? 1 : 0));
    return {A.size(0), A.size(1)};
}

struct Described {
    flute_linear w;
    int64_t N;
    Tensor keep1, keep2;    // re-aligned blobs, alive until the launch is queued
};

uint32_t gs_mask(const std::vector<int> &allowed) {
    uint32_t m = 0;
    for (int g : allowed) m |= 1u << (31 - __builtin_clz((unsigned)g));
    return m;
}

const std::vector<int> kGsAll = {16, 32, 64, 128, 256, 512, 1024, 2048};
const std::vector<int> kGsPlain = {64, 128, 256, 512, 1024, 2048};

// The checks of one weight's tensors: flute_describe_linear; this function records what it was
// handed and re-aligns blobs that torch may hand over as views.
Described describe(const char *who, const Tensor &A, int64_t K, const Tensor &indices,
                   const Tensor &lut, int64_t b1, const Tensor &indices2, const Tensor &lut2,
                   int64_t b2, const Tensor &resB, const Tensor &resA, const Tensor &bias,
                   int64_t gs, const c10::optional<Tensor> &signs, c10::optional<Tensor> awq,
                   int64_t rot_block, const std::vector<int> &gs_allowed, int64_t max_rank) {
    Described d;
    d.keep1 = (indices.defined() && indices.is_cuda()) ? aligned16(indices) : indices;
    d.keep2 = (b2 > 0 && indices2.defined() && indices2.is_cuda()) ? aligned16(indices2) : indices2;
    Record rA, rI, rL, rI2, rL2, rRB, rRA, rBias, rS, rAwq;
    record(rA, &A);
    record(rI, &d.keep1);
    record(rL, &lut);
    record(rI2, &d.keep2);
    record(rL2, &lut2);
    record(rRB, &resB);
    record(rRA, &resA);
    record(rBias, &bias);
    record(rS, signs.has_value() ? &*signs : nullptr);
    record(rAwq, awq.has_value() ? &*awq : nullptr);
    flute_operands ops = {};
    ops.A = rA.t;
    ops.indices = rI.t;
    ops.lut = rL.t;
    ops.indices2 = rI2.t;
    ops.lut2 = rL2.t;
    ops.resB = rRB.t;
    ops.resA = rRA.t;
    ops.bias = rBias.t;
    ops.signs = rS.t;
    ops.awq = rAwq.t;
    ops.K = K;
    ops.b1 = (int32_t)b1;
    ops.b2 = (int32_t)b2;
    ops.group_size = (gs >= INT32_MIN && gs <= INT32_MAX) ? (int32_t)gs : -1;
    ops.rot_block = (int32_t)rot_block;
    ops.max_rank = (int32_t)max_rank;
    ops.gs_allowed = gs_mask(gs_allowed);
    check_status(flute_describe_linear(who, &ops, &d.w, &d.N));
    return d;
}

Tensor gemv(const char *who, const Tensor &A_in, const Tensor &indices, const Tensor &lut,
            int64_t b1, const Tensor &indices2, const Tensor &lut2, int64_t b2, const Tensor &resB,
            const Tensor &resA, const Tensor &bias, int64_t gs,
            const c10::optional<Tensor> &signs, const c10::optional<Tensor> &awq, int64_t split,
            int64_t rot_block, const std::vector<int> &gs_allowed, int64_t max_rank) {
    const Shape2 s = check_2d_input(who, A_in, true);
    if (s.K == 0 || indices.numel() == 0) {
        // degenerate shapes never reach the device (src/kernel_gemv.cu:456-461 upstream)
        const int64_t N = (s.K == 0 && lut.dim() == 2) ? lut.size(0) * gs : 0;
        return torch::zeros({1, N}, A_in.options());
    }
    Described d = describe(who, A_in, s.K, indices, lut, b1, indices2, lut2, b2, resB, resA, bias,
                           gs, signs, awq, rot_block, gs_allowed, max_rank);
    const Tensor A = aligned16(A_in);
    c10::DeviceGuard guard(A.device());
    Tensor C = torch::empty({1, d.N}, A.options());
    check_status(flute_gemv(&d.w, A.data_ptr(), C.data_ptr(), act_code(A), (int)split, stream_of(A)));
    return C;
}

Tensor gemm(const char *who, const Tensor &A_in, const Tensor &indices, const Tensor &lut,
            int64_t b1, const Tensor &indices2, const Tensor &lut2, int64_t b2, const Tensor &resB,
            const Tensor &resA, const Tensor &bias, int64_t gs) {
    const Shape2 s = check_2d_input(who, A_in, false);
    if (s.K == 0 || s.M == 0 || indices.numel() == 0) {
        const int64_t rb = (s.K * b1) / 8;
        const int64_t N = s.K == 0 ? 0 : indices.numel() / (rb > 1 ? rb : 1);
        return torch::zeros({s.M, N}, A_in.options());
    }
    Described d = describe(who, A_in, s.K, indices, lut, b1, indices2, lut2, b2, resB, resA, bias,
                           gs, c10::nullopt, c10::nullopt, 0, kGsAll, 256);
    const Tensor A = aligned16(A_in);
    c10::DeviceGuard guard(A.device());
    Tensor C = torch::empty({s.M, d.N}, A.options());
    check_status(flute_gemm(&d.w, A.data_ptr(), C.data_ptr(), (int)s.M, s.K, d.N, act_code(A),
                            stream_of(A)));
    return C;
}

// ---- M = 1 GEMV family --------------------------------------------------------------

Tensor qgemm_gemv_stream(const Tensor &A, const Tensor &indices, const Tensor &lut, int64_t b1,
                         const Tensor &indices2, const Tensor &lut2, int64_t b2,
                         const Tensor &resB, const Tensor &resA, const Tensor &bias, int64_t gs) {
    return gemv("qgemm_gemv_stream", A, indices, lut, b1, indices2, lut2, b2, resB, resA, bias, gs,
                c10::nullopt, c10::nullopt, 0, 0, kGsPlain, 16);
}

Tensor qgemm_gemv_fht_stream(const Tensor &A, const Tensor &indices, const Tensor &lut, int64_t b1,
                             const Tensor &indices2, const Tensor &lut2, int64_t b2,
                             const Tensor &resB, const Tensor &resA, const Tensor &bias, int64_t gs,
                             const c10::optional<Tensor> &signs, const c10::optional<Tensor> &s) {
    return gemv("qgemm_gemv_fht_stream", A, indices, lut, b1, indices2, lut2, b2, resB, resA, bias,
                gs, signs, s, 0, 0, kGsPlain, 16);
}

Tensor qgemm_gemv_splitk_stream(const Tensor &A, const Tensor &indices, const Tensor &lut,
                                int64_t b1, const Tensor &indices2, const Tensor &lut2, int64_t b2,
                                const Tensor &resB, const Tensor &resA, const Tensor &bias,
                                int64_t gs, int64_t split) {
    return gemv("qgemm_gemv_splitk_stream", A, indices, lut, b1, indices2, lut2, b2, resB, resA,
                bias, gs, c10::nullopt, c10::nullopt, split, 0, kGsAll, 256);
}

Tensor qgemm_gemv_splitk_fht_stream(const Tensor &A, const Tensor &indices, const Tensor &lut,
                                    int64_t b1, const Tensor &indices2, const Tensor &lut2,
                                    int64_t b2, const Tensor &resB, const Tensor &resA,
                                    const Tensor &bias, int64_t gs,
                                    const c10::optional<Tensor> &signs,
                                    const c10::optional<Tensor> &s, int64_t split,
                                    int64_t rot_block) {
    return gemv("qgemm_gemv_splitk_fht_stream", A, indices, lut, b1, indices2, lut2, b2, resB, resA,
                bias, gs, signs, s, split, rot_block, kGsAll, 256);
}

// ---- segment-table entries -----------------------------------------------------------

constexpr int kSegCols = 15;   // q1 lut1 q2 lut2 resB resA bias C N R b1 b2 gs signs s

int64_t check_seg_inputs(const char *who, const Tensor &A, const Tensor &seg_table, int64_t rows) {
    TORCH_CHECK(A.dim() == 2 && A.size(0) == 1 && is_act(A) && A.is_contiguous(), who,
                ": A must be a contiguous [1, K] float16/bfloat16 tensor");
    TORCH_CHECK(seg_table.device().is_cpu() && seg_table.scalar_type() == at::kLong &&
                    seg_table.dim() == 2 && seg_table.size(1) == kSegCols,
                who, ": seg_table must be a CPU int64 [count, 15] tensor");
    const int64_t count = seg_table.size(0);
    TORCH_CHECK(rows < 0 || count == rows, who, ": seg_table must have ", rows, " rows (got ",
                count, ")");
    TORCH_CHECK(rows >= 0 || (count >= 1 && count <= 4), who,
                ": 1..4 segments per launch (got ", count, ")");
    return count;
}

void seg_descs(const char *who, const Tensor &A, const Tensor &seg_table, int lut_dtype,
               std::vector<flute_linear> &descs, std::vector<void *> &outs) {
    const int64_t K = A.size(1);
    const Tensor table = seg_table.contiguous();
    const int64_t *v = table.data_ptr<int64_t>();
    const int64_t count = table.size(0);
    descs.assign(count, flute_linear{});
    outs.assign(count, nullptr);
    static const char *names[] = {"q1", "q2", "resB", "resA", "signs", "s"};
    static const int cols[] = {0, 2, 4, 5, 13, 14};
    for (int64_t i = 0; i < count; ++i) {
        const int64_t *r = v + i * kSegCols;
        for (int c = 0; c < 6; ++c)
            TORCH_CHECK(r[cols[c]] % 16 == 0, who, ": segment ", i, " pointer ", names[c],
                        " must be 16-byte aligned");
        TORCH_CHECK(r[0] != 0 && r[1] != 0, who, ": segment ", i, " has no stream-1 indices/lut");
        TORCH_CHECK(r[12] > 0, who, ": segment ", i, " group_size must be positive");
        flute_linear &w = descs[i];
        const int64_t N = r[8], R = r[9], b1 = r[10], b2 = r[11], gs = r[12];
        w.q1 = (const void *)r[0];
        w.lut1 = (const void *)r[1];
        w.q2 = (const void *)r[2];
        w.lut2 = (const void *)r[3];
        w.resB = (const void *)r[4];
        w.resA = (const void *)r[5];
        w.bias = (const void *)r[6];
        w.signs = (const float *)r[13];
        w.awq = (const float *)r[14];
        w.N = (int)N;
        w.K = (int)K;
        w.R = (int)R;
        w.b1 = (int)b1;
        w.b2 = (int)b2;
        w.group_size = (int)gs;
        w.q1_bytes = N * K * b1 / 8;
        w.q2_bytes = N * K * b2 / 8;
        w.lut_rows = (int)((N + gs - 1) / gs);
        w.lut_dtype = lut_dtype;
        outs[i] = (void *)r[7];
    }
}

// lut_dtype: None (float16) or a torch.dtype
int lut_code(const pybind11::object &lut_dtype) {
    if (lut_dtype.is_none()) return FLUTE_F16;
    return lut_dtype.is(pybind11::module_::import("torch").attr("bfloat16")) ? FLUTE_BF16 : FLUTE_F16;
}

void qgemm_gemv_multi(const Tensor &A_in, const Tensor &seg_table,
                      const pybind11::object &lut_dtype, int64_t split) {
    const char *who = "qgemm_gemv_multi";
    check_seg_inputs(who, A_in, seg_table, -1);
    TORCH_CHECK(A_in.is_cuda(), who, ": A must be a CUDA (HIP) tensor");
    std::vector<flute_linear> descs;
    std::vector<void *> outs;
    seg_descs(who, A_in, seg_table, lut_code(lut_dtype), descs, outs);
    for (size_t i = 0; i < outs.size(); ++i)
        TORCH_CHECK(outs[i] != nullptr, who, ": segment ", i, " has no output pointer");
    const Tensor A = aligned16(A_in);
    c10::DeviceGuard guard(A.device());
    check_status(flute_gemv_multi(descs.data(), (int)descs.size(), A.data_ptr(), outs.data(),
                                  act_code(A), (int)split, stream_of(A)));
}

Tensor qgemm_gemv_mlp(const Tensor &A_in, const Tensor &seg_table, const Tensor &C,
                      const pybind11::object &lut_dtype, int64_t split) {
    const char *who = "qgemm_gemv_mlp";
    check_seg_inputs(who, A_in, seg_table, 2);
    TORCH_CHECK(C.scalar_type() == A_in.scalar_type() && C.is_contiguous(), who,
                ": C must be a contiguous ", dtype_name(A_in), " output buffer");
    const Tensor table = seg_table.contiguous();   // alive while v is read
    const int64_t *v = table.data_ptr<int64_t>();
    const int64_t N = v[8];
    TORCH_CHECK(v[kSegCols + 8] == N && C.numel() == N, who, ": gate/up/C must agree in N");
    TORCH_CHECK(A_in.is_cuda() && C.is_cuda(), who, ": A and C must be CUDA (HIP) tensors");
    TORCH_CHECK(C.device() == A_in.device(), who, ": C must live on A's device ",
                A_in.device().str());
    std::vector<flute_linear> descs;
    std::vector<void *> outs;
    seg_descs(who, A_in, seg_table, lut_code(lut_dtype), descs, outs);
    const Tensor A = aligned16(A_in);
    c10::DeviceGuard guard(A.device());
    check_status(flute_gemv_mlp(&descs[0], &descs[1], A.data_ptr(), C.data_ptr(), act_code(A),
                                (int)split, stream_of(A)));
    return C;
}

// ---- GEMM family ------------------------------------------------------------------------

Tensor qgemm_cutlass_streaming(const Tensor &A, const Tensor &indices, const Tensor &lut,
                               int64_t b1, int64_t gs, int64_t q_layout) {
    TORCH_CHECK(q_layout == 1, "qgemm_cutlass_streaming: only q_layout=1 (the idxN blob) is served");
    const Tensor e8 = torch::empty({0}, A.options().dtype(at::kByte));
    const Tensor e16 = torch::empty({0}, A.options());
    return gemm("qgemm_cutlass_streaming", A, indices, lut, b1, e8, e16, 0, e16, e16, e16, gs);
}

Tensor qgemm_dual_stream(const Tensor &A, const Tensor &indices, const Tensor &lut, int64_t b1,
                         const Tensor &indices2, const Tensor &lut2, int64_t b2,
                         const Tensor &resB, const Tensor &resA, const Tensor &bias, int64_t gs) {
    return gemm("qgemm_dual_stream", A, indices, lut, b1, indices2, lut2, b2, resB, resA, bias, gs);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    namespace py = pybind11;
    m.doc() = "compiled PyTorch-ROCm binding of the idxN LUT linear layer (libflute_hip.so)";
    m.def("abi_version", []() { return flute_abi_version(); });
    m.def("qgemm_gemv_stream", &qgemm_gemv_stream);
    m.def("qgemm_gemv_fht_stream", &qgemm_gemv_fht_stream);
    m.def("qgemm_gemv_splitk_stream", &qgemm_gemv_splitk_stream, py::arg("A"), py::arg("indices"),
          py::arg("lut"), py::arg("bitwidth"), py::arg("indices2"), py::arg("lut2"),
          py::arg("bitwidth2"), py::arg("resB"), py::arg("resA"), py::arg("bias"),
          py::arg("group_size"), py::arg("split") = 0);
    m.def("qgemm_gemv_splitk_fht_stream", &qgemm_gemv_splitk_fht_stream, py::arg("A"),
          py::arg("indices"), py::arg("lut"), py::arg("bitwidth"), py::arg("indices2"),
          py::arg("lut2"), py::arg("bitwidth2"), py::arg("resB"), py::arg("resA"), py::arg("bias"),
          py::arg("group_size"), py::arg("signs"), py::arg("s"), py::arg("split") = 0,
          py::arg("rot_block") = 0);
    m.def("qgemm_gemv_multi", &qgemm_gemv_multi, py::arg("A"), py::arg("seg_table"),
          py::arg("lut_dtype") = py::none(), py::arg("split") = 0);
    m.def("qgemm_gemv_mlp", &qgemm_gemv_mlp, py::arg("A"), py::arg("seg_table"), py::arg("C"),
          py::arg("lut_dtype") = py::none(), py::arg("split") = 0);
    m.def("qgemm_cutlass_streaming", &qgemm_cutlass_streaming, py::arg("A"), py::arg("indices"),
          py::arg("lut"), py::arg("bitwidth"), py::arg("group_size"), py::arg("q_layout") = 1);
    m.def("qgemm_dual_stream", &qgemm_dual_stream, py::arg("A"), py::arg("indices"), py::arg("lut"),
          py::arg("bitwidth"), py::arg("indices2"), py::arg("lut2"), py::arg("bitwidth2"),
          py::arg("resB"), py::arg("resA"), py::arg("bias"), py::arg("group_size") = 512);
}
