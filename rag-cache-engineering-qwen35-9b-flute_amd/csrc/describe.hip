// The argument checks of one weight's operands as a binding sees them (shapes, dtypes,
// contiguity, devices), in one place: the ctypes mirror (flute_extended/_C.py) and the compiled
// PyTorch binding (torch_binding.cpp) both marshal their tensors into flute_tensor records and
// call this, so the checks, their order and their messages exist once.  They are the checks of
// upstream's bindings (src/bindings.cpp:230-546, src/kernel_gemv.cu:379-474): "absent" operands
// are empty tensors, N comes from the blob's byte count, every violation is an error with a
// message.  Host code only.
#include <string>

#include "host_common.h"

namespace flute {

namespace {

bool is_act(const flute_tensor &t) { return t.dtype == FLUTE_F16 || t.dtype == FLUTE_BF16; }
bool populated(const flute_tensor &t) { return t.present && t.numel > 0; }

// the name Python prints for a dtype
std::string dtype_name(const flute_tensor &t) {
    if (t.dtype_name) return t.dtype_name;
    switch (t.dtype) {
        case FLUTE_F16: return "torch.float16";
        case FLUTE_BF16: return "torch.bfloat16";
        case FLUTE_F32: return "torch.float32";
        case FLUTE_U8: return "torch.uint8";
        default: return "another dtype";
    }
}
// a shape as Python prints a tuple
std::string shape_of(const flute_tensor &t) {
    std::string s = "(";
    for (int i = 0; i < t.ndim && i < 4; ++i) s += (i ? ", " : "") + std::to_string((long long)t.size[i]);
    if (t.ndim == 1) s += ",";
    return s + ")";
}
std::string gs_list(uint32_t mask) {
    std::string s;
    for (int i = 0; i < 32; ++i)
        if (mask & (1u << i)) s += (s.empty() ? "" : "/") + std::to_string(1u << i);
    return s;
}
bool gs_in(int64_t gs, uint32_t mask) {
    return gs > 0 && gs < ((int64_t)1 << 31) && (gs & (gs - 1)) == 0 &&
           (mask & (1u << __builtin_ctzll((unsigned long long)gs)));
}

}  // namespace

}  // namespace flute

using namespace flute;

#define FLUTE_REFUSE(cond, ...) FLUTE_REQUIRE(cond, FLUTE_ERR_INVALID, __VA_ARGS__)

extern "C" flute_status flute_check_input(const char *who, const flute_tensor *A, int need_m1) {
    FLUTE_REFUSE(who && A, "flute_check_input: NULL argument");
    FLUTE_REFUSE(A->ndim == 2, "%s: A must be 2-D [M, K]", who);
    FLUTE_REFUSE(is_act(*A), "%s: A must be float16 or bfloat16 (got %s)", who, dtype_name(*A).c_str());
    const long long M = A->size[0], K = A->size[1];
    FLUTE_REFUSE(!need_m1 || M == 1,
                 "%s: the decode GEMV serves M == 1 (got M=%lld) - route larger M through "
                 "qgemm_dual_stream / qgemm_per_group_lut", who, M);
    FLUTE_REFUSE(K % 64 == 0, "%s: K must be a multiple of 64 (the idxN blob's 64-k tiles; got K=%lld)",
                 who, K);
    FLUTE_REFUSE(A->contiguous, "%s: A must be contiguous", who);
    return FLUTE_OK;
}

extern "C" flute_status flute_describe_linear(const char *who, const flute_operands *ops,
                                              flute_linear *out, int64_t *N_out) {
    FLUTE_REFUSE(who && ops && out && N_out, "flute_describe_linear: NULL argument");
    const flute_tensor &A = ops->A, &indices = ops->indices, &lut = ops->lut, &indices2 = ops->indices2,
                       &lut2 = ops->lut2, &resB = ops->resB, &resA = ops->resA, &bias = ops->bias,
                       &signs = ops->signs, &awq = ops->awq;
    const long long K = ops->K, b1 = ops->b1, b2 = ops->b2, gs = ops->group_size;
    const std::string act = dtype_name(A);
    FLUTE_REFUSE(b1 >= 1 && b1 <= 4, "%s: bitwidth must be 1, 2, 3 or 4 (got %lld)", who, b1);
    FLUTE_REFUSE(b2 >= 0 && b2 <= 4, "%s: bitwidth2 must be 0 (single stream) or 1..4 (got %lld)", who, b2);
    FLUTE_REFUSE(gs_in(gs, ops->gs_allowed), "%s: group_size must be one of %s (got %lld)", who,
                 gs_list(ops->gs_allowed).c_str(), gs);
    FLUTE_REFUSE(indices.dtype == FLUTE_U8, "%s: stream-1 indices must be uint8", who);
    FLUTE_REFUSE(is_act(lut), "%s: stream-1 lut must be float16 (or bfloat16 with bfloat16 activations)", who);
    FLUTE_REFUSE(!(lut.dtype == FLUTE_BF16 && A.dtype != FLUTE_BF16),
                 "%s: a bfloat16 lut needs bfloat16 activations", who);
    const long long row_bytes1 = (K * b1) / 8;
    FLUTE_REFUSE(K != 0, "%s: K == 0 reaches the kernel path", who);
    const long long N = row_bytes1 > 0 ? indices.numel / row_bytes1 : 0;
    FLUTE_REFUSE(N > 0 && N * row_bytes1 == indices.numel,
                 "%s: stream-1 byte count %lld is not N*(K*%lld/8) for any N (K = %lld)", who,
                 (long long)indices.numel, b1, K);
    FLUTE_REFUSE(N % 128 == 0, "%s: idxN layout requires N %% 128 == 0 (got N = %lld)", who, N);
    const long long rows = (N + gs - 1) / gs;
    FLUTE_REFUSE(lut.ndim == 2 && lut.size[0] == rows && lut.size[1] == (1 << b1),
                 "%s: stream-1 lut must be [ceil(N/group_size), 2^bitwidth] = [%lld, %d] (got %s)", who,
                 rows, 1 << b1, shape_of(lut).c_str());
    FLUTE_REFUSE(indices.contiguous && lut.contiguous, "%s: stream-1 indices and lut must be contiguous", who);
    const bool has_s2 = b2 > 0;
    if (has_s2) {
        FLUTE_REFUSE(indices2.dtype == FLUTE_U8, "%s: stream-2 indices must be uint8", who);
        FLUTE_REFUSE(lut2.dtype == lut.dtype, "%s: stream-2 lut must have the dtype of stream 1 (%s)", who,
                     dtype_name(lut).c_str());
        FLUTE_REFUSE(indices2.numel == N * ((K * b2) / 8), "%s: stream-2 byte count %lld != N*K*%lld/8 = %lld",
                     who, (long long)indices2.numel, b2, N * ((K * b2) / 8));
        FLUTE_REFUSE(lut2.ndim == 2 && lut2.size[0] == rows && lut2.size[1] == (1 << b2),
                     "%s: stream-2 lut must be [ceil(N/group_size), 2^bitwidth2] = [%lld, %d] (got %s)", who,
                     rows, 1 << b2, shape_of(lut2).c_str());
        FLUTE_REFUSE(indices2.contiguous && lut2.contiguous, "%s: stream-2 indices/lut must be contiguous", who);
    }
    const bool has_res = populated(resB);
    FLUTE_REFUSE(has_res == populated(resA),
                 "%s: resB and resA must be supplied together (both empty or both populated)", who);
    long long R = 0;
    if (has_res) {
        FLUTE_REFUSE(resB.dtype == A.dtype && resA.dtype == A.dtype,
                     "%s: resB/resA must have the activation dtype %s", who, act.c_str());
        FLUTE_REFUSE(resB.ndim == 2 && resA.ndim == 2, "%s: resB must be (R, K) and resA (N, R)", who);
        R = resB.size[0];
        FLUTE_REFUSE(R >= 1 && R <= ops->max_rank, "%s: residual rank must be 1..%d (got R=%lld)", who,
                     ops->max_rank, R);
        FLUTE_REFUSE(resB.size[1] == K && resA.size[0] == N && resA.size[1] == R,
                     "%s: residual shape mismatch: resB %s, resA %s for N=%lld, K=%lld", who,
                     shape_of(resB).c_str(), shape_of(resA).c_str(), N, K);
        FLUTE_REFUSE(resB.contiguous && resA.contiguous, "%s: resB/resA must be contiguous", who);
    }
    const bool has_bias = populated(bias);
    if (has_bias)
        FLUTE_REFUSE(bias.dtype == A.dtype && bias.ndim == 1 && bias.size[0] == N && bias.contiguous,
                     "%s: bias must be a contiguous (N,) %s tensor (N=%lld)", who, act.c_str(), N);
    const bool has_signs = signs.present != 0;
    if (has_signs)
        FLUTE_REFUSE(signs.dtype == FLUTE_F32 && signs.ndim == 1 && signs.numel == K && signs.contiguous,
                     "%s: signs must be a contiguous (K,) float32 vector (K=%lld)", who, K);
    const bool has_awq = populated(awq);
    if (has_awq) {
        FLUTE_REFUSE(has_signs, "%s: awq scale without rotation signs", who);
        FLUTE_REFUSE(awq.dtype == FLUTE_F32 && awq.ndim == 1 && awq.numel == K && awq.contiguous,
                     "%s: awq scale must be a contiguous (K,) float32 vector (K=%lld)", who, K);
    }

    // ---- device ----------------------------------------------------------------------
    const flute_tensor *tensors[10];
    int count = 0;
    tensors[count++] = &A;
    tensors[count++] = &indices;
    tensors[count++] = &lut;
    if (has_s2) {
        tensors[count++] = &indices2;
        tensors[count++] = &lut2;
    }
    if (has_res) {
        tensors[count++] = &resB;
        tensors[count++] = &resA;
    }
    if (has_bias) tensors[count++] = &bias;
    if (has_signs) tensors[count++] = &signs;
    if (has_awq) tensors[count++] = &awq;
    for (int i = 0; i < count; ++i) {
        FLUTE_REFUSE(tensors[i]->device >= 0, "%s: all tensors must be CUDA (HIP) tensors", who);
        FLUTE_REFUSE(tensors[i]->device == A.device, "%s: all tensors must live on A's device cuda:%d", who,
                     A.device);
    }

    flute_linear w = {};
    w.q1 = indices.data;
    w.lut1 = lut.data;
    w.q1_bytes = indices.numel;
    if (has_s2) {
        w.q2 = indices2.data;
        w.lut2 = lut2.data;
        w.q2_bytes = indices2.numel;
    }
    if (has_res) {
        w.resB = resB.data;
        w.resA = resA.data;
    }
    if (has_bias) w.bias = bias.data;
    if (has_signs) w.signs = (const float *)signs.data;
    if (has_awq) w.awq = (const float *)awq.data;
    w.lut_rows = (int32_t)rows;
    w.N = (int32_t)N;
    w.K = (int32_t)K;
    w.R = (int32_t)R;
    w.b1 = (int32_t)b1;
    w.b2 = (int32_t)b2;
    w.group_size = (int32_t)gs;
    w.lut_dtype = lut.dtype == FLUTE_BF16 ? FLUTE_BF16 : FLUTE_F16;
    w.rot_block = ops->rot_block;
    *out = w;
    *N_out = N;
    return FLUTE_OK;
}
