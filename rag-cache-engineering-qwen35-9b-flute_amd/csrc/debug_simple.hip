// Scalar differential twin of the LUT GEMM: one thread per output element, no matrix
// cores, no LDS table, no tiling.  Every weight is decoded from its bit position and
// looked up in the LUT in global memory; the products are summed in fp32 in ascending k
// and rounded once.  It exists to check the fast kernels against an independent reading
// of the same bytes (the role of src/kernel_debug_simple.cu upstream, which stages
// scalars into the tensor-core path; here nothing at all is shared with the fast path).
#include "host_common.h"

namespace flute {

namespace {

struct SimpleParams {
    const uint8_t *q;      // logical packed rows [N, K*b/8] (layout 0) or idxN blob (layout 1)
    const uint16_t *lut;   // [lut_rows, 2^b]
    const uint16_t *A;     // [M, lda]
    uint16_t *C;           // [M, ldc]
    int64_t lda, ldc;
    int M, N, K, bits, gs, lut_rows, layout, lut_bf16, act_bf16;
};

// b-bit field at bit offset `bit` of a byte string (fields may straddle a byte).
__device__ __forceinline__ uint32_t field(const uint8_t *bytes, int64_t bit, int b) {
    const int64_t byte = bit >> 3;
    const int sh = (int)(bit & 7);
    uint32_t v = bytes[byte];
    if (sh + b > 8) v |= (uint32_t)bytes[byte + 1] << 8;
    return (v >> sh) & ((1u << b) - 1u);
}

// Code of element (n, k).  Logical rows: LSB-first along k (docs/QUANTIZATION.md:40-51
// upstream).  idxN blob (flute_extended/idxN.py:37-55 upstream): tile (n/128, k/64) of
// 1024*b bytes, chunk th = wx*32 + lane of 16*b bytes, pair p at bit 2*b*p, where
//   n % 128 = wx*64 + v*16 + d*8 + (lane >> 2)
//   k % 64  = kt*16 + 2*(lane & 3) + 8*s2 + e,   p = kt*16 + v*4 + d*2 + s2.
__device__ __forceinline__ uint32_t code_of(const SimpleParams &p, int n, int k) {
    const int b = p.bits;
    if (p.layout == 0) return field(p.q + (int64_t)n * (p.K * b / 8), (int64_t)k * b, b);
    const int t = n >> 7, r = n & 127, g = k >> 6, kk = k & 63;
    const int wx = r >> 6, v = (r >> 4) & 3, d = (r >> 3) & 1, lane_hi = r & 7;
    const int kt = kk >> 4, s2 = (kk >> 3) & 1, lane_lo = (kk >> 1) & 3, e = kk & 1;
    const int th = wx * 32 + lane_hi * 4 + lane_lo;
    const int pair = kt * 16 + v * 4 + d * 2 + s2;
    const uint8_t *chunk = p.q + (((int64_t)t * (p.K >> 6) + g) * 64 + th) * (16 * b);
    return field(chunk, (int64_t)2 * b * pair + b * e, b);
}

__global__ void __launch_bounds__(256) debug_simple_kernel(const SimpleParams p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.M * p.N) return;
    const int m = (int)(idx / p.N), n = (int)(idx % p.N);
    const int row = min(n / p.gs, p.lut_rows - 1);
    const uint16_t *lr = p.lut + ((int64_t)row << p.bits);
    const uint16_t *a = p.A + (int64_t)m * p.lda;
    float acc = 0.0f;
    for (int k = 0; k < p.K; ++k) {
        const uint16_t wv = lr[code_of(p, n, k)];
        const float w = p.lut_bf16 ? bf2f(wv) : h2f(wv);
        const float x = p.act_bf16 ? bf2f(a[k]) : h2f(a[k]);
        acc = fmaf(x, w, acc);
    }
    p.C[(int64_t)m * p.ldc + n] = round_act(acc, p.act_bf16);
}

}  // namespace

}  // namespace flute

using namespace flute;

extern "C" flute_status flute_gemm_debug_simple(const void *q, int64_t q_bytes, int layout,
                                                const void *lut, int lut_rows, int lut_dtype,
                                                int bits, int group_size, int N, int K,
                                                const void *A, void *C, int M, int64_t lda,
                                                int64_t ldc, int act_dtype, void *stream) {
    const char *who = "flute_gemm_debug_simple";
    FLUTE_REQUIRE(bits >= 1 && bits <= 4, FLUTE_ERR_INVALID, "%s: bitwidth must be 1..4 (got %d)",
                  who, bits);
    FLUTE_REQUIRE(layout == 0 || layout == 1, FLUTE_ERR_INVALID,
                  "%s: layout must be 0 (logical packed rows) or 1 (idxN blob)", who);
    FLUTE_REQUIRE(N > 0 && K > 0 && (K * bits) % 8 == 0, FLUTE_ERR_INVALID,
                  "%s: N and K must be positive and K*bitwidth a whole number of bytes", who);
    FLUTE_REQUIRE(layout == 0 || (N % 128 == 0 && K % 64 == 0), FLUTE_ERR_INVALID,
                  "%s: the idxN layout requires N %% 128 == 0 and K %% 64 == 0 (got N=%d, K=%d)",
                  who, N, K);
    FLUTE_REQUIRE(q_bytes == (int64_t)N * K * bits / 8, FLUTE_ERR_INVALID,
                  "%s: %lld index bytes are not N*K*%d/8 = %lld", who, (long long)q_bytes, bits,
                  (long long)((int64_t)N * K * bits / 8));
    FLUTE_REQUIRE(is_pow2(group_size) && group_size >= 16 && group_size <= 2048, FLUTE_ERR_INVALID,
                  "%s: group_size must be one of 16/32/64/128/256/512/1024/2048 (got %d)", who,
                  group_size);
    FLUTE_REQUIRE(lut_rows == (N + group_size - 1) / group_size, FLUTE_ERR_INVALID,
                  "%s: lut must have ceil(N/group_size) = %d rows (got %d)", who,
                  (N + group_size - 1) / group_size, lut_rows);
    FLUTE_REQUIRE((lut_dtype == FLUTE_F16 || lut_dtype == FLUTE_BF16) &&
                      (act_dtype == FLUTE_F16 || act_dtype == FLUTE_BF16),
                  FLUTE_ERR_INVALID, "%s: lut and activations must be float16 or bfloat16", who);
    FLUTE_REQUIRE(M >= 0 && lda >= K && ldc >= N, FLUTE_ERR_INVALID,
                  "%s: M must be >= 0 and the row strides must cover a row", who);
    if (M == 0) return FLUTE_OK;
    FLUTE_REQUIRE(q && lut && A && C, FLUTE_ERR_INVALID, "%s: NULL operand", who);
    SimpleParams p;
    p.q = (const uint8_t *)q;
    p.lut = (const uint16_t *)lut;
    p.A = (const uint16_t *)A;
    p.C = (uint16_t *)C;
    p.lda = lda;
    p.ldc = ldc;
    p.M = M;
    p.N = N;
    p.K = K;
    p.bits = bits;
    p.gs = group_size;
    p.lut_rows = lut_rows;
    p.layout = layout;
    p.lut_bf16 = lut_dtype == FLUTE_BF16;
    p.act_bf16 = act_dtype == FLUTE_BF16;
    const int64_t total = (int64_t)M * N;
    FLUTE_REQUIRE((total + 255) / 256 <= 0x7fffffff, FLUTE_ERR_UNSUPPORTED, "%s: M*N exceeds the grid",
                  who);
    hipLaunchKernelGGL(debug_simple_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}
