// Embedding rows out of a palettized table: a gather through the idxN layout, the
// second stream, the low-rank residual and the un-rotation of tied (rotated) tables,
// in the dtype ladder of the upstream module (scripts/palettized_modules.py:1998-2015,
// 2298-2335):
//     w   = lut1[n / gs][idx1[n, :]]  (+ lut2[...] in the LUT's 16-bit type, stream 1 first)
//     row = float(w) + resA[n, :] @ resB                (fp32)
//     row = row @ T^T  when the table is rotated          (adjoint transform, fp32)
//     out = row rounded once to the LUT's type
#include "fht_dev.h"
#include "host_common.h"

#include <atomic>

namespace flute {

namespace {

constexpr int kEmbThreads = 256;

struct EmbParams {
    const uint8_t *q[2];
    const uint16_t *lut[2];
    const uint16_t *resA, *resB;
    const float *signs;
    const int64_t *ids;
    uint16_t *out;
    int bits[2];
    int nstreams;
    int N, K, gs, lut_rows, R;
    int bf16;        // LUT / output / residual dtype
    int block;       // rotation block (0: descending power-of-two segments)
};

// The two values of logical pair (n, k), k even, of one stream.
__device__ __forceinline__ void pair_values(const uint8_t *q, const uint16_t *lut, int b, int G,
                                            int n, int k, int grp, uint32_t &e0, uint32_t &e1) {
    const int t = n >> 7, r = n & 127;
    const int wx = r >> 6, v = (r >> 4) & 3, d = (r >> 3) & 1, r8 = r & 7;
    const int g = k >> 6, kk = k & 63;
    const int kt = kk >> 4, s2 = (kk >> 3) & 1, c4 = (kk >> 1) & 3;
    const int th = wx * 32 + r8 * 4 + c4;
    const int p = kt * 16 + v * 4 + d * 2 + s2;
    const uint8_t *chunk = q + (((size_t)t * G + g) * 64 + th) * (16 * b);
    const int bit = 2 * b * p, byte = bit >> 3;
    uint32_t w = chunk[byte];
    if (byte + 1 < 16 * b) w |= (uint32_t)chunk[byte + 1] << 8;
    const uint32_t code = (w >> (bit & 7)) & ((1u << (2 * b)) - 1u);
    const uint16_t *row = lut + ((size_t)grp << b);
    e0 = row[code & ((1u << b) - 1u)];
    e1 = row[code >> b];
}

__device__ __forceinline__ float to_f(uint32_t h, int bf16) {
    return bf16 ? bf2f((uint16_t)h) : h2f((uint16_t)h);
}

// One workgroup per requested row.
__global__ void __launch_bounds__(kEmbThreads) embedding_kernel(const EmbParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    float *buf = (float *)lds;
    const int tid = threadIdx.x;
    const int64_t n64 = p.ids[blockIdx.x];
    uint16_t *out = p.out + (size_t)blockIdx.x * p.K;
    if (n64 < 0 || n64 >= p.N) {                  // refused on the host; never read out of range
        for (int k = tid; k < p.K; k += kEmbThreads) out[k] = 0;
        return;
    }
    const int n = (int)n64;
    const int G = p.K >> 6;
    const int grp = min(n / p.gs, p.lut_rows - 1);

    auto pair_row = [&](int k, float &f0, float &f1) {
        uint32_t a0, a1;
        pair_values(p.q[0], p.lut[0], p.bits[0], G, n, k, grp, a0, a1);
        f0 = to_f(a0, p.bf16);
        f1 = to_f(a1, p.bf16);
        if (p.nstreams == 2) {
            uint32_t b0, b1;
            pair_values(p.q[1], p.lut[1], p.bits[1], G, n, k, grp, b0, b1);
            // the 16-bit add of the module: exact sum, one rounding to the LUT's type
            f0 = to_f(round_act(f0 + to_f(b0, p.bf16), p.bf16), p.bf16);
            f1 = to_f(round_act(f1 + to_f(b1, p.bf16), p.bf16), p.bf16);
        }
        if (p.R > 0) {
            float r0 = 0.0f, r1 = 0.0f;
            for (int r = 0; r < p.R; ++r) {
                const float a = to_f(p.resA[(size_t)n * p.R + r], p.bf16);
                r0 = fmaf(a, to_f(p.resB[(size_t)r * p.K + k], p.bf16), r0);
                r1 = fmaf(a, to_f(p.resB[(size_t)r * p.K + k + 1], p.bf16), r1);
            }
            f0 += r0;
            f1 += r1;
        }
    };

    if (p.signs == nullptr) {
        for (int k = tid * 2; k < p.K; k += kEmbThreads * 2) {
            float f0, f1;
            pair_row(k, f0, f1);
            *(uint32_t *)(out + k) =
                (uint32_t)round_act(f0, p.bf16) | ((uint32_t)round_act(f1, p.bf16) << 16);
        }
        return;
    }
    // rotated table: the adjoint transform of the row, segment by segment
    for (int off = 0; off < p.K;) {
        int count, nst;
        if (p.block > 0) {
            nst = 31 - __builtin_clz((unsigned)p.block);
            count = min((16384 / p.block) * p.block, p.K - off);
        } else {
            nst = 31 - __builtin_clz((unsigned)(p.K - off));
            count = 1 << nst;
        }
        for (int j = tid * 2; j < count; j += kEmbThreads * 2) {
            float f0, f1;
            pair_row(off + j, f0, f1);
            buf[fht_slot(j)] = f0 * p.signs[off + j];
            buf[fht_slot(j + 1)] = f1 * p.signs[off + j + 1];
        }
        __syncthreads();
        fht_lds(buf, count, nst, tid, kEmbThreads);
        const float inv = inv_sqrt_pow2(nst);
        for (int j = tid * 2; j < count; j += kEmbThreads * 2)
            *(uint32_t *)(out + off + j) =
                (uint32_t)round_act(buf[fht_slot(j)] * inv, p.bf16) |
                ((uint32_t)round_act(buf[fht_slot(j + 1)] * inv, p.bf16) << 16);
        __syncthreads();
        off += count;
    }
}

}  // namespace

}  // namespace flute

using namespace flute;

extern "C" flute_status flute_embedding(const flute_linear *w, const int64_t *ids, int64_t count,
                                        void *out, void *stream) {
    flute_status st = validate_linear(w, 1, "flute_embedding");
    if (st != FLUTE_OK) return st;
    FLUTE_REQUIRE(count >= 0 && count <= 0x7fffffffLL, FLUTE_ERR_INVALID,
                  "flute_embedding: count must be in [0, 2^31)");
    if (count == 0) return FLUTE_OK;
    FLUTE_REQUIRE(ids != nullptr && out != nullptr, FLUTE_ERR_INVALID,
                  "flute_embedding: ids and out must not be NULL");
    FLUTE_REQUIRE(w->bias == nullptr, FLUTE_ERR_INVALID, "flute_embedding: an embedding has no bias");
    FLUTE_REQUIRE(w->awq == nullptr, FLUTE_ERR_INVALID,
                  "flute_embedding: an embedding table carries no activation scale");
    FLUTE_REQUIRE(((uintptr_t)ids & 7) == 0, FLUTE_ERR_INVALID,
                  "flute_embedding: ids are int64 and must be 8-byte aligned");
    FLUTE_REQUIRE(((uintptr_t)out & 3) == 0, FLUTE_ERR_INVALID,
                  "flute_embedding: out must be 4-byte aligned");
    EmbParams p = {};
    p.q[0] = (const uint8_t *)w->q1;
    p.q[1] = (const uint8_t *)w->q2;
    p.lut[0] = (const uint16_t *)w->lut1;
    p.lut[1] = (const uint16_t *)w->lut2;
    p.bits[0] = w->b1;
    p.bits[1] = w->b2;
    p.nstreams = w->b2 > 0 ? 2 : 1;
    p.resA = (const uint16_t *)w->resA;
    p.resB = (const uint16_t *)w->resB;
    p.R = w->R;
    p.signs = w->signs;
    p.ids = ids;
    p.out = (uint16_t *)out;
    p.N = w->N;
    p.K = w->K;
    p.gs = w->group_size;
    p.lut_rows = w->lut_rows;
    p.bf16 = w->lut_dtype == FLUTE_BF16;
    p.block = w->rot_block;
    size_t lds = 0;
    if (w->signs) {
        if (w->rot_block > 0) {
            FLUTE_REQUIRE(is_pow2(w->rot_block) && w->rot_block >= 32 && w->rot_block <= 16384 &&
                              w->K % w->rot_block == 0,
                          FLUTE_ERR_INVALID,
                          "flute_embedding: rotation block must be a power of two in [32, 16384] "
                          "dividing K");
            lds = (size_t)(w->K <= 16384 ? w->K : (16384 / w->rot_block) * w->rot_block) * 4;
        } else {
            lds = (size_t)make_segments(w->K, 0).len[0] * 4;
        }
        static std::atomic<bool> attr_done{false};   // threads may race to the first call: the call is idempotent
        if (!attr_done) {
            FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)embedding_kernel,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
            attr_done = true;
        }
    }
    hipLaunchKernelGGL(embedding_kernel, dim3((unsigned)count), dim3(kEmbThreads), lds,
                       (hipStream_t)stream, p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}
