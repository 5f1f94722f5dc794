// Standalone Walsh-Hadamard rotation: one workgroup per row, the butterfly of
// fht_dev.h in LDS, fp32 throughout, one rounding to the I/O type.
#include "fht_dev.h"
#include "host_common.h"

#include <atomic>

#include <cmath>

namespace flute {

namespace {

constexpr int kFhtThreads = 256;

struct FhtParams {
    const void *x;
    void *out;
    const float *signs;
    const float *awq;
    int K;
    int dtype;      // flute_dtype of x and out
    int adjoint;
    int block;      // > 0: equal blocks
    int chunk;      // columns transformed per pass in block mode
};

__device__ __forceinline__ float load_any(const void *p, int64_t i, int dtype) {
    if (dtype == FLUTE_F32) return ((const float *)p)[i];
    return load_act(p, i, dtype == FLUTE_BF16);
}
__device__ __forceinline__ void store_any(void *p, int64_t i, int dtype, float v) {
    if (dtype == FLUTE_F32) ((float *)p)[i] = v;
    else ((uint16_t *)p)[i] = round_act(v, dtype == FLUTE_BF16);
}

// forward:  out = ((x [*awq]) @ H) * signs * inv [/ awq]   (fht.py:206-222, 646-651 upstream)
// adjoint:  out = ((x * signs) @ H) * inv                  (fht.py:225-238 upstream)
__global__ void __launch_bounds__(kFhtThreads) fht_kernel(const FhtParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    float *buf = (float *)lds;
    const int tid = threadIdx.x;
    const int64_t row = (int64_t)blockIdx.x * p.K;
    // block mode: chunks of whole blocks; otherwise the descending power-of-two
    // segments of K (fht.py:118-134 upstream)
    for (int off = 0; off < p.K;) {
        int count, nstages;
        if (p.block > 0) {
            count = min(p.chunk, p.K - off);
            nstages = 31 - __builtin_clz((unsigned)p.block);
        } else {
            nstages = 31 - __builtin_clz((unsigned)(p.K - off));
            count = 1 << nstages;
        }
        const float inv = inv_sqrt_pow2(nstages);
        // Eight columns per thread and step; the loads of a step (row, signs, scale) are
        // independent and issued together, so each phase is one memory round trip.
#pragma unroll 2
        for (int j = tid * 8; j < count; j += kFhtThreads * 8) {
            float f[8], m[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) f[q] = load_any(p.x, row + off + j + q, p.dtype);
            if (p.adjoint || p.awq) {
                const float *mul = p.adjoint ? p.signs : p.awq;
#pragma unroll
                for (int q = 0; q < 8; ++q) m[q] = mul[off + j + q];
#pragma unroll
                for (int q = 0; q < 8; ++q) f[q] *= m[q];
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) buf[fht_slot(j + q)] = f[q];
        }
        __syncthreads();
        fht_lds(buf, count, nstages, tid, kFhtThreads);
#pragma unroll 2
        for (int j = tid * 8; j < count; j += kFhtThreads * 8) {
            float sg[8], sc[8];
            if (!p.adjoint) {
#pragma unroll
                for (int q = 0; q < 8; ++q) sg[q] = p.signs[off + j + q];
                if (p.awq) {
#pragma unroll
                    for (int q = 0; q < 8; ++q) sc[q] = p.awq[off + j + q];
                }
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                float t = buf[fht_slot(j + q)];
                if (p.adjoint) {
                    t = t * inv;
                } else {
                    t = t * sg[q] * inv;
                    if (p.awq) t = t / sc[q];
                }
                store_any(p.out, row + off + j + q, p.dtype, t);
            }
        }
        __syncthreads();
        off += count;
    }
}

}  // namespace

}  // namespace flute

using namespace flute;

extern "C" flute_status flute_fht(const void *x, const float *signs, const float *awq, void *out,
                                  int M, int K, int dtype, int adjoint, int block, void *stream) {
    FLUTE_REQUIRE(x && out && signs, FLUTE_ERR_INVALID, "flute_fht: x, signs and out must not be NULL");
    FLUTE_REQUIRE(dtype == FLUTE_F16 || dtype == FLUTE_BF16 || dtype == FLUTE_F32, FLUTE_ERR_INVALID,
                  "flute_fht: dtype must be float16, bfloat16 or float32");
    FLUTE_REQUIRE(M >= 0, FLUTE_ERR_INVALID, "flute_fht: M must be >= 0");
    FLUTE_REQUIRE(K >= 32 && K % 32 == 0 && K <= 65504, FLUTE_ERR_INVALID,
                  "flute_fht: K must be a multiple of 32 in [32, 65504] (got %d)", K);
    FLUTE_REQUIRE(!(awq && adjoint), FLUTE_ERR_INVALID,
                  "flute_fht: the awq-compensated transform exists in the forward direction only");
    FhtParams p;
    p.x = x;
    p.out = out;
    p.signs = signs;
    p.awq = awq;
    p.K = K;
    p.dtype = dtype;
    p.adjoint = adjoint ? 1 : 0;
    p.block = block;
    p.chunk = 0;
    size_t lds_bytes;
    if (block > 0) {
        FLUTE_REQUIRE(is_pow2(block) && block >= 32 && block <= 16384 && K % block == 0,
                      FLUTE_ERR_INVALID,
                      "flute_fht: block must be a power of two in [32, 16384] dividing K (got %d)",
                      block);
        p.chunk = K <= 16384 ? K : (16384 / block) * block;
        lds_bytes = (size_t)p.chunk * 4;
    } else {
        const Segs segs = make_segments(K, 0);
        FLUTE_REQUIRE(segs.len[0] <= 16384, FLUTE_ERR_UNSUPPORTED,
                      "flute_fht: segment of %d columns exceeds the 16384-column LDS tile",
                      segs.len[0]);
        lds_bytes = (size_t)segs.len[0] * 4;
    }
    if (M == 0) return FLUTE_OK;
    static std::atomic<bool> attr_done{false};   // threads may race to the first call: the call is idempotent
    if (!attr_done) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)fht_kernel,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
        attr_done = true;
    }
    hipLaunchKernelGGL(fht_kernel, dim3(M), dim3(kFhtThreads), lds_bytes, (hipStream_t)stream, p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}
