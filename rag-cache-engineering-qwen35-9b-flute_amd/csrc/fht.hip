// Standalone Walsh-Hadamard rotation: one workgroup per row, the butterfly of
// fht_dev.h in LDS, fp32 throughout, one rounding to the I/O type.
#include "fht_dev.h"
#include "host_common.h"

#include <atomic>

#include <cmath>
#include <cstdlib>

namespace flute {

namespace {

constexpr int kFhtThreads = 256;

struct FhtParams {
    const void *x;
    void *out;
    const float *signs;
    const float *awq;
    int64_t ldx, ldo;   // row strides of x and out in elements
    int K;
    int dtype;      // flute_dtype of x and out
    int adjoint;
    int block;      // > 0: equal blocks
    int chunk;      // columns transformed per pass in block mode
    // Operand-order output for the LUT GEMM instead of rows (ap != NULL): the rotated row
    // m is rounded to `dtype`, converted to the LUT's 16-bit type and written where the
    // GEMM's activation pre-pass would put it, Ap[g][j][m / 16][lane][8]; rows from M up
    // to the padded count are written as zeros.
    uint32_t *ap;
    int ap_M, ap_mblk_pad, ap_bf16, ap_block_xor;
    int vec_io;     // x and out rows allow 16-byte accesses (16-bit types only)
    int vec_mul;    // signs and awq allow 16-byte loads
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
// Eight consecutive columns k0...k0+7 (k0 a multiple of 8) of row m in operand order:
// k = g*64 + (2j + ktl)*16 + 2*kg + 8*s2 + e lives in lane kg*16 + m%16 of block m/16,
// dword ktl*2 + s2, half e; so the eight values are the (e = 0, 1) pairs of the four
// lanes kg = 0...3 at one dword position.
__device__ __forceinline__ void store_operand_order(const FhtParams &p, int m, int k0,
                                                    const uint16_t (&v)[8]) {
    const int g = k0 >> 6, kl = k0 & 63;
    const int jh = kl >> 5, s = ((kl >> 4) & 1) * 2 + ((kl >> 3) & 1);
    const int64_t unit = ((int64_t)(g * 2 + jh) * p.ap_mblk_pad + ((m >> 4) ^ image_block_xor(g, p.ap_block_xor))) * 64 + (m & 15);
#pragma unroll
    for (int kg = 0; kg < 4; ++kg)
        p.ap[(unit + kg * 16) * 4 + s] = (uint32_t)v[2 * kg] | ((uint32_t)v[2 * kg + 1] << 16);
}

__device__ __forceinline__ void load_mul8(const float *m, int k, int vec, float (&v)[8]) {
    if (vec) {
        const float4 a = *(const float4 *)(m + k), b = *(const float4 *)(m + k + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = m[k + q];
    }
}

// Eight consecutive columns of a row as fp32, already multiplied by what the direction
// applies before the butterfly (signs for the adjoint, the scale for the compensated
// forward transform); sg/sc keep the multipliers the output needs.
__device__ __forceinline__ void load_cols8(const FhtParams &p, int64_t row, int k, float (&f)[8],
                                           float (&sg)[8], float (&sc)[8]) {
    const int bf16 = p.dtype == FLUTE_BF16;
    if (p.vec_io) {
        const uint4 raw = *(const uint4 *)((const uint16_t *)p.x + row + k);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint16_t h = (uint16_t)(w[q >> 1] >> (16 * (q & 1)));
            f[q] = bf16 ? bf2f(h) : h2f(h);
        }
    } else {
#pragma unroll
        for (int q = 0; q < 8; ++q) f[q] = load_any(p.x, row + k + q, p.dtype);
    }
    load_mul8(p.signs, k, p.vec_mul, sg);
    if (p.awq) load_mul8(p.awq, k, p.vec_mul, sc);
    if (p.adjoint || p.awq) {
#pragma unroll
        for (int q = 0; q < 8; ++q) f[q] *= p.adjoint ? sg[q] : sc[q];
    }
}

// The transformed eight columns out: scaled, (forward) signed and de-scaled, one rounding
// to the I/O type, as rows or in the GEMM's operand order.
__device__ __forceinline__ void store_cols8(const FhtParams &p, int64_t orow, int k, float inv,
                                            const float (&f)[8], const float (&sg)[8],
                                            const float (&sc)[8]) {
    const int bf16 = p.dtype == FLUTE_BF16;
    uint16_t op[8];
    float t[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) t[q] = p.adjoint ? f[q] * inv : f[q] * sg[q] * inv;
    if (!p.adjoint && p.awq) {          // one uniform branch: as a select per value every launch paid for the divisions
#pragma unroll
        for (int q = 0; q < 8; ++q) t[q] = t[q] / sc[q];
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        if (p.dtype != FLUTE_F32) {
            uint16_t a = round_act(t[q], bf16);
            if (p.ap && bf16 != p.ap_bf16) a = round_act(bf16 ? bf2f(a) : h2f(a), p.ap_bf16);
            op[q] = a;
        }
    }
    if (p.ap) {
        store_operand_order(p, blockIdx.x, k, op);
    } else if (p.dtype == FLUTE_F32) {
#pragma unroll
        for (int q = 0; q < 8; ++q) ((float *)p.out)[orow + k + q] = t[q];
    } else if (p.vec_io) {
        *(uint4 *)((uint16_t *)p.out + orow + k) =
            make_uint4((uint32_t)op[0] | ((uint32_t)op[1] << 16),
                       (uint32_t)op[2] | ((uint32_t)op[3] << 16),
                       (uint32_t)op[4] | ((uint32_t)op[5] << 16),
                       (uint32_t)op[6] | ((uint32_t)op[7] << 16));
    } else {
#pragma unroll
        for (int q = 0; q < 8; ++q) ((uint16_t *)p.out)[orow + k + q] = op[q];
    }
}

// Stages of length 1, 2, 4 between a thread's own eight columns.
__device__ __forceinline__ void stages_in_thread(float (&f)[8]) {
#pragma unroll
    for (int len = 1; len < 8; len <<= 1) {
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            if ((q & len) == 0) {
                const float a = f[q], c = f[q | len];
                f[q] = a + c;
                f[q | len] = a - c;
            }
        }
    }
}

// One stage against the lane whose number differs in bit M (M = 1 ... 16: ds_swizzle,
// the LDS crossbar without a memory access).  The lower lane of a pair keeps a + b and
// the upper a - b, formed as fma(mine, +-1, other): the product is exact, so every value
// sees the same single rounding per stage as in the buffered butterfly.
template <int M>
__device__ __forceinline__ void stage_across_lanes(float (&f)[8], int lane) {
    const float sgn = (lane & M) ? -1.0f : 1.0f;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const float other = __int_as_float(
            __builtin_amdgcn_ds_swizzle(__float_as_int(f[q]), (M << 10) | 0x1f));
        f[q] = fmaf(f[q], sgn, other);
    }
}

// Equal blocks of at most 256 columns without the LDS buffer: three stages in a thread's
// registers, the stages of length 8 ... block/2 across lanes, in the same ascending order
// as the buffered butterfly and bit-identical to it.  One memory round trip, no barrier.
// The lanes of a block are always in the same step of the loop (a step covers 2048
// columns, a multiple of every block), so a lane's partners are active.
__device__ __forceinline__ void fht_blocks_inwave(const FhtParams &p, int64_t row, int64_t orow,
                                                  int tid) {
    const int nst = 31 - __builtin_clz((unsigned)p.block);
    const float inv = inv_sqrt_pow2(nst);
    const int lane = tid & 63;
    const int pair_lanes = p.block >> 3;               // lanes of one block: 4 ... 32
    // one step at a time: holding several steps of loads in registers measured slower
    // (K = 4096: 5.4 us against 3.8 us per launch)
    for (int j = tid * 8; j < p.K; j += kFhtThreads * 8) {
        float f[8], sg[8], sc[8];
        load_cols8(p, row, j, f, sg, sc);
        stages_in_thread(f);
        if (pair_lanes > 1) stage_across_lanes<1>(f, lane);
        if (pair_lanes > 2) stage_across_lanes<2>(f, lane);
        if (pair_lanes > 4) stage_across_lanes<4>(f, lane);
        if (pair_lanes > 8) stage_across_lanes<8>(f, lane);
        if (pair_lanes > 16) stage_across_lanes<16>(f, lane);
        store_cols8(p, orow, j, inv, f, sg, sc);
    }
}

// One power-of-two segment of 512 ... 8192 columns starting at column `off`.  The first
// nine stages (lengths 1 ... 256) run as in fht_blocks_inwave, the last of them against
// the lane 32 away (ds_bpermute); the remaining stages (lengths 512 ... b/2, at most
// four) are one pass over the fp32 buffer in LDS.  Same butterflies in the same ascending
// order as fht_lds alone, so bit-identical; one memory round trip instead of two, two
// barriers instead of five, a third of the LDS traffic.  A thread holds up to S steps of
// eight columns; b/8 is a multiple of 64, so wavefronts are active as a whole, and a
// step a thread does not have repeats its first one (loads stay unconditional).
template <int S>
__device__ __forceinline__ void fht_segment_fast(const FhtParams &p, int64_t row, int64_t orow,
                                                 int off, int b, int nst, float *buf, int tid) {
    const float inv = inv_sqrt_pow2(nst);
    const int lane = tid & 63;
    const int j0 = tid * 8;
    constexpr int STEP = kFhtThreads * 8;
    const bool one = j0 < b;
    float f[S][8], sg[S][8], sc[S][8];
    if (one) {
#pragma unroll
        for (int h = 0; h < S; ++h)
            load_cols8(p, row, off + (j0 + h * STEP < b ? j0 + h * STEP : j0), f[h], sg[h], sc[h]);
#pragma unroll
        for (int h = 0; h < S; ++h) stages_in_thread(f[h]);
#pragma unroll
        for (int h = 0; h < S; ++h) stage_across_lanes<1>(f[h], lane);
#pragma unroll
        for (int h = 0; h < S; ++h) stage_across_lanes<2>(f[h], lane);
#pragma unroll
        for (int h = 0; h < S; ++h) stage_across_lanes<4>(f[h], lane);
#pragma unroll
        for (int h = 0; h < S; ++h) stage_across_lanes<8>(f[h], lane);
#pragma unroll
        for (int h = 0; h < S; ++h) stage_across_lanes<16>(f[h], lane);
        const float sgn = (lane & 32) ? -1.0f : 1.0f;
        const int partner = (lane ^ 32) << 2;
#pragma unroll
        for (int h = 0; h < S; ++h)
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const float other = __int_as_float(
                    __builtin_amdgcn_ds_bpermute(partner, __float_as_int(f[h][q])));
                f[h][q] = fmaf(f[h][q], sgn, other);
            }
    }
    if (nst > 9) {                                     // uniform: stages of length 512 and up
        if (one) {
#pragma unroll
            for (int h = 0; h < S; ++h) {
                if (j0 + h * STEP < b) {
                    const int s0 = fht_slot(j0 + h * STEP);   // multiple of 8: slot(j + q) = s0 ^ q
#pragma unroll
                    for (int q = 0; q < 8; ++q) buf[s0 ^ q] = f[h][q];
                }
            }
        }
        __syncthreads();
        switch (nst - 9) {
            case 1: fht_pass<1>(buf, b, 9, tid, kFhtThreads); break;
            case 2: fht_pass<2>(buf, b, 9, tid, kFhtThreads); break;
            case 3: fht_pass<3>(buf, b, 9, tid, kFhtThreads); break;
            default: fht_pass<4>(buf, b, 9, tid, kFhtThreads); break;
        }
        __syncthreads();
        if (one) {
#pragma unroll
            for (int h = 0; h < S; ++h) {
                if (j0 + h * STEP < b) {
                    const int s0 = fht_slot(j0 + h * STEP);
#pragma unroll
                    for (int q = 0; q < 8; ++q) f[h][q] = buf[s0 ^ q];
                }
            }
        }
        __syncthreads();                               // the next segment reuses the buffer
    }
    if (one) {
#pragma unroll
        for (int h = 0; h < S; ++h)
            if (j0 + h * STEP < b) store_cols8(p, orow, off + j0 + h * STEP, inv, f[h], sg[h], sc[h]);
    }
}

// MAXS: steps of eight columns a thread may hold in the register-resident segment path
// (0: every segment through the LDS buffer; 2: segments up to 4096 columns in registers;
// 4: up to 8192, at twice the registers).
template <int MAXS>
__global__ void __launch_bounds__(kFhtThreads) fht_kernel(const FhtParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    float *buf = (float *)lds;
    const int tid = threadIdx.x;
    const int64_t row = (int64_t)blockIdx.x * p.ldx;
    const int64_t orow = (int64_t)blockIdx.x * p.ldo;
    if (p.ap && (int)blockIdx.x >= p.ap_M) {           // padding row of the operand image
        const uint16_t zero[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int j = tid * 8; j < p.K; j += kFhtThreads * 8)
            store_operand_order(p, blockIdx.x, j, zero);
        return;
    }
    if (p.block > 0 && p.block <= 256) {
        fht_blocks_inwave(p, row, orow, tid);
        return;
    }
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
        if constexpr (MAXS > 0) {
            if (p.block == 0 && count >= 512 && count <= kFhtThreads * 8 * MAXS) {
                if (MAXS == 2 || count <= kFhtThreads * 16)
                    fht_segment_fast<2>(p, row, orow, off, count, nstages, buf, tid);
                else
                    fht_segment_fast<MAXS>(p, row, orow, off, count, nstages, buf, tid);
                off += count;
                continue;
            }
        }
        const float inv = inv_sqrt_pow2(nstages);
        // The output multipliers of a thread's first two steps are requested together
        // with the row, so the output phase does not start with a memory round trip.
        const int j0 = tid * 8, j1 = j0 + kFhtThreads * 8;
        float sg0[8], sg1[8], sc0[8], sc1[8];
        auto load_mul = [&](int j, float (&sg)[8], float (&sc)[8]) {
            if (p.adjoint) return;
#pragma unroll
            for (int q = 0; q < 8; ++q) sg[q] = p.signs[off + j + q];
            if (p.awq) {
#pragma unroll
                for (int q = 0; q < 8; ++q) sc[q] = p.awq[off + j + q];
            }
        };
        if (j0 < count) load_mul(j0, sg0, sc0);
        if (j1 < count) load_mul(j1, sg1, sc1);
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
        auto emit = [&](int j, const float (&sg)[8], const float (&sc)[8]) {
            uint16_t op[8];
            float tt[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const float b = buf[fht_slot(j + q)];
                tt[q] = p.adjoint ? b * inv : b * sg[q] * inv;
            }
            if (!p.adjoint && p.awq) {
#pragma unroll
                for (int q = 0; q < 8; ++q) tt[q] = tt[q] / sc[q];
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const float t = tt[q];
                if (p.ap) {
                    const int in_bf16 = p.dtype == FLUTE_BF16;
                    uint16_t a = round_act(t, in_bf16);
                    if (in_bf16 != p.ap_bf16) a = round_act(in_bf16 ? bf2f(a) : h2f(a), p.ap_bf16);
                    op[q] = a;
                } else {
                    store_any(p.out, orow + off + j + q, p.dtype, t);
                }
            }
            if (p.ap) store_operand_order(p, blockIdx.x, off + j, op);
        };
        if (j0 < count) emit(j0, sg0, sc0);
        if (j1 < count) emit(j1, sg1, sc1);
        for (int j = j1 + kFhtThreads * 8; j < count; j += kFhtThreads * 8) {
            float sg[8], sc[8];
            load_mul(j, sg, sc);
            emit(j, sg, sc);
        }
        __syncthreads();
        off += count;
    }
}

}  // namespace

}  // namespace flute

namespace flute {

flute_status fht_launch(const void *x, int64_t ldx, const float *signs, const float *awq, void *out,
                        int64_t ldo, int M, int K, int dtype, int adjoint, int block,
                        hipStream_t stream, const FhtOperandOut *operand) {
    FhtParams p;
    p.x = x;
    p.out = out;
    p.signs = signs;
    p.awq = awq;
    p.ldx = ldx;
    p.ldo = ldo;
    p.K = K;
    p.dtype = dtype;
    p.adjoint = adjoint ? 1 : 0;
    p.block = block;
    p.chunk = 0;
    p.ap = operand ? operand->ap : nullptr;
    p.ap_M = M;
    p.ap_mblk_pad = operand ? operand->mblk_pad : 0;
    p.ap_block_xor = operand ? operand->block_xor : 0;
    p.ap_bf16 = operand ? operand->lut_bf16 : 0;
    const bool io16 = dtype != FLUTE_F32;
    p.vec_io = io16 && ((uintptr_t)x & 15) == 0 && ldx % 8 == 0 &&
               (operand || (((uintptr_t)out & 15) == 0 && ldo % 8 == 0));
    p.vec_mul = ((uintptr_t)signs & 15) == 0 && (!awq || ((uintptr_t)awq & 15) == 0);
    size_t lds_bytes;
    bool wide = false;
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
        wide = segs.len[0] > kFhtThreads * 16 && segs.len[0] <= kFhtThreads * 32;
    }
    const int rows = operand ? operand->mblk_pad * 16 : M;
    if (rows == 0) return FLUTE_OK;
    static std::atomic<bool> attr_done{false};   // threads may race to the first call: the call is idempotent
    if (!attr_done) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)fht_kernel<2>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)fht_kernel<0>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)fht_kernel<4>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
        attr_done = true;
    }
    // Which variant: the register-resident segment path wins wherever it applies, except
    // that its wide form (segments of 8192 columns, 270 registers, one workgroup per CU)
    // loses to the buffered kernel once there are many rows (K = 12288: 12.4 us against
    // 21.0 us for one row, 52.6 us against 40.3 us for 1024 rows).  FLUTE_FHT_STEPS = 0, 2
    // or 4 forces a variant (tuning and test knob).
    int steps = wide ? (rows <= 512 ? 4 : 0) : 2;
    {
        const int v = tuning().fht_steps;
        if (v == 0 || v == 2 || v == 4) steps = v;
    }
    if (steps == 0)
        hipLaunchKernelGGL(fht_kernel<0>, dim3(rows), dim3(kFhtThreads), lds_bytes, stream, p);
    else if (steps == 4)
        hipLaunchKernelGGL(fht_kernel<4>, dim3(rows), dim3(kFhtThreads), lds_bytes, stream, p);
    else
        hipLaunchKernelGGL(fht_kernel<2>, dim3(rows), dim3(kFhtThreads), lds_bytes, stream, p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}

}  // namespace flute

using namespace flute;

extern "C" flute_status flute_fht(const void *x, const float *signs, const float *awq, void *out,
                                  int M, int K, int dtype, int adjoint, int block, void *stream) {
    FLUTE_REQUIRE(x && out && signs, FLUTE_ERR_INVALID, "flute_fht: x, signs and out must not be NULL");
    FLUTE_REQUIRE(dtype == FLUTE_F16 || dtype == FLUTE_BF16 || dtype == FLUTE_F32, FLUTE_ERR_INVALID,
                  "flute_fht: dtype must be float16, bfloat16 or float32");
    FLUTE_REQUIRE(M >= 0, FLUTE_ERR_INVALID, "flute_fht: M must be >= 0");
    {
        const uintptr_t elem = dtype == FLUTE_F32 ? 3 : 1;
        FLUTE_REQUIRE(((uintptr_t)x & elem) == 0 && ((uintptr_t)out & elem) == 0, FLUTE_ERR_INVALID,
                      "flute_fht: x and out must be aligned to their element size");
        FLUTE_REQUIRE(((uintptr_t)signs & 3) == 0 && ((uintptr_t)awq & 3) == 0, FLUTE_ERR_INVALID,
                      "flute_fht: signs and awq are fp32 and must be 4-byte aligned");
    }
    FLUTE_REQUIRE(K >= 32 && K % 32 == 0 && K <= 65504, FLUTE_ERR_INVALID,
                  "flute_fht: K must be a multiple of 32 in [32, 65504] (got %d)", K);
    FLUTE_REQUIRE(!(awq && adjoint), FLUTE_ERR_INVALID,
                  "flute_fht: the awq-compensated transform exists in the forward direction only");
    return fht_launch(x, K, signs, awq, out, K, M, K, dtype, adjoint, block, (hipStream_t)stream,
                      nullptr);
}
