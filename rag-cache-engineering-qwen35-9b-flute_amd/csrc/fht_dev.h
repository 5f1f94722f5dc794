// Walsh-Hadamard butterfly on an fp32 LDS buffer, shared by the standalone
// rotation kernel and the GEMV prologue so that both produce the same bits.
//
// The transform is the stage-doubling butterfly of fht.py:174-192 upstream: for
// len = 1, 2, 4, ... every pair (i, i + len) whose index i has bit log2(len)
// clear becomes (a + b, a - b).  Each pair operation is a single fp32 add and a
// single fp32 subtract, and a value is touched by exactly one pair per stage, so
// the result does not depend on which thread executes which pair: it is
// bit-identical to the scalar loop as long as the stages run in ascending order.
//
// Stages are executed four at a time in registers (radix-16 passes): a thread
// gathers the 16 values whose indices differ only in the four bits of the pass,
// runs the four stages locally, and scatters them back.  One barrier per pass
// instead of one per stage.
#pragma once

#include "common.h"

namespace flute {

// float(1 / sqrt(2^n)), identical to rounding the fp64 quotient: the value is
// 2^-(n/2) for even n and float(sqrt(2)) * 2^-((n+1)/2) for odd n, and scaling
// by a power of two is exact.
__device__ __forceinline__ float inv_sqrt_pow2(int n) {
    return ldexpf((n & 1) ? 1.41421356237309504880f : 1.0f, -((n + 1) >> 1));
}

// Physical LDS slot of logical element i: a linear XOR swizzle of the five bank
// bits by higher index bits.  In the first radix-16 pass 32 consecutive lanes
// differ in index bits 4..8, in the second in bits 0..3 and 8; the swizzle maps
// both patterns (and plain consecutive indices) onto 32 distinct banks.
__device__ __forceinline__ int fht_slot(int i) {
    return i ^ ((i >> 5) & 7) ^ (((i >> 8) & 1) * 24);
}

template <int R>
__device__ __forceinline__ void fht_pass(float *buf, int b, int sh0, int tid, int nthreads) {
    constexpr int E = 1 << R;
    const int ngroups = b >> R;
    const int lowmask = (1 << sh0) - 1;
    for (int gi = tid; gi < ngroups; gi += nthreads) {
        const int base = ((gi >> sh0) << (sh0 + R)) | (gi & lowmask);
        float v[E];
#pragma unroll
        for (int j = 0; j < E; ++j) v[j] = buf[fht_slot(base + (j << sh0))];
#pragma unroll
        for (int q = 0; q < R; ++q) {
#pragma unroll
            for (int j = 0; j < E; ++j) {
                if ((j & (1 << q)) == 0) {
                    const float a = v[j], c = v[j | (1 << q)];
                    v[j] = a + c;
                    v[j | (1 << q)] = a - c;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < E; ++j) buf[fht_slot(base + (j << sh0))] = v[j];
    }
}

// In-place transform of `count` values held at buf[fht_slot(0..count-1)], as
// count / b independent blocks of b = 2^nstages consecutive values (count a
// multiple of b; b >= 2).  Must be called by every thread of the workgroup; the
// buffer must be complete (barrier) on entry and is complete on exit.
template <int RMAX = 4>
__device__ __forceinline__ void fht_lds(float *buf, int count, int nstages, int tid,
                                        int nthreads) {
    // RMAX = stages per pass: 4 keeps 16 values in registers, 3 keeps 8 (for callers
    // that are short of registers); the order of the stages, and so every bit of the
    // result, is the same.
    int sh0 = 0;
    while (nstages - sh0 >= RMAX) {
        fht_pass<RMAX>(buf, count, sh0, tid, nthreads);
        __syncthreads();
        sh0 += RMAX;
    }
    const int rem = nstages - sh0;
    if (RMAX > 3 && rem == 3) fht_pass<3>(buf, count, sh0, tid, nthreads);
    else if (rem == 2) fht_pass<2>(buf, count, sh0, tid, nthreads);
    else if (rem == 1) fht_pass<1>(buf, count, sh0, tid, nthreads);
    if (rem) __syncthreads();
}

}  // namespace flute
