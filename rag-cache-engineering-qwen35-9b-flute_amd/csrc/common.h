// Shared host/device helpers for the gfx950 idxN LUT kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flute_hip.h"

namespace flute {

// ---- error reporting (thread-local message behind flute_last_error) --------
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define FLUTE_REQUIRE(cond, code, ...)            \
    do {                                          \
        if (!(cond)) {                            \
            ::flute::set_error(__VA_ARGS__);      \
            return (code);                        \
        }                                         \
    } while (0)

#define FLUTE_HIP_CHECK(expr)                                                   \
    do {                                                                        \
        hipError_t _e = (expr);                                                 \
        if (_e != hipSuccess) {                                                 \
            ::flute::set_error("%s failed: %s", #expr, hipGetErrorString(_e));  \
            return FLUTE_ERR_HIP;                                               \
        }                                                                       \
    } while (0)

// ---- geometry of the idxN blob (flute_extended/idxN.py:37-55 upstream) -----
constexpr int kTileRows = 128;   // output rows per tile
constexpr int kTileK = 64;       // k values per tile
constexpr int kWave = 64;        // one wavefront owns one tile: lane = chunk

// MI355X: 256 CUs in 8 XCDs, 160 KB of LDS per CU.
constexpr int kNumCU = 256;
constexpr int kLdsPerCU = 160 * 1024;

// Descending power-of-two segments of K (fht.py:118-134 upstream).
struct Segs {
    int n;
    int off[16];
    int len[16];
};

inline Segs make_segments(int K, int block) {
    Segs s;
    s.n = 0;
    if (block > 0) {                 // equal blocks are handled by the kernels
        s.n = 1;
        s.off[0] = 0;
        s.len[0] = block;
        return s;
    }
    int off = 0, rem = K;
    while (rem > 0 && s.n < 16) {
        int b = 1;
        while ((b << 1) <= rem) b <<= 1;
        s.off[s.n] = off;
        s.len[s.n] = b;
        ++s.n;
        off += b;
        rem -= b;
    }
    return s;
}

// Activation image of the LUT GEMM, order of the 16-row blocks inside their groups of four: block
// b of K tile g is stored at position b ^ image_block_xor(g, mode).  mode 0: as they come.  mode 1
// (workgroups of four k ways): g & 3.  mode 2 (eight k ways): bit 2 and bit 1 of g swapped into
// bits 1 and 0.  The k way that owns tile g then finds in position j the block its hand-overs at
// the end of the kernel expect there (gemm_kernel.h).
__host__ __device__ inline int image_block_xor(int g, int mode) {
    return mode == 1 ? (g & 3) : mode == 2 ? (((g & 4) >> 1) | ((g & 2) >> 1)) : 0;
}

// A 64-bit address put together from two 32-bit halves that come out of builtins returning
// `int` (__builtin_amdgcn_readfirstlane): each half is taken as unsigned first.  Converting the
// int straight to uint64_t sign-extends it, and a low half with bit 31 set then sets all 32 upper
// bits of the result: an address outside every allocation.
__host__ __device__ __forceinline__ uint64_t join_address_halves(int lo, int hi) {
    return (uint64_t)(uint32_t)lo | ((uint64_t)(uint32_t)hi << 32);
}

// Reads one dword of every 64-byte line of the kernel-argument block with
// independent scalar loads and waits for them once.  The descriptor fields are
// then fetched through a chain of dependent scalar loads (segment -> stream ->
// pointers); with the lines already in the scalar cache each link costs a cache
// hit instead of a trip to L2 or memory.
template <int BYTES>
__device__ __forceinline__ void warm_kernargs(const void *kernargs) {
    const uint32_t *ka = (const uint32_t *)kernargs;
    uint32_t seen = 0;
#pragma unroll
    for (int o = 0; o < BYTES; o += 64) seen |= ka[o / 4];
    asm volatile("" ::"s"(seen));
}

// ---- 16-bit float conversions on the device --------------------------------
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float h2f(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}
__device__ __forceinline__ uint16_t f2h(float f) {     // round to nearest even
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}
__device__ __forceinline__ float bf2f(uint16_t h) {
    return __builtin_bit_cast(float, (uint32_t)h << 16);
}
__device__ __forceinline__ uint16_t f2bf(float f) {    // round to nearest even (v_cvt_pk_bf16_f32)
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float load_act(const void *p, int64_t i, int is_bf16) {
    uint16_t h = ((const uint16_t *)p)[i];
    return is_bf16 ? bf2f(h) : h2f(h);
}
__device__ __forceinline__ uint16_t round_act(float f, int is_bf16) {
    return is_bf16 ? f2bf(f) : f2h(f);
}

// acc += a.x*b.x + a.y*b.y, 16-bit operands packed in a dword, fp32 accumulate.
template <bool BF16>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    if constexpr (BF16) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                               __builtin_bit_cast(bf16x2_t, b), acc, false);
    } else {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a),
                                      __builtin_bit_cast(half2_t, b), acc, false);
    }
}

// ---- bfloat16 activations in front of float16 arithmetic -------------------------
// A float16 LUT fixes the arithmetic type to float16 (the dequantised weight must be the
// LUT entry exactly), but bfloat16 activations reach from 1e-38 to 3e38 and float16 only
// from 6e-8 to 65504.  The staged row is therefore scaled by a power of two chosen from
// its largest magnitude (exact: only the exponent changes), the products are summed in
// fp32 as usual, and the row sums are scaled back before anything else is added.  The
// result is what unscaled arithmetic would give wherever that does not overflow, and
// stays finite and correct where it would.

// Largest biased exponent among eight bfloat16 values.
__device__ __forceinline__ uint32_t bf16_max_exp8(uint4 v) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t e = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        e = max(e, (w[q] >> 7) & 0xffu);
        e = max(e, (w[q] >> 23) & 0xffu);
    }
    return e;
}

// Maximum over the wavefront, in scalar registers: four DPP steps fold each row of 16
// lanes, four lane reads fold the rows.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_max(uint32_t v) {
    const uint32_t moved = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
    return max(v, moved);
}
__device__ __forceinline__ uint32_t wavefront_max(uint32_t v) {
    v = dpp_max<0xB1>(v);    // quad_perm [1,0,3,2]
    v = dpp_max<0x4E>(v);    // quad_perm [2,3,0,1]
    v = dpp_max<0x141>(v);   // row_half_mirror
    v = dpp_max<0x140>(v);   // row_mirror
    const uint32_t a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const uint32_t c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return max(max(a, b), max(c, d));
}

// Maximum over the workgroup; slots = one LDS word per wavefront.  One barrier.
__device__ __forceinline__ uint32_t workgroup_max(uint32_t v, uint32_t *slots, int tid,
                                                  int nthreads) {
    v = wavefront_max(v);
    if ((tid & 63) == 0) slots[tid >> 6] = v;
    __syncthreads();
    uint32_t r = 0;
    for (int w = 0; w < (nthreads >> 6); ++w) r = max(r, slots[w]);
    return r;
}

// Shift that brings a row whose largest biased exponent is emax to magnitudes in [1, 2):
// the largest value then has 15 binades of float16 range above it and 14 normal (24 in
// all) below.  Zero rows and non-finite values keep their values (shift 0).
__device__ __forceinline__ int bf16_row_shift(uint32_t emax) {
    return (emax == 0 || emax == 255) ? 0 : (int)emax - 127;
}

// Eight bfloat16 values -> eight float16 values of x * 2^-shift.
__device__ __forceinline__ uint4 bf16_to_f16_scaled8(uint4 v, int shift) {
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float lo = ldexpf(bf2f((uint16_t)(w[q] & 0xffffu)), -shift);
        const float hi = ldexpf(bf2f((uint16_t)(w[q] >> 16)), -shift);
        w[q] = (uint32_t)f2h(lo) | ((uint32_t)f2h(hi) << 16);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// The same conversion in packed 16-bit integer arithmetic, two values per instruction, for
// the lean GEMV whose prologue is bound by vector-instruction issue.  The largest magnitude
// goes to float16's top binade (biased exponent 30; bfloat16's largest mantissa stays below
// 65504), which leaves 29 normal binades below it: adj = max(emax - 30, 0) is subtracted
// from every biased exponent and the row sums are scaled back by 2^(adj - 112).  Values
// more than 29 binades below the largest one are flushed (the one binade at the edge maps
// to a float16 subnormal of at most the same size): a relative error below 2^-29 of the
// largest magnitude.  Rows that hold an infinity or a NaN (emax = 255) must take the
// float route above.
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));

// Running maximum of the magnitudes (sign cleared) of eight bfloat16 values, per half.
__device__ __forceinline__ uint32_t bf16_max_mag8(uint32_t m, uint4 v) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    u16x2_t r = __builtin_bit_cast(u16x2_t, m);
#pragma unroll
    for (int q = 0; q < 4; ++q)
        r = __builtin_elementwise_max(r, __builtin_bit_cast(u16x2_t, w[q] & 0x7fff7fffu));
    return __builtin_bit_cast(uint32_t, r);
}
// Largest biased exponent held in a packed pair of magnitudes.
__device__ __forceinline__ uint32_t bf16_mag_exp(uint32_t m) { return max(m & 0xffffu, m >> 16) >> 7; }

__device__ __forceinline__ uint4 bf16_to_f16_top8(uint4 v, uint32_t adj) {
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
    const uint32_t a = adj << 7;
    const u16x2_t av = __builtin_bit_cast(u16x2_t, a | (a << 16));
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        u16x2_t t = __builtin_bit_cast(u16x2_t, w[q] & 0x7fff7fffu);
        t = __builtin_elementwise_sub_sat(t, av);   // exponent - adj, flushed below
        t = t << (unsigned short)3;                 // 8.7 -> 5.10 field positions
        w[q] = (__builtin_bit_cast(uint32_t, t) & 0x7fff7fffu) | (w[q] & 0x80008000u);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

}  // namespace flute
