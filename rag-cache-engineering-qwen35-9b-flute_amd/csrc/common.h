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

}  // namespace flute
