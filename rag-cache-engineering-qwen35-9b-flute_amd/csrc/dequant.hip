// Dense dump of one palettized stream: W[n, k] = LUT[n / gs][idx[n, k]] (or, with the LUT
// grouped along K, LUT[n][k / 128][idx[n, k]]) written as the LUT's own 16-bit values, so the result can be compared bit for bit with
// a gather on the host.
#include "host_common.h"

namespace flute {

namespace {

// b-bit field f (0..127) of a 16*b-byte chunk, LSB first at bit b*f
// (flute_extended/idxN.py:46-47,158-232 upstream).
__device__ __forceinline__ uint32_t chunk_field(const uint8_t *chunk, int b, int f) {
    const int bit = b * f;
    const int byte = bit >> 3;
    uint32_t v = chunk[byte];
    if (byte + 1 < 16 * b) v |= (uint32_t)chunk[byte + 1] << 8;
    return (v >> (bit & 7)) & ((1u << b) - 1u);
}

// One workgroup per (128-row tile t, 64-k tile g); thread = (chunk th, quarter kt).
__global__ void __launch_bounds__(256) dequant_kernel(const uint8_t *q, const uint16_t *lut,
                                                      uint16_t *W, int N, int K, int gs, int b,
                                                      int lut_rows, int k_group) {
    const int G = K >> 6;
    const int t = blockIdx.x / G, g = blockIdx.x % G;
    const int th = threadIdx.x & 63, kt = threadIdx.x >> 6;
    const int wx = th >> 5, lane = th & 31;
    const uint8_t *chunk = q + ((size_t)t * G + g) * (1024 * b) + th * 16 * b;
    for (int r = 0; r < 16; ++r) {
        const int p = kt * 16 + r;
        const int v = (p >> 2) & 3, d = (p >> 1) & 1, s2 = p & 1;
        const int n = t * 128 + wx * 64 + v * 16 + d * 8 + (lane >> 2);
        const int k = g * 64 + kt * 16 + 2 * (lane & 3) + 8 * s2;
        const int grp = k_group ? n * (K >> 7) + (k >> 7) : min(n / gs, lut_rows - 1);
        const uint16_t *row = lut + ((size_t)grp << b);
        const uint32_t lo = row[chunk_field(chunk, b, 2 * p)];
        const uint32_t hi = row[chunk_field(chunk, b, 2 * p + 1)];
        *(uint32_t *)(W + (size_t)n * K + k) = lo | (hi << 16);
    }
}

}  // namespace

}  // namespace flute

using namespace flute;

extern "C" flute_status flute_dequant(const flute_linear *w, int which, void *W_out, void *stream) {
    flute_status st = validate_linear(w, 1 | kModeKGroupOk, "flute_dequant");
    if (st != FLUTE_OK) return st;
    FLUTE_REQUIRE(W_out != nullptr, FLUTE_ERR_INVALID, "flute_dequant: output is NULL");
    FLUTE_REQUIRE(((uintptr_t)W_out & 3) == 0, FLUTE_ERR_INVALID,
                  "flute_dequant: output must be 4-byte aligned (two weights per store)");
    FLUTE_REQUIRE(which == 1 || (which == 2 && w->b2 > 0), FLUTE_ERR_INVALID,
                  "flute_dequant: stream %d is not present", which);
    const uint8_t *q = (const uint8_t *)(which == 1 ? w->q1 : w->q2);
    const uint16_t *lut = (const uint16_t *)(which == 1 ? w->lut1 : w->lut2);
    const int b = which == 1 ? w->b1 : w->b2;
    const int tiles = (w->N / 128) * (w->K / 64);
    hipLaunchKernelGGL(dequant_kernel, dim3(tiles), dim3(256), 0, (hipStream_t)stream, q, lut,
                       (uint16_t *)W_out, w->N, w->K, w->group_size, b, w->lut_rows, w->k_group);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}
