/*
 * CPU oracle (plain C) for the idxN LUT-palettized linear layer.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/liboracle.so, loaded by tests/
 * and by bench.py's cpu_baseline leg as the checker / the timed CPU port.
 * The product library never links or loads it.
 *
 * Each function cites the upstream file:line it restates (paths relative to
 * the upstream tree).  This file is written independently of
 * flute_oracle.py so that the two can be compared byte for byte.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* IEEE binary16 -> binary32, exact. */
static float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                       /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static float bf16_to_float(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* Field f (0..127) of a chunk, b bits wide, LSB first at bit offset b*f
 * (flute_extended/flute_extended/idxN.py:46-47,158-232). */
static inline unsigned chunk_field(const uint8_t *chunk, int b, int f) {
    int bit = b * f;
    unsigned lo = chunk[bit >> 3];
    unsigned hi = ((bit >> 3) + 1 < 16 * b) ? chunk[(bit >> 3) + 1] : 0u;
    return (((hi << 8) | lo) >> (bit & 7)) & ((1u << b) - 1u);
}

/* Tile-local coordinates of pair p of chunk th (idxN.py:46-51). */
static inline void pair_rc(int th, int p, int *row, int *k) {
    int wx = th >> 5, lane = th & 31;
    int kt = p >> 4, v = (p >> 2) & 3, d = (p >> 1) & 1, s2 = p & 1;
    *row = wx * 64 + v * 16 + d * 8 + (lane >> 2);
    *k = kt * 16 + 2 * (lane & 3) + 8 * s2;
}

/* blob -> logical [N, K] indices (idxN.py:267-291).  Returns 0, or -1 when the
 * shape is not storable (idxN.py:95-108). */
int oracle_unpack_idxn(const uint8_t *blob, int N, int K, int b, uint8_t *idx) {
    if (b < 1 || b > 4 || N % 128 || K % 64) return -1;
    int G = K / 64;
    for (int t = 0; t < N / 128; ++t)
        for (int g = 0; g < G; ++g) {
            const uint8_t *tile = blob + ((size_t)t * G + g) * 1024 * b;
            for (int th = 0; th < 64; ++th) {
                const uint8_t *chunk = tile + th * 16 * b;
                for (int p = 0; p < 64; ++p) {
                    int r, k;
                    pair_rc(th, p, &r, &k);
                    uint8_t *dst = idx + (size_t)(t * 128 + r) * K + g * 64 + k;
                    dst[0] = (uint8_t)chunk_field(chunk, b, 2 * p);
                    dst[1] = (uint8_t)chunk_field(chunk, b, 2 * p + 1);
                }
            }
        }
    return 0;
}

/* logical [N, K] indices -> blob (idxN.py:235-264). */
int oracle_pack_idxn(const uint8_t *idx, int N, int K, int b, uint8_t *blob) {
    if (b < 1 || b > 4 || N % 128 || K % 64) return -1;
    int G = K / 64;
    memset(blob, 0, (size_t)N * K * b / 8);
    for (int t = 0; t < N / 128; ++t)
        for (int g = 0; g < G; ++g) {
            uint8_t *tile = blob + ((size_t)t * G + g) * 1024 * b;
            for (int th = 0; th < 64; ++th) {
                uint8_t *chunk = tile + th * 16 * b;
                for (int p = 0; p < 64; ++p) {
                    int r, k;
                    pair_rc(th, p, &r, &k);
                    const uint8_t *src = idx + (size_t)(t * 128 + r) * K + g * 64 + k;
                    for (int j = 0; j < 2; ++j) {
                        unsigned val = src[j];
                        if (val >> b) return -2;
                        int bit = b * (2 * p + j);
                        unsigned sh = val << (bit & 7);
                        chunk[bit >> 3] |= (uint8_t)sh;
                        if (sh >> 8) chunk[(bit >> 3) + 1] |= (uint8_t)(sh >> 8);
                    }
                }
            }
        }
    return 0;
}

/* W[n, k] = LUT[n / gs, idx[n, k]] as fp32
 * (scripts/palettized_modules.py:125-162).  lut_is_bf16 selects the LUT's
 * 16-bit format. */
int oracle_dequant(const uint8_t *blob, const uint16_t *lut, int lut_is_bf16,
                   int N, int K, int gs, int b, float *W) {
    uint8_t *idx = (uint8_t *)malloc((size_t)N * K);
    if (!idx) return -3;
    int rc = oracle_unpack_idxn(blob, N, K, b, idx);
    if (rc) { free(idx); return rc; }
    int ngroups = (N + gs - 1) / gs;
    for (int n = 0; n < N; ++n) {
        int grp = n / gs;
        if (grp > ngroups - 1) grp = ngroups - 1;
        const uint16_t *row = lut + ((size_t)grp << b);
        for (int k = 0; k < K; ++k) {
            uint16_t h = row[idx[(size_t)n * K + k]];
            W[(size_t)n * K + k] = lut_is_bf16 ? bf16_to_float(h) : half_to_float(h);
        }
    }
    free(idx);
    return 0;
}

/* y[n] = sum_k x[k] * W[n, k] in fp32, ascending k: the M = 1 case of
 * x.float() @ W.t() (palettized_modules.py:1241-1251) with the unpack and the
 * gather done per call, as the upstream reference does when indices are not
 * cached (palettized_modules.py:811-824).  x is fp32 here; the caller
 * converts. */
int oracle_gemv(const float *x, const uint8_t *blob, const uint16_t *lut,
                int lut_is_bf16, int N, int K, int gs, int b, float *y) {
    float *W = (float *)malloc((size_t)N * K * sizeof(float));
    if (!W) return -3;
    int rc = oracle_dequant(blob, lut, lut_is_bf16, N, K, gs, b, W);
    if (rc) { free(W); return rc; }
    for (int n = 0; n < N; ++n) {
        float acc = 0.0f;
        const float *w = W + (size_t)n * K;
        for (int k = 0; k < K; ++k) acc += x[k] * w[k];
        y[n] = acc;
    }
    free(W);
    return 0;
}

/* In-place stage-doubling Walsh-Hadamard butterfly on b fp32 values: for
 * len = 1, 2, 4, ... each pair (i, i+len) of a 2*len group -> (a+b, a-b)
 * (fht.py:174-192). */
static void butterfly(float *v, int b) {
    for (int len = 1; len < b; len <<= 1)
        for (int base = 0; base < b; base += 2 * len)
            for (int o = 0; o < len; ++o) {
                float a = v[base + o], c = v[base + o + len];
                v[base + o] = a + c;
                v[base + o + len] = a - c;
            }
}

/* out = x @ T per row: ((x @ H) * s) * (1/sqrt(b)) over the descending
 * power-of-two segments of K (fht.py:118-134, 206-222).  adjoint != 0 gives
 * x @ T^T = ((x * s) @ H) * (1/sqrt(b)) (fht.py:225-238). */
int oracle_fht(const float *x, const float *signs, int M, int K, int adjoint, float *out) {
    for (int m = 0; m < M; ++m) {
        int off = 0, rem = K;
        while (rem > 0) {
            int b = 1;
            while ((b << 1) <= rem) b <<= 1;
            float *seg = out + (size_t)m * K + off;
            for (int j = 0; j < b; ++j) {
                float v = x[(size_t)m * K + off + j];
                seg[j] = adjoint ? v * signs[off + j] : v;
            }
            butterfly(seg, b);
            float inv = (float)(1.0 / sqrt((double)b));
            for (int j = 0; j < b; ++j)
                seg[j] = adjoint ? seg[j] * inv : (seg[j] * signs[off + j]) * inv;
            off += b;
            rem -= b;
        }
    }
    return 0;
}

/* The upstream split policy (src/gemv_host.cpp:29-38): keep doubling the
 * split while the grid is short of 160 workgroups, the split is below 16 and
 * every K-quarter of every split still owns at least one 64-k tile. */
int oracle_pick_split_upstream(int tiles, int G) {
    int s = 1;
    while (tiles * s < 160 && s < 16 && G >= 8 * s && G % (8 * s) == 0) s *= 2;
    return s;
}
