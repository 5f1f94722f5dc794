// M = 1 LUT GEMV for gfx950 (wave64), the decode kernel of the idxN layer.
//
// Ownership.  A workgroup OWNS a slice of RW output rows of one 128-row tile
// (RW = 8, 16 or 32: 1, 2 or 4 of the tile's sixteen 8-row chunk groups) and,
// when K is split, one K range.  Its wavefronts all work on the same rows and
// divide the 64-k tiles of the range between them; a workgroup runs every
// stream that feeds its rows (one or two streams of a weight; gate and up of a
// merged MLP) one after the other, so without a K split no partial result ever
// leaves the workgroup.
//
// Reading the blob (flute_extended/idxN.py:37-55 upstream).  In a tile of
// 1024*b bytes, chunk group cg = (wx, r8) is the 64*b contiguous bytes of the
// four chunks i = 0..3 that cover rows wx*64 + v*16 + d*8 + r8 (v<4, d<2).
// A lane reads 4*b bytes: quarter kt of one chunk, i.e. 16 k-pairs
// q = v*4 + d*2 + s2 of columns kt*16 + 2*i + 8*s2 (+1).  With LPG = 2*RW lanes
// per 64-k tile, lane l = (cg_local, i, kt) and a wavefront load covers 64/LPG
// tiles at once, each as one contiguous run of LPG*4*b bytes.  A lane therefore
// keeps 8 fp32 row accumulators (v, d) for its whole K share; the lanes that
// share rows are folded once at the end (DPP inside 16 lanes, then across).
//
// Dequantisation.  The group's LUT (2^b 16-bit values) is expanded once per
// workgroup into a paired table in LDS indexed by a whole packed byte (b = 4:
// byte -> {W[k], W[k+1]}; b = 2: byte -> 4 values; b = 1: byte -> 8 values;
// b = 3: 6-bit pair field -> 2 values).  Every entry is replicated across a
// power-of-two stride so that each lane reads its own bank: one conflict-free
// ds_read per lookup whatever the codes are.  With a 256-byte stride the address
// is {replica byte, code byte} and is formed by a single v_perm_b32.  A pair
// feeds v_dot2_f32_f16 / v_dot2_f32_bf16 against the matching activation pair:
// 2 MACs per instruction, fp32 accumulate.
//
// K split (narrow N only).  Row partials go to a workspace through
// device-coherent stores; the last workgroup to take a ticket for a row slice
// folds them in fixed order.  Deterministic and replayable: tickets return to 0.
#pragma once

#include "common.h"
#include "fht_dev.h"

namespace flute {

constexpr int kGemvMaxThreads = 512;
constexpr int kGemvMaxSegs = 4;
constexpr int kGemvMaxRank = 256;

struct GemvStream {
    const uint8_t *q;       // idxN blob
    const uint16_t *lut;    // [lut_rows, 2^bits]
    int bits;
    int es;                 // log2(LDS bytes between consecutive table entries)
};

struct GemvSeg {            // one weight
    GemvStream st[2];
    const uint16_t *resA;   // (N, R) or null
    const uint16_t *bias;   // (N,) or null
    const float *xb;        // (R,) residual coefficients x . resB[r], fp32, or null
    const uint16_t *xsrc;   // (K,) this weight's own input row, or null for the shared one
    const float *signs;     // (K,) or null: rotate the input first
    const float *awq;       // (K,) or null
    uint16_t *out;          // (N,)
    int nstreams;
    int N;
    int R;
    int gs;
    int lut_rows;
    int col0;               // first grid column (row slice) of this weight
    int n0;                 // first column of this weight in a partial-sum row
    int ticket0;            // first ticket of this weight
};

constexpr int kGemvRedBytes = 2 * 8 * 32 * 4;   // partial row sums of two outputs, eight wavefronts

struct GemvParams {
    GemvSeg seg[kGemvMaxSegs];
    const uint16_t *x;      // (K,) activations
    float *P;               // partial sums: [split][p_stride]
    int *tickets;
    int nsegs;
    int K;
    int split;
    int gs_tiles;           // 64-k tiles per split
    int lpg_log2;           // log2(lanes per 64-k tile) = log2(2 * RW): 4, 5 or 6
    int p_stride;           // floats per partial-sum row
    int silu_mul;           // 1: out = silu(seg 0) * seg 1, written to seg[0].out
    int act_bf16;           // activations, residual, bias and outputs are bf16
    int fht_block;          // > 0: equal rotation blocks of this many columns
    int lds_x;              // LDS byte offsets
    int lds_red;            // row sums [2][8][32] fp32, ticket flag (16 B), 8 words for a row maximum
    int slices;             // > 0: a workgroup walks the row slices blockIdx.x, + gridDim.x, ... below this
    int xcd_runs;           // lean kernel, one column space: workgroup b takes slice (b % 8) * (grid / 8) + b / 8
};

// ---- small device helpers ---------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
    return v + __builtin_bit_cast(float, moved);
}

// Workspace traffic between workgroups goes through device-scope atomic
// stores and loads: they bypass the non-coherent cache levels (each XCD has its
// own L2), so no cache write-back or invalidate is needed around the ticket.
__device__ __forceinline__ void ws_store(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ws_load(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A store is visible device-wide once it has been acknowledged; the ticket that
// announces the stores of a workgroup may only be taken after that.  (A barrier does
// not wait for outstanding memory operations.)
__device__ __forceinline__ void ws_stores_done() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0)

// Sum over the 16 lanes of a DPP row; every lane of the row ends with the total.
__device__ __forceinline__ float row16_sum(float v) {
    v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);   // row_half_mirror
    v = dpp_add<0x140>(v);   // row_mirror
    return v;
}

// Table geometry per width: entries, log2(bytes per entry).
template <int B> struct TableShape;
template <> struct TableShape<4> { static constexpr int kEntries = 256, kEntryLog2 = 2; };
template <> struct TableShape<3> { static constexpr int kEntries = 64,  kEntryLog2 = 2; };
template <> struct TableShape<2> { static constexpr int kEntries = 256, kEntryLog2 = 3; };
template <> struct TableShape<1> { static constexpr int kEntries = 256, kEntryLog2 = 4; };

// Dword `sub` of the table entry of code byte `e`: two LUT values packed low/high.
template <int B>
__device__ __forceinline__ uint32_t table_dword(const uint16_t *lut, int e, int sub) {
    int c0, c1;
    if constexpr (B == 4) { c0 = e & 15; c1 = e >> 4; }
    else if constexpr (B == 3) { c0 = e & 7; c1 = e >> 3; }
    else if constexpr (B == 2) { c0 = (e >> (4 * sub)) & 3; c1 = (e >> (4 * sub + 2)) & 3; }
    else { c0 = (e >> (2 * sub)) & 1; c1 = (e >> (2 * sub + 1)) & 1; }
    return (uint32_t)lut[c0] | ((uint32_t)lut[c1] << 16);
}

// One quarter-chunk (4*B bytes of this lane) in two steps, so that the refill of
// the index registers can be issued between them: every table lookup of the
// quarter goes out first (the LDS latency is paid once per quarter, not once per
// lookup), then the looked-up pairs meet the activation pairs xa (s2 = 0) and xb
// (s2 = 1).  lane_off[v] = table base of row block v plus this lane's replica
// offset.  Whatever the width, a quarter looks up 16 dwords.
template <int B>
__device__ __forceinline__ void quarter_lookups(const uint32_t (&w)[B], const uint8_t *lds,
                                                const uint32_t (&lane_off)[4], int es,
                                                uint32_t (&e)[16]) {
    auto byte_addr = [&](uint32_t word, int j, uint32_t off) -> uint32_t {
        return (((word >> (8 * j)) & 0xffu) << es) + off;
    };
    if constexpr (B == 4) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int j = 0; j < 4; ++j)             // byte j: d = j >> 1, s2 = j & 1
                e[v * 4 + j] = *(const uint32_t *)(lds + byte_addr(w[v], j, lane_off[v]));
    } else if constexpr (B == 2) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int d = 0; d < 2; ++d) {           // byte (v & 1) * 2 + d of dword v >> 1
                const uint2 t = *(const uint2 *)(lds + byte_addr(w[v >> 1], (v & 1) * 2 + d, lane_off[v]));
                e[(v * 2 + d) * 2] = t.x;
                e[(v * 2 + d) * 2 + 1] = t.y;
            }
    } else if constexpr (B == 1) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {               // byte v of the single dword
            const uint4 t = *(const uint4 *)(lds + byte_addr(w[0], v, lane_off[v]));
            e[v * 4] = t.x;
            e[v * 4 + 1] = t.y;
            e[v * 4 + 2] = t.z;
            e[v * 4 + 3] = t.w;
        }
    } else {                                        // B == 3: one 24-bit group per v
        const uint32_t grp[4] = {
            w[0],
            __builtin_amdgcn_alignbit(w[1], w[0], 24),
            __builtin_amdgcn_alignbit(w[2], w[1], 16),
            w[2] >> 8,
        };
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int f = 0; f < 4; ++f) {           // field f: d = f >> 1, s2 = f & 1
                const uint32_t code = (grp[v] >> (6 * f)) & 63u;
                e[v * 4 + f] = *(const uint32_t *)(lds + (code << es) + lane_off[v]);
            }
    }
}

template <int B, bool BF16>
__device__ __forceinline__ void quarter_dots(const uint32_t (&e)[16], uint32_t xa, uint32_t xb,
                                             float (&acc)[8]) {
    if constexpr (B == 4 || B == 3) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[v * 2 + (j >> 1)] = dot2<BF16>(e[v * 4 + j], (j & 1) ? xb : xa, acc[v * 2 + (j >> 1)]);
    } else if constexpr (B == 2) {
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            acc[a] = dot2<BF16>(e[a * 2], xa, acc[a]);
            acc[a] = dot2<BF16>(e[a * 2 + 1], xb, acc[a]);
        }
    } else {
#pragma unroll
        for (int a = 0; a < 8; ++a) {               // a = v * 2 + d: dwords (z, w) of entry v for d = 1
            acc[a] = dot2<BF16>(e[a * 2], xa, acc[a]);
            acc[a] = dot2<BF16>(e[a * 2 + 1], xb, acc[a]);
        }
    }
}

// A wavefront-uniform pointer pinned into scalar registers.  Loads written as
// (uniform base + 32-bit lane offset) then keep that form; otherwise the loop
// optimiser turns every such load into its own 64-bit per-lane pointer, carried in
// vector registers across the K loop.
typedef const __attribute__((address_space(1))) uint8_t *GlobalBytes;
__device__ __forceinline__ GlobalBytes uniform_ptr(const uint8_t *ptr) {
    const uint64_t b = (uint64_t)ptr;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    return (GlobalBytes)(((uint64_t)hi << 32) | lo);      // global, not generic: no flat loads
}

template <int B>
__device__ __forceinline__ void load_quarter(uint32_t (&w)[B], GlobalBytes p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    typedef const __attribute__((address_space(1))) u32x4 *G16;
    typedef const __attribute__((address_space(1))) u32x2 *G8;
    typedef const __attribute__((address_space(1))) uint32_t *G4;
    if constexpr (B == 4) {
        const u32x4 v = *(G16)p;
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    } else if constexpr (B == 3) {
        G4 q = (G4)p;
        w[0] = q[0]; w[1] = q[1]; w[2] = q[2];
    } else if constexpr (B == 2) {
        const u32x2 v = *(G8)p;
        w[0] = v.x; w[1] = v.y;
    } else {
        w[0] = *(G4)p;
    }
}

// Eight consecutive floats (signs, scales), as two 16-byte loads when the array is
// 16-byte aligned (k is a multiple of 8).  Element-wise loads here each touch 64
// lanes x 4 bytes spread over 2 KB, and the vector memory pipe is then the bottleneck
// of the whole rotation.
__device__ __forceinline__ void load_f8(const float *src, int k, float (&v)[8]) {
    if (((uintptr_t)src & 15) == 0) {                  // uniform
        const float4 a = *(const float4 *)(src + k), b = *(const float4 *)(src + k + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = src[k + q];
    }
}

// Eight consecutive activations (16 bytes) as floats.
__device__ __forceinline__ void load_act8(const uint16_t *x, int k, int is_bf16, float (&f)[8]) {
    const uint4 v = *(const uint4 *)(x + k);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint16_t lo = (uint16_t)(w[j] & 0xffffu), hi = (uint16_t)(w[j] >> 16);
        f[2 * j] = is_bf16 ? bf2f(lo) : h2f(lo);
        f[2 * j + 1] = is_bf16 ? bf2f(hi) : h2f(hi);
    }
}

// xs holds kc bfloat16 values in natural order, written by every thread of the
// workgroup; converts them in place to float16 of x * 2^-shift and returns the shift.
// Barriers inside: before (the writes), between, and none after (the caller's next
// barrier publishes the result).
__device__ __forceinline__ int normalise_staged_row(uint16_t *xs, int kc, uint32_t *slots, int tid,
                                                    int nthreads) {
    __syncthreads();
    uint32_t e = 0;
    for (int j = tid * 8; j < kc; j += nthreads * 8) e = max(e, bf16_max_exp8(*(const uint4 *)(xs + j)));
    const int shift = bf16_row_shift(workgroup_max(e, slots, tid, nthreads));
    for (int j = tid * 8; j < kc; j += nthreads * 8)
        *(uint4 *)(xs + j) = bf16_to_f16_scaled8(*(const uint4 *)(xs + j), shift);
    return shift;
}

// Eight rotated values, divided by the AWQ scales where there are any, rounded to the activation
// type and packed.  The two conditions are uniform and sit outside the loops over the values: as
// selects inside them (which is what an `if` around one division becomes) every launch paid for the
// divisions and for both conversions, 25 vector instructions per value where 3 are needed.
__device__ __forceinline__ void pack_act8(float (&t)[8], const float *sc, int act_bf16, uint32_t (&o)[4]) {
    if (sc != nullptr) {
#pragma unroll
        for (int q = 0; q < 8; ++q) t[q] = t[q] / sc[q];
    }
    if (act_bf16) {
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = (uint32_t)f2bf(t[2 * q]) | ((uint32_t)f2bf(t[2 * q + 1]) << 16);
    } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = (uint32_t)f2h(t[2 * q]) | ((uint32_t)f2h(t[2 * q + 1]) << 16);
    }
}

// Output side of the fused rotation, eight columns per step: value * sign * inv
// (/ awq), rounded to the activation type exactly as the standalone kernel rounds,
// then converted to the compute type.  The eight sign (and scale) loads of a step are
// independent and issued together, so a step costs one memory round trip, not eight.
template <bool BF16>
__device__ __forceinline__ void rotated_out8(const float *buf, int j, const float *signs,
                                             const float *awq, int g, float inv, int act_bf16,
                                             uint16_t *dst) {
    float sg[8], sc[8];
    load_f8(signs, g, sg);
    if (awq) load_f8(awq, g, sc);
    uint32_t o[4];
    const int s0 = fht_slot(j);                        // j is a multiple of 8: slot(j + q) = s0 ^ q
    float t[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) t[q] = buf[s0 ^ q] * sg[q] * inv;
    pack_act8(t, awq ? sc : nullptr, act_bf16, o);
    *(uint4 *)dst = make_uint4(o[0], o[1], o[2], o[3]);
}

// Input side: eight activations (times the scale when compensated) into the swizzled
// fp32 buffer.
__device__ __forceinline__ void rotated_in8(float *buf, int j, const uint16_t *x, int g,
                                            const float *awq, int act_bf16) {
    float f[8], sc[8];
    load_act8(x, g, act_bf16, f);
    if (awq) {
        load_f8(awq, g, sc);
#pragma unroll
        for (int q = 0; q < 8; ++q) f[q] *= sc[q];
    }
    const int s0 = fht_slot(j);                        // j is a multiple of 8: slot(j + q) = s0 ^ q
#pragma unroll
    for (int q = 0; q < 8; ++q) buf[s0 ^ q] = f[q];
}

// Equal rotation blocks of at most 256 columns, without the fp32 LDS buffer: a thread
// holds eight consecutive columns, so the stages of length 1, 2, 4 are butterflies
// between its own registers, and the stages of length 8 .. block/2 pair it with the
// lane whose number differs in one bit (ds_swizzle, the LDS crossbar without a memory
// access).  The lower lane of a pair keeps a + b and the upper a - b, formed as
// fma(mine, +-1, other): the product is exact, so every value sees the same single
// rounding per stage, in the same ascending order, as in the buffered butterfly and
// the result is bit-identical.  The loads of all (at most two) steps of a thread go
// out before the first butterfly: one memory round trip for the whole rotation, no
// barrier.  Lanes of one block are in the same step, so a step's partners are active.
template <bool BF16>
__device__ __forceinline__ void rotate_blocks_inwave(const uint16_t *x, const float *signs,
                                                     const float *awq, uint16_t *xs, int k0,
                                                     int kc, int block, int act_bf16, int tid,
                                                     int nthreads) {
    const int nst = 31 - __builtin_clz((unsigned)block);
    const float inv = inv_sqrt_pow2(nst);
    const int lane = tid & 63;
    const int pair_lanes = block >> 3;                 // lanes of one block: 4 .. 32
    for (int j0 = tid * 8; j0 < kc; j0 += 2 * nthreads * 8) {
        float f[2][8], sg[2][8], sc[2][8];
        const int j1 = j0 + nthreads * 8;
        const bool two = j1 < kc;                      // same for every lane of a block
        load_act8(x, k0 + j0, act_bf16, f[0]);
        load_act8(x, k0 + (two ? j1 : j0), act_bf16, f[1]);
        load_f8(signs, k0 + j0, sg[0]);
        load_f8(signs, k0 + (two ? j1 : j0), sg[1]);
        if (awq) {
            load_f8(awq, k0 + j0, sc[0]);
            load_f8(awq, k0 + (two ? j1 : j0), sc[1]);
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                f[0][q] *= sc[0][q];
                f[1][q] *= sc[1][q];
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int len = 1; len < 8; len <<= 1) {
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    if ((q & len) == 0) {
                        const float a = f[h][q], c = f[h][q | len];
                        f[h][q] = a + c;
                        f[h][q | len] = a - c;
                    }
                }
            }
        }
        // and_mask 0x1f, or_mask 0, xor_mask m: lane ^ m inside each half of the wavefront
#define FLUTE_XOR_STAGE(m)                                                                   \
        if (pair_lanes > (m)) {                                                              \
            const float sgn = (lane & (m)) ? -1.0f : 1.0f;                                   \
            _Pragma("unroll") for (int h = 0; h < 2; ++h)                                    \
                _Pragma("unroll") for (int q = 0; q < 8; ++q) {                              \
                    const float other = __int_as_float(__builtin_amdgcn_ds_swizzle(          \
                        __float_as_int(f[h][q]), ((m) << 10) | 0x1f));                       \
                    f[h][q] = fmaf(f[h][q], sgn, other);                                     \
                }                                                                            \
        }
        FLUTE_XOR_STAGE(1)
        FLUTE_XOR_STAGE(2)
        FLUTE_XOR_STAGE(4)
        FLUTE_XOR_STAGE(8)
        FLUTE_XOR_STAGE(16)
#undef FLUTE_XOR_STAGE
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h == 1 && !two) break;
            uint32_t o[4];
            float t[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) t[q] = f[h][q] * sg[h][q] * inv;
            pack_act8(t, awq ? sc[h] : nullptr, act_bf16, o);   // (the activation type; the caller converts bf16 -> f16 if needed)
            *(uint4 *)(xs + (h ? j1 : j0)) = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
}

// One rotation segment of b = 512 .. 16 * nthreads columns starting at column `off`,
// all of it inside the staged slice.  The first nine stages (lengths 1 .. 256) run as
// in rotate_blocks_inwave, the last of them against the lane 32 away; what is left
// (lengths 512 .. b/2, at most four stages) is one pass over the fp32 buffer in LDS.
// Same butterflies in the same ascending order as fht_lds alone: bit-identical.
// Against the buffered transform this halves the LDS traffic, drops two of five
// barriers and needs one memory round trip instead of three.
template <bool BF16>
__device__ __forceinline__ void rotate_segment_fast(const uint16_t *x, const float *signs,
                                                    const float *awq, float *buf, uint16_t *xs,
                                                    int off, int xs_off, int b, int act_bf16,
                                                    int tid, int nthreads) {
    const int nst = 31 - __builtin_clz((unsigned)b);
    const float inv = inv_sqrt_pow2(nst);
    const int lane = tid & 63;
    const int j0 = tid * 8, j1 = j0 + nthreads * 8;
    const bool one = j0 < b, two = j1 < b;             // whole wavefronts: b/8 is a multiple of 64
    float f[2][8], sg[2][8], sc[2][8];
    if (one) {
        load_act8(x, off + j0, act_bf16, f[0]);
        load_act8(x, off + (two ? j1 : j0), act_bf16, f[1]);
        load_f8(signs, off + j0, sg[0]);
        load_f8(signs, off + (two ? j1 : j0), sg[1]);
        if (awq) {
            load_f8(awq, off + j0, sc[0]);
            load_f8(awq, off + (two ? j1 : j0), sc[1]);
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                f[0][q] *= sc[0][q];
                f[1][q] *= sc[1][q];
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int len = 1; len < 8; len <<= 1) {
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    if ((q & len) == 0) {
                        const float a = f[h][q], c = f[h][q | len];
                        f[h][q] = a + c;
                        f[h][q | len] = a - c;
                    }
                }
            }
        }
#define FLUTE_XOR_STAGE(m)                                                                   \
        {                                                                                    \
            const float sgn = (lane & (m)) ? -1.0f : 1.0f;                                   \
            _Pragma("unroll") for (int h = 0; h < 2; ++h)                                    \
                _Pragma("unroll") for (int q = 0; q < 8; ++q) {                              \
                    const float other = __int_as_float(__builtin_amdgcn_ds_swizzle(          \
                        __float_as_int(f[h][q]), ((m) << 10) | 0x1f));                       \
                    f[h][q] = fmaf(f[h][q], sgn, other);                                     \
                }                                                                            \
        }
        FLUTE_XOR_STAGE(1)
        FLUTE_XOR_STAGE(2)
        FLUTE_XOR_STAGE(4)
        FLUTE_XOR_STAGE(8)
        FLUTE_XOR_STAGE(16)
#undef FLUTE_XOR_STAGE
        {
            const float sgn = (lane & 32) ? -1.0f : 1.0f;
            const int partner = (lane ^ 32) << 2;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const float other = __int_as_float(
                        __builtin_amdgcn_ds_bpermute(partner, __float_as_int(f[h][q])));
                    f[h][q] = fmaf(f[h][q], sgn, other);
                }
        }
    }
    if (nst > 9) {                                     // uniform: stages of length 512 and up
        if (one) {
            const int s0 = fht_slot(j0), s1 = fht_slot(j1);
#pragma unroll
            for (int q = 0; q < 8; ++q) buf[s0 ^ q] = f[0][q];
            if (two) {
#pragma unroll
                for (int q = 0; q < 8; ++q) buf[s1 ^ q] = f[1][q];
            }
        }
        __syncthreads();
        switch (nst - 9) {
            case 1: fht_pass<1>(buf, b, 9, tid, nthreads); break;
            case 2: fht_pass<2>(buf, b, 9, tid, nthreads); break;
            case 3: fht_pass<3>(buf, b, 9, tid, nthreads); break;
            default: fht_pass<4>(buf, b, 9, tid, nthreads); break;
        }
        __syncthreads();
        if (one) {
            const int s0 = fht_slot(j0), s1 = fht_slot(j1);
#pragma unroll
            for (int q = 0; q < 8; ++q) f[0][q] = buf[s0 ^ q];
            if (two) {
#pragma unroll
                for (int q = 0; q < 8; ++q) f[1][q] = buf[s1 ^ q];
            }
        }
    }
    if (one) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h == 1 && !two) break;
            uint32_t o[4];
            float t[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) t[q] = f[h][q] * sg[h][q] * inv;
            pack_act8(t, awq ? sc[h] : nullptr, act_bf16, o);   // (the activation type; the caller converts bf16 -> f16 if needed)
            *(uint4 *)(xs + xs_off + (h ? j1 : j0)) = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
}

// Stage the activation slice [k0, k0 + kc) into LDS as 16-bit values of the
// compute type (the LUT's type), 16 bytes per thread per step so that the whole
// slice is one round trip to memory.  With signs, the rotation of every segment
// that overlaps the slice is computed first in the fp32 scratch at the start of
// LDS (where the tables are built afterwards), rounded to the activation type
// exactly as the standalone rotation kernel rounds, and only then converted.
// bfloat16 activations in front of a float16 LUT are scaled by a power of two on the
// way (normalise_staged_row); the shift is returned and is 0 otherwise.
// Ends with the slice complete and the scratch free (barrier included).
template <bool BF16>
__device__ int stage_x(const GemvParams &p, const uint16_t *x, const float *signs,
                       const float *awq, uint8_t *lds, int k0, int kc, int tid, int nthreads) {
    uint16_t *xs = (uint16_t *)(lds + p.lds_x);
    const bool convert = !BF16 && p.act_bf16;          // uniform
    auto finish = [&]() -> int {
        int shift = 0;
        if (convert)
            shift = normalise_staged_row(xs, kc, (uint32_t *)(lds + p.lds_red + kGemvRedBytes + 16),
                                         tid, nthreads);
        __syncthreads();
        return shift;
    };
    if (signs == nullptr) {
        for (int j = tid * 8; j < kc; j += nthreads * 8)
            *(uint4 *)(xs + j) = *(const uint4 *)(x + k0 + j);
        return finish();
    }
    float *buf = (float *)lds;
    if (p.fht_block > 0 && p.fht_block <= 256) {
        rotate_blocks_inwave<BF16>(x, signs, awq, xs, k0, kc, p.fht_block, p.act_bf16, tid, nthreads);
        return finish();
    }
    if (p.fht_block > 0) {
        // equal blocks: the slice is a whole number of blocks
#pragma unroll 2
        for (int j = tid * 8; j < kc; j += nthreads * 8)
            rotated_in8(buf, j, x, k0 + j, awq, p.act_bf16);
        __syncthreads();
        const int nst = 31 - __builtin_clz((unsigned)p.fht_block);
        fht_lds(buf, kc, nst, tid, nthreads);
        const float inv = inv_sqrt_pow2(nst);
#pragma unroll 2
        for (int j = tid * 8; j < kc; j += nthreads * 8)
            rotated_out8<BF16>(buf, j, signs, awq, k0 + j, inv, p.act_bf16, xs + j);
        return finish();
    }
    // descending power-of-two segments of K (fht.py:118-134 upstream)
    for (int off = 0, rem = p.K; rem > 0;) {
        const int nst = 31 - __builtin_clz((unsigned)rem);
        const int b = 1 << nst;
        const int lo = max(off, k0), hi = min(off + b, k0 + kc);
        if (lo < hi && lo == off && hi == off + b && b >= 512 && b <= 16 * nthreads &&
            (nthreads & 63) == 0 && nst <= 13) {
            rotate_segment_fast<BF16>(x, signs, awq, buf, xs, off, off - k0, b, p.act_bf16, tid,
                                      nthreads);
            __syncthreads();                       // scratch is reused by the next segment
        } else if (lo < hi) {                      // uniform across the workgroup
#pragma unroll 2
            for (int j = tid * 8; j < b; j += nthreads * 8)
                rotated_in8(buf, j, x, off + j, awq, p.act_bf16);
            __syncthreads();
            fht_lds(buf, b, nst, tid, nthreads);
            const float inv = inv_sqrt_pow2(nst);
            // lo, hi, off are multiples of 8 (segments and slices are multiples of 32)
#pragma unroll 2
            for (int k = lo + tid * 8; k < hi; k += nthreads * 8)
                rotated_out8<BF16>(buf, k - off, signs, awq, k, inv, p.act_bf16, xs + (k - k0));
            __syncthreads();                       // scratch is reused by the next segment
        }
        off += b;
        rem -= b;
    }
    return finish();
}

// Geometry of this lane inside its workgroup, fixed for the whole kernel.
struct LaneGeom {
    int tid, nthreads, w, nwaves, L;
    int gsub;        // which of the 64/LPG tiles of a wavefront load this lane reads
    int l;           // lane within the tile: (cg_local, i, kt)
    int t;           // 128-row tile
    int cg0;         // first chunk group of the row slice
    int cg;          // this lane's chunk group
    int g_lo;        // first 64-k tile of the K range
    int units;       // wavefront loads covering the K range
    int gpi;         // 64-k tiles per wavefront load
};

// Per-lane state of one stream pass between its phases.
template <int B>
struct StreamRegs {
    static constexpr int kPrefetch = B == 4 ? 4 : 8;   // loads in flight per lane (a unit is 4*B bytes of it)
    static constexpr int kEarly = B == 4 ? 1 : 2;      // loads issued ahead of the table build
    static constexpr int kEDW = 1 << (TableShape<B>::kEntryLog2 - 2);
    uint32_t q[kPrefetch][B];
    uint32_t val[kEDW];      // this thread's table entry (fast path)
    const uint8_t *qrow;
    uint32_t lane0, step;
    int my_units;
    int grp0, ngrp;
    bool fast_table;         // one (group, entry) item per thread: values already in val
};

// Phase 1 - global loads only: the first index bytes of this lane and the LUT
// values of the table entry this thread will write.  Nothing here waits.
template <int B>
__device__ __forceinline__ void stream_issue(const GemvParams &p, const GemvSeg &sg,
                                             const GemvStream &st, const LaneGeom &gm,
                                             StreamRegs<B> &r) {
    constexpr int E = TableShape<B>::kEntries;
    constexpr int PF = StreamRegs<B>::kPrefetch;
    const int G = p.K >> 6;
    // uniform 64-bit base of this tile row's K range + a 32-bit lane offset (a
    // tile row is at most 4 MB)
    r.qrow = st.q + ((size_t)gm.t * G + gm.g_lo) * (1024 * B);
    const uint32_t unit_bytes = (uint32_t)gm.gpi * (1024 * B);
    r.lane0 = (uint32_t)gm.gsub * (1024 * B) + (uint32_t)gm.cg0 * (64 * B) +
              (uint32_t)gm.l * (4 * B) + (uint32_t)gm.w * unit_bytes;
    r.step = (uint32_t)gm.nwaves * unit_bytes;
    // wavefront counts, group sizes, slices per tile and table sizes are powers of two:
    // shifts and masks instead of integer divisions throughout the prologue
    const int nw_log2 = __builtin_ctz(gm.nwaves);
    r.my_units = gm.units > gm.w ? (gm.units - gm.w + gm.nwaves - 1) >> nw_log2 : 0;
    const int gs = sg.gs;
    const int gs_log2 = __builtin_ctz(gs);
    const int ngrp_all = gs >= 128 ? 1 : 128 >> gs_log2;
    r.grp0 = min((gm.t * 128) >> gs_log2, sg.lut_rows - 1);
    r.ngrp = min(ngrp_all, sg.lut_rows - r.grp0);
    const int items = r.ngrp * E;
    r.fast_table = items <= gm.nthreads;
    if (r.fast_table) {
        const int item = (items & (items - 1)) == 0 ? (gm.tid & (items - 1)) : gm.tid % items;
        const uint16_t *lut = st.lut + ((size_t)(r.grp0 + item / E) << B);
#pragma unroll
        for (int s = 0; s < StreamRegs<B>::kEDW; ++s) r.val[s] = table_dword<B>(lut, item % E, s);
    }
    // Every load is unconditional (a wavefront with fewer than PF units re-reads the
    // first unit of the K range into the registers it will not consume), issued in
    // the order of use and addressed as a uniform base plus one lane-constant
    // offset: the compiler then knows how many loads are in flight at each point and
    // waits for exactly the one a unit needs.
    // Only the first kEarly loads go out here; the rest follow the table build
    // (stream_issue_rest).  A full batch ahead of it would put every other
    // workgroup's activation and LUT loads behind it in the CU's memory queue.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < StreamRegs<B>::kEarly; ++n) {
        const uint8_t *base = n < r.my_units ? r.qrow + (size_t)n * r.step
                                             : r.qrow - (size_t)gm.w * unit_bytes;
        load_quarter<B>(r.q[n], uniform_ptr(base) + r.lane0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int B>
__device__ __forceinline__ void stream_issue_rest(const LaneGeom &gm, StreamRegs<B> &r) {
    constexpr int PF = StreamRegs<B>::kPrefetch;
    const uint32_t unit_bytes = (uint32_t)gm.gpi * (1024 * B);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = StreamRegs<B>::kEarly; n < PF; ++n) {
        const uint8_t *base = n < r.my_units ? r.qrow + (size_t)n * r.step
                                             : r.qrow - (size_t)gm.w * unit_bytes;
        load_quarter<B>(r.q[n], uniform_ptr(base) + r.lane0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Phase 2 - expand the LUT rows into replicated paired tables at the start of
// LDS.  Table of group q starts at q * (E << es); entry e at e << es and repeats
// every entry-size bytes inside its stride.  A thread owns one (group, entry)
// and a share of its replicas; the walk starts at a lane-dependent replica so
// that a wavefront writes 64 different banks.
template <int B>
__device__ __forceinline__ void stream_tables(const GemvStream &st, const LaneGeom &gm,
                                              uint8_t *lds, const StreamRegs<B> &r) {
    constexpr int E = TableShape<B>::kEntries;
    constexpr int EL = TableShape<B>::kEntryLog2;
    constexpr int EDW = StreamRegs<B>::kEDW;
    const int es = st.es;
    const int items = r.ngrp * E;
    const int nrep = 1 << (es - EL);
    const bool pow2 = (items & (items - 1)) == 0;   // always, unless the LUT ends inside the tile
    const int items_log2 = 31 - __builtin_clz((unsigned)items);
    int shares = pow2 ? gm.nthreads >> items_log2 : gm.nthreads / items;
    if (shares < 1) shares = 1;
    if (shares > nrep) shares = nrep;
    const int per = pow2 ? nrep >> (31 - __builtin_clz((unsigned)shares)) : nrep / shares;
    for (int it = gm.tid; it < items * shares; it += gm.nthreads) {
        const int item = pow2 ? (it & (items - 1)) : it % items;
        const int share = pow2 ? it >> items_log2 : it / items;
        const int qg = item / E, e = item % E;
        uint32_t val[EDW];
        if (r.fast_table) {
#pragma unroll
            for (int s = 0; s < EDW; ++s) val[s] = r.val[s];
        } else {
            const uint16_t *lut = st.lut + ((size_t)(r.grp0 + qg) << B);
#pragma unroll
            for (int s = 0; s < EDW; ++s) val[s] = table_dword<B>(lut, e, s);
        }
        uint8_t *ent = lds + (size_t)qg * (E << es) + ((size_t)e << es);
        if (es >= 4) {
            // the replicas of an entry are contiguous: 16 bytes per store
            uint4 pat;
            if constexpr (EDW == 1) pat = make_uint4(val[0], val[0], val[0], val[0]);
            else if constexpr (EDW == 2) pat = make_uint4(val[0], val[1], val[0], val[1]);
            else pat = make_uint4(val[0], val[1], val[2], val[3]);
            const int pieces = (per << EL) >> 4;    // 16-byte pieces of this thread's share
            if (pieces > 0) {
                uint8_t *mine = ent + (size_t)share * per * (1 << EL);
                for (int k = 0; k < pieces; ++k)
                    *(uint4 *)(mine + (((k + gm.tid) & (pieces - 1)) << 4)) = pat;
                continue;
            }
        }
        for (int k = 0; k < per; ++k) {
            const int rep = share * per + ((k + gm.tid) & (per - 1));
            uint32_t *dst = (uint32_t *)(ent + (rep << EL));
#pragma unroll
            for (int s = 0; s < EDW; ++s) dst[s] = val[s];
        }
    }
}

// Phase 3 - stream the index bytes of this lane against the staged activations.
template <int B, bool BF16>
__device__ __forceinline__ void stream_loop(const GemvParams &p, const GemvSeg &sg,
                                            const GemvStream &st, const LaneGeom &gm,
                                            uint8_t *lds, StreamRegs<B> &r, float (&acc)[8]) {
    constexpr int E = TableShape<B>::kEntries;
    constexpr int EL = TableShape<B>::kEntryLog2;
    constexpr int PF = StreamRegs<B>::kPrefetch;
    const int es = st.es;
    const int gs = sg.gs;
    const int slot_mask = (1 << (es - EL)) - 1;
    uint32_t lane_off[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int row_local = (gm.cg >> 3) * 64 + v * 16;
        int qg = gs >= 128 ? 0 : row_local >> __builtin_ctz(gs);
        qg = min(qg, r.ngrp - 1);
        lane_off[v] = (uint32_t)(qg * (E << es) + ((gm.L & slot_mask) << EL));
    }
    const uint32_t *xs32 = (const uint32_t *)(lds + p.lds_x);
    const int xi = gm.gsub * 32 + (gm.l & 3) * 8 + ((gm.l >> 2) & 3);   // + unit * gpi * 32
    auto lookups = [&](const uint32_t (&wq)[B], uint32_t (&e)[16]) {
        quarter_lookups<B>(wq, lds, lane_off, es, e);
    };
    // The staged activations of consecutive units of this wavefront are xstep
    // dwords apart; one running index serves every unit (a separate address per
    // unrolled unit would be hoisted out of the loop and held in registers).
    const int xstep = gm.nwaves * gm.gpi * 32;
    int xo = gm.w * gm.gpi * 32 + xi;
    auto dots = [&](const uint32_t (&e)[16]) {
        quarter_dots<B, BF16>(e, xs32[xo], xs32[xo + 4], acc);
        xo += xstep;
        asm volatile("" : "+v"(xo));                          // keep it one running register
    };
    // The loop is cut so that every load inside its main part is unconditional; a
    // conditional refill in a loop makes the compiler wait for all loads in flight
    // at the loop head, which serialises the memory stream and the arithmetic.
    const int U = r.my_units;
    int nb = 0;
    __builtin_amdgcn_s_setprio(2);
    for (; nb + 2 * PF <= U; nb += PF) {                      // every refill exists
#pragma unroll
        for (int n = 0; n < PF; ++n) {
            uint32_t e[16];
            lookups(r.q[n], e);
            __builtin_amdgcn_sched_barrier(0);                // refills stay where they are
            load_quarter<B>(r.q[n], uniform_ptr(r.qrow + (size_t)(nb + n + PF) * r.step) + r.lane0);
            __builtin_amdgcn_sched_barrier(0);
            dots(e);
        }
    }
    if (nb + PF >= U) {                                       // the last group, no refills
#pragma unroll
        for (int n = 0; n < PF; ++n) {
            if (nb + n < U) {                                 // uniform within the wavefront
                uint32_t e[16];
                lookups(r.q[n], e);
                dots(e);
            }
        }
    } else {
        // A unit count that is not a multiple of PF: the rest runs with conditional
        // refills (and the early waits they cause).
        for (; nb < U; nb += PF) {
#pragma unroll
            for (int n = 0; n < PF; ++n) {
                const int m = nb + n;
                if (m < U) {
                    uint32_t e[16];
                    lookups(r.q[n], e);
                    if (m + PF < U)
                        load_quarter<B>(r.q[n], uniform_ptr(r.qrow + (size_t)(m + PF) * r.step) + r.lane0);
                    dots(e);
                }
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                       // vmcnt(0): nothing is in flight any more
}

// One stream pass whose loads were not issued ahead: all three phases in a row.
// Ends with a barrier so that the table region may be rewritten.
template <int B, bool BF16>
__device__ void run_stream(const GemvParams &p, const GemvSeg &sg, const GemvStream &st,
                           const LaneGeom &gm, uint8_t *lds, float (&acc)[8]) {
    StreamRegs<B> r;
    stream_issue<B>(p, sg, st, gm, r);
    stream_tables<B>(st, gm, lds, r);
    stream_issue_rest<B>(gm, r);
    __syncthreads();
    stream_loop<B, BF16>(p, sg, st, gm, lds, r, acc);
    __syncthreads();
}

// BFIX = 1..4: every stream of the launch has this width (the common case, one
// instantiation per width); BFIX = 10 * b1 + b2: every weight's first stream is b1 bits wide
// and its second one, where it has one, b2 (the mixed pairs of deployed artifacts: the code of
// two widths only, which keeps the kernel in the register budget of three wavefronts per SIMD);
// BFIX == 0: any mix, chosen per stream at run time (all four widths inlined: it spills).
template <bool BF16, int BFIX>
__device__ __forceinline__ void run_stream_any(const GemvParams &p, const GemvSeg &sg,
                                               const GemvStream &st, const LaneGeom &gm,
                                               uint8_t *lds, float (&acc)[8], int si) {
    if constexpr (BFIX >= 10) {
        if (si == 0) run_stream<BFIX / 10, BF16>(p, sg, st, gm, lds, acc);
        else run_stream<BFIX % 10, BF16>(p, sg, st, gm, lds, acc);
        return;
    } else if constexpr (BFIX != 0) {
        run_stream<BFIX, BF16>(p, sg, st, gm, lds, acc);
        return;
    }
    switch (st.bits) {
        case 4: run_stream<4, BF16>(p, sg, st, gm, lds, acc); break;
        case 3: run_stream<3, BF16>(p, sg, st, gm, lds, acc); break;
        case 2: run_stream<2, BF16>(p, sg, st, gm, lds, acc); break;
        default: run_stream<1, BF16>(p, sg, st, gm, lds, acc); break;
    }
}

// Tile-local row of accumulator a of chunk group cg.
__device__ __forceinline__ int row_of(int cg, int a) {
    return (cg >> 3) * 64 + (a >> 1) * 16 + (a & 1) * 8 + (cg & 7);
}

template <bool BF16, int BFIX>
__global__ void __launch_bounds__(kGemvMaxThreads, 3) gemv_kernel(const GemvParams p) {
    extern __shared__ __align__(16) uint8_t lds[];

    // Read the weight descriptors straight from the kernel-argument segment
    // (constant address space): a dynamic index then costs a scalar load with an
    // offset instead of a select chain over every field of every descriptor.
    const GemvParams *kp = (const GemvParams *)(const void *)__builtin_amdgcn_kernarg_segment_ptr();
    warm_kernargs<(int)sizeof(GemvParams)>(kp);
    // Wavefront priority falls as a workgroup advances (3 in the prologue, 2 in the
    // K loops, 0 from the last fold on): a SIMD serves its oldest wavefront first, and
    // the workgroup that arrived last on a CU would otherwise lag through the launch.
    __builtin_amdgcn_s_setprio(3);
    int si0 = 0;
    if (!p.silu_mul) {
#pragma unroll
        for (int i = 1; i < kGemvMaxSegs; ++i)
            if (i < p.nsegs && (int)blockIdx.x >= p.seg[i].col0) si0 = i;
    }
    const GemvSeg sg = kp->seg[si0];

    LaneGeom gm;
    gm.tid = threadIdx.x;
    gm.nthreads = blockDim.x;
    gm.w = __builtin_amdgcn_readfirstlane(gm.tid >> 6);
    gm.nwaves = gm.nthreads >> 6;
    gm.L = gm.tid & 63;
    const int lpg = 1 << p.lpg_log2;
    gm.gsub = gm.L >> p.lpg_log2;
    gm.l = gm.L & (lpg - 1);
    gm.gpi = 64 >> p.lpg_log2;
    const int rw = lpg >> 1;                        // rows per workgroup
    const int spt = 128 / rw;                       // row slices per tile
    int sl = (int)blockIdx.x - sg.col0;
    const int spt_log2 = 8 - p.lpg_log2;            // spt = 128 / rw = 256 >> lpg_log2
    if (p.xcd_runs) {                               // a contiguous run of this weight's slices per XCD
        const int per = ((sg.N >> 7) << spt_log2) >> 3;
        sl = (sl & 7) * per + (sl >> 3);
    }
    gm.t = sl >> spt_log2;
    gm.cg0 = (sl & (spt - 1)) * (rw >> 3);
    gm.cg = gm.cg0 + (gm.l >> 4);
    const int s = blockIdx.y;
    gm.g_lo = s * p.gs_tiles;
    gm.units = p.gs_tiles >> (6 - p.lpg_log2);      // gpi = 64 >> lpg_log2
    const int k0 = gm.g_lo * 64, kc = p.gs_tiles * 64;

    float *red = (float *)(lds + p.lds_red);        // [2][nwaves][32] row sums
    const int nout = p.silu_mul ? 2 : 1;
    // With one width for the whole launch and a plain (unrotated) input, the first
    // pass issues its loads in the order activations, LUT values, index bytes before
    // anything is staged, so that the three kinds travel together and each consumer
    // waits only for what was issued before it.  A rotated input is staged first: the
    // rotation needs most of the register file, and index loads held across it would
    // be spilled (and waited for) on the spot.
    constexpr int BF = BFIX >= 10 ? BFIX / 10 : (BFIX != 0 ? BFIX : 4);   // width of a first stream
    constexpr int XV = 2;                           // 16-byte activation loads per thread
    StreamRegs<BF> first;
    const uint16_t *x0 = sg.xsrc ? sg.xsrc : p.x;
    // bfloat16 activations with a float16 LUT are scaled on the way into LDS: that needs
    // the whole slice first, so such launches stage through stage_x
    const bool x_ahead = BFIX != 0 && sg.signs == nullptr && !(!BF16 && p.act_bf16);   // uniform
    int xshift = 0;                                 // the staged slice holds x * 2^-xshift
    if (x_ahead) {
        uint4 xv[XV];
#pragma unroll
        for (int i = 0; i < XV; ++i) {
            const int j = (i * gm.nthreads + gm.tid) * 8;
            xv[i] = *(const uint4 *)(x0 + k0 + (j < kc ? j : 0));
        }
        if constexpr (BFIX != 0) stream_issue<BF>(p, sg, sg.st[0], gm, first);
        uint16_t *xs = (uint16_t *)(lds + p.lds_x);
#pragma unroll
        for (int i = 0; i < XV; ++i) {
            const int j = (i * gm.nthreads + gm.tid) * 8;
            if (j < kc) *(uint4 *)(xs + j) = xv[i];
        }
        for (int j = (XV * gm.nthreads + gm.tid) * 8; j < kc; j += gm.nthreads * 8)
            *(uint4 *)(xs + j) = *(const uint4 *)(x0 + k0 + j);
        // no barrier here: the one after the table build publishes both
    } else {
        xshift = stage_x<BF16>(p, x0, sg.signs, sg.awq, lds, k0, kc, gm.tid, gm.nthreads);
        if constexpr (BFIX != 0) stream_issue<BF>(p, sg, sg.st[0], gm, first);
    }
    int out_shift[2] = {0, 0};
    const uint16_t *staged_x = x0;
    const float *staged_signs = sg.signs, *staged_awq = sg.awq;

    for (int so = 0; so < nout; ++so) {
        const GemvSeg og = kp->seg[so == 1 ? 1 : si0];
        const uint16_t *xin = og.xsrc ? og.xsrc : p.x;
        if (so > 0 && (xin != staged_x || og.signs != staged_signs || og.awq != staged_awq)) {
            xshift = stage_x<BF16>(p, xin, og.signs, og.awq, lds, k0, kc, gm.tid, gm.nthreads);
            staged_x = xin;
            staged_signs = og.signs;
            staged_awq = og.awq;
        }
        out_shift[so] = xshift;
        float acc[8];
#pragma unroll
        for (int a = 0; a < 8; ++a) acc[a] = 0.0f;
        for (int si = 0; si < og.nstreams; ++si) {
            const GemvStream st = kp->seg[so == 1 ? 1 : si0].st[si];
            if (BFIX != 0 && so == 0 && si == 0) {
                if constexpr (BFIX != 0) {
                    stream_tables<BF>(st, gm, lds, first);
                    stream_issue_rest<BF>(gm, first);
                    __syncthreads();
                    stream_loop<BF, BF16>(p, og, st, gm, lds, first, acc);
                    __syncthreads();
                }
            } else {
                run_stream_any<BF16, BFIX>(p, og, st, gm, lds, acc, si);
            }
        }

        // fold the lanes that share rows: 16 (i, kt) lanes, then the tiles of a load
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            float v = row16_sum(acc[a]);
            if (p.lpg_log2 <= 5) v += __shfl_xor(v, 32);
            if (p.lpg_log2 == 4) v += __shfl_xor(v, 16);
            acc[a] = v;
        }
        if (gm.L < lpg && (gm.L & 15) == 0) {
#pragma unroll
            for (int a = 0; a < 8; ++a)
                red[(so * gm.nwaves + gm.w) * 32 + (gm.L >> 4) * 8 + a] = acc[a];
        }
    }
    __builtin_amdgcn_s_setprio(0);
    __syncthreads();

    // ---- one thread per owned row: fold the wavefronts in fixed order ----------
    const bool owner = gm.tid < rw;
    const int cg_o = gm.cg0 + (gm.tid >> 3);
    const int n = gm.t * 128 + row_of(cg_o, gm.tid & 7);
    float yv[2] = {0.0f, 0.0f};
    if (owner) {
#pragma unroll
        for (int so = 0; so < 2; ++so) {
            if (so >= nout) break;
            float y = 0.0f;
            for (int w = 0; w < gm.nwaves; ++w) y += red[(so * gm.nwaves + w) * 32 + gm.tid];
            yv[so] = ldexpf(y, out_shift[so]);      // undo the activation scaling (exact)
        }
    }

    if (p.split > 1) {
        // publish the partials of this K range, take a ticket, let the last
        // arrival finish the rows
        int *flag = (int *)(red + 2 * gm.nwaves * 32);
        if (owner) {
#pragma unroll
            for (int so = 0; so < 2; ++so) {
                if (so >= nout) break;
                const int og_n0 = kp->seg[so == 1 ? 1 : si0].n0;
                ws_store(p.P + (size_t)s * p.p_stride + og_n0 + n, yv[so]);
            }
        }
        // the stores are acknowledged by the device-coherent level before the ticket
        ws_stores_done();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (gm.tid == 0) {
            const int old = __hip_atomic_fetch_add(p.tickets + sg.ticket0 + sl, 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
            *flag = (old == p.split - 1);
        }
        __syncthreads();
        if (!*flag) return;
        if (owner) {
#pragma unroll
            for (int so = 0; so < 2; ++so) {
                if (so >= nout) break;
                const float *col = p.P + kp->seg[so == 1 ? 1 : si0].n0 + n;
                float y = 0.0f;
                for (int sb = 0; sb < p.split; sb += 8) {     // 8 independent loads in flight
                    float part[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        part[j] = (sb + j < p.split) ? ws_load(col + (size_t)(sb + j) * p.p_stride)
                                                     : 0.0f;
#pragma unroll
                    for (int j = 0; j < 8; ++j) y += part[j];
                }
                yv[so] = y;
            }
        }
        if (gm.tid == 0)
            __hip_atomic_store(p.tickets + sg.ticket0 + sl, 0, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }

    if (owner) {
#pragma unroll
        for (int so = 0; so < 2; ++so) {
            if (so >= nout) break;
            const GemvSeg og = kp->seg[so == 1 ? 1 : si0];
            float y = yv[so];
            if (og.R > 0) {
                const uint16_t *ra = og.resA + (size_t)n * og.R;
                for (int r = 0; r < og.R; ++r)
                    y = fmaf(og.xb[r], p.act_bf16 ? bf2f(ra[r]) : h2f(ra[r]), y);
            }
            if (og.bias) y += p.act_bf16 ? bf2f(og.bias[n]) : h2f(og.bias[n]);
            yv[so] = y;
        }
        float y = yv[0];
        if (p.silu_mul) y = (yv[0] / (1.0f + expf(-yv[0]))) * yv[1];
        sg.out[n] = round_act(y, p.act_bf16);
    }
}

}  // namespace flute
