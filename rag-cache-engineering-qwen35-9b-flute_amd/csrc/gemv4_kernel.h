// Lean specialisation of the M = 1 LUT GEMV for the common case: every stream
// 4 bits wide and one LUT group per 128-row tile (group_size >= 128).  Same
// ownership, table format and K-split protocol as gemv_kernel.h; what differs is
// how a looked-up weight pair meets the activations.
//
// Matrix cores instead of dot products.  The K loop is bound by the rate at which
// a CU issues LDS lookups (about one wavefront lookup per nanosecond), so every
// vector instruction next to a lookup costs time.  The looked-up pairs are
// therefore fed to v_mfma_f32_16x16x32 as they come out of the table:
//   * lane L = (kg, rb, kt) = (L >> 4, (L >> 2) & 3, L & 3) reads quarter kt of
//     chunk (cg0 + cgl, kg) of tile gsub, where rb = (gsub, cgl) splits by the
//     slice width.  Four lanes with equal L >> 2 read 64 contiguous bytes and a
//     wavefront load covers 1 KB of whole 64-byte pieces.
//   * a 16-byte load holds, per row (v, d) of the lane's eight rows, the bytes
//     s2 = 0, 1 = four consecutive-pair k values.  Two loads give eight k values
//     per row: one A operand of the 16x16x32 product per (v, d), whose matrix row
//     is i = (rb, kt) and whose k block is kg.
//   * the k values of a lane depend on kt, which is part of the matrix row.  The B
//     operand therefore carries, in column j = (rb', kt'), the activations of
//     quarter kt' of tile gsub(rb'): the product D[i][j] is the wanted partial sum
//     where kt' = kt and gsub(rb') = gsub(rb), and the other columns are ignored.
//     The matrix cores are idle otherwise, so the unused columns cost nothing.
//   * D[i][j] sits in lane (j + 16 * (i >> 2)), register i & 3: the lanes with
//     rb' = rb keep register kt', a quad sum folds kt', and one LDS exchange folds
//     the tiles of a load and the wavefronts.
// Per weight pair this leaves two address instructions and the lookup; the
// multiply-accumulate and the cross-lane reduction of the dot-product form are gone.
//
// Activations are staged per wavefront: a wavefront loads, converts and stores exactly
// the units of K it will read back, so the only workgroup barrier of the prologue is the
// one that publishes the table, and a power-of-two scale (bfloat16 activations in front
// of a float16 LUT) is a wavefront-local matter.
//
// The LUT row (32 bytes) comes through the scalar cache, so it does not queue
// behind the index loads of the other workgroups of the CU in the vector memory
// pipe; index loads are non-temporal (read once).
//
// Walking grids (template argument WALK).  A launch with more row slices than workgroups
// fit the device at once (very wide outputs) is started as one resident workgroup per slot;
// with four slices or more each a workgroup takes a contiguous run of them (consecutive
// slices mostly share a 128-row tile, hence the LUT row, and the table is then kept instead
// of rebuilt; the partial row sums alternate between two LDS areas so that the barrier
// which would publish the table can go too), with fewer it takes b, b + gridDim.x, ...
// It stages the activations once; the change of slice is handled like the change of stream
// inside a slice: the next slice's LUT row and first index loads are requested under the
// last products of the current one, the owners of the finished rows fold and store them
// while the other wavefronts go on.  The sums of a row are formed in the same order as in
// a one-slice launch.
#pragma once

#include <type_traits>

#include "gemv_kernel.h"

#ifdef FLUTE_STAMPS
// Instrumented builds only: per-wavefront phase times of the lean kernel (s_memrealtime, 10 ns
// units), written to the buffer flute_debug_gemv_stamps() was given; gemv_phase_stamps.py reads them.
// (One copy of the pointer per translation unit: the setter reaches the instantiations of gemv.hip.)
__device__ long long *g_gemv_stamps = nullptr;
#define FLUTE_GEMV_STAMP(slot)                                                                  \
    do {                                                                                        \
        if (g_gemv_stamps && (threadIdx.x & 63) == 0)                                           \
            g_gemv_stamps[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x / 64) * 8 + \
                          (threadIdx.x >> 6) * 8 + (slot)] =                                    \
                (long long)__builtin_amdgcn_s_memrealtime();                                    \
    } while (0)
#else
#define FLUTE_GEMV_STAMP(slot) do { } while (0)
#endif

namespace flute {

typedef _Float16 gv_h8_t __attribute__((ext_vector_type(8)));
typedef __bf16 gv_bf8_t __attribute__((ext_vector_type(8)));
typedef float gv_f4_t __attribute__((ext_vector_type(4)));
typedef uint32_t gv_u4_t __attribute__((ext_vector_type(4)));

template <bool BF16>
__device__ __forceinline__ gv_f4_t gv_mfma(gv_u4_t a, gv_u4_t b, gv_f4_t c) {
    if constexpr (BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gv_bf8_t, a),
                                                       __builtin_bit_cast(gv_bf8_t, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(gv_h8_t, a),
                                                      __builtin_bit_cast(gv_h8_t, b), c, 0, 0, 0);
    }
}

// The value that lane (CTRL & 3) of this lane's quad holds (CTRL = that lane number in all four
// two-bit fields of a quad_perm control).
template <int CTRL>
__device__ __forceinline__ float quad_lane(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Index bytes are read once: non-temporal loads, so they do not displace the activations
// and LUT rows that every workgroup shares from the caches.
// One quarter of a chunk of a B-bit stream: 16 pairs of codes, 4 * B bytes, read once.
template <int B>
struct IdxQuarter {
    uint32_t d[B];
};
template <int B>
__device__ __forceinline__ IdxQuarter<B> load_idx(const uint8_t *p) {
    typedef uint32_t vec_t __attribute__((ext_vector_type(B == 3 ? 3 : B)));
    typedef const __attribute__((address_space(1))) vec_t *GlobalVec;              // global, not flat
    IdxQuarter<B> r;
    if constexpr (B == 1) {
        typedef const __attribute__((address_space(1))) uint32_t *GlobalWord;
        r.d[0] = __builtin_nontemporal_load((GlobalWord)(uintptr_t)p);
    } else {
        const vec_t v = __builtin_nontemporal_load((GlobalVec)(uintptr_t)p);
#pragma unroll
        for (int i = 0; i < B; ++i) r.d[i] = v[i];
    }
    return r;
}
// The 2B-bit code of pair pp (0..15) of a quarter (all indices constant after unrolling).
template <int B>
__device__ __forceinline__ uint32_t quarter_code(const IdxQuarter<B> &q, int pp) {
    const int bit = 2 * B * pp, dw = bit >> 5, sh = bit & 31;
    if (sh + 2 * B <= 32) return __builtin_amdgcn_ubfe(q.d[dw], sh, 2 * B);
    return __builtin_amdgcn_alignbit(q.d[dw + 1 < B ? dw + 1 : dw], q.d[dw], sh) & ((1u << (2 * B)) - 1u);
}

// One LUT row of 2^B 16-bit values through the scalar cache (the pointer is
// wavefront-uniform and 4-byte aligned); dwords beyond the row stay zero.
template <int B = 4>
__device__ __forceinline__ void load_lut_row(const uint16_t *lut, uint32_t (&d)[8]) {
    typedef const __attribute__((address_space(4))) uint32_t *ConstWord;
    ConstWord p = (ConstWord)(const void *)lut;
#pragma unroll
    for (int i = 0; i < 8; ++i) d[i] = i < (1 << B) / 2 ? p[i] : 0u;
}

// Value c (0..15) of a LUT row held as eight uniform dwords.
__device__ __forceinline__ uint32_t lut_value(const uint32_t (&d)[8], int c) {
    const int i = c >> 1;
    const uint32_t a = (i & 1) ? d[1] : d[0], b = (i & 1) ? d[3] : d[2];
    const uint32_t e = (i & 1) ? d[5] : d[4], f = (i & 1) ? d[7] : d[6];
    const uint32_t ab = (i & 2) ? b : a, ef = (i & 2) ? f : e;
    const uint32_t w = (i & 4) ? ef : ab;
    return (c & 1) ? (w >> 16) : (w & 0xffffu);
}

// Eight consecutive columns of an equal-block rotation held by one lane, block/8 lanes side
// by side: the stages of length 1, 2, 4 are butterflies between the lane's own values, the
// longer ones pair it with the lane one bit away (ds_swizzle) as in rotate_blocks_inwave,
// with the same single rounding per stage, so the result is bit-identical to the standalone
// rotation; sign, scale 1/sqrt(block) and the rounding to the activation type included.
template <bool ACT_BF16>
__device__ __forceinline__ void rotate_piece(uint4 &v, const float (&sg)[8], const float (&sc)[8],
                                             bool has_awq, float inv, int pair_lanes, int lane) {
    float f[8];
    const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint16_t lo = (uint16_t)(wv[e] & 0xffffu), hi = (uint16_t)(wv[e] >> 16);
        f[2 * e] = ACT_BF16 ? bf2f(lo) : h2f(lo);
        f[2 * e + 1] = ACT_BF16 ? bf2f(hi) : h2f(hi);
    }
    if (has_awq) {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] *= sc[e];
    }
#pragma unroll
    for (int len = 1; len < 8; len <<= 1) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if ((e & len) == 0) {
                const float a = f[e], c = f[e | len];
                f[e] = a + c;
                f[e | len] = a - c;
            }
        }
    }
    // and_mask 0x1f, or_mask 0, xor_mask m: lane ^ m inside each half of the wavefront
#define FLUTE_XOR_STAGE(m)                                                                   \
    if (pair_lanes > (m)) {                                                                  \
        const float sgn = (lane & (m)) ? -1.0f : 1.0f;                                       \
        _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                      \
            const float other = __int_as_float(__builtin_amdgcn_ds_swizzle(                  \
                __float_as_int(f[e]), ((m) << 10) | 0x1f));                                  \
            f[e] = fmaf(f[e], sgn, other);                                                   \
        }                                                                                    \
    }
    FLUTE_XOR_STAGE(1)
    FLUTE_XOR_STAGE(2)
    FLUTE_XOR_STAGE(4)
    FLUTE_XOR_STAGE(8)
    FLUTE_XOR_STAGE(16)
#undef FLUTE_XOR_STAGE
    uint32_t o[4];
    float t[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) t[e] = f[e] * sg[e] * inv;
    pack_act8(t, has_awq ? sc : nullptr, ACT_BF16 ? 1 : 0, o);   // the standalone kernel's rounding
    v = make_uint4(o[0], o[1], o[2], o[3]);
}

// a | byte J of w, in one instruction (the compiler's own choice is a shift and an and-or).
template <int J>
__device__ __forceinline__ uint32_t or_byte(uint32_t a, uint32_t w) {
    uint32_t r;
    if constexpr (J == 0)
        asm("v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(a), "v"(w));
    else if constexpr (J == 1)
        asm("v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(a), "v"(w));
    else if constexpr (J == 2)
        asm("v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(a), "v"(w));
    else
        asm("v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(a), "v"(w));
    return r;
}

// A LUT grouped along K: 16-byte pieces of LUT rows a thread stages at most.
constexpr int kKGroupPieces = 8;

// LPGL = log2(lanes per 64-k tile) = log2(2 * rows per workgroup): 4, 5, 6.
// NW   = wavefronts per workgroup (4 or 8).
// PF   = index loads a lane keeps in flight (2 or 4).  The host picks a PF that
//        divides the loads of a wavefront, which it makes equal for all wavefronts
//        and even (two loads feed one matrix product).
// The table stride is 128 bytes (32 replicas of a 4-byte entry, 32 KB): three
// four-wavefront workgroups fit a CU.
// WALK: the instantiation for resident grids that walk over the row slices (p.slices > 0);
// launches of one workgroup per slice use the one without that control path.
// BA, BB: widths of every weight's first stream and (where it has one) second stream.  (4, 4) is
// the kernel described above: one table, rebuilt between the passes.  Any other pair (the mixed
// pairs of deployed artifacts, (3, 3)) has small tables: both are built before an output's first
// loop (the first at offset 0, the second behind it) and the two K loops run back to back, with
// no barrier and no table build between them.
// KG: the LUT is grouped along K instead of along N: one row of sixteen values per (output row,
// 128-wide K group), W[n, k] = LUT[n][k / 128][idx[n, k]] (a variant no upstream artifact has;
// single weight, one 4-bit stream).  No pair table then (it would be 1 KB per 128 weights): the
// workgroup stages the LUT rows of its row slice and K range in LDS, group-major, every 16-bit
// value widened to a dword that holds it in both halves (rows 64 bytes apart), and a weight is one
// 32-bit read at (code * 4) in its row; two reads are joined with one bit-field insert.  (16-bit
// LDS reads of a half-size table measured four times slower per read than 32-bit ones.)  A row is
// sixteen dwords on sixteen different banks and equal dwords are broadcast, so the lanes of a
// lookup (two rows per wavefront instruction, padded onto the other sixteen banks) do not conflict.
// DEEP (two tables, PF = 4, a 1-bit first stream): that stream keeps eight loads in flight instead
// of four.  Its loads are four bytes per lane, so a group of four is consumed long before its
// refill can be back; the deeper ring costs four registers.  The host picks it when a wavefront's
// loads are a multiple of eight ((1, 4) at 4096 -> 12288: 10.5 -> 9.7 us; with the 1-bit stream
// second it measured no gain, so the host puts it first).
template <int LPGL, int NW, int PF, bool BF16, bool WALK = false, int BA = 4, int BB = 4, bool KG = false,
          bool DEEP = false>
__global__ void __launch_bounds__(NW * 64, 3) gemv4_kernel(const GemvParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int ES = 7;
    constexpr int NT = NW * 64;
    constexpr int LPG = 1 << LPGL;
    constexpr int GPI = 64 >> LPGL;                 // 64-k tiles per wavefront load
    constexpr int RW = LPG >> 1;                    // rows per workgroup
    constexpr int SPT = 128 / RW;                   // row slices per tile
    constexpr int SH = LPGL - 4;                    // bits of rb that pick the chunk group
    constexpr int XV = 4;                           // 16-byte activation loads a lane holds at once
    constexpr int PF0 = 2;                          // index loads issued ahead of the table build
    constexpr int STRIDE = 1 << ES;                 // table bytes per entry
    constexpr int CHUNKS = STRIDE / 16;             // 16-byte pieces of one entry's replicas
    constexpr int SHARES = NT / 256;                // threads per table entry
    constexpr int CPT = CHUNKS / SHARES;            // pieces written per thread
    static_assert(NT >= 256, "one thread per table entry at least");
    static_assert(PF % 2 == 0 && PF >= PF0, "loads are consumed in pairs");
    static_assert(!WALK || NW == 4, "the alternating sum areas of a walking grid are sized for four wavefronts");
    constexpr bool TWO = !(BA == 4 && BB == 4);     // two resident tables
    static_assert(!TWO || !WALK, "walking grids: the (4, 4) kernel");
    static_assert(!KG || (!TWO && !WALK), "K-grouped LUTs: one 4-bit stream, one slice per workgroup");
    static_assert(!DEEP || (TWO && PF == 4 && BA == 1), "the deep ring is for a 1-bit first stream");
    constexpr int DA = (DEEP && BA == 1) ? 2 * PF : PF;  // loads in flight, first / second stream
    constexpr int DB = (DEEP && BB == 1) ? 2 * PF : PF;
    constexpr int KG_GROUP = RW * 64 + (RW / 8) * 64;   // LDS bytes of one K group's rows
    // A 1-bit stream (two tables only) is looked up a nibble at a time: four weights of one row =
    // two operand dwords from one 8-byte entry, sixteen entries, 32 replicas 8 bytes apart (4 KB).
    // Half the lookups and address instructions of the pair-at-a-time form.
    constexpr int TAB1 = 16 * 256;
    constexpr int TAB_A = (TWO && BA == 1) ? TAB1 : (1 << (2 * BA)) * STRIDE;  // bytes of the first table

    FLUTE_GEMV_STAMP(0);
    const GemvParams *kp = (const GemvParams *)(const void *)__builtin_amdgcn_kernarg_segment_ptr();
    warm_kernargs<(int)sizeof(GemvParams)>(kp);
    // several independent weights in one launch: the descriptor is picked by grid column
    int si0 = 0;
    if (p.nsegs > 1 && !p.silu_mul) {
#pragma unroll
        for (int i = 1; i < kGemvMaxSegs; ++i)
            if (i < p.nsegs && (int)blockIdx.x >= p.seg[i].col0) si0 = i;
    }

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int L = tid & 63;
    const int kg = L >> 4, rb = (L >> 2) & 3, kt = L & 3;
    const int gsub = rb >> SH;                      // tile of the load this lane reads
    const int cgl = rb & ((1 << SH) - 1);           // chunk group inside the row slice
    // The row slice of this workgroup.  A walking workgroup keeps the staged activations and
    // takes, from four slices per workgroup on, a contiguous run of the p.slices slices (the
    // first p.slices % gridDim.x workgroups one more than the others): consecutive slices
    // mostly lie in one 128-row tile and then share their LUT row, i.e. their table.  With
    // fewer slices each it takes blockIdx.x, + gridDim.x, ...: the neighbours then read the
    // four slices of a tile at the same time, which the memory system likes better.
    constexpr bool walk = WALK;                     // unsplit launches of one column space
    int sl = (int)blockIdx.x - kp->seg[si0].col0;
    if (!walk && p.xcd_runs) {
        // Consecutive workgroups go to consecutive XCDs.  Every XCD takes a contiguous run of slices
        // instead of every eighth one: the slices of a 128-row tile (their pieces of each 4 KB
        // index tile, their LUT row) then meet in one L2.  Measured 1 - 5 % (most on narrow outputs).
        // (per weight of a grouped launch: the host checks that every weight's slices come in eights)
        const int per = ((kp->seg[si0].N >> 7) * SPT) >> 3;
        sl = (sl & 7) * per + (sl >> 3);
    }
    int sl_end = sl + 1, sl_step = 1;
    if constexpr (walk) {
        const int per = p.slices / (int)gridDim.x, extra = p.slices % (int)gridDim.x;
        const int b = (int)blockIdx.x;
        if (per >= 4 && p.xcd_runs) {
            // an eighth of the slices per XCD, divided evenly over its workgroups: the runs of an
            // XCD lie side by side and every XCD streams the same share
            const int x = b & 7, j = b >> 3, nx = (int)gridDim.x >> 3;
            const int each = p.slices >> 3, odd = p.slices & 7;
            const int first = x * each + min(x, odd), count = each + (x < odd ? 1 : 0);
            const int per_x = count / nx, extra_x = count % nx;
            sl = first + j * per_x + min(j, extra_x);
            sl_end = sl + per_x + (j < extra_x ? 1 : 0);
        } else if (per >= 4) {
            sl = b * per + min(b, extra);
            sl_end = sl + per + (b < extra ? 1 : 0);
        } else {
            sl_end = p.slices;
            sl_step = (int)gridDim.x;
        }
    }
    const int s = blockIdx.y;
    const int g_lo = s * p.gs_tiles;
    const int units = p.gs_tiles / GPI;
    const int my_units = units / NW;                // the host makes this exact, even, >= PF
    const int k0 = g_lo * 64, kc = p.gs_tiles * 64;
    const int G = p.K >> 6;

    uint16_t *xs = (uint16_t *)(lds + p.lds_x);
    float *red = (float *)(lds + p.lds_red);        // [2][NW][4][8] partial row sums

    // lane-constant pieces of the addresses
    // (a B-bit stream: tiles of 1024 * B bytes, chunk groups of 64 * B, chunks of 16 * B,
    // quarters of 4 * B)
    const uint32_t lane_unit = (uint32_t)gsub * 1024u + (uint32_t)cgl * 64u + (uint32_t)kg * 16u +
                               (uint32_t)kt * 4u + (uint32_t)w * (GPI * 1024u);
    const uint32_t lane0 = lane_unit * BA, lane0B = lane_unit * BB;
    constexpr uint32_t step = NW * GPI * 1024u * BA, stepB = NW * GPI * 1024u * BB;
    // Lookup addresses are formed as absolute LDS addresses, so the (zero) base of
    // the dynamic LDS block is folded into the per-lane replica offset once.
    typedef const __attribute__((address_space(3))) uint32_t *LdsWord;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    // The kernel has no static LDS, so its dynamic block starts at address 0 and a lane's slot
    // stays below the table stride: (code << 7) and the slot share no bits, which lets the
    // address of byte 0 be formed as shift + and-or, two instructions like the other bytes.
    __builtin_assume(lds_base == 0);
    const uint32_t slot = lds_base + (uint32_t)(L & 31) * 4u;
    const uint32_t slot1 = lds_base + (uint32_t)(L & 31) * 8u;       // (nibble table of a 1-bit stream)
    const uint32_t slotA = (TWO && BA == 1) ? slot1 : slot;
    const uint32_t slotB = ((TWO && BB == 1) ? slot1 : slot) + (TWO ? TAB_A : 0);
    const int e_own = tid & 255;                    // table entry this thread writes
    const int share = tid >> 8;

    const int nout = p.silu_mul ? 2 : 1;

    // A pass is one (output, stream) of this workgroup's rows: one output with one
    // stream for a plain weight, two streams for a dual-stream weight, two outputs
    // for the gate/up pair.  Every pass covers the same K range with the same lane
    // geometry; only the index blob and the LUT row change.
    auto pass_ptrs = [&](int sl_, int so_, int si_, const uint8_t *&qr, const uint16_t *&lutp) {
        const int sg = so_ == 1 ? 1 : si0;
        const GemvStream st = kp->seg[sg].st[si_];
        const int t = sl_ / SPT, cg0 = (sl_ % SPT) * (RW >> 3);
        const int grp = min((t * 128) >> __builtin_ctz(kp->seg[sg].gs), kp->seg[sg].lut_rows - 1);
        const int B = si_ ? BB : BA;
        qr = st.q + ((size_t)t * G + g_lo) * (1024u * B) + (uint32_t)cg0 * (64u * B);
        lutp = st.lut + ((size_t)grp << B);
    };
    // Index loads are addressed as (uniform base + unit offset) in scalar registers
    // plus one lane-constant 32-bit offset, so no per-load address lives in vector
    // registers; every load is unconditional, so the compiler knows how many are in
    // flight at each point and waits for exactly the ones a product needs.
    auto first_units = [&](const uint8_t *qr, IdxQuarter<BA> (&qq)[DA], int from) {
#pragma unroll
        for (int n = 0; n < DA; ++n) {
            if (n >= from) {
                qq[n] = load_idx<BA>(qr + (size_t)n * step + lane0);
                __builtin_amdgcn_sched_barrier(0);  // issue order = consumption order
            }
        }
    };

    // Paired table: entry e -> {lut[e & 15], lut[e >> 4]}, replicated over the stride;
    // 16 bytes per store, starting at a lane-dependent piece so that a wavefront
    // spreads over the banks.
    auto write_table = [&](const uint32_t (&row)[8]) {
        const uint32_t v = lut_value(row, e_own & 15) | (lut_value(row, e_own >> 4) << 16);
        const uint4 v4 = make_uint4(v, v, v, v);
        uint8_t *ent = lds + e_own * STRIDE + share * (CPT * 16);
#pragma unroll
        for (int k = 0; k < CPT; ++k) *(uint4 *)(ent + (((k + tid) & (CPT - 1)) << 4)) = v4;
    };
    // A table of a narrower stream (4^B entries, at most 64): one thread per entry writes all
    // the replicas of its entry.
    auto write_small_table = [&](const uint32_t (&row)[8], auto width, uint32_t base) {
        constexpr int B = decltype(width)::value;
        if constexpr (B == 1) {
            if (tid < 16) {                         // entry = four bits b0..b3 -> {l[b0] l[b1]} {l[b2] l[b3]}
                const uint32_t lo = lut_value(row, tid & 1) | (lut_value(row, (tid >> 1) & 1) << 16);
                const uint32_t hi = lut_value(row, (tid >> 2) & 1) | (lut_value(row, tid >> 3) << 16);
                const uint4 v4 = make_uint4(lo, hi, lo, hi);
                uint8_t *ent = lds + base + tid * 256;
#pragma unroll
                for (int k = 0; k < 16; ++k) *(uint4 *)(ent + (((k + tid) & 15) << 4)) = v4;
            }
            return;
        }
        if (tid < (1 << (2 * B))) {
            const uint32_t v = lut_value(row, tid & ((1 << B) - 1)) | (lut_value(row, tid >> B) << 16);
            const uint4 v4 = make_uint4(v, v, v, v);
            uint8_t *ent = lds + base + tid * STRIDE;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) *(uint4 *)(ent + (((k + tid) & (CHUNKS - 1)) << 4)) = v4;
        }
    };
    // K-grouped LUT: the rows of this slice for the K groups of this launch's K range, 16 bytes
    // per piece, consecutive threads on consecutive pieces of a row in memory.  At most eight
    // pieces per thread (the host checks); a thread beyond the end re-reads piece 0.
    constexpr int KG_MAX = kKGroupPieces;
    uint4 slab_v[KG ? KG_MAX : 1];
    const int kg_row_pieces = (kc >> 7) * 2;        // 16-byte pieces of one row's K groups of the range
    const int kg_pieces = RW * kg_row_pieces;
    // piece tid + i NT = (row kg_r, piece kg_pc of the row), stepped without a division per piece:
    // one division for the thread's first piece, the step NT = (kg_dr rows, kg_dp pieces) is uniform
    int kg_r = 0, kg_pc = 0;
    const int kg_dr = __builtin_amdgcn_readfirstlane(NT / max(kg_row_pieces, 1));
    const int kg_dp = NT - kg_dr * kg_row_pieces;
    auto slab_issue = [&]() {
        if constexpr (KG) {
            const int t0 = sl / SPT, cg0 = (sl % SPT) * (RW >> 3);
            const uint16_t *lutk = kp->seg[si0].st[0].lut + ((size_t)(k0 >> 7) << 4);
            const int row_stride = (p.K >> 7) << 4;             // 16-bit values per output row
            int r = tid / kg_row_pieces, pc = tid - r * kg_row_pieces;
            kg_r = r;
            kg_pc = pc;
#pragma unroll
            for (int i = 0; i < KG_MAX; ++i) {
                if (i * NT < kg_pieces) {                       // (uniform: whole rounds beyond the end are skipped)
                    const bool in = r < RW;                     // (the last round: threads beyond the end re-read piece 0)
                    const int rr = in ? r : 0, pp = in ? pc : 0;
                    const int n = t0 * 128 + row_of(cg0 + (rr >> 3), rr & 7);
                    slab_v[i] = *(const uint4 *)(lutk + (size_t)n * row_stride + pp * 8);
                    r += kg_dr;
                    pc += kg_dp;
                    if (pc >= kg_row_pieces) {
                        pc -= kg_row_pieces;
                        ++r;
                    }
                }
            }
        }
    };
    auto slab_write = [&]() {
        if constexpr (KG) {
            int r = kg_r, pc = kg_pc;
#pragma unroll
            for (int i = 0; i < KG_MAX; ++i) {
                if (i * NT < kg_pieces) {
                    if (r < RW) {
                        // eight 16-bit values -> eight dwords, each value in both halves
                        const uint4 v = slab_v[i];
                        auto both = [](uint32_t two, int hi) -> uint32_t {
                            return hi ? (two >> 16) | (two & 0xffff0000u) : (two & 0xffffu) | (two << 16);
                        };
                        uint8_t *dst = lds + (pc >> 1) * KG_GROUP + r * 64 + (r >> 3) * 64 + (pc & 1) * 32;
                        *(uint4 *)dst = make_uint4(both(v.x, 0), both(v.x, 1), both(v.y, 0), both(v.y, 1));
                        *(uint4 *)(dst + 16) = make_uint4(both(v.z, 0), both(v.z, 1), both(v.w, 0), both(v.w, 1));
                    }
                    r += kg_dr;
                    pc += kg_dp;
                    if (pc >= kg_row_pieces) {
                        pc -= kg_row_pieces;
                        ++r;
                    }
                }
            }
        }
    };
    // the tables of one output: the first stream's, and (two resident tables) the second's
    auto write_tables = [&](const uint32_t (&rowA)[8], const uint32_t (&rowB)[8], bool second) {
        if constexpr (KG) {
            slab_write();
            return;
        }
        if constexpr (BA == 4) write_table(rowA);
        else write_small_table(rowA, std::integral_constant<int, BA>(), 0u);
        if constexpr (TWO) {
            if (second) {
                if constexpr (BB == 4) {
                    // (a 4-bit second stream behind a narrow first one: the full-size writer at the
                    // second table's base)
                    const uint32_t v = lut_value(rowB, e_own & 15) | (lut_value(rowB, e_own >> 4) << 16);
                    const uint4 v4 = make_uint4(v, v, v, v);
                    uint8_t *ent = lds + TAB_A + e_own * STRIDE + share * (CPT * 16);
#pragma unroll
                    for (int k = 0; k < CPT; ++k) *(uint4 *)(ent + (((k + tid) & (CPT - 1)) << 4)) = v4;
                } else {
                    write_small_table(rowB, std::integral_constant<int, BB>(), (uint32_t)TAB_A);
                }
            }
        }
    };

    // Activations in operand order: for load unit u (GPI tiles) the 8 bytes
    // {k, k+1, k+8, k+9} of (kg, tile, kt) lie together, so a lane reads the B half of
    // a product as one 8-byte LDS word.  Eight consecutive activations (one tile,
    // quarter and s2; kg = 0..3) scatter to four such words.
    auto stage8 = [&](int j, uint4 v) {
        const int g = j >> 6, kk = j & 63;
        const int u = g / GPI, gs_ = g % GPI;
        uint32_t *dst = (uint32_t *)xs + u * (32 * GPI) + ((gs_ * 4 + (kk >> 4)) << 1) + ((kk >> 3) & 1);
        dst[0] = v.x;
        dst[GPI * 8] = v.y;
        dst[GPI * 16] = v.z;
        dst[GPI * 24] = v.w;
    };

    // Wavefront priority falls as a workgroup advances: 3 in the prologue, 2 while
    // there is more to stream, 1 in the last group, 0 from the fold on.  A SIMD holds
    // one wavefront of each resident workgroup and serves the oldest first; without
    // this the workgroup that arrived last on a CU lags through the whole launch.
    __builtin_amdgcn_s_setprio(3);
    int so = 0, si = 0;
    const uint8_t *qrow;
    const uint16_t *lut;
    pass_ptrs(sl, 0, 0, qrow, lut);
    uint32_t lrow[8], lrowB[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
    if constexpr (!KG) load_lut_row<BA>(lut, lrow);
    bool second0 = false;                           // two tables: this output has a second stream
    if constexpr (TWO) {
        second0 = kp->seg[si0].nstreams == 2;
        if (second0) {
            const uint8_t *q_unused;
            const uint16_t *lutB;
            pass_ptrs(sl, 0, 1, q_unused, lutB);
            load_lut_row<BB>(lutB, lrowB);
        }
    }
    const uint16_t *staged_x = kp->seg[si0].xsrc ? kp->seg[si0].xsrc : p.x;
    const float *staged_signs = kp->seg[si0].signs, *staged_awq = kp->seg[si0].awq;
    const bool x_plain = staged_signs == nullptr;   // plain copy
    IdxQuarter<BA> q[DA];
    IdxQuarter<BB> q2[DB];
    // bfloat16 activations in front of a float16 LUT: the staged units hold x * 2^-xshift,
    // xshift chosen per wavefront (per workgroup when the input is rotated)
    const bool convert = !BF16 && p.act_bf16;       // uniform
    int xshift = 0;
    // A wavefront stages the units it consumes (unit m of wavefront w is unit w + m * NW of
    // the K range): a 16-byte piece per lane, UPL units per wavefront load.
    constexpr int UPL = 8 / GPI;                    // units per wavefront load
    constexpr int LPU = 64 / UPL;                   // lanes (16-byte pieces) per unit
    const int xu = L / LPU, xp = L % LPU;
    auto x_piece = [&](int i) -> int {              // local k of piece i of this lane, or -1
        const int m = i * UPL + xu;
        return m < my_units ? (w + m * NW) * (64 * GPI) + xp * 8 : -1;
    };
    const int x_loads = (my_units + UPL - 1) / UPL;
    const bool x_short = x_loads <= XV;             // uniform
    // Equal rotation blocks that fit a unit of K (the block-128 form) are transformed by the
    // wavefront that consumes the unit, in the registers its pieces arrive in: sixteen lanes
    // hold a block of 128 columns eight to a lane, exactly the arrangement of the butterflies
    // in rotate_blocks_inwave, so the rotated launch keeps the wavefront-local staging (no
    // workgroup barrier, operand order) of the plain one.
    const bool rot_inwave = !x_plain && x_short && p.fht_block >= 16 && p.fht_block <= 64 * GPI;
    const bool x_direct = x_plain || rot_inwave;    // staged in operand order
    // Eight-wavefront workgroups (one or two per CU) pass the barrier that publishes the table
    // before they wait for their activations, which every wavefront stages for itself: each then
    // starts its loop when its own loads are in instead of when the slowest of the eight has staged
    // (12288 -> 4096: 8.15 -> 7.94 us, 4096 -> 1024: 4.55 -> 4.45 us).  Four-wavefront workgroups,
    // three to a CU, measured 2 % slower that way and keep the barrier behind the staging.
    constexpr bool EARLY = !KG && !TWO && NW == 8;
    bool early_done = false;
    if (x_direct && x_short) {
        // The usual case: activations first, then two index loads, the table (its LUT
        // row arrives through the scalar cache meanwhile), the rest of the loads, and
        // the activations into LDS.
        uint4 xv[XV];
#pragma unroll
        for (int i = 0; i < XV; ++i) {
            const int j = x_piece(i);
            xv[i] = *(const uint4 *)(staged_x + k0 + (j >= 0 ? j : 0));
        }
        // signs and scales of a rotated input travel with the activations, ahead of the index
        // bytes: waiting for them then does not mean waiting for the index loads
        float sgv[XV][8], scv[XV][8];
        if (rot_inwave) {
#pragma unroll
            for (int i = 0; i < XV; ++i) {
                if (i >= x_loads) break;
                const int j = x_piece(i);
                load_f8(staged_signs, k0 + (j >= 0 ? j : 0), sgv[i]);
                if (staged_awq) load_f8(staged_awq, k0 + (j >= 0 ? j : 0), scv[i]);
            }
        }
        slab_issue();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < PF0; ++n) {
            q[n] = load_idx<BA>(qrow + (size_t)n * step + lane0);
            __builtin_amdgcn_sched_barrier(0);
        }
        FLUTE_GEMV_STAMP(1);                        // (waits for the scalar loads: the LUT row is in)
        write_tables(lrow, lrowB, second0);
        FLUTE_GEMV_STAMP(2);
        first_units(qrow, q, PF0);
        if (EARLY) {
            __syncthreads();
            early_done = true;
        }
        if (rot_inwave) {
            const int nst = 31 - __builtin_clz((unsigned)p.fht_block);
            const float inv = inv_sqrt_pow2(nst);
            const int pair_lanes = p.fht_block >> 3;    // lanes of one block: 2 .. 32
#pragma unroll
            for (int i = 0; i < XV; ++i) {
                if (i >= x_loads) break;
                if (p.act_bf16) rotate_piece<true>(xv[i], sgv[i], scv[i], staged_awq != nullptr, inv, pair_lanes, L);
                else rotate_piece<false>(xv[i], sgv[i], scv[i], staged_awq != nullptr, inv, pair_lanes, L);
            }
        }
        if (convert) {
            uint32_t m = 0;
#pragma unroll
            for (int i = 0; i < XV; ++i)
                if (i < x_loads) m = bf16_max_mag8(m, xv[i]);  // idle lanes hold piece 0 of the slice: harmless
            const uint32_t emax = wavefront_max(bf16_mag_exp(m));
            if (emax == 255) {                      // an infinity or a NaN: keep it
#pragma unroll
                for (int i = 0; i < XV; ++i) xv[i] = bf16_to_f16_scaled8(xv[i], 0);
            } else {
                const uint32_t adj = emax > 30 ? emax - 30 : 0;
                xshift = (int)adj - 112;
#pragma unroll
                for (int i = 0; i < XV; ++i)
                    if (i < x_loads) xv[i] = bf16_to_f16_top8(xv[i], adj);
            }
        }
#pragma unroll
        for (int i = 0; i < XV; ++i) {
            const int j = i < x_loads ? x_piece(i) : -1;
            if (j >= 0) stage8(j, xv[i]);
        }
        FLUTE_GEMV_STAMP(3);
    } else if (x_plain) {
        // A long K range: two passes over this wavefront's pieces when a scale is needed
        // (the second one reads them from the cache).
        uint32_t adj = 0;
        bool finite = true;                         // uniform
        if (convert) {
            uint32_t m = 0;
            for (int i = 0; i < x_loads; ++i) {
                const int j = x_piece(i);
                if (j >= 0) m = bf16_max_mag8(m, *(const uint4 *)(staged_x + k0 + j));
            }
            const uint32_t emax = wavefront_max(bf16_mag_exp(m));
            finite = emax != 255;
            adj = (finite && emax > 30) ? emax - 30 : 0;
            if (finite) xshift = (int)adj - 112;
        }
        for (int i = 0; i < x_loads; ++i) {
            const int j = x_piece(i);
            if (j >= 0) {
                const uint4 v = *(const uint4 *)(staged_x + k0 + j);
                stage8(j, !convert ? v : finite ? bf16_to_f16_top8(v, adj) : bf16_to_f16_scaled8(v, 0));
            }
        }
        slab_issue();
        write_tables(lrow, lrowB, second0);
        __builtin_amdgcn_sched_barrier(0);
        first_units(qrow, q, 0);
    } else {
        // A rotated input: the rotation leaves the slice in natural order; the first
        // index loads travel while it runs.
#pragma unroll
        for (int n = 0; n < PF0; ++n) {
            q[n] = load_idx<BA>(qrow + (size_t)n * step + lane0);
            __builtin_amdgcn_sched_barrier(0);
        }
        xshift = stage_x<BF16>(p, staged_x, staged_signs, staged_awq, lds, k0, kc, tid, NT);
        slab_issue();
        write_tables(lrow, lrowB, second0);
        __builtin_amdgcn_sched_barrier(0);
        first_units(qrow, q, PF0);
    }

    gv_f4_t acc[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) acc[a] = (gv_f4_t){0.0f, 0.0f, 0.0f, 0.0f};

    const uint2 *xs64 = (const uint2 *)xs;
    const uint32_t *xs32 = (const uint32_t *)xs;
    const int xoff = (kg * GPI + gsub) * 4 + kt;    // operand order: 8-byte word of this lane
    const int xnat = gsub * 32 + kt * 8 + kg;       // natural order: first dword of this lane

    // ---- one thread per owned row: fold the wavefronts and the tiles of a load, then the
    //      residual, the bias, the gate and the store -----------------------------------
    const int cgl_o = tid >> 3, a_o = tid & 7;
    auto row_n = [&](int sl_) -> int {
        return (sl_ / SPT) * 128 + row_of((sl_ % SPT) * (RW >> 3) + cgl_o, a_o);
    };
    auto fold_rows = [&](float (&yv)[2], int par_) {
        yv[0] = yv[1] = 0.0f;
#pragma unroll
        for (int so = 0; so < 2; ++so) {
            if (so >= nout) break;
            float y = 0.0f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww)
#pragma unroll
                for (int gb = 0; gb < GPI; ++gb)
                    y += red[par_ * (2 * NW * 32) + (so * NW + ww) * 32 + ((gb << SH) | cgl_o) * 8 + a_o];
            yv[so] = y;
        }
    };
    auto finish_rows = [&](int sl_, float (&yv)[2]) {
        const int n = row_n(sl_);
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
        kp->seg[si0].out[n] = round_act(y, p.act_bf16);
    };

    // ---- K loop pieces, generic in the width of the stream ----------------------------------
    // One step = two units (two loads of this lane) = 32 lookups and 8 matrix products.
    auto operand_b = [&](int m0, int m1) -> gv_u4_t {
        const int u0 = w + m0 * NW, u1 = w + m1 * NW;
        if (x_direct) {
            const uint2 xa = xs64[u0 * (16 * GPI) + xoff], xb = xs64[u1 * (16 * GPI) + xoff];
            return (gv_u4_t){xa.x, xa.y, xb.x, xb.y};
        }
        const int a0 = u0 * (32 * GPI) + xnat, a1 = u1 * (32 * GPI) + xnat;
        return (gv_u4_t){xs32[a0], xs32[a0 + 4], xs32[a1], xs32[a1 + 4]};
    };
    // per row group v, eight lookups feed two matrix products; pair pp = v * 4 + d * 2 + s2 of a
    // quarter, an operand is (s2 = 0, 1) of both units
    // (K-grouped LUT: ga, gb = LDS byte offsets of the two units' K groups plus this lane's rows)
    auto unit_pair = [&](const auto &qa, const auto &qb, gv_u4_t Bop, uint32_t tslot, auto width,
                         uint32_t ga = 0, uint32_t gb = 0) {
        constexpr int B = decltype(width)::value;
        if constexpr (KG) {
            // Row group v needs sixteen 16-bit reads (dword v of both units: four bytes of two
            // codes).  Their addresses are formed while the reads of group v - 1 are in flight, and
            // the reads go out behind that group's products: address arithmetic, LDS round trip
            // and matrix products of neighbouring groups overlap instead of following each other.
            auto addresses = [&](int v, uint32_t (&ad)[16]) {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint32_t wq = u ? qb.d[v] : qa.d[v];
                    const uint32_t base = (u ? gb : ga) + (uint32_t)(2 * v * 64);
                    // Entry offsets (code * 4) of the four low and the four high codes, one to a
                    // byte: two instructions per set, then one byte-select OR per address (a row
                    // of entries is 64 bytes and 64-byte aligned, so OR is the sum).
                    const uint32_t lo = (wq << 2) & 0x3c3c3c3cu, hi = (wq >> 2) & 0x3c3c3c3cu;
                    // byte j of the dword: row 2 v + (j >> 1), the two codes of one pair
                    ad[u * 8 + 0] = or_byte<0>(base, lo);
                    ad[u * 8 + 1] = or_byte<0>(base, hi);
                    ad[u * 8 + 2] = or_byte<1>(base, lo);
                    ad[u * 8 + 3] = or_byte<1>(base, hi);
                    ad[u * 8 + 4] = or_byte<2>(base, lo) + 64u;
                    ad[u * 8 + 5] = or_byte<2>(base, hi) + 64u;
                    ad[u * 8 + 6] = or_byte<3>(base, lo) + 64u;
                    ad[u * 8 + 7] = or_byte<3>(base, hi) + 64u;
                }
            };
            auto reads = [&](const uint32_t (&ad)[16], uint32_t (&r)[16]) {
#pragma unroll
                for (int i = 0; i < 16; ++i) r[i] = *(LdsWord)ad[i];
            };
            auto products = [&](int v, const uint32_t (&r)[16]) {
                // (every dword holds its value in both halves: low half of one, high half of the other)
                auto pr = [&](int i) -> uint32_t { return (r[2 * i] & 0xffffu) | (r[2 * i + 1] & 0xffff0000u); };
                // pairs 0..3: unit a, bytes 0..3; pairs 4..7: unit b
                const gv_u4_t A0 = {pr(0), pr(1), pr(4), pr(5)};
                const gv_u4_t A1 = {pr(2), pr(3), pr(6), pr(7)};
                acc[v * 2] = gv_mfma<BF16>(A0, Bop, acc[v * 2]);
                acc[v * 2 + 1] = gv_mfma<BF16>(A1, Bop, acc[v * 2 + 1]);
            };
            uint32_t ad[16], r[16];
            addresses(0, ad);
            reads(ad, r);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if (v < 3) addresses(v + 1, ad);
                __builtin_amdgcn_sched_barrier(0);
                products(v, r);
                __builtin_amdgcn_sched_barrier(0);
                if (v < 3) reads(ad, r);
                __builtin_amdgcn_sched_barrier(0);
            }
            return;
        }
        if constexpr (B == 1) {
            typedef uint32_t pair_t __attribute__((ext_vector_type(2)));
            typedef const __attribute__((address_space(3))) pair_t *LdsPair;
            const uint32_t wa = qa.d[0], wb = qb.d[0];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                // byte v of the quarter: low nibble = the four weights of row 2 v, high nibble = row 2 v + 1
                const pair_t a0 = *(LdsPair)((__builtin_amdgcn_ubfe(wa, 8 * v, 4) << 8) + tslot);
                const pair_t a1 = *(LdsPair)((__builtin_amdgcn_ubfe(wa, 8 * v + 4, 4) << 8) + tslot);
                const pair_t b0 = *(LdsPair)((__builtin_amdgcn_ubfe(wb, 8 * v, 4) << 8) + tslot);
                const pair_t b1 = *(LdsPair)((__builtin_amdgcn_ubfe(wb, 8 * v + 4, 4) << 8) + tslot);
                const gv_u4_t A0 = {a0.x, a0.y, b0.x, b0.y};
                const gv_u4_t A1 = {a1.x, a1.y, b1.x, b1.y};
                acc[v * 2] = gv_mfma<BF16>(A0, Bop, acc[v * 2]);
                acc[v * 2 + 1] = gv_mfma<BF16>(A1, Bop, acc[v * 2 + 1]);
            }
            return;
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            auto look = [&](const IdxQuarter<B> &qq, int j) -> uint32_t {
                if constexpr (B == 4 && !TWO) {
                    // a whole byte of dword v; byte 0: shift, then one and-or (the slot lies
                    // below the stride, the table at offset 0)
                    const uint32_t wq = qq.d[v];
                    if (j == 0) return *(LdsWord)(((wq << ES) & (0xffu << ES)) | tslot);
                    return *(LdsWord)((((wq >> (8 * j)) & 0xffu) << ES) + tslot);
                } else {
                    return *(LdsWord)((quarter_code<B>(qq, v * 4 + j) << ES) + tslot);
                }
            };
            const gv_u4_t A0 = {look(qa, 0), look(qa, 1), look(qb, 0), look(qb, 1)};
            const gv_u4_t A1 = {look(qa, 2), look(qa, 3), look(qb, 2), look(qb, 3)};
            acc[v * 2] = gv_mfma<BF16>(A0, Bop, acc[v * 2]);
            acc[v * 2 + 1] = gv_mfma<BF16>(A1, Bop, acc[v * 2 + 1]);
        }
    };
    // K-grouped LUT: LDS offset of unit m's K group (tile (w + m NW) GPI + gsub of the range, two
    // tiles per group) plus this lane's first row (chunk group cgl: eight rows and one pad).
    auto kg_off = [&](int m) -> uint32_t {
        if constexpr (!KG) return 0u;
        return (uint32_t)((((w + m * NW) * GPI + gsub) >> 1) * KG_GROUP + cgl * (8 * 64 + 64));
    };
    // The K range of one stream of width B held in qc, refilled from qcur; the last group's
    // registers are refilled with the first loads of what follows: a stream of width BN from
    // qnext into qn (nothing when last).
    auto k_loop = [&](auto &qc, const uint8_t *qcur, uint32_t lane_c, uint32_t step_c, uint32_t tslot,
                      auto width, auto &qn, const uint8_t *qnext, uint32_t lane_n, uint32_t step_n,
                      auto width_next, bool has_next, bool output_ends = true) {
        constexpr int B = decltype(width)::value, BN = decltype(width_next)::value;
        // the ring depths are the extents of the register arrays
        constexpr int D = (int)(sizeof(qc) / sizeof(qc[0])), DN = (int)(sizeof(qn) / sizeof(qn[0]));
        int nb = 0;
        __builtin_amdgcn_s_setprio(2);
        for (; nb + 2 * D <= my_units; nb += D) {            // every refill exists
#pragma unroll
            for (int n = 0; n < D; n += 2) {
                const gv_u4_t Bop = operand_b(nb + n, nb + n + 1);
                unit_pair(qc[n], qc[n + 1], Bop, tslot, width, kg_off(nb + n), kg_off(nb + n + 1));
                __builtin_amdgcn_sched_barrier(0);
                qc[n] = load_idx<B>(qcur + (size_t)(nb + n + D) * step_c + lane_c);
                qc[n + 1] = load_idx<B>(qcur + (size_t)(nb + n + 1 + D) * step_c + lane_c);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (!has_next && output_ends) __builtin_amdgcn_s_setprio(1);
        if (has_next) {
#pragma unroll
            for (int n = 0; n < D; n += 2) {
                const gv_u4_t Bop = operand_b(nb + n, nb + n + 1);
                unit_pair(qc[n], qc[n + 1], Bop, tslot, width, kg_off(nb + n), kg_off(nb + n + 1));
                __builtin_amdgcn_sched_barrier(0);
                if (n < DN) {
                    qn[n] = load_idx<BN>(qnext + (size_t)n * step_n + lane_n);
                    qn[n + 1] = load_idx<BN>(qnext + (size_t)(n + 1) * step_n + lane_n);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int n = D; n < DN; ++n) qn[n] = load_idx<BN>(qnext + (size_t)n * step_n + lane_n);
        } else {
#pragma unroll
            for (int n = 0; n < D; n += 2) {
                const gv_u4_t Bop = operand_b(nb + n, nb + n + 1);
                unit_pair(qc[n], qc[n + 1], Bop, tslot, width, kg_off(nb + n), kg_off(nb + n + 1));
            }
        }
        if (!has_next && output_ends) __builtin_amdgcn_s_setprio(0);
    };
    // ---- end of an output: D[i][j] with i = (rb, kt) in (lane >> 4, register) and
    //      j = (rb', kt') in lane & 15.  The lanes with rb' == rb keep register kt';
    //      a quad sum folds kt'; the activation scaling is undone here (exact). -----
    auto end_of_output = [&](int so_, int par_) {
        const bool keep = rb == kg;                 // here L >> 4 is the matrix row block
        float v[8];
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            // lane kt' of a quad holds the wanted term in register kt': each register is
            // read from its own lane of the quad, summed as (0 + 1) + (2 + 3).  The sums are
            // formed by every lane, in front of the branch: there the lane reads fold into the
            // additions (five instructions a sum instead of seven).
            v[a] = (quad_lane<0x00>(acc[a][0]) + quad_lane<0x55>(acc[a][1])) +
                   (quad_lane<0xAA>(acc[a][2]) + quad_lane<0xFF>(acc[a][3]));
            asm volatile("" : "+v"(v[a]));
            acc[a] = (gv_f4_t){0.0f, 0.0f, 0.0f, 0.0f};
        }
        if (keep && kt == 0) {
#pragma unroll
            for (int a = 0; a < 8; ++a)
                red[par_ * (2 * NW * 32) + (so_ * NW + w) * 32 + rb * 8 + a] = ldexpf(v[a], xshift);
        }
    };
    const auto WA = std::integral_constant<int, BA>();
    const auto WB = std::integral_constant<int, BB>();

    int par = 0;                                    // walking: the partial sums alternate between two areas
    if constexpr (TWO) {
        // ---- two resident tables: per output, [both tables] barrier, loop A, loop B ----------
        for (so = 0; so < nout; ++so) {
            const int sg = so == 1 ? 1 : si0;
            const bool second = kp->seg[sg].nstreams == 2;
            if (so > 0) write_tables(lrow, lrowB, second);  // (the first output's: in the prologue)
            // the LUT rows of the next output travel under this output's loops
            const bool more = so + 1 < nout;
            const uint8_t *qa_next = qrow, *qb_cur = qrow, *q_unused;
            const uint16_t *lutn;
            bool second_next = false;
            if (second) pass_ptrs(sl, so, 1, qb_cur, lutn);
            if (more) {
                second_next = kp->seg[1].nstreams == 2;
                pass_ptrs(sl, so + 1, 0, qa_next, lutn);
                load_lut_row<BA>(lutn, lrow);
                if (second_next) {
                    pass_ptrs(sl, so + 1, 1, q_unused, lutn);
                    load_lut_row<BB>(lutn, lrowB);
                }
            }
            // the second stream's first loads go out before the first stream's loop: its registers
            // are free from here on, and its data is then there when its loop starts
            if (second) {
#pragma unroll
                for (int n = 0; n < DB; ++n) {
                    q2[n] = load_idx<BB>(qb_cur + (size_t)n * stepB + lane0B);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __syncthreads();                        // publishes the tables (and the staged activations)
            if (second) {
                k_loop(q, qrow, lane0, step, slotA, WA, q2, qb_cur, lane0B, stepB, WB, false, false);
                k_loop(q2, qb_cur, lane0B, stepB, slotB, WB, q, qa_next, lane0, step, WA, more);
            } else {
                k_loop(q, qrow, lane0, step, slotA, WA, q, qa_next, lane0, step, WA, more);
            }
            end_of_output(so, 0);
            if (!more) break;
            __syncthreads();                        // the table region is rewritten next
            qrow = qa_next;
        }
    } else {
    bool same_table = false;                        // walking: the next slice reuses the table
    for (bool first = true;; first = false) {
        const int sg = so == 1 ? 1 : si0;
        if (!first && !same_table) {
            // every output of the launch reads the same staged activations (the host
            // sends launches whose outputs differ in input or rotation to the general
            // kernel), so only the table changes between passes
            write_table(lrow);
        }

        // ---- the pass after this one: its LUT row is fetched now and its first index
        //      loads replace this pass's last ones as they are consumed, so the memory
        //      stream does not stop between passes. -----------------------------------
        int nso = so, nsi = si + 1, nsl = sl;
        if (nsi == kp->seg[sg].nstreams) {
            nsi = 0;
            nso = so + 1;
        }
        const bool out_ends = nso != so;
        bool slice_ends = false;
        if (nso == nout && walk && sl + sl_step < sl_end) {
            nsl = sl + sl_step;                     // on to the first pass of the next slice
            nso = 0;
            slice_ends = true;
        }
        const bool has_next = nso < nout;
        const uint8_t *qnext = qrow;
        const uint16_t *lutn = lut;
        bool next_same = false;
        if (has_next) {
            pass_ptrs(nsl, nso, nsi, qnext, lutn);
            // one output of one stream per slice and the same LUT row: the table stands
            next_same = walk && slice_ends && nout == 1 && kp->seg[sg].nstreams == 1 && lutn == lut;
            if (!next_same) load_lut_row(lutn, lrow);
        }
        // publishes the table; with the table kept, the alternating sum areas make it unnecessary
        if (!same_table && !(first && early_done)) __syncthreads();
        if (first) FLUTE_GEMV_STAMP(4);

        k_loop(q, qrow, lane0, step, slot, WA, q, qnext, lane0, step, WA, has_next);
        if (!has_next) FLUTE_GEMV_STAMP(5);

        if (out_ends) end_of_output(so, par);
        if (!has_next) break;
        __syncthreads();                            // the table region is rewritten next
        if (slice_ends) {
            // The partial sums of the finished slice are complete behind the barrier above; the
            // next slice writes the other area, and this one again only two barriers later.
            if (tid < RW) {
                float yv[2];
                fold_rows(yv, par);
                finish_rows(sl, yv);
            }
            sl = nsl;
            par ^= 1;
        }
        same_table = next_same;
        so = nso;
        si = nsi;
        qrow = qnext;
        lut = lutn;
    }
    }
    FLUTE_GEMV_STAMP(6);
    __syncthreads();
    FLUTE_GEMV_STAMP(7);

    if (tid >= RW && p.split == 1) return;
    const bool owner = tid < RW;
    const int n = row_n(sl);
    float yv[2] = {0.0f, 0.0f};
    if (owner) fold_rows(yv, par);

    if (p.split > 1) {
        int *flag = (int *)(red + 2 * NW * 32);
        if (owner) {
#pragma unroll
            for (int so = 0; so < 2; ++so) {
                if (so >= nout) break;
                ws_store(p.P + (size_t)s * p.p_stride + kp->seg[so == 1 ? 1 : si0].n0 + n, yv[so]);
            }
        }
        ws_stores_done();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(p.tickets + kp->seg[si0].ticket0 + sl, 1,
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
                for (int sb = 0; sb < p.split; sb += 8) {
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
        if (tid == 0)
            __hip_atomic_store(p.tickets + kp->seg[si0].ticket0 + sl, 0, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }

    if (owner) finish_rows(sl, yv);
}

// The launch of the K-grouped instantiations (its own translation unit).  nw: wavefronts per
// workgroup, pf: loads in flight (pick as for the lean kernel), p.lpg_log2 in 4..6.
flute_status launch_gemv_kgroup(const GemvParams &p, int grid_x, int nw, int pf, size_t lds_bytes,
                                bool lut_bf16, hipStream_t stream);

// The launches of the two-table instantiations (their own translation units).  pair = 10 * BA + BB;
// pf: 2 or 4, 8 = four with the deep ring of a 1-bit first stream.
flute_status launch_gemv_pair_1bit(const GemvParams &p, int pair, int grid_x, int nw, int pf,
                                   size_t lds_bytes, bool lut_bf16, hipStream_t stream);
flute_status launch_gemv_pair_wide(const GemvParams &p, int pair, int grid_x, int nw, int pf,
                                   size_t lds_bytes, bool lut_bf16, hipStream_t stream);

}  // namespace flute
