// LUT GEMM for M > 1 on the gfx950 matrix cores:  C[M, N] = A[M, K] @ W^T,
// W[n, k] = LUT[n / gs][idx[n, k]], fp32 accumulate, one rounding.
//
// The weights never exist as a dense tile anywhere.  A lane loads one 16*b-byte
// chunk of the idxN blob, which holds 8 rows x 16 k of one 128 x 64 tile, turns
// the codes into 16-bit LUT values through a pair table in LDS (one lookup = two
// weights) and feeds the result straight into v_mfma_f32_16x16x32 as the
// row-side operand.  The blob's chunk order is the operand order of that
// instruction up to a lane permutation:
//
//   MFMA lane l:  rho = l & 15 (operand row), kg = l >> 4 (k group of 8 values)
//   chunk         th  = (rho >> 3) * 32 + (rho & 7) * 4 + kg     (wx, lane>>2, lane&3)
//   operand (v, d, j), j = half of the 64-k tile:
//       row  n = t*128 + wx*64 + v*16 + d*8 + (rho & 7)
//       slot s = ktl*4 + s2*2 + e  ->  k = g*64 + (2j + ktl)*16 + 2*kg + 8*s2 + e
//
// so one chunk yields the 16 operands (v, d, j) of its 16 rows, and the
// activations only have to present the same k order: a pre-pass writes them as
// Ap[g][j][m / 16][lane = kg*16 + m % 16][8 values], one 16-byte load per operand.
// The product is formed as C^T (rows of W on the MFMA row side), so a lane ends
// up with four consecutive n of one m.
//
// Workgroup = KW x MW wavefronts on one 128-row tile: wavefront (kw, mw) walks the
// k-tiles kw, kw + KW, ... for MB blocks of 16 rows of A.  Partial sums meet in a
// tree through LDS, then (gridDim.z > 1) across workgroups through fp32 partials
// and a ticket; the last arrival folds them in a fixed order.
#pragma once

#include <type_traits>

#include "common.h"

namespace flute {

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));

#ifdef FLUTE_STAMPS
// Instrumented builds only: per-wavefront phase times (s_memrealtime, 10 ns units) and the shader
// clock count across the K loop, written to the buffer flute_debug_stamps() was given.
__device__ long long *g_gemm_stamps = nullptr;
#define FLUTE_STAMP(slot)                                                                       \
    do {                                                                                        \
        if (g_gemm_stamps && (threadIdx.x & 63) == 0)                                           \
            g_gemm_stamps[(((size_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * \
                              (blockDim.x / 64) * 8 + (threadIdx.x >> 6) * 8 + (slot)] =        \
                (slot) == 7 ? (long long)__builtin_readcyclecounter()                           \
                            : (long long)__builtin_amdgcn_s_memrealtime();                      \
    } while (0)
#else
#define FLUTE_STAMP(slot) do { } while (0)
#endif
struct GemmParams {
    const uint8_t *q[2];
    const uint16_t *lut[2];
    const u4_t *Ap;        // permuted activations, LUT dtype, rows padded to 16
    void *C;
    const float *xb;       // [M, R] fp32 residual coefficients (A @ resB^T) or NULL
    const uint16_t *resA;  // [N, R] activation dtype
    const uint16_t *bias;  // [N] activation dtype
    float *P;              // split-K partial images
    int *tickets;
    int64_t ldc;
    int bits[2];
    int tab_off[2];        // byte offset of each stream's pair tables in LDS
    int rep_log2[2];       // log2 of the table replication (lanes per entry)
    int stage_off;         // byte offset of the per-wavefront tile staging buffers (4 KB, lean loop: 8 KB)
    int lean;              // 1: the launch uses the lean loop's instantiation
    int prog_off;          // lean loop: byte offset of one progress word per wavefront
    int balance;           // lean loop: 1 = the wavefront of a SIMD that is behind gets the higher priority
    int scatter;           // four blocks per wavefront: the mode of image_block_xor the image was written with;
                           // not 0: the k ways hand blocks to each other instead of reducing through the tree
    int nstreams;
    int M, N, K, G, gs, lut_rows, R;
    int mblk_total;        // ceil(M / 16)
    int mblk_pad;          // blocks Ap holds per half tile: gridDim.y * MW * MB
    int ksplit, gper;      // gridDim.z and k-tiles per z slice
    int z_base, ztotal;    // partial tiles: this launch writes [z_base, z_base + gridDim.z) of
                           // ztotal (several launches, one per stream, may share a fold)
    int out_bf16;          // dtype of C, resA, bias
    int vec_store;         // C rows allow 16-byte stores
    const u4_t *A8;        // direct mode: A itself, rows of lda8 16-byte pieces, no pre-pass
    int64_t lda8;
    int a_bf16;            // dtype of A in direct mode
    const int *rowshift;   // [M] or NULL: row m of the operands holds A[m] * 2^-rowshift[m]
};

// Activation pre-pass: Ap[g][j][mb][lane][slot] in the LUT's 16-bit type.
// block_xor: the mode of image_block_xor (common.h).
__global__ void __launch_bounds__(256) gemm_prep_kernel(const uint16_t *A, u4_t *Ap, int M,
                                                        int64_t lda, int G, int mblk,
                                                        int in_bf16, int out_bf16, int pairs,
                                                        const int *rowshift, int block_xor) {
    const int64_t total = (int64_t)G * 2 * mblk * 64;
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total;
         o += (int64_t)gridDim.x * blockDim.x) {
        const int lane = (int)(o & 63);
        const int64_t rest = o >> 6;
        const int gj = (int)(rest / mblk);
        const int g = gj >> 1, j = gj & 1;
        const int mb = (int)(rest % mblk) ^ image_block_xor(g, block_xor);
        const int m = mb * 16 + (lane & 15), kg = lane >> 4;
        uint32_t out[4] = {0u, 0u, 0u, 0u};
        if (m < M) {
            const int shift = rowshift ? rowshift[m] : 0;
#pragma unroll
            for (int s = 0; s < 4; ++s) {              // s = ktl*2 + s2
                const int k = g * 64 + (2 * j + (s >> 1)) * 16 + 2 * kg + 8 * (s & 1);
                // k is even: one 32-bit load per pair where the rows are 4-byte aligned
                uint16_t a0, a1;
                if (pairs) {
                    const uint32_t pair = *(const uint32_t *)(A + m * lda + k);
                    a0 = (uint16_t)(pair & 0xffffu);
                    a1 = (uint16_t)(pair >> 16);
                } else {
                    a0 = A[m * lda + k];
                    a1 = A[m * lda + k + 1];
                }
                if (in_bf16 != out_bf16) {
                    a0 = round_act(ldexpf(in_bf16 ? bf2f(a0) : h2f(a0), -shift), out_bf16);
                    a1 = round_act(ldexpf(in_bf16 ? bf2f(a1) : h2f(a1), -shift), out_bf16);
                }
                out[s] = (uint32_t)a0 | ((uint32_t)a1 << 16);
            }
        }
        u4_t v = {out[0], out[1], out[2], out[3]};
        Ap[o] = v;
    }
}

// The same image for 16-byte aligned rows, without gathers: a thread loads one 16-byte piece
// (eight consecutive k) of a row, the four threads that share a 32-k segment transpose their
// 4 x 4 dwords among themselves (thread q ends up with dword q of every piece, which is
// operand kg = q), and each stores one operand.  A wavefront owns one (segment, 16-row block):
// it reads sixteen 64-byte pieces of rows and writes one whole 1 KB block of the image.
template <int J>
__device__ __forceinline__ uint32_t quad_bcast(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, J * 0x55, 0xf, 0xf, true);
}
__global__ void __launch_bounds__(256) gemm_prep_quad_kernel(const uint16_t *A, u4_t *Ap, int M,
                                                             int64_t lda, int G, int mblk,
                                                             int in_bf16, int out_bf16,
                                                             const int *rowshift,
                                                             const uint32_t *warm, int warm_lines,
                                                             int block_xor) {
    // The launch that follows starts with a chain of dependent loads (its arguments, then the
    // LUT rows): one thread per 64-byte line touches the LUT here, so that the rows come from
    // the memory-side cache there instead of from memory.
    {
        const int line = blockIdx.x * blockDim.x + threadIdx.x;
        if (line < warm_lines) {
            const uint32_t seen = __builtin_nontemporal_load(warm + (size_t)line * 16);
            asm volatile("" ::"v"(seen));
        }
    }
    const int segs = 2 * G;                             // 32-k segments per row
    const int64_t total = (int64_t)mblk * 16 * segs * 4;
    // the four threads of a quad share their row and their loop bound
    for (int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total;
         o += (int64_t)gridDim.x * blockDim.x) {
        const int q = (int)(o & 3);
        const int64_t wv = o >> 6;
        int gj, mblock;
        if (total >> 6 <= 0x7fffffff) {                 // uniform; a 64-bit division costs some hundred instructions
            gj = (int)((uint32_t)wv % (uint32_t)segs);
            mblock = (int)((uint32_t)wv / (uint32_t)segs);
        } else {
            gj = (int)(wv % segs);
            mblock = (int)(wv / segs);
        }
        const int m = mblock * 16 + (int)((o >> 2) & 15);
        u4_t raw = {0u, 0u, 0u, 0u};
        if (m < M) {
            raw = *(const u4_t *)(A + (int64_t)m * lda + gj * 32 + q * 8);
            if (in_bf16 != out_bf16) {
                const int shift = rowshift ? rowshift[m] : 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint16_t lo = (uint16_t)(raw[e] & 0xffffu), hi = (uint16_t)(raw[e] >> 16);
                    const float flo = ldexpf(in_bf16 ? bf2f(lo) : h2f(lo), -shift);
                    const float fhi = ldexpf(in_bf16 ? bf2f(hi) : h2f(hi), -shift);
                    raw[e] = (uint32_t)round_act(flo, out_bf16) | ((uint32_t)round_act(fhi, out_bf16) << 16);
                }
            }
        }
        // piece j of a segment holds its dwords 4j .. 4j + 3; operand kg is the dwords
        // {kg, kg + 4, kg + 8, kg + 12} = element kg of the pieces 0 .. 3
        u4_t out;
#define FLUTE_TAKE(J)                                                                          \
        {                                                                                      \
            const uint32_t b0 = quad_bcast<J>(raw[0]), b1 = quad_bcast<J>(raw[1]);             \
            const uint32_t b2 = quad_bcast<J>(raw[2]), b3 = quad_bcast<J>(raw[3]);             \
            out[J] = (q & 2) ? ((q & 1) ? b3 : b2) : ((q & 1) ? b1 : b0);                      \
        }
        FLUTE_TAKE(0) FLUTE_TAKE(1) FLUTE_TAKE(2) FLUTE_TAKE(3)
#undef FLUTE_TAKE
        Ap[((int64_t)gj * mblk + ((m >> 4) ^ image_block_xor(gj >> 1, block_xor))) * 64 + q * 16 + (m & 15)] = out;
    }
}

// bfloat16 rows in front of float16 operands: shift[m] = the power of two that brings the
// largest magnitude of row m to [1, 2) (bf16_row_shift), one workgroup per row.
__global__ void __launch_bounds__(256) gemm_rowshift_kernel(const uint16_t *A, int64_t lda, int K,
                                                            int *shift) {
    __shared__ uint32_t slots[4];
    const uint16_t *row = A + (int64_t)blockIdx.x * lda;
    uint32_t e = 0;
    if ((((uintptr_t)row) & 15) == 0) {                // uniform per row
        for (int k = threadIdx.x * 8; k < K; k += 256 * 8) {
            if (k + 8 <= K) e = max(e, bf16_max_exp8(*(const uint4 *)(row + k)));
            else for (int q = k; q < K; ++q) e = max(e, (uint32_t)(row[q] >> 7) & 0xffu);
        }
    } else {
        for (int k = threadIdx.x; k < K; k += 256) e = max(e, (uint32_t)(row[k] >> 7) & 0xffu);
    }
    e = workgroup_max(e, slots, threadIdx.x, 256);
    if (threadIdx.x == 0) shift[blockIdx.x] = bf16_row_shift(e);
}

// xb[m, r] = sum_k A[m, k] * resB[r, k] in fp32 (one workgroup per (r, m)).
__global__ void __launch_bounds__(256) gemm_coeff_kernel(const uint16_t *A, int64_t lda,
                                                         const uint16_t *resB, float *xb, int K,
                                                         int R, int is_bf16) {
    const int r = blockIdx.x, m = blockIdx.y;
    float s = 0.0f;
    for (int k = threadIdx.x; k < K; k += 256)
        s = fmaf(load_act(A, m * lda + k, is_bf16), load_act(resB, (int64_t)r * K + k, is_bf16), s);
    __shared__ float red[256];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) xb[(int64_t)m * R + r] = red[0];
}

// Partial sums cross workgroups (and so the per-XCD L2s) inside one launch: they are
// written through and read around the L2 with device-scope (sc1) accesses, the same
// instructions a relaxed agent-scope atomic compiles to, but 16 bytes at a time.
__device__ __forceinline__ void ws_store16(float *p, f4_t v) {
    // s_nop: a store of more than 8 bytes reads its data registers after issue, and the
    // compiler does not know what this statement is, so it would not keep the next write to
    // those registers away from it
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void ws_stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Four 16-byte device-scope loads in flight, complete on return.
__device__ __forceinline__ void ws_load16x4(const float *p0, const float *p1, const float *p2,
                                            const float *p3, f4_t &a, f4_t &b, f4_t &c, f4_t &d) {
    asm volatile(
        "global_load_dwordx4 %0, %4, off sc1\n"
        "global_load_dwordx4 %1, %5, off sc1\n"
        "global_load_dwordx4 %2, %6, off sc1\n"
        "global_load_dwordx4 %3, %7, off sc1\n"
        "s_waitcnt vmcnt(0)"
        : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d)
        : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
        : "memory");
}


template <bool BF16>
__device__ __forceinline__ f4_t mfma16(u4_t w, u4_t a, f4_t acc) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, w),
                                                       __builtin_bit_cast(bf8_t, a), acc, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8_t, w),
                                                      __builtin_bit_cast(h8_t, a), acc, 0, 0, 0);
}

// The 2B-bit code of pair p of a chunk held as 4*B dwords (all indices constant
// after unrolling).
template <int B>
__device__ __forceinline__ uint32_t pair_code(const uint32_t (&Q)[4 * B], int p) {
    const int bit = 2 * B * p, dw = bit >> 5, sh = bit & 31;
    if (sh + 2 * B <= 32) return __builtin_amdgcn_ubfe(Q[dw], sh, 2 * B);
    return __builtin_amdgcn_alignbit(Q[dw + 1 < 4 * B ? dw + 1 : dw], Q[dw], sh) &
           ((1u << (2 * B)) - 1u);
}

template <int B>
__device__ __forceinline__ void load_chunk(uint32_t (&Q)[4 * B], const uint8_t *chunk) {
    const u4_t *src = (const u4_t *)chunk;
#pragma unroll
    for (int i = 0; i < B; ++i) {
        const u4_t v = __builtin_nontemporal_load(src + i);
        Q[4 * i + 0] = v[0];
        Q[4 * i + 1] = v[1];
        Q[4 * i + 2] = v[2];
        Q[4 * i + 3] = v[3];
    }
}

// The four lookups of operand (j, v, d).  PERM (4-bit codes, 64-lane replication,
// table on a 64 KB boundary of LDS): the code is a whole byte of the chunk and the
// entry stride is 256 bytes, so one v_perm_b32 drops it into byte 1 of the lane's
// column address.
template <int B, bool PERM>
__device__ __forceinline__ u4_t fetch_operand(const uint32_t (&Q)[4 * B], int j, int v, int d,
                                              uint32_t lbase, int code_shift) {
    typedef const __attribute__((address_space(3))) uint32_t *LdsWord;
    u4_t w;
#pragma unroll
    for (int s = 0; s < 4; ++s) {                      // s = ktl*2 + s2
        const int p = (2 * j + (s >> 1)) * 16 + v * 4 + d * 2 + (s & 1);
        uint32_t addr;
        if constexpr (PERM) {
            static_assert(B == 4, "byte codes");
            addr = __builtin_amdgcn_perm(Q[p >> 2], lbase, 0x03020000u | ((4u + (p & 3)) << 8));
        } else {
            addr = (pair_code<B>(Q, p) << code_shift) + lbase;
        }
        w[s] = *(LdsWord)addr;
    }
    return w;
}

// Half (32 k) of a 64-k tile of one stream: 8 operands x MB MFMAs.  The lookups
// run one pair of operands ahead of the MFMAs that consume them, in two
// alternating register sets, so the LDS latency hides behind matrix work.
//   lbase[v] : LDS byte address of this lane's column of the table that serves
//              rows (wx, v) (the LUT group may depend on wx and v when gs < 128)
template <int B, int MB, bool BF16, bool PERM = false>
__device__ __forceinline__ void half_mma(const uint32_t (&Q)[4 * B], int j, const u4_t (&Aj)[MB],
                                         f4_t (&acc)[MB][8], const uint32_t (&lbase)[4],
                                         int code_shift) {
    constexpr int AHEAD = 2;                             // pairs of operands in flight
    u4_t W[AHEAD + 1][2];
#pragma unroll
    for (int v = 0; v < AHEAD; ++v) {
        W[v][0] = fetch_operand<B, PERM>(Q, j, v, 0, lbase[v], code_shift);
        W[v][1] = fetch_operand<B, PERM>(Q, j, v, 1, lbase[v], code_shift);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        if (v + AHEAD < 4) {
            W[(v + AHEAD) % (AHEAD + 1)][0] =
                fetch_operand<B, PERM>(Q, j, v + AHEAD, 0, lbase[v + AHEAD], code_shift);
            W[(v + AHEAD) % (AHEAD + 1)][1] =
                fetch_operand<B, PERM>(Q, j, v + AHEAD, 1, lbase[v + AHEAD], code_shift);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                acc[mb][v * 2 + d] =
                    mfma16<BF16>(W[v % (AHEAD + 1)][d], Aj[mb], acc[mb][v * 2 + d]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Direct mode of the one-block fast path: a lane has loaded eight consecutive k of its row
// (piece c = lane >> 4 of the 32-k half tile), the matrix cores want the pairs
// (2*kg, 2*kg + 1) of all four pieces.  With the four lanes that share a row (16 apart)
// this is a 4 x 4 transpose of dwords: in round r every lane offers dword (kg + r) & 3 and
// reads the offer of piece (kg - r) & 3, which is that piece's dword kg.
__device__ __forceinline__ u4_t quad_transpose(u4_t v, int lane) {
    const int kg = lane >> 4;
    u4_t out = v;                                      // round 0: own piece, dword kg stays
#pragma unroll
    for (int r = 1; r < 4; ++r) {
        const int give = (kg + r) & 3, take = (kg - r) & 3;
        const uint32_t offer = (give & 2) ? ((give & 1) ? v[3] : v[2]) : ((give & 1) ? v[1] : v[0]);
        const uint32_t got = (uint32_t)__builtin_amdgcn_ds_bpermute(
            (take * 16 + (lane & 15)) << 2, (int)offer);
#pragma unroll
        for (int q = 0; q < 4; ++q) out[q] = (take == q) ? got : out[q];
    }
    // out[q] for q != kg now holds piece q's dword kg; the own piece contributes v[kg] at q = kg
    const uint32_t own = (kg & 2) ? ((kg & 1) ? v[3] : v[2]) : ((kg & 1) ? v[1] : v[0]);
#pragma unroll
    for (int q = 0; q < 4; ++q) out[q] = (kg == q) ? own : out[q];
    return out;
}

// B1 > 0: single stream of that width.  B1 == 0: widths read from the
// parameters, one or two streams.
// DIRECT (one block per wavefront on the fast path only): the activations are read from A
// itself and put into operand order in registers; no pre-pass launch.
// Block mb of an activation half: 16 bytes per lane at src + mb KB, as a statement the compiler
// does not take for a load (no wait of its own follows).
__device__ __forceinline__ void lean_load16(u4_t &dst, const u4_t *src, int mb) {
    switch (mb) {                                       // the offset is an immediate
        case 0: asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(dst) : "v"(src) : "memory"); break;
        case 1: asm volatile("global_load_dwordx4 %0, %1, off offset:1024" : "=&v"(dst) : "v"(src) : "memory"); break;
        case 2: asm volatile("global_load_dwordx4 %0, %1, off offset:2048" : "=&v"(dst) : "v"(src) : "memory"); break;
        default: asm volatile("global_load_dwordx4 %0, %1, off offset:3072" : "=&v"(dst) : "v"(src) : "memory"); break;
    }
}

// LEAN (four blocks per wavefront, one 4-bit stream, one LUT group per tile): every vector memory
// instruction of the kernel is written out and so is every wait for one.  The tile goes straight
// into LDS (global_load_lds_dwordx4), which frees the sixteen registers a tile in flight would
// hold; the compiler cannot count such loads next to its own (it answers one in flight with
// vmcnt(0) in front of the next use of any loaded register), hence all or nothing.
template <int MB, int KW, int MW, bool BF16, int B1, bool PERM = false, bool DIRECT = false,
          bool LEAN = false>
__global__ void __launch_bounds__(64 * KW * MW) gemm_kernel(const GemmParams p) {
    static_assert(!DIRECT || (PERM && MB == 1), "direct activations: one block, fast path");
    static_assert(!LEAN || (PERM && !DIRECT && MB >= 2 && B1 == 4), "lean loop: fast path, operand image");
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int NT = 64 * KW * MW;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kw = wave % KW, mw = wave / KW;
    const int t = blockIdx.x;
    FLUTE_STAMP(0);
    const int mb0 = (blockIdx.y * MW + mw) * MB;       // first 16-row block of this wavefront
    const int z = blockIdx.z;
    const int rho = lane & 15, kg = lane >> 4;
    const int wx = rho >> 3;
    const int th = wx * 32 + (rho & 7) * 4 + kg;

    const int gbeg = z * p.gper, gend = min(p.G, gbeg + p.gper);
    const bool active = mb0 < p.mblk_total;            // whole wavefront
    const int g0 = gbeg + kw;
    int left = (active && g0 < gend) ? (gend - g0 + KW - 1) / KW : 0;   // tiles of this wavefront
    // u4 units between the halves of a tile (direct mode: 32 k of a row are four pieces)
    const int64_t jstep = DIRECT ? 4 : (int64_t)p.mblk_pad * 64;
    // Ap is padded to whole workgroups of blocks (zeros), so every block index below
    // gridDim.y * MW * MB is loadable.
    // A wavefront without tiles addresses the first tile of the K range instead: its
    // loads below are then unconditional like everyone's, and the compiler can count them.
    const int g_first = left > 0 ? g0 : gbeg;
    const int a_row = mb0 * 16 + rho;                  // direct mode: this lane's row of A
    const bool a_row_valid = a_row < p.M;
    const int a_shift = (DIRECT && p.rowshift && a_row_valid) ? p.rowshift[a_row] : 0;
    const u4_t *ap = DIRECT
        ? p.A8 + (int64_t)(a_row_valid ? a_row : 0) * p.lda8 + (int64_t)g_first * 8 + kg
        : p.Ap + ((int64_t)g_first * 2 * p.mblk_pad + mb0) * 64 + lane;
    // direct mode: raw piece -> operand (rows beyond M are zero; the activations are
    // presented in the LUT's 16-bit type)
    auto operand_of = [&](u4_t raw) -> u4_t {
        if (!a_row_valid) raw = u4_t{0u, 0u, 0u, 0u};
        if (p.a_bf16 != (int)BF16) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint16_t lo16 = (uint16_t)(raw[q] & 0xffffu), hi16 = (uint16_t)(raw[q] >> 16);
                const float flo = ldexpf(p.a_bf16 ? bf2f(lo16) : h2f(lo16), -a_shift);
                const float fhi = ldexpf(p.a_bf16 ? bf2f(hi16) : h2f(hi16), -a_shift);
                raw[q] = (uint32_t)round_act(flo, BF16) | ((uint32_t)round_act(fhi, BF16) << 16);
            }
        }
        return quad_transpose(raw, lane);
    };
    auto load_a = [&](u4_t (&Aj)[MB], const u4_t *src) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) Aj[mb] = src[mb * 64];
    };
    // fast path: first tile and first activation operands are requested before the
    // tables are built, so their latency hides behind the build
    u4_t R[4], A0[MB], A1[MB];
    const uint8_t *tp = p.q[0] + ((int64_t)t * p.G + g_first) * 4096 + lane * 16;
    auto load_tile = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) R[i] = __builtin_nontemporal_load((const u4_t *)(tp + i * 1024));
    };
    const int ngrp = p.gs >= 128 ? 1 : 128 / p.gs;
    uint32_t lutv[2] = {0u, 0u};                       // fast path: LUT row(s), one value per lane
    if constexpr (PERM) {
#pragma unroll
        for (int gl = 0; gl < 2; ++gl) {
            if (LEAN || gl >= ngrp) break;
            int row = p.gs >= 128 ? (t * 128) / p.gs : t * ngrp + gl;
            row = min(row, p.lut_rows - 1);
            lutv[gl] = p.lut[0][((size_t)row << 4) + (lane & 15)];
        }
        // Unconditional, after the LUT row: the table build below then waits for the LUT
        // values only, not for the first tile (a conditional load here made that wait a
        // wait for everything).
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!LEAN) {
            load_tile();
            load_a(A0, ap);
            load_a(A1, ap + jstep);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    // ---- lean loop: hand-written loads ------------------------------------------------
    // LDS staging: two 4 KB buffers per wavefront; tile n lives in buffer n & 1.  Lane L of row i
    // asks for the 16-byte piece that belongs at position L of that row (the same layout the
    // register path writes: slot order and rotation of the quarters).
    const uint32_t lds_base0 =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    const uint32_t lean_stage =
        __builtin_amdgcn_readfirstlane(lds_base0 + p.stage_off + (uint32_t)wave * 8192u);
    const int lean_kt = ((lane & 3) - (lane >> 4)) & 3;
    const uint32_t lean_even = (uint32_t)((lane >> 2) * 64 + lean_kt * 16);
    const uint32_t lean_odd = (uint32_t)(((lane >> 2) ^ 1) * 64 + lean_kt * 16);
    const uint8_t *lean_tq = p.q[0] + ((int64_t)t * p.G + g_first) * 4096;   // wavefront-uniform
    auto lean_tile = [&](int buf) {                    // four loads, straight into LDS
        const uint32_t m0v = lean_stage + (uint32_t)buf * 4096u;
        // (the pointer is the same in every lane; the compiler cannot see that through the
        // wavefront-dependent tile count)
        const uint64_t a64 = (uint64_t)(uintptr_t)lean_tq;
        const uint8_t *tq_s = (const uint8_t *)(uintptr_t)join_address_halves(
            __builtin_amdgcn_readfirstlane((int)(uint32_t)a64),
            __builtin_amdgcn_readfirstlane((int)(uint32_t)(a64 >> 32)));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %1, %3 offset:0 nt\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:1024 nt\n\t"
                     "global_load_lds_dwordx4 %1, %3 offset:2048 nt\n\t"
                     "global_load_lds_dwordx4 %2, %3 offset:3072 nt"
                     :: "s"(m0v), "v"(lean_even), "v"(lean_odd), "s"(tq_s) : "memory", "m0");
    };
    if constexpr (LEAN) {
        int row = (t * 128) / p.gs;
        row = min(row, p.lut_rows - 1);
        const uint16_t *lp = p.lut[0] + ((size_t)row << 4) + (lane & 15);
        uint32_t lv;
        asm volatile("global_load_ushort %0, %1, off" : "=&v"(lv) : "v"(lp) : "memory");
        lean_tile(0);                                  // tile 0
        static_assert(MB == 4 || MB == 2, "operands of a half");
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) lean_load16(A0[mb], ap, mb);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) lean_load16(A1[mb], ap + jstep, mb);
        // the LUT value is the oldest load: 4 + 2 MB younger ones may stay in flight
        asm volatile("s_waitcnt vmcnt(%1)" : "+v"(lv) : "n"(4 + 2 * MB) : "memory");
        lutv[0] = lv;
    }

    // ---- pair tables ------------------------------------------------------------
    if constexpr (PERM) {
        // 64 replicas per entry: a wavefront writes one entry per instruction, every
        // lane the same dword, built from two lane reads of the LUT row it holds.
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
#pragma unroll
        for (int gl = 0; gl < 2; ++gl) {
            if (gl >= ngrp) break;
            const uint32_t lv = lutv[gl];
            uint32_t *tab = (uint32_t *)(smem + p.tab_off[0]) + (gl << 14);
            for (int code = wave_u; code < 256; code += NT / 64) {
                const uint32_t lo = __builtin_amdgcn_readlane(lv, code & 15);
                const uint32_t hi = __builtin_amdgcn_readlane(lv, code >> 4);
                tab[code * 64 + lane] = lo | (hi << 16);
            }
        }
    } else {
        for (int s = 0; s < p.nstreams; ++s) {
            const int b = B1 > 0 ? B1 : p.bits[s];
            const int rl = p.rep_log2[s];
            const int total = ngrp << (2 * b + rl);
            uint32_t *tab = (uint32_t *)(smem + p.tab_off[s]);
            const uint16_t *lut = p.lut[s];
            for (int i = tid; i < total; i += NT) {
                const int code = (i >> rl) & ((1 << (2 * b)) - 1);
                const int gl = i >> (rl + 2 * b);
                int row = p.gs >= 128 ? (t * 128) / p.gs : t * ngrp + gl;
                row = min(row, p.lut_rows - 1);
                const uint16_t *lr = lut + ((size_t)row << b);
                tab[i] = (uint32_t)lr[code & ((1 << b) - 1)] | ((uint32_t)lr[code >> b] << 16);
            }
        }
    }
    if constexpr (LEAN) {
        if (lane == 0)
            *(uint32_t *)(smem + p.prog_off + wave * 4) = (uint32_t)__builtin_amdgcn_readfirstlane(left);
    }
    __syncthreads();
    FLUTE_STAMP(1);
    FLUTE_STAMP(7);

    f4_t acc[MB][8];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[mb][i] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};

    const uint32_t lds_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    auto table_bases = [&](uint32_t (&lb)[4], int s, int b) {
        const int rl = p.rep_log2[s];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = wx * 64 + v * 16;
            const int gl = p.gs >= 128 ? 0 : row / p.gs;
            lb[v] = lds_base + p.tab_off[s] +
                    (((gl << (2 * b + rl)) + (lane & ((1 << rl) - 1))) << 2);
        }
    };

    if (active) {
        if constexpr (PERM) {
            // 4-bit fast path.  A 64-byte chunk per lane is the worst pattern for the
            // vector memory pipe (one 64-byte sector per lane and instruction), so the
            // 4 KB tile is fetched as four fully contiguous 1 KB rows instead, dropped
            // into a per-wavefront LDS buffer and read back chunk by chunk.  Slot
            // order and a rotation of the four quarters keep both sides free of bank
            // conflicts: piece (chunk c, quarter kt) lives at
            //     (c ^ ((c >> 4) & 1)) * 64 + ((kt + (c >> 2)) & 3) * 16.
            typedef __attribute__((address_space(3))) u4_t *LdsQuad;
            uint32_t lb[4];
            table_bases(lb, 0, 4);
            const uint32_t stage = lds_base + p.stage_off + wave * 4096;
            const int rotw = ((lane & 3) + ((lane >> 4) & 3)) & 3;
            const uint32_t wb_even = stage + (lane >> 2) * 64 + rotw * 16;
            const uint32_t wb_odd = stage + ((lane >> 2) ^ 1) * 64 + rotw * 16;
            const int slot = th ^ ((th >> 4) & 1);
            uint32_t rb[4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) rb[kt] = stage + slot * 64 + ((kt + (rho & 3)) & 3) * 16;

            uint32_t Q[16];
            constexpr int64_t qstep = (int64_t)KW * 4096;
            const int64_t astep = DIRECT ? (int64_t)KW * 8 : (int64_t)KW * 2 * p.mblk_pad * 64;
            auto stage_write = [&]() {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    *(LdsQuad)(uintptr_t)(((i & 1) ? wb_odd : wb_even) + i * 1024) = R[i];
            };
            auto stage_read = [&]() {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) {
                    const u4_t v = *(LdsQuad)(uintptr_t)rb[kt];
                    Q[4 * kt + 0] = v[0];
                    Q[4 * kt + 1] = v[1];
                    Q[4 * kt + 2] = v[2];
                    Q[4 * kt + 3] = v[3];
                }
            };
            if constexpr (LEAN) {
                // One round = one tile of this wavefront.  Vector memory instructions of a round,
                // in issue order: the tile after next (4, into the LDS buffer just read out), the
                // next tile's first-half operands (MB), its second-half operands (MB).  Inside a
                // half the weight operands are outermost: an operand serves all blocks of rows
                // and is replaced by the next half's right away, so lookups and products
                // alternate four by four (measured against blocks of rows outermost with the
                // lookups bunched behind the last two blocks: 1 % faster; the explicit waits of
                // either order cost no time, a wavefront's loads are there when it asks).
                // The products of an accumulator come in the same order as in the other loop.
                u4_t W[8];
                uint32_t Q8[8];
                const uint32_t lb0 = lb[0];
                const uint32_t rbase = lean_stage + slot * 64;
                const int rot = rho & 3;
                uint32_t cur = 0;                         // LDS buffer of this round's tile: 0 or 4096
                auto read_codes = [&](int j, uint32_t boff) {
#pragma unroll
                    for (int kk = 0; kk < 2; ++kk) {
                        const u4_t v = *(LdsQuad)(uintptr_t)(rbase + boff + (((2 * j + kk + rot) & 3) << 4));
                        Q8[4 * kk + 0] = v[0];
                        Q8[4 * kk + 1] = v[1];
                        Q8[4 * kk + 2] = v[2];
                        Q8[4 * kk + 3] = v[3];
                    }
                };
                auto operand = [&](int o) -> u4_t {
                    typedef const __attribute__((address_space(3))) uint32_t *LdsWord;
                    const int v = o >> 1, d = o & 1;
                    u4_t w;
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4)       // q4 = ktl * 2 + s2
                        w[q4] = *(LdsWord)__builtin_amdgcn_perm(
                            Q8[(q4 >> 1) * 4 + v], lb0, 0x03020000u | ((4u + d * 2 + (q4 & 1)) << 8));
                    return w;
                };
                // `between` runs after the first operand's products: work that has to follow LDS
                // reads issued in front of the half finds them complete there
                auto half = [&](u4_t (&Aj)[MB], const u4_t *next, auto &&between) {
#pragma unroll
                    for (int o = 0; o < 8; ++o) {
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) acc[mb][o] = mfma16<BF16>(W[o], Aj[mb], acc[mb][o]);
                        if (o == 0) {
                            __builtin_amdgcn_sched_barrier(0);
                            between();
                        }
                        W[o] = operand(o);
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) lean_load16(Aj[mb], next, mb);
                    __builtin_amdgcn_sched_barrier(0);
                };
                auto wait_half = [&](u4_t (&Aj)[MB], auto younger) {
                    if constexpr (MB == 4)
                        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(Aj[0]), "+v"(Aj[1]), "+v"(Aj[2]), "+v"(Aj[3])
                                     : "n"(decltype(younger)::value) : "memory");
                    else
                        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(Aj[0]), "+v"(Aj[1])
                                     : "n"(decltype(younger)::value) : "memory");
                };
                // (the same in every lane: a scalar count gives a scalar loop)
                left = __builtin_amdgcn_readfirstlane(left);
                if (left > 0) {
                    // tile 0 is the oldest load in flight: both activation halves may stay
                    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * MB) : "memory");
                    read_codes(0, 0);
#pragma unroll
                    for (int o = 0; o < 8; ++o) W[o] = operand(o);
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    if (left > 1) lean_tq += qstep;
                    lean_tile(1);                         // tile 1 (or a harmless reload)
                }
                const int wave_hi = __builtin_amdgcn_readfirstlane(wave >> 2);
                // Progress of the two wavefronts of a SIMD (w and w + 4): every round a wavefront
                // posts the tiles it has left and reads the other's figure of a round ago; the one
                // that is behind (or level) runs at the higher priority.  Against taking turns tile
                // by tile (FLUTE_GEMM_NO_BALANCE) the second wavefront of a SIMD leaves the loop
                // 0.8 us after the first instead of 1.9 us; worth 1 % at M = 256, nothing elsewhere.
                typedef __attribute__((address_space(3))) uint32_t *LdsProg;
                const uint32_t prog_mine = lds_base0 + p.prog_off + (uint32_t)wave * 4u;
                const uint32_t prog_other = lds_base0 + p.prog_off + (uint32_t)(wave ^ 4) * 4u;
                int other_left = left;
                while (left > 0) {
                    uint32_t seen = 0;
                    if (p.balance) {
                        if (left >= other_left) __builtin_amdgcn_s_setprio(1);
                        else __builtin_amdgcn_s_setprio(0);
                        *(LdsProg)(uintptr_t)prog_mine = (uint32_t)left;
                        seen = *(LdsProg)(uintptr_t)prog_other;
                    } else {
                        if ((left + wave_hi) & 1) __builtin_amdgcn_s_setprio(1);
                        else __builtin_amdgcn_s_setprio(0);
                    }
                    const u4_t *apn = left > 1 ? ap + astep : ap;
                    // this tile's first-half operands (and, older, the tile itself) have arrived;
                    // the second-half operands may still be in flight
                    wait_half(A0, std::integral_constant<int, MB>());
                    read_codes(1, cur);                   // this tile, second half
                    __builtin_amdgcn_sched_barrier(0);
                    half(A0, apn, [&] {
                        // the tile after next goes into the buffer just read out: not before
                        // those reads have returned (four products later they have)
                            asm volatile("s_waitcnt lgkmcnt(0)"
                                     : "+v"(Q8[0]), "+v"(Q8[1]), "+v"(Q8[2]), "+v"(Q8[3]), "+v"(Q8[4]),
                                       "+v"(Q8[5]), "+v"(Q8[6]), "+v"(Q8[7]) :: "memory");
                        if (left > 2) lean_tq += qstep;
                        lean_tile(cur != 0);
                        __builtin_amdgcn_sched_barrier(0);
                    });
                    // second-half operands and (older) the next tile have arrived; the tile after
                    // next and the next first-half operands may be in flight
                    wait_half(A1, std::integral_constant<int, 4 + MB>());
                    read_codes(0, cur ^ 4096u);           // next tile, first half
                    __builtin_amdgcn_sched_barrier(0);
                    half(A1, apn + jstep, [] {});
                    ap = apn;
                    cur ^= 4096u;
                    --left;
                    if (p.balance) other_left = __builtin_amdgcn_readfirstlane((int)seen);
                }
                // nothing may land in LDS or in a register once the tree reuses them
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            } else {
            if (left > 0) {
                stage_write();                            // first tile, requested before the tables
                if (left > 1) tp += qstep;
                load_tile();                              // second tile (or a harmless reload)
            }
            while (left > 0) {
                // The two wavefronts of a SIMD (wavefront w and w + 4) take turns at the higher
                // priority, tile by tile, so that neither falls a tile behind the other
                // (measured with the builds interleaved: about 1 % at M = 256 and M = 1024).
                if ((left + (wave >> 2)) & 1) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
                stage_read();                             // this tile's chunk
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (DIRECT) {
                    const u4_t T0[1] = {operand_of(A0[0])};
                    half_mma<4, MB, BF16, true>(Q, 0, T0, acc, lb, 8);
                } else {
                    half_mma<4, MB, BF16, true>(Q, 0, A0, acc, lb, 8);
                }
                if (left > 1) ap += astep;
                load_a(A0, ap);                           // half a tile ahead of its use
                // issue order activations -> tile: the wait for these activations at the
                // top of the next iteration then does not include the tile load
                __builtin_amdgcn_sched_barrier(0);
                stage_write();                            // next tile, requested a whole tile ago
                if (left > 2) tp += qstep;
                load_tile();                              // the tile after it
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (DIRECT) {
                    const u4_t T1[1] = {operand_of(A1[0])};
                    half_mma<4, MB, BF16, true>(Q, 1, T1, acc, lb, 8);
                } else {
                    half_mma<4, MB, BF16, true>(Q, 1, A1, acc, lb, 8);
                }
                load_a(A1, ap + jstep);
                __builtin_amdgcn_sched_barrier(0);
                --left;
            }
            }
            __builtin_amdgcn_s_setprio(0);
        } else if constexpr (B1 > 0) {
            uint32_t lb[4];
            table_bases(lb, 0, B1);
            const int cs = p.rep_log2[0] + 2;
            uint32_t Qa[4 * B1], Qb[4 * B1];
            const uint8_t *qp = p.q[0] + (((int64_t)t * p.G + g0) * 64 + th) * (16 * B1);
            constexpr int64_t qstep = (int64_t)KW * 64 * 16 * B1;
            const int64_t astep = (int64_t)KW * 2 * p.mblk_pad * 64;
            if (left > 0) {
                load_chunk<B1>(Qa, qp);
                load_a(A0, ap);
                load_a(A1, ap + jstep);
            }
            // One tile: the next chunk is requested first (a whole tile ahead), the
            // activation halves of the next tile as soon as their registers are free.
            auto step = [&](const uint32_t (&Qc)[4 * B1], uint32_t (&Qn)[4 * B1], bool more) {
                if (more) {                              // else: harmless reload of this tile
                    qp += qstep;
                    ap += astep;
                }
                load_chunk<B1>(Qn, qp);
                __builtin_amdgcn_sched_barrier(0);
                half_mma<B1, MB, BF16, PERM>(Qc, 0, A0, acc, lb, cs);
                load_a(A0, ap);
                __builtin_amdgcn_sched_barrier(0);
                half_mma<B1, MB, BF16, PERM>(Qc, 1, A1, acc, lb, cs);
                load_a(A1, ap + jstep);
                __builtin_amdgcn_sched_barrier(0);
            };
            while (left > 0) {
                step(Qa, Qb, left > 1);
                if (--left == 0) break;
                step(Qb, Qa, left > 1);
                --left;
            }
        } else {
            for (int g = gbeg + kw; g < gend; g += KW) {
                u4_t A0[MB], A1[MB];
                const u4_t *ap = p.Ap + ((int64_t)g * 2 * p.mblk_pad + mb0) * 64 + lane;
                load_a(A0, ap);
                load_a(A1, ap + jstep);
                for (int s = 0; s < p.nstreams; ++s) {
                    uint32_t lb[4];
                    const int cs = p.rep_log2[s] + 2;
                    const int64_t tile = (int64_t)t * p.G + g;
                    switch (p.bits[s]) {
                        case 1: {
                            uint32_t Q[4];
                            table_bases(lb, s, 1);
                            load_chunk<1>(Q, p.q[s] + (tile * 64 + th) * (16 * 1));
                            half_mma<1, MB, BF16>(Q, 0, A0, acc, lb, cs);
                            half_mma<1, MB, BF16>(Q, 1, A1, acc, lb, cs);
                        } break;
                        case 2: {
                            uint32_t Q[8];
                            table_bases(lb, s, 2);
                            load_chunk<2>(Q, p.q[s] + (tile * 64 + th) * (16 * 2));
                            half_mma<2, MB, BF16>(Q, 0, A0, acc, lb, cs);
                            half_mma<2, MB, BF16>(Q, 1, A1, acc, lb, cs);
                        } break;
                        case 3: {
                            uint32_t Q[12];
                            table_bases(lb, s, 3);
                            load_chunk<3>(Q, p.q[s] + (tile * 64 + th) * (16 * 3));
                            half_mma<3, MB, BF16>(Q, 0, A0, acc, lb, cs);
                            half_mma<3, MB, BF16>(Q, 1, A1, acc, lb, cs);
                        } break;
                        default: {
                            uint32_t Q[16];
                            table_bases(lb, s, 4);
                            load_chunk<4>(Q, p.q[s] + (tile * 64 + th) * (16 * 4));
                            half_mma<4, MB, BF16>(Q, 0, A0, acc, lb, cs);
                            half_mma<4, MB, BF16>(Q, 1, A1, acc, lb, cs);
                        } break;
                    }
                }
            }
        }
    }

    // a lean loop's loads land in LDS and registers without the compiler's knowledge: none may
    // be in flight when the tree reuses either (wavefronts without work have issued some too)
    if constexpr (LEAN) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // ---- tree over the KW wavefronts of one m group, through LDS ------------------
    f4_t *red = (f4_t *)smem;                           // slot = [MB*8][64] f4
#ifdef FLUTE_STAMPS
    if (g_gemm_stamps && lane == 0) {
        long long *sl = g_gemm_stamps + (((size_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * (NT / 64) * 8 + wave * 8;
        sl[7] = (long long)__builtin_readcyclecounter() - sl[7];
    }
#endif
    FLUTE_STAMP(2);
    __syncthreads();                                    // tables are dead from here
    FLUTE_STAMP(3);
    // Four blocks of rows per wavefront and the image in the order of image_block_xor: accumulator j
    // of k way kw holds block j ^ x(kw).  Instead of the tree every wavefront hands the blocks it
    // does not keep to the k way that keeps them: accumulators 2 and 3 to the k way whose 0 and 1
    // they are, then accumulator 1 to the one whose 0 it is; with eight k ways two of them then
    // hold the same block and the odd one gives its sums to the even one.  The same bytes cross
    // LDS as in the tree and the sums are the same (every addition commutes), but all eight
    // wavefronts move them, barriers go, and four or eight wavefronts write the totals tile.
    const bool scattered = MB == 4 && KW * MW == 8 && p.scatter != 0;
    if constexpr (MB == 4 && KW * MW == 8) {
        if (scattered) {
            constexpr int P1 = KW == 4 ? 2 : 4, P2 = KW == 4 ? 1 : 2;   // partners of the two hand-overs
            f4_t *mine1 = red + (size_t)wave * 1024;
            const f4_t *theirs1 = red + (size_t)(wave ^ P1) * 1024;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                mine1[i * 64 + lane] = acc[2][i];
                mine1[(8 + i) * 64 + lane] = acc[3][i];
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                acc[0][i] += theirs1[i * 64 + lane];
                acc[1][i] += theirs1[(8 + i) * 64 + lane];
            }
            __syncthreads();
            // second hand-over: behind the region the totals tile takes (17 * 4 KB from the start)
            f4_t *mine2 = red + 4352 + (size_t)wave * 512;
            const f4_t *theirs2 = red + 4352 + (size_t)(wave ^ P2) * 512;
#pragma unroll
            for (int i = 0; i < 8; ++i) mine2[i * 64 + lane] = acc[1][i];
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[0][i] += theirs2[i * 64 + lane];
            if constexpr (KW == 8) {
                // k ways kw and kw ^ 1 hold the same block: between the (smaller) totals tile
                // and the second hand-over's areas
                f4_t *pair3 = red + 2176 + (size_t)(wave >> 1) * 512;
                if (kw & 1) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) pair3[i * 64 + lane] = acc[0][i];
                }
                __syncthreads();
                if (!(kw & 1)) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[0][i] += pair3[i * 64 + lane];
                }
            }
        }
    }
#pragma unroll
    for (int step = KW / 2; step >= 1; step >>= 1) {
        if (scattered) break;
        if (kw >= step && kw < 2 * step) {
            f4_t *slot = red + (size_t)((kw - step) * MW + mw) * (MB * 8 * 64);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int i = 0; i < 8; ++i) slot[(mb * 8 + i) * 64 + lane] = acc[mb][i];
        }
        __syncthreads();
        if (kw < step) {
            const f4_t *slot = red + (size_t)(kw * MW + mw) * (MB * 8 * 64);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[mb][i] += slot[(mb * 8 + i) * 64 + lane];
        }
        __syncthreads();
    }

    FLUTE_STAMP(4);
    // ---- totals of the workgroup as a row-major fp32 tile in LDS --------------------
    constexpr int ROWS = MW * MB * 16;                  // rows of C this workgroup owns
    constexpr int LDT = 128 + 4;                        // padded row: conflict-free both ways
    float *tile = (float *)smem;
    if (scattered) {                                    // the totals of block x(kw) are in accumulator 0
        if (KW == 4 || !(kw & 1)) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = (mw * MB + image_block_xor(kw, p.scatter)) * 16 + rho;
            const int n0 = (kg >> 1) * 64 + (i >> 1) * 16 + (i & 1) * 8 + (kg & 1) * 4;
            *(f4_t *)(tile + row * LDT + n0) = acc[0][i];
        }
        }
    } else if (kw == 0) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int row = (mw * MB + mb) * 16 + rho;
                const int n0 = (kg >> 1) * 64 + (i >> 1) * 16 + (i & 1) * 8 + (kg & 1) * 4;
                *(f4_t *)(tile + row * LDT + n0) = acc[mb][i];
            }
    }
    __syncthreads();

    FLUTE_STAMP(5);
    // Every thread now serves pieces of 8 consecutive outputs of one row: 16 threads
    // write one 256-byte row segment of C.
    constexpr int PIECES = ROWS * 16;
    const int unit = blockIdx.y * gridDim.x + blockIdx.x;           // (m chunk, n tile)
    const size_t image = (size_t)ROWS * 128;                        // floats per unit per z
    const size_t zstride = (size_t)gridDim.x * gridDim.y * image;
    if (p.ztotal > 1) {
        // across workgroups: partial tiles + ticket; the last arrival folds them in z order
        float *mine = p.P + (size_t)(p.z_base + z) * zstride + (size_t)unit * image;
        for (int idx = tid; idx < PIECES; idx += NT) {
            const int ml = idx >> 4, n8 = idx & 15;
            ws_store16(mine + ml * 128 + n8 * 8, *(const f4_t *)(tile + ml * LDT + n8 * 8));
            ws_store16(mine + ml * 128 + n8 * 8 + 4, *(const f4_t *)(tile + ml * LDT + n8 * 8 + 4));
        }
        ws_stores_done();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        int *flag = (int *)(tile + ROWS * LDT);
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(p.tickets + unit, 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
            *flag = (old == p.ztotal - 1);
        }
        __syncthreads();
        if (!*flag) return;
        if (tid == 0)
            __hip_atomic_store(p.tickets + unit, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- epilogue: residual, bias, one rounding, store -------------------------------
    for (int idx = tid; idx < PIECES; idx += NT) {
        const int ml = idx >> 4, n8 = idx & 15;
        const int m = blockIdx.y * ROWS + ml;
        if (m >= p.M) continue;
        const int n0 = t * 128 + n8 * 8;
        float y[8];
        if (p.ztotal > 1) {
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = 0.0f;
            const float *src = p.P + (size_t)unit * image + ml * 128 + n8 * 8;
            for (int z0 = 0; z0 < p.ztotal; z0 += 2) {
                const float *s0 = src + z0 * zstride;
                const float *s1 = z0 + 1 < p.ztotal ? s0 + zstride : s0;
                f4_t a, b, c, d;
                ws_load16x4(s0, s0 + 4, s1, s1 + 4, a, b, c, d);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    y[e] += a[e];
                    y[4 + e] += b[e];
                }
                if (z0 + 1 < p.ztotal) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        y[e] += c[e];
                        y[4 + e] += d[e];
                    }
                }
            }
        } else {
            const f4_t lo = *(const f4_t *)(tile + ml * LDT + n8 * 8);
            const f4_t hi = *(const f4_t *)(tile + ml * LDT + n8 * 8 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                y[e] = lo[e];
                y[4 + e] = hi[e];
            }
        }
        if (p.rowshift) {                               // undo the row's activation scaling (exact)
            const int sh = p.rowshift[m];
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = ldexpf(y[e], sh);
        }
        if (p.R > 0) {
            const float *xr = p.xb + (size_t)m * p.R;
            for (int r = 0; r < p.R; ++r) {
                const float c = xr[r];
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    y[e] = fmaf(c, load_act(p.resA, (int64_t)(n0 + e) * p.R + r, p.out_bf16), y[e]);
            }
        }
        if (p.bias) {
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] += load_act(p.bias, n0 + e, p.out_bf16);
        }
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            o[e] = (uint32_t)round_act(y[2 * e], p.out_bf16) |
                   ((uint32_t)round_act(y[2 * e + 1], p.out_bf16) << 16);
        uint16_t *dst = (uint16_t *)p.C + (size_t)m * p.ldc + n0;
        if (p.vec_store) {
            *(u4_t *)dst = u4_t{o[0], o[1], o[2], o[3]};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                dst[2 * e] = (uint16_t)o[e];
                dst[2 * e + 1] = (uint16_t)(o[e] >> 16);
            }
        }
    }
    FLUTE_STAMP(6);
}

}  // namespace flute
