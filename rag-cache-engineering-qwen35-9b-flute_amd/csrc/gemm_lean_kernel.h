// LUT GEMM for 64 rows of A and more per workgroup on the single-stream 4-bit fast path (one LUT
// group per 128-row tile): the same arithmetic as gemm_kernel (weights looked up through a pair
// table in LDS straight into v_mfma_f32_16x16x32, activations from the operand image), with
//   * every vector memory instruction and every wait for one written out: the 4 KB tile goes
//     straight into LDS (global_load_lds_dwordx4, two buffers per wavefront), which frees the
//     registers a tile in flight would hold; the compiler cannot count such loads next to its
//     own (it answers one in flight with vmcnt(0) in front of the next use of any loaded
//     register), hence all or nothing;
//   * a resident grid: a workgroup walks over a contiguous run of work items (tile, chunk of
//     rows, K slice), so launches with more items than CUs pay one launch, not several rounds;
//   * a fold across the K ways of a workgroup that leaves every wavefront with a share of the
//     totals (each wavefront sends the others what they own and sums what it owns, two rounds
//     through LDS), which it finishes and stores itself from registers: no totals tile, and the
//     partial images of a K split across workgroups are written from registers as well.
#pragma once

#include "gemm_kernel.h"

namespace flute {

// LDS the kernel needs: 64 KB table, two 4 KB tile buffers per wavefront, the ticket flag.
constexpr int kLeanStageOff = 64 * 1024;
constexpr int kLeanFlagOff = 128 * 1024;
constexpr int kLeanLdsBytes = kLeanFlagOff + 16;

template <int KW, int MW, bool BF16>
__global__ void __launch_bounds__(64 * KW * MW) gemm_lean_kernel(const GemmParams p) {
    constexpr int MB = 4;
    constexpr int NT = 64 * KW * MW;
    constexpr int NW = KW * MW;
    static_assert(NW == 8, "eight wavefronts: two per SIMD");
    constexpr int IPO = 32 / KW;                        // accumulators a wavefront owns after the fold
    constexpr int HALF = IPO / 2;                       // ... and sends per owner and round
    // one round of the fold: MW * KW * (KW - 1) * HALF slots of 1 KB
    static_assert(MW * KW * (KW - 1) * HALF * 1024 <= kLeanFlagOff, "fold scratch");
    extern __shared__ __align__(16) unsigned char smem[];
    typedef __attribute__((address_space(3))) u4_t *LdsQuad;
    typedef const __attribute__((address_space(3))) uint32_t *LdsWord;

    // the parameters span several 64-byte lines; fetched as the code needs them, each new line
    // would be a trip to memory of its own in front of the first load
    // (written as one statement: the compiler moves plain loads of this kind behind the first
    // uses)
    {
        static_assert(sizeof(GemmParams) <= 256, "four lines");
        const void *ka = (const void *)__builtin_amdgcn_kernarg_segment_ptr();
        uint32_t l0, l1, l2, l3;
        asm volatile("s_load_dword %0, %4, 0x0\n\ts_load_dword %1, %4, 0x40\n\t"
                     "s_load_dword %2, %4, 0x80\n\ts_load_dword %3, %4, 0xc0\n\ts_waitcnt lgkmcnt(0)"
                     : "=&s"(l0), "=&s"(l1), "=&s"(l2), "=&s"(l3) : "s"(ka) : "memory");
    }
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kw = wave % KW, mw = wave / KW;
    const int rho = lane & 15, kg = lane >> 4;
    const int wx = rho >> 3;
    const int th = wx * 32 + (rho & 7) * 4 + kg;
    FLUTE_STAMP(0);

    const uint32_t lds_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    // Tile staging: tile n of a wavefront lives in buffer n & 1.  Lane L of row i asks for the
    // 16-byte piece that belongs at position L of that row, so that piece (chunk c, quarter kt)
    // ends up at (c ^ ((c >> 4) & 1)) * 64 + ((kt + (c >> 2)) & 3) * 16: both the landing and
    // the chunk-wise read-back are free of bank conflicts.
    const uint32_t stage = __builtin_amdgcn_readfirstlane(lds_base + kLeanStageOff + (uint32_t)wave * 8192u);
    const int land_kt = ((lane & 3) - (lane >> 4)) & 3;
    const uint32_t land_even = (uint32_t)((lane >> 2) * 64 + land_kt * 16);
    const uint32_t land_odd = (uint32_t)(((lane >> 2) ^ 1) * 64 + land_kt * 16);
    const int slot = th ^ ((th >> 4) & 1);
    const uint32_t rbase = stage + slot * 64;
    const int rot = rho & 3;
    const uint32_t lb0 = lds_base + ((uint32_t)lane << 2);       // this lane's column of the table
    const int wave_hi = __builtin_amdgcn_readfirstlane(wave >> 2);
    constexpr int64_t qstep = (int64_t)KW * 4096;
    const int64_t jstep = (int64_t)p.mblk_pad * 64;     // u4 units between the halves of a tile
    const int64_t astep = (int64_t)KW * 2 * p.mblk_pad * 64;

    // Work items [it_beg, it_end) of this workgroup; item = (unit, K slice), unit = (tile, chunk
    // of rows) with the chunks of a tile adjacent.  32-bit arithmetic (64-bit division costs
    // about a microsecond on this target); the first item is decoded by division, the others by
    // carrying.
    const uint32_t nwg = gridDim.x;
    const uint32_t it_beg = (uint32_t)blockIdx.x * (uint32_t)p.items / nwg;
    const uint32_t it_end = ((uint32_t)blockIdx.x + 1u) * (uint32_t)p.items / nwg;
    int z = (int)(it_beg % (uint32_t)p.ksplit);
    int unit = (int)(it_beg / (uint32_t)p.ksplit);
    int mc = (int)((uint32_t)unit % (uint32_t)p.mchunks), t = (int)((uint32_t)unit / (uint32_t)p.mchunks);
    for (uint32_t it = it_beg; it < it_end; ++it) {
        if (it != it_beg) {
            if (++z == p.ksplit) {
                z = 0;
                ++unit;
                if (++mc == p.mchunks) {
                    mc = 0;
                    ++t;
                }
            }
        }
        // the fold's scratch is the memory of the table and of the tile buffers
        if (it != it_beg) __syncthreads();

        const int mb0 = (mc * MW + mw) * MB;            // first 16-row block of this wavefront
        const int gbeg = z * p.gper, gend = min(p.G, gbeg + p.gper);
        const bool active = mb0 < p.mblk_total;         // whole wavefront
        const int g0 = gbeg + kw;
        int left = (active && g0 < gend) ? (gend - g0 + KW - 1) / KW : 0;   // tiles of this wavefront
        left = __builtin_amdgcn_readfirstlane(left);
        // A wavefront without tiles addresses the first tile of the K range: its loads are
        // then unconditional like everyone's.  The operand image is padded to whole workgroups
        // of blocks (zeros), so every block index of the grid is loadable.
        const int g_first = left > 0 ? g0 : gbeg;
        const u4_t *ap = p.Ap + ((int64_t)g_first * 2 * p.mblk_pad + mb0) * 64 + lane;
        const uint8_t *tq = p.q[0] + ((int64_t)t * p.G + g_first) * 4096;   // wavefront-uniform
        auto load_tile = [&](int buf) {                 // four loads, straight into LDS
            const uint32_t m0v = stage + (uint32_t)buf * 4096u;
            // (the pointer is the same in every lane; the compiler cannot see that through the
            // wavefront-dependent tile count)
            const uint64_t a64 = (uint64_t)(uintptr_t)tq;
            const uint8_t *tq_s = (const uint8_t *)(uintptr_t)join_address_halves(
                __builtin_amdgcn_readfirstlane((int)(uint32_t)a64),
                __builtin_amdgcn_readfirstlane((int)(uint32_t)(a64 >> 32)));
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                         "global_load_lds_dwordx4 %1, %3 offset:0 nt\n\t"
                         "global_load_lds_dwordx4 %2, %3 offset:1024 nt\n\t"
                         "global_load_lds_dwordx4 %1, %3 offset:2048 nt\n\t"
                         "global_load_lds_dwordx4 %2, %3 offset:3072 nt"
                         :: "s"(m0v), "v"(land_even), "v"(land_odd), "s"(tq_s) : "memory", "m0");
        };

        // ---- first loads, then the pair table ------------------------------------------
        u4_t A0[MB], A1[MB];
        uint32_t lv;
        {
            int row = (t * 128) / p.gs;
            row = min(row, p.lut_rows - 1);
            const uint16_t *lp = p.lut[0] + ((size_t)row << 4) + (lane & 15);
            FLUTE_STAMP(5);
            asm volatile("global_load_ushort %0, %1, off" : "=&v"(lv) : "v"(lp) : "memory");
            load_tile(0);                               // tile 0
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) lean_load16(A0[mb], ap, mb);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) lean_load16(A1[mb], ap + jstep, mb);
            // the LUT value is the oldest load: 4 + 2 MB younger ones may stay in flight
            asm volatile("s_waitcnt vmcnt(%1)" : "+v"(lv) : "n"(4 + 2 * MB) : "memory");
            FLUTE_STAMP(4);
        }
        {
            // 64 replicas per entry at a stride of 256 bytes: a wavefront writes one entry per
            // instruction, every lane the same dword, from two lane reads of the LUT row
            uint32_t *tab = (uint32_t *)smem;
            for (int code = wave; code < 256; code += NW) {
                const uint32_t lo = __builtin_amdgcn_readlane(lv, code & 15);
                const uint32_t hi = __builtin_amdgcn_readlane(lv, code >> 4);
                tab[code * 64 + lane] = lo | (hi << 16);
            }
        }
        __syncthreads();
        FLUTE_STAMP(1);
        FLUTE_STAMP(7);

        f4_t acc[MB][8];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[mb][i] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};

        // ---- K loop ---------------------------------------------------------------------
        // One round = one tile of this wavefront.  Vector memory instructions of a round, in issue
        // order: the tile after next (4, into the LDS buffer just read out), the next tile's
        // first-half operands (MB), its second-half operands (MB).  Inside a half the weight
        // operands are outermost: an operand serves all blocks of rows and is replaced by the
        // next half's right away, so lookups and products alternate four by four.
        {
            u4_t W[8];
            uint32_t Q8[8];
            uint32_t cur = 0;                             // LDS buffer of this round's tile: 0 or 4096
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
            // The four lookups of operand o = (v, d) of the half whose codes Q8 holds: the code
            // is a whole byte and the entry stride 256 bytes, so one v_perm_b32 drops it into
            // byte 1 of the lane's column address.
            auto operand = [&](int o) -> u4_t {
                const int v = o >> 1, d = o & 1;
                u4_t w;
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4)           // q4 = ktl * 2 + s2
                    w[q4] = *(LdsWord)__builtin_amdgcn_perm(
                        Q8[(q4 >> 1) * 4 + v], lb0, 0x03020000u | ((4u + d * 2 + (q4 & 1)) << 8));
                return w;
            };
            // `between` runs after the first operand's products: work that has to follow the LDS
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
                asm volatile("s_waitcnt vmcnt(%4)" : "+v"(Aj[0]), "+v"(Aj[1]), "+v"(Aj[2]), "+v"(Aj[3])
                             : "n"(decltype(younger)::value) : "memory");
            };
            if (left > 0) {
                // tile 0 is the oldest load in flight: both activation halves may stay
                asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * MB) : "memory");
                read_codes(0, 0);
#pragma unroll
                for (int o = 0; o < 8; ++o) W[o] = operand(o);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (left > 1) tq += qstep;
                load_tile(1);                             // tile 1 (or a harmless reload)
            }
            while (left > 0) {
                // the two wavefronts of a SIMD take turns at the higher priority, tile by tile
                if ((left + wave_hi) & 1) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
                const u4_t *apn = left > 1 ? ap + astep : ap;
                // this tile's first-half operands (and, older, the next tile) have arrived; the
                // second-half operands may still be in flight
                wait_half(A0, std::integral_constant<int, MB>());
                read_codes(1, cur);                       // this tile, second half
                __builtin_amdgcn_sched_barrier(0);
                half(A0, apn, [&] {
                    // the tile after next goes into the buffer just read out: not before those
                    // reads have returned
                    asm volatile("s_waitcnt lgkmcnt(0)"
                                 : "+v"(Q8[0]), "+v"(Q8[1]), "+v"(Q8[2]), "+v"(Q8[3]), "+v"(Q8[4]),
                                   "+v"(Q8[5]), "+v"(Q8[6]), "+v"(Q8[7]) :: "memory");
                    if (left > 2) tq += qstep;
                    load_tile(cur != 0);
                    __builtin_amdgcn_sched_barrier(0);
                });
                // second-half operands and (older) the next tile have arrived; the tile after
                // next and the next first-half operands may be in flight
                wait_half(A1, std::integral_constant<int, 4 + MB>());
                read_codes(0, cur ^ 4096u);               // next tile, first half
                __builtin_amdgcn_sched_barrier(0);
                half(A1, apn + jstep, [] {});
                ap = apn;
                cur ^= 4096u;
                --left;
            }
            __builtin_amdgcn_s_setprio(0);
        }
        // the loads land in LDS and registers without the compiler's knowledge: none may be in
        // flight when the fold reuses either (wavefronts without work have issued some too)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#ifdef FLUTE_STAMPS
        if (g_gemm_stamps && lane == 0) {
            long long *sl = g_gemm_stamps + ((size_t)blockIdx.x * NW + wave) * 8;
            sl[7] = (long long)__builtin_readcyclecounter() - sl[7];
        }
#endif
        FLUTE_STAMP(2);

        // ---- fold across the K ways --------------------------------------------------------
        // Accumulator f = mb * 8 + o belongs to the way f / IPO.  In each of two rounds a
        // wavefront sends every other way HALF of the accumulators that way owns and sums its own
        // HALF over the ways in the order 0 .. KW - 1 (its own term from registers).
        f4_t *scr = (f4_t *)smem;                       // slots of 64 f4
        f4_t tot[IPO];
        __syncthreads();                                // table and tile buffers are dead from here
        FLUTE_STAMP(3);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
#pragma unroll
            for (int ow = 0; ow < KW; ++ow) {
                if (ow != kw) {
                    const int sender = kw < ow ? kw : kw - 1;
                    f4_t *dst = scr + (size_t)(((mw * KW + ow) * (KW - 1) + sender) * HALF) * 64 + lane;
#pragma unroll
                    for (int l = 0; l < HALF; ++l) {
                        const int f = ow * IPO + r * HALF + l;
                        dst[l * 64] = acc[f >> 3][f & 7];
                    }
                }
            }
            __syncthreads();
#pragma unroll
            for (int ow = 0; ow < KW; ++ow) {
                if (ow == kw) {
#pragma unroll
                    for (int l = 0; l < HALF; ++l) {
                        const int f = ow * IPO + r * HALF + l;
                        f4_t v = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int s = 0; s < KW; ++s) {
                            if (s == ow) {
                                v += acc[f >> 3][f & 7];
                            } else {
                                const int sender = s < ow ? s : s - 1;
                                v += scr[(size_t)((((mw * KW + ow) * (KW - 1) + sender) * HALF) + l) * 64 + lane];
                            }
                        }
                        tot[r * HALF + l] = v;
                    }
                }
            }
            if (r == 0) __syncthreads();
        }

        // ---- across workgroups: partial images from registers, ticket, the last arrival sums ---
        constexpr size_t IMG = (size_t)NW * IPO * 256;  // floats per (K slice, unit)
        if (p.ztotal > 1) {
            float *mine = p.P + ((size_t)(p.z_base + z) * p.units + unit) * IMG +
                          (size_t)wave * IPO * 256 + lane * 4;
#pragma unroll
            for (int l = 0; l < IPO; ++l) ws_store16(mine + l * 256, tot[l]);
            ws_stores_done();
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
            int *flag = (int *)(smem + kLeanFlagOff);
            if (tid == 0) {
                const int old = __hip_atomic_fetch_add(p.tickets + unit, 1, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
                *flag = (old == p.ztotal - 1);
            }
            __syncthreads();
            if (!*flag) continue;                       // (uniform) not the last of this unit
            if (tid == 0)
                __hip_atomic_store(p.tickets + unit, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float *src = p.P + (size_t)unit * IMG + (size_t)wave * IPO * 256 + lane * 4;
            const size_t zstride = (size_t)p.units * IMG;
#pragma unroll
            for (int l = 0; l < IPO; ++l) tot[l] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
            for (int z0 = 0; z0 < p.ztotal; ++z0) {     // fixed order: the same sums every run
                const float *s0 = src + (size_t)z0 * zstride;
                static_assert(IPO % 4 == 0, "four loads in flight");
#pragma unroll
                for (int l = 0; l < IPO; l += 4) {
                    f4_t a, b, c, d;
                    ws_load16x4(s0 + l * 256, s0 + (l + 1) * 256, s0 + (l + 2) * 256, s0 + (l + 3) * 256,
                                a, b, c, d);
                    tot[l] += a;
                    tot[l + 1] += b;
                    tot[l + 2] += c;
                    tot[l + 3] += d;
                }
            }
        }

        // ---- residual, bias, one rounding, store ----------------------------------------------
        // A total holds four consecutive outputs of row m; the totals o = 2a and 2a + 1 of the lanes
        // kg and kg ^ 1 (sixteen lanes apart) together are sixteen consecutive outputs.  After the
        // rounding the two lanes swap a half each (v_permlane16_swap), so that every lane stores
        // eight consecutive outputs, 16 bytes.
        static_assert(IPO % 2 == 0, "totals come in pairs");
#pragma unroll
        for (int l = 0; l < IPO; l += 2) {
            const int f = kw * IPO + l;
            const int mb = f >> 3, o = f & 7;           // o even
            const int m = ((mc * MW + mw) * MB + mb) * 16 + rho;
            const bool valid = m < p.M;
            const int mr = valid ? m : p.M - 1;         // operands of a row beyond M: any valid row
            const int n0 = t * 128 + (kg >> 1) * 64 + (o >> 1) * 16 + (kg & 1) * 4;   // + 8 for o + 1
            uint32_t packed[2][2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float y[4] = {tot[l + h][0], tot[l + h][1], tot[l + h][2], tot[l + h][3]};
                const int nh = n0 + 8 * h;
                if (p.rowshift) {                       // undo the row's activation scaling (exact)
                    const int sh = p.rowshift[mr];
#pragma unroll
                    for (int e = 0; e < 4; ++e) y[e] = ldexpf(y[e], sh);
                }
                if (p.R > 0) {
                    const float *xr = p.xb + (size_t)mr * p.R;
                    for (int r = 0; r < p.R; ++r) {
                        const float c = xr[r];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            y[e] = fmaf(c, load_act(p.resA, (int64_t)(nh + e) * p.R + r, p.out_bf16), y[e]);
                    }
                }
                if (p.bias) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) y[e] += load_act(p.bias, nh + e, p.out_bf16);
                }
                packed[h][0] = (uint32_t)round_act(y[0], p.out_bf16) | ((uint32_t)round_act(y[1], p.out_bf16) << 16);
                packed[h][1] = (uint32_t)round_act(y[2], p.out_bf16) | ((uint32_t)round_act(y[3], p.out_bf16) << 16);
            }
            // even rows of sixteen lanes keep their first total and get the partner's first; odd
            // rows get the partner's second and keep their second
            const auto s0 = __builtin_amdgcn_permlane16_swap(packed[0][0], packed[1][0], false, false);
            const auto s1 = __builtin_amdgcn_permlane16_swap(packed[0][1], packed[1][1], false, false);
            const int ns = (kg & 1) ? n0 + 4 : n0;      // first of this lane's eight outputs
            if (valid) {
                uint16_t *dst = (uint16_t *)p.C + (size_t)m * p.ldc + ns;
                if (p.vec_store) {
                    *(u4_t *)dst = u4_t{s0[0], s1[0], s0[1], s1[1]};
                } else {
                    const uint32_t out[4] = {s0[0], s1[0], s0[1], s1[1]};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        dst[2 * e] = (uint16_t)out[e];
                        dst[2 * e + 1] = (uint16_t)(out[e] >> 16);
                    }
                }
            }
        }
        FLUTE_STAMP(6);
    }
}

}  // namespace flute
