// Lean specialisation of the M = 1 LUT GEMV for the common case: every stream
// 4 bits wide and one LUT group per 128-row tile (group_size >= 128).  Same
// ownership, lane mapping, table format and K-split protocol as gemv_kernel.h;
// the row-slice width, the wavefront count and the table stride are template
// constants so that the prologue and the per-load overhead shrink to a few
// dozen instructions.
#pragma once

#include "gemv_kernel.h"

namespace flute {

// LPGL = log2(lanes per 64-k tile) = log2(2 * rows per workgroup): 4, 5, 6.
// NW   = wavefronts per workgroup.
// PF   = index loads a lane keeps in flight (2, 3 or 4).  A few loads per
//        wavefront, refilled as they are consumed, serve every wavefront of the grid
//        in turn; a deep queue (a wavefront's whole K range requested at once) is
//        served wavefront by wavefront, and the last ones served start their
//        arithmetic when the memory stream is already over.  The host picks the
//        largest PF that divides the units of a wavefront, so that the K loop has no
//        partial group.
// The table stride is 128 bytes (32 replicas of a 4-byte entry, 32 KB): three
// four-wavefront workgroups fit a CU.
template <int LPGL, int NW, int PF, bool BF16>
__global__ void __launch_bounds__(NW * 64, 3) gemv4_kernel(const GemvParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int ES = 7;
    constexpr int NT = NW * 64;
    constexpr int LPG = 1 << LPGL;
    constexpr int GPI = 64 >> LPGL;                 // 64-k tiles per wavefront load
    constexpr int RW = LPG >> 1;                    // rows per workgroup
    constexpr int SPT = 128 / RW;                   // row slices per tile
    constexpr int XV = 2;                           // 16-byte activation loads per thread
    constexpr int PF0 = 1;                          // index loads issued ahead of the table build
    constexpr int STRIDE = 1 << ES;                 // table bytes per entry
    constexpr int CHUNKS = STRIDE / 16;             // 16-byte pieces of one entry's replicas
    constexpr int SHARES = NT / 256;                // threads per table entry
    constexpr int CPT = CHUNKS / SHARES;            // pieces written per thread
    static_assert(NT >= 256, "one thread per table entry at least");

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
    const int gsub = L >> LPGL;
    const int l = L & (LPG - 1);
    const int sl = (int)blockIdx.x - kp->seg[si0].col0;
    const int t = sl / SPT;
    const int cg0 = (sl % SPT) * (RW >> 3);
    const int s = blockIdx.y;
    const int g_lo = s * p.gs_tiles;
    const int units = p.gs_tiles / GPI;
    const int my_units = units > w ? (units - w + NW - 1) / NW : 0;
    const int k0 = g_lo * 64, kc = p.gs_tiles * 64;
    const int G = p.K >> 6;

    uint16_t *xs = (uint16_t *)(lds + p.lds_x);
    const uint32_t *xs32 = (const uint32_t *)xs;
    float *red = (float *)(lds + p.lds_red);        // [2][NW][32] row sums

    // lane-constant pieces of the addresses
    const uint32_t unit_bytes = GPI * 4096u;
    const uint32_t lane0 = (uint32_t)gsub * 4096u + (uint32_t)cg0 * 256u + (uint32_t)l * 16u +
                           (uint32_t)w * unit_bytes;
    constexpr uint32_t step = NW * GPI * 4096u;
    const int xi = gsub * 32 + (l & 3) * 8 + ((l >> 2) & 3) + w * (GPI * 32);
    // Lookup addresses are formed as absolute LDS addresses, so the (zero) base of
    // the dynamic LDS block is folded into the per-lane replica offset once
    // instead of being added after every v_perm.
    typedef const __attribute__((address_space(3))) uint32_t *LdsWord;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const uint32_t slot = lds_base + (uint32_t)(L & 31) * 4u;
    const int e_own = tid & 255;                    // table entry this thread writes
    const int share = tid >> 8;

    const int nout = p.silu_mul ? 2 : 1;

    // A pass is one (output, stream) of this workgroup's rows: one output with one
    // stream for a plain weight, two streams for a dual-stream weight, two outputs
    // for the gate/up pair.  Every pass covers the same K range with the same lane
    // geometry; only the index blob and the LUT row change.
    auto pass_ptrs = [&](int so_, int si_, const uint8_t *&qr, const uint16_t *&lutp) {
        const int sg = so_ == 1 ? 1 : si0;
        const GemvStream st = kp->seg[sg].st[si_];
        const int grp = min((t * 128) >> __builtin_ctz(kp->seg[sg].gs), kp->seg[sg].lut_rows - 1);
        qr = st.q + ((size_t)t * G + g_lo) * 4096u;
        lutp = st.lut + ((size_t)grp << 4);
    };
    // A wavefront with fewer than PF loads re-reads the first unit of the K range
    // (always present) into the registers it will not consume: every load below is
    // unconditional, so the compiler knows how many are in flight at each point and
    // waits for exactly the one it needs.  One conditional load in a loop makes it
    // wait for all of them at the loop head, which serialises the memory stream and
    // the arithmetic.
    // Index loads are addressed as (uniform base + unit offset) in scalar registers
    // plus one lane-constant 32-bit offset, so no per-load address lives in vector
    // registers.
    auto unit_load = [&](const uint8_t *qr, int unit) -> uint4 {
        const uint8_t *base = unit < my_units ? qr + (size_t)unit * step
                                              : qr - (size_t)w * unit_bytes;
        return *(const uint4 *)(base + lane0);
    };
    auto first_units = [&](const uint8_t *qr, uint4 (&qq)[PF]) {
#pragma unroll
        for (int n = 0; n < PF; ++n) {
            qq[n] = unit_load(qr, n);
            __builtin_amdgcn_sched_barrier(0);      // issue order = consumption order
        }
    };

    // Paired table: entry e -> {lut[e & 15], lut[e >> 4]}, replicated over the stride;
    // 16 bytes per store, starting at a lane-dependent piece so that a wavefront
    // spreads over the banks.
    auto write_table = [&](uint32_t lo_, uint32_t hi_) {
        const uint32_t v = lo_ | (hi_ << 16);
        const uint4 v4 = make_uint4(v, v, v, v);
        uint8_t *ent = lds + e_own * STRIDE + share * (CPT * 16);
#pragma unroll
        for (int k = 0; k < CPT; ++k) *(uint4 *)(ent + (((k + tid) & (CPT - 1)) << 4)) = v4;
    };

    FLUTE_TRACE(0);
    // Wavefront priority falls as a workgroup advances: 3 in the prologue, 2 while
    // there is more to stream, 1 in the last group, 0 from the fold on.  A SIMD holds
    // one wavefront of each resident workgroup and serves the oldest first; without
    // this the workgroup that arrived last on a CU lags through the whole launch and
    // ends more than a microsecond after the first.
    __builtin_amdgcn_s_setprio(3);
    // ---- first pass: activations, LUT values and the first index bytes.  The order
    //      of the loads is the order they are needed in, and the scheduler is kept
    //      from changing it: a wait for an early load also waits for everything
    //      issued before it. ---------------------------------------------------------
    int so = 0, si = 0;
    const uint8_t *qrow;
    const uint16_t *lut;
    pass_ptrs(0, 0, qrow, lut);
    const uint16_t *staged_x = kp->seg[si0].xsrc ? kp->seg[si0].xsrc : p.x;
    const float *staged_signs = kp->seg[si0].signs, *staged_awq = kp->seg[si0].awq;
    const bool x_direct = staged_signs == nullptr;  // plain copy
    const bool x_short = kc <= XV * NT * 8;         // uniform
    uint4 q[PF];
    uint32_t lo, hi;
    if (x_direct && x_short) {
        // The usual case.  A few index loads go out ahead of the table build so that
        // the memory stream starts early; the rest follow once the table is written.
        // (All of them at once would put every other workgroup's activation and LUT
        // loads behind a full batch of index bytes in the CU's memory queue.)
        uint4 xv[XV];
#pragma unroll
        for (int i = 0; i < XV; ++i) {
            const int j = (i * NT + tid) * 8;
            xv[i] = *(const uint4 *)(staged_x + k0 + (j < kc ? j : 0));
        }
        __builtin_amdgcn_sched_barrier(0);
        lo = lut[e_own & 15];
        hi = lut[e_own >> 4];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < PF0; ++n) {
            q[n] = unit_load(qrow, n);
            __builtin_amdgcn_sched_barrier(0);
        }
        FLUTE_TRACE(1);
#pragma unroll
        for (int i = 0; i < XV; ++i) {
            const int j = (i * NT + tid) * 8;
            if (j < kc) *(uint4 *)(xs + j) = to_compute_type<BF16>(xv[i], p.act_bf16);
        }
        write_table(lo, hi);
#pragma unroll
        for (int n = PF0; n < PF; ++n) {
            q[n] = unit_load(qrow, n);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else if (x_direct) {
        // A long K range: everything the table and the staged activations need is
        // fetched and written first (the index registers carry the activations
        // meanwhile), then the index loads start.
#pragma unroll
        for (int n = 0; n < PF; ++n) {
            const int j = (n * NT + tid) * 8;
            q[n] = *(const uint4 *)(staged_x + k0 + (j < kc ? j : 0));
        }
        __builtin_amdgcn_sched_barrier(0);
        lo = lut[e_own & 15];
        hi = lut[e_own >> 4];
        __builtin_amdgcn_sched_barrier(0);
        FLUTE_TRACE(1);
#pragma unroll
        for (int n = 0; n < PF; ++n) {
            const int j = (n * NT + tid) * 8;
            if (j < kc) *(uint4 *)(xs + j) = to_compute_type<BF16>(q[n], p.act_bf16);
        }
        for (int j = (PF * NT + tid) * 8; j < kc; j += NT * 8)
            *(uint4 *)(xs + j) =
                to_compute_type<BF16>(*(const uint4 *)(staged_x + k0 + j), p.act_bf16);
        write_table(lo, hi);
        __builtin_amdgcn_sched_barrier(0);
        first_units(qrow, q);
    } else {
        // A rotated input: the LUT values and the first index loads travel while the
        // rotation runs.
        lo = lut[e_own & 15];
        hi = lut[e_own >> 4];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < PF0; ++n) {
            q[n] = unit_load(qrow, n);
            __builtin_amdgcn_sched_barrier(0);
        }
        FLUTE_TRACE(1);
        stage_x<BF16>(p, staged_x, staged_signs, staged_awq, lds, k0, kc, tid, NT);
        write_table(lo, hi);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = PF0; n < PF; ++n) {
            q[n] = unit_load(qrow, n);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    float acc[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) acc[a] = 0.0f;

    for (bool first = true;; first = false) {
        const int sg = so == 1 ? 1 : si0;
        if (!first) {
            // every output of the launch reads the same staged activations (the host
            // sends launches whose outputs differ in input or rotation to the general
            // kernel), so only the table changes between passes
            write_table(lo, hi);
        }

        // ---- the pass after this one: its LUT values are fetched now and its first
        //      index loads replace this pass's last ones as they are consumed, so the
        //      memory stream does not stop between passes.  Without a next pass the
        //      same LUT values are read again (harmless, and keeps the load count
        //      unconditional). -----------------------------------------------------------
        int nso = so, nsi = si + 1;
        if (nsi == kp->seg[sg].nstreams) {
            nsi = 0;
            nso = so + 1;
        }
        const bool has_next = nso < nout;
        const uint8_t *qnext = qrow;
        const uint16_t *lutn = lut;
        if (has_next) pass_ptrs(nso, nsi, qnext, lutn);
        __builtin_amdgcn_sched_barrier(0);
        lo = lutn[e_own & 15];
        hi = lutn[e_own >> 4];
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
#ifdef FLUTE_GEMV_TRACE
        if (first) FLUTE_TRACE(2); else if (so == 1 && si == 0) FLUTE_TRACE(7);
#endif

        // ---- K loop -----------------------------------------------------------------
        // One unit = one 16-byte load of this lane.  Its sixteen table lookups go out
        // together and are consumed together, so the LDS latency is paid once per
        // load, not once per dword.
        auto lookups = [&](const uint4 &qv, uint32_t (&e)[4][4]) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t wv = v == 0 ? qv.x : v == 1 ? qv.y : v == 2 ? qv.z : qv.w;
#pragma unroll
                for (int j = 0; j < 4; ++j) {       // byte j: d = j >> 1, s2 = j & 1
                    e[v][j] = *(LdsWord)((((wv >> (8 * j)) & 0xffu) << ES) + slot);
                }
            }
        };
        auto dots = [&](const uint32_t (&e)[4][4], int m) {
            const int xo = xi + m * (NW * GPI * 32);
            const uint32_t xa = xs32[xo];
            const uint32_t xb = xs32[xo + 4];
#pragma unroll
            for (int v = 0; v < 4; ++v)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[v * 2 + (j >> 1)] =
                        dot2<BF16>(e[v][j], (j & 1) ? xb : xa, acc[v * 2 + (j >> 1)]);
        };
        int nb = 0;
        __builtin_amdgcn_s_setprio(2);
        for (; nb + 2 * PF <= my_units; nb += PF) {          // every refill exists
#pragma unroll
            for (int n = 0; n < PF; ++n) {
                uint32_t e[4][4];
                lookups(q[n], e);
                // pinned: the scheduler would otherwise sink all refills to the end of
                // the body, draining the prefetch queue once per group
                __builtin_amdgcn_sched_barrier(0);
                q[n] = *(const uint4 *)(qrow + (size_t)(nb + n + PF) * step + lane0);
                __builtin_amdgcn_sched_barrier(0);
                dots(e, nb + n);
            }
        }
        if (!has_next) __builtin_amdgcn_s_setprio(1);
        if (nb + PF == my_units && has_next) {                // a full last group, refilled
#pragma unroll                                                //   from the next pass
            for (int n = 0; n < PF; ++n) {
                uint32_t e[4][4];
                lookups(q[n], e);
                __builtin_amdgcn_sched_barrier(0);
                q[n] = *(const uint4 *)(qnext + (size_t)n * step + lane0);
                __builtin_amdgcn_sched_barrier(0);
                dots(e, nb + n);
            }
        } else if (nb + PF >= my_units) {                     // the last group, no refills
#pragma unroll
            for (int n = 0; n < PF; ++n) {
                if (nb + n < my_units) {                      // uniform within the wavefront
                    uint32_t e[4][4];
                    lookups(q[n], e);
                    dots(e, nb + n);
                }
            }
            if (has_next) first_units(qnext, q);
        } else {                                              // a partial group follows
            for (; nb < my_units; nb += PF) {
#pragma unroll
                for (int n = 0; n < PF; ++n) {
                    const int m = nb + n;
                    if (m < my_units) {
                        uint32_t e[4][4];
                        lookups(q[n], e);
                        if (m + PF < my_units)
                            q[n] = *(const uint4 *)(qrow + (size_t)(m + PF) * step + lane0);
                        dots(e, m);
                    }
                }
            }
            __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): see below
            if (has_next) first_units(qnext, q);
        }
#ifdef FLUTE_GEMV_TRACE
        if (!has_next) FLUTE_TRACE(3); else if (first) FLUTE_TRACE(6);
#endif

        if (!has_next) __builtin_amdgcn_s_setprio(0);
        // ---- end of an output: fold the lanes that share rows ------------------------
        if (nso != so) {
#pragma unroll
            for (int a = 0; a < 8; ++a) {
                float v = row16_sum(acc[a]);
                if constexpr (LPGL <= 5) v += __shfl_xor(v, 32);
                if constexpr (LPGL == 4) v += __shfl_xor(v, 16);
                acc[a] = v;
            }
            if (L < LPG && (L & 15) == 0) {
#pragma unroll
                for (int a = 0; a < 8; ++a) red[(so * NW + w) * 32 + (L >> 4) * 8 + a] = acc[a];
            }
#pragma unroll
            for (int a = 0; a < 8; ++a) acc[a] = 0.0f;
        }
        if (!has_next) break;
        __syncthreads();                            // the table region is rewritten next
        so = nso;
        si = nsi;
        qrow = qnext;
        lut = lutn;
    }
    __syncthreads();
    FLUTE_TRACE(4);

    // ---- one thread per owned row --------------------------------------------------
    if (tid >= RW && p.split == 1) return;
    const bool owner = tid < RW;
    const int n = t * 128 + row_of(cg0 + (tid >> 3), tid & 7);
    float yv[2] = {0.0f, 0.0f};
    if (owner) {
#pragma unroll
        for (int so = 0; so < 2; ++so) {
            if (so >= nout) break;
            float y = 0.0f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) y += red[(so * NW + ww) * 32 + tid];
            yv[so] = y;
        }
    }

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
        kp->seg[si0].out[n] = round_act(y, p.act_bf16);
    }
    FLUTE_TRACE(5);
}

}  // namespace flute
