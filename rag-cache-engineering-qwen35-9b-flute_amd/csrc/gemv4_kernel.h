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
// ES   = log2(table stride): 8 (v_perm addressing, 64 KB) or 7 (32 KB).
// MULTI = several independent weights share the launch (the descriptor is then
//         picked by grid column, which costs a dependent scalar load).
template <int LPGL, int NW, int ES, bool BF16, bool MULTI>
__global__ void __launch_bounds__(NW * 64) gemv4_kernel(const GemvParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int NT = NW * 64;
    constexpr int LPG = 1 << LPGL;
    constexpr int GPI = 64 >> LPGL;                 // 64-k tiles per wavefront load
    constexpr int RW = LPG >> 1;                    // rows per workgroup
    constexpr int SPT = 128 / RW;                   // row slices per tile
    constexpr int PF = NW == 4 ? 8 : 4;             // wavefront loads in flight per lane
    constexpr int XV = 2;                           // 16-byte activation loads per thread
#ifndef FLUTE_GEMV4_LB
#define FLUTE_GEMV4_LB 4
#endif
    constexpr int LB = FLUTE_GEMV4_LB;              // dwords of a load looked up per batch
    constexpr int STRIDE = 1 << ES;                 // table bytes per entry
    constexpr int CHUNKS = STRIDE / 16;             // 16-byte pieces of one entry's replicas
    constexpr int SHARES = NT / 256;                // threads per table entry
    constexpr int CPT = CHUNKS / SHARES;            // pieces written per thread
    static_assert(NT >= 256, "one thread per table entry at least");

    const GemvParams *kp = (const GemvParams *)(const void *)__builtin_amdgcn_kernarg_segment_ptr();
    int si0 = 0;
    if (MULTI && !p.silu_mul) {
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
    const uint32_t slot = lds_base + (ES == 8 ? (uint32_t)L * 4u : (uint32_t)(L & 31) * 4u);
    const int e_own = tid & 255;                    // table entry this thread writes
    const int share = tid >> 8;

    const int nout = p.silu_mul ? 2 : 1;
    const uint16_t *staged_x = nullptr;
    const float *staged_signs = nullptr, *staged_awq = nullptr;
    bool staged = false;

    FLUTE_TRACE(0);
    for (int so = 0; so < nout; ++so) {
        const int si_seg = so == 1 ? 1 : si0;
        const uint16_t *xin = kp->seg[si_seg].xsrc ? kp->seg[si_seg].xsrc : p.x;
        const float *signs = kp->seg[si_seg].signs, *awq = kp->seg[si_seg].awq;
        const int nstreams = kp->seg[si_seg].nstreams;
        const int lut_rows = kp->seg[si_seg].lut_rows;
        const int grp = min((t * 128) / kp->seg[si_seg].gs, lut_rows - 1);
        const bool restage = !staged || xin != staged_x || signs != staged_signs || awq != staged_awq;
        const bool x_direct = restage && signs == nullptr;     // plain copy: loads issued first

        float acc[8];
#pragma unroll
        for (int a = 0; a < 8; ++a) acc[a] = 0.0f;

        for (int si = 0; si < nstreams; ++si) {
            const GemvStream st = kp->seg[si_seg].st[si];
            // ---- loads, in the order they are needed: activations, LUT, indices ----
            uint4 xv[XV];
            if (si == 0 && x_direct) {
#pragma unroll
                for (int i = 0; i < XV; ++i) {
                    const int j = (i * NT + tid) * 8;
                    xv[i] = make_uint4(0u, 0u, 0u, 0u);
                    if (j < kc) xv[i] = *(const uint4 *)(xin + k0 + j);
                }
            }
            const uint16_t *lut = st.lut + ((size_t)grp << 4);
            const uint32_t lo = lut[e_own & 15], hi = lut[e_own >> 4];
            const uint8_t *qrow = st.q + ((size_t)t * G + g_lo) * 4096u;
            uint4 q[PF];
#pragma unroll
            for (int n = 0; n < PF; ++n) {
                q[n] = make_uint4(0u, 0u, 0u, 0u);
                if (n < my_units) q[n] = *(const uint4 *)(qrow + (lane0 + (uint32_t)n * step));
            }

            FLUTE_TRACE(1);
            // ---- activations into LDS ---------------------------------------------
            if (si == 0 && restage) {
                if (x_direct) {
#pragma unroll
                    for (int i = 0; i < XV; ++i) {
                        const int j = (i * NT + tid) * 8;
                        if (j < kc) *(uint4 *)(xs + j) = to_compute_type<BF16>(xv[i], p.act_bf16);
                    }
                    for (int j = (XV * NT + tid) * 8; j < kc; j += NT * 8)
                        *(uint4 *)(xs + j) =
                            to_compute_type<BF16>(*(const uint4 *)(xin + k0 + j), p.act_bf16);
                } else {
                    stage_x<BF16>(p, xin, signs, awq, lds, k0, kc, tid, NT);
                }
                staged = true;
                staged_x = xin;
                staged_signs = signs;
                staged_awq = awq;
            }

            // ---- paired table: entry e -> {lut[e & 15], lut[e >> 4]}, replicated over
            //      the stride; 16 bytes per store, starting at a lane-dependent piece so
            //      that a wavefront spreads over the banks --------------------------------
            {
                const uint32_t v = lo | (hi << 16);
                const uint4 v4 = make_uint4(v, v, v, v);
                uint8_t *ent = lds + e_own * STRIDE + share * (CPT * 16);
#pragma unroll
                for (int k = 0; k < CPT; ++k)
                    *(uint4 *)(ent + (((k + tid) & (CPT - 1)) << 4)) = v4;
            }
            __syncthreads();
            FLUTE_TRACE(2);

            // ---- K loop -----------------------------------------------------------
            for (int nb = 0; nb < my_units; nb += PF) {
#pragma unroll
                for (int n = 0; n < PF; ++n) {
                    const int m = nb + n;
                    if (m < my_units) {             // uniform within the wavefront
                        const int xo = xi + m * (NW * GPI * 32);
                        const uint32_t xa = xs32[xo];
                        const uint32_t xb = xs32[xo + 4];
                        // The lookups of LB dwords of the load go out together and are
                        // consumed together, so their LDS latency is paid once per batch,
                        // not once per dword.
#pragma unroll
                        for (int vb = 0; vb < 4; vb += LB) {
                            uint32_t e[LB][4];
#pragma unroll
                            for (int v = 0; v < LB; ++v) {
                                const uint32_t wv = vb + v == 0 ? q[n].x
                                                  : vb + v == 1 ? q[n].y
                                                  : vb + v == 2 ? q[n].z : q[n].w;
#pragma unroll
                                for (int j = 0; j < 4; ++j) {   // byte j: d = j >> 1, s2 = j & 1
                                    uint32_t addr;
                                    if constexpr (ES == 8) {
                                        addr = __builtin_amdgcn_perm(wv, slot,
                                                                     0x03020000u | ((4u + j) << 8));
                                    } else {
                                        addr = (((wv >> (8 * j)) & 0xffu) << ES) + slot;
                                    }
                                    e[v][j] = *(LdsWord)addr;
                                }
                            }
                            if (vb + LB == 4 && m + PF < my_units)   // indices consumed: refill
                                q[n] = *(const uint4 *)(qrow + (lane0 + (uint32_t)(m + PF) * step));
#pragma unroll
                            for (int v = 0; v < LB; ++v)
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    acc[(vb + v) * 2 + (j >> 1)] = dot2<BF16>(
                                        e[v][j], (j & 1) ? xb : xa, acc[(vb + v) * 2 + (j >> 1)]);
                        }
                    }
                }
            }
            FLUTE_TRACE(3);
            __syncthreads();                       // the table region is rewritten next
        }

        // fold the lanes that share rows
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
