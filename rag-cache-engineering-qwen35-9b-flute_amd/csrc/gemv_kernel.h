// M = 1 LUT GEMV for gfx950 (wave64), the decode kernel of the idxN layer.
//
// Work decomposition.  The unit of work is one STREAM of one weight, one
// 128-row tile t, one K-split s:  workgroup (x = tile column, y = s), 256
// threads = 4 wavefronts.  Wavefront u owns QUARTER u of every 64-k tile of
// the split: the 16 consecutive thread-chunks [16u, 16u+16) of the idxN tile,
// which are 256*b contiguous bytes.  Lane L reads the 4*b bytes at L*4*b of
// that quarter — one fully coalesced load per tile per wavefront — and those
// bytes are exactly quarter kt = L & 3 of chunk c = 16u + (L >> 2), i.e.
//
//     rows  n = t*128 + (u>>1)*64 + v*16 + d*8 + 4*(u&1) + (L>>4)   (v<4, d<2)
//     cols  k = g*64 + (L&3)*16 + 2*((L>>2)&3) + 8*s2  and k+1     (s2<2)
//
// so a lane keeps 8 fp32 row accumulators for the whole K range and the 16
// lanes L&15 that share a row are folded once at the end with DPP.
//
// Dequantisation.  The per-group LUT (2^b 16-bit values) is expanded once per
// workgroup into a paired table in LDS that is indexed by a whole packed byte
// (b = 4: byte -> {W[k], W[k+1]}; b = 2: byte -> 4 values; b = 1: byte -> 8
// values; b = 3: 6-bit pair field -> 2 values).  Every entry is replicated
// across a power-of-two stride so that each lane reads its own bank: a lookup
// is one ds_read with no bank conflicts whatever the codes are.  With a 256-byte
// stride the address is {slot byte, code byte} and is formed by one v_perm_b32.
// A looked-up pair feeds v_dot2_f32_f16 / v_dot2_f32_bf16 against the matching
// activation pair: 2 MACs per instruction, fp32 accumulate.
//
// Split-K.  Row partials of every (stream, split) slot go to a workspace
// P[slot][column]; the last workgroup to arrive at an output tile (a ticket
// counter per tile) folds the slots in fixed order, adds the low-rank residual
// and the bias in fp32, applies SiLU*mul for the merged gate/up mode, rounds
// once and resets the ticket, so the launch is deterministic and replayable.
#pragma once

#include "common.h"
#include "fht_dev.h"

namespace flute {

constexpr int kGemvThreads = 256;
constexpr int kGemvMaxJobs = 8;
constexpr int kGemvMaxSegs = 4;
constexpr int kGemvMaxRank = 256;
constexpr int kPrefetch = 8;          // 64-k tiles of index data in flight per lane

struct GemvJob {            // one stream of one weight
    const uint8_t *q;       // idxN blob
    const uint16_t *lut;    // [rows, 2^bits]
    int tile0;              // first grid column of this job
    int ntiles;             // N / 128
    int bits;
    int seg;
    int es;                 // log2(LDS bytes between consecutive table entries)
    int slot0;              // first partial-sum slot of this stream
};

struct GemvSeg {            // one weight
    const uint16_t *resB;   // (R, K) or null
    const uint16_t *resA;   // (N, R) or null
    const uint16_t *bias;   // (N,) or null
    const float *signs;     // (K,) or null: rotate the input first
    const float *awq;       // (K,) or null
    uint16_t *out;          // (N,)
    int N;
    int R;
    int gs;
    int lut_rows;
    int nslots;             // partial-sum slots of this weight (streams * split)
    int arrivals;           // workgroups that must arrive before an output tile is finished
    int n0;                 // first column of this weight in a partial-sum row
    int r0;                 // first residual column of this weight
    int ticket0;            // first ticket of this weight
};

struct GemvParams {
    GemvJob job[kGemvMaxJobs];
    GemvSeg seg[kGemvMaxSegs];
    const uint16_t *x;      // (K,) activations
    float *P;               // partial sums: [slot][p_stride]
    int *tickets;
    int njobs;
    int K;
    int split;
    int gs_tiles;           // 64-k tiles per split
    int p_stride;           // floats per partial-sum row
    int silu_mul;           // 1: out = silu(seg 0) * seg 1, written to seg[0].out
    int act_bf16;           // activations, residual, bias and outputs are bf16
    int fht_block;          // > 0: equal rotation blocks of this many columns
    int lds_x;              // LDS byte offsets
    int lds_red;
    int lds_xb;
};

// ---- small device helpers ---------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
    return v + __builtin_bit_cast(float, moved);
}

// Sum over the 16 lanes of a DPP row; every lane of the row ends with the total.
__device__ __forceinline__ float row16_sum(float v) {
    v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);   // row_half_mirror
    v = dpp_add<0x140>(v);   // row_mirror
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

// Table geometry per width: entries, bytes per entry.
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

// Expand `ngrp` LUT rows into replicated paired tables at tab (LDS).  Table of
// group q starts at q * (kEntries << es); entry e at e << es; the entry repeats
// every kEntryBytes inside its stride.  A thread owns one (group, entry) at a
// time and walks the replicas starting at a lane-dependent one, so that the 64
// lanes of a wavefront write 64 different banks.
template <int B>
__device__ __forceinline__ void build_tables(uint8_t *tab, const uint16_t *lut_rows, int ngrp,
                                             int es, int tid) {
    constexpr int E = TableShape<B>::kEntries;
    constexpr int EL = TableShape<B>::kEntryLog2;
    constexpr int EDW = 1 << (EL - 2);              // dwords per entry
    const int nrep = 1 << (es - EL);                // replicas per entry
    for (int item = tid; item < ngrp * E; item += kGemvThreads) {
        const int q = item / E, e = item % E;
        const uint16_t *lut = lut_rows + ((size_t)q << B);
        uint32_t val[EDW];
#pragma unroll
        for (int s = 0; s < EDW; ++s) val[s] = table_dword<B>(lut, e, s);
        uint8_t *ent = tab + (size_t)q * (E << es) + ((size_t)e << es);
        for (int r = 0; r < nrep; ++r) {
            const int rep = (r + tid) & (nrep - 1);
            uint32_t *dst = (uint32_t *)(ent + (rep << EL));
#pragma unroll
            for (int s = 0; s < EDW; ++s) dst[s] = val[s];
        }
    }
}

// One quarter-tile (4*B bytes of this lane) against the activation pairs xa
// (s2 = 0) and xb (s2 = 1).  lane_off[v] = table base of row block v plus this
// lane's replica offset.
template <int B, bool BF16, bool PERM>
__device__ __forceinline__ void consume_tile(const uint32_t (&w)[B], uint32_t xa, uint32_t xb,
                                             const uint8_t *lds, const uint32_t (&lane_off)[4],
                                             int es, float (&acc)[8]) {
    if constexpr (B == 4) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {          // byte j: d = j >> 1, s2 = j & 1
                uint32_t addr;
                if constexpr (PERM) {
                    addr = __builtin_amdgcn_perm(w[v], lane_off[v], 0x03020000u | ((4u + j) << 8));
                } else {
                    addr = (((w[v] >> (8 * j)) & 0xffu) << es) + lane_off[v];
                }
                const uint32_t e = *(const uint32_t *)(lds + addr);
                acc[v * 2 + (j >> 1)] = dot2<BF16>(e, (j & 1) ? xb : xa, acc[v * 2 + (j >> 1)]);
            }
        }
    } else if constexpr (B == 2) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                const int j = (v & 1) * 2 + d;      // byte j of dword v >> 1
                uint32_t addr;
                if constexpr (PERM) {
                    addr = __builtin_amdgcn_perm(w[v >> 1], lane_off[v],
                                                 0x03020000u | ((4u + j) << 8));
                } else {
                    addr = (((w[v >> 1] >> (8 * j)) & 0xffu) << es) + lane_off[v];
                }
                const uint2 e = *(const uint2 *)(lds + addr);
                acc[v * 2 + d] = dot2<BF16>(e.x, xa, acc[v * 2 + d]);
                acc[v * 2 + d] = dot2<BF16>(e.y, xb, acc[v * 2 + d]);
            }
        }
    } else if constexpr (B == 1) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {               // byte v of the single dword
            uint32_t addr;
            if constexpr (PERM) {
                addr = __builtin_amdgcn_perm(w[0], lane_off[v], 0x03020000u | ((4u + v) << 8));
            } else {
                addr = (((w[0] >> (8 * v)) & 0xffu) << es) + lane_off[v];
            }
            const uint4 e = *(const uint4 *)(lds + addr);
            acc[v * 2 + 0] = dot2<BF16>(e.x, xa, acc[v * 2 + 0]);
            acc[v * 2 + 0] = dot2<BF16>(e.y, xb, acc[v * 2 + 0]);
            acc[v * 2 + 1] = dot2<BF16>(e.z, xa, acc[v * 2 + 1]);
            acc[v * 2 + 1] = dot2<BF16>(e.w, xb, acc[v * 2 + 1]);
        }
    } else {                                        // B == 3: 24-bit group per v
        const uint32_t grp[4] = {
            w[0],
            __builtin_amdgcn_alignbit(w[1], w[0], 24),
            __builtin_amdgcn_alignbit(w[2], w[1], 16),
            w[2] >> 8,
        };
#pragma unroll
        for (int v = 0; v < 4; ++v) {
#pragma unroll
            for (int f = 0; f < 4; ++f) {          // field f: d = f >> 1, s2 = f & 1
                const uint32_t code = (grp[v] >> (6 * f)) & 63u;
                const uint32_t e = *(const uint32_t *)(lds + (code << es) + lane_off[v]);
                acc[v * 2 + (f >> 1)] = dot2<BF16>(e, (f & 1) ? xb : xa, acc[v * 2 + (f >> 1)]);
            }
        }
    }
}

template <int B>
__device__ __forceinline__ void load_quarter(uint32_t (&w)[B], const uint8_t *p) {
    if constexpr (B == 4) {
        const uint4 v = *(const uint4 *)p;
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    } else if constexpr (B == 3) {
        const uint32_t *q = (const uint32_t *)p;
        w[0] = q[0]; w[1] = q[1]; w[2] = q[2];
    } else if constexpr (B == 2) {
        const uint2 v = *(const uint2 *)p;
        w[0] = v.x; w[1] = v.y;
    } else {
        w[0] = *(const uint32_t *)p;
    }
}

// Stage the activation slice [k0, k0 + kc) into LDS as 16-bit values of the
// compute type (the LUT's type).  With signs, the rotation of every segment
// that overlaps the slice is computed first in the fp32 scratch (which aliases
// the not-yet-built tables), rounded to the activation type exactly as the
// standalone rotation kernel rounds, and only then converted.
template <bool BF16>
__device__ void stage_x(const GemvParams &p, const GemvSeg &sg, uint8_t *lds, int k0, int kc,
                        int tid) {
    uint16_t *xs = (uint16_t *)(lds + p.lds_x);
    if (sg.signs == nullptr) {
        for (int j = tid; j < kc; j += kGemvThreads) {
            const float f = load_act(p.x, k0 + j, p.act_bf16);
            xs[j] = BF16 ? f2bf(f) : f2h(f);
        }
        return;
    }
    float *buf = (float *)lds;
    if (p.fht_block > 0) {
        // equal blocks: the slice is a whole number of blocks
        for (int j = tid; j < kc; j += kGemvThreads) {
            float f = load_act(p.x, k0 + j, p.act_bf16);
            if (sg.awq) f *= sg.awq[k0 + j];
            buf[fht_slot(j)] = f;
        }
        __syncthreads();
        const int nst = 31 - __builtin_clz((unsigned)p.fht_block);
        fht_lds(buf, kc, nst, tid, kGemvThreads);
        const float inv = inv_sqrt_pow2(nst);
        for (int j = tid; j < kc; j += kGemvThreads) {
            float t = buf[fht_slot(j)] * sg.signs[k0 + j] * inv;
            if (sg.awq) t = t / sg.awq[k0 + j];
            const uint16_t a = round_act(t, p.act_bf16);
            const float back = p.act_bf16 ? bf2f(a) : h2f(a);
            xs[j] = BF16 ? f2bf(back) : f2h(back);
        }
        __syncthreads();
        return;
    }
    // descending power-of-two segments of K (fht.py:118-134 upstream)
    for (int off = 0, rem = p.K; rem > 0;) {
        const int nst = 31 - __builtin_clz((unsigned)rem);
        const int b = 1 << nst;
        const int lo = max(off, k0), hi = min(off + b, k0 + kc);
        if (lo < hi) {                             // uniform across the workgroup
            for (int j = tid; j < b; j += kGemvThreads) {
                float f = load_act(p.x, off + j, p.act_bf16);
                if (sg.awq) f *= sg.awq[off + j];
                buf[fht_slot(j)] = f;
            }
            __syncthreads();
            fht_lds(buf, b, nst, tid, kGemvThreads);
            const float inv = inv_sqrt_pow2(nst);
            for (int k = lo + tid; k < hi; k += kGemvThreads) {
                float t = buf[fht_slot(k - off)] * sg.signs[k] * inv;
                if (sg.awq) t = t / sg.awq[k];
                const uint16_t a = round_act(t, p.act_bf16);
                const float back = p.act_bf16 ? bf2f(a) : h2f(a);
                xs[k - k0] = BF16 ? f2bf(back) : f2h(back);
            }
            __syncthreads();                       // scratch is reused by the next segment
        }
        off += b;
        rem -= b;
    }
}

// Finish one output row: fold the partial-sum slots in ascending order, add the
// residual and the bias.  Everything in fp32.
__device__ __forceinline__ float fold_row(const GemvParams &p, const GemvSeg &sg, int n,
                                          bool from_workspace, float own) {
    float y;
    if (from_workspace) {
        y = 0.0f;
        for (int s = 0; s < sg.nslots; ++s)
            y += __hip_atomic_load(p.P + (size_t)s * p.p_stride + sg.n0 + n, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    } else {
        y = own;
    }
    return y;
}

template <int B, bool BF16>
__device__ void gemv_body(const GemvParams &p, const GemvJob &jb, const GemvSeg &sg,
                          uint8_t *lds) {
    const int tid = threadIdx.x;
    const int u = tid >> 6;                         // quarter of the tile
    const int L = tid & 63;
    const int t = blockIdx.x - jb.tile0;
    const int s = blockIdx.y;
    const int G = p.K >> 6;
    const int g0 = s * p.gs_tiles;
    const int k0 = g0 * 64, kc = p.gs_tiles * 64;

    // ---- issue the first index loads before the prologue: up to kPrefetch tiles
    //      of this lane are in flight at any time -------------------------------
    const uint8_t *qbase = jb.q + ((size_t)t * G + g0) * (1024 * B) + u * (256 * B) + L * (4 * B);
    uint32_t q[kPrefetch][B];
#pragma unroll
    for (int i = 0; i < kPrefetch; ++i) {
#pragma unroll
        for (int j = 0; j < B; ++j) q[i][j] = 0u;
        if (i < p.gs_tiles) load_quarter<B>(q[i], qbase + (size_t)i * (1024 * B));
    }

    // ---- activations (and rotation) into LDS ----------------------------------
    stage_x<BF16>(p, sg, lds, k0, kc, tid);
    __syncthreads();

    // ---- residual partials of this K slice: only stream 1 carries them --------
    const bool direct = (sg.arrivals == 1);
    float *xB = (float *)(lds + p.lds_xb);
    if (sg.R > 0 && jb.slot0 == 0) {
        const uint16_t *xs = (const uint16_t *)(lds + p.lds_x);
        for (int r = u; r < sg.R; r += 4) {
            const uint16_t *brow = sg.resB + (size_t)r * p.K + k0;
            float part = 0.0f;
            for (int k = L; k < kc; k += 64) {
                const float xv = BF16 ? bf2f(xs[k]) : h2f(xs[k]);
                part = fmaf(xv, p.act_bf16 ? bf2f(brow[k]) : h2f(brow[k]), part);
            }
            part = wave_sum(part);
            if (L == 0) {
                if (direct) xB[r] = part;
                else p.P[(size_t)s * p.p_stride + sg.r0 + r] = part;
            }
        }
    }

    // ---- paired tables of the groups this tile touches ------------------------
    constexpr int E = TableShape<B>::kEntries;
    constexpr int EL = TableShape<B>::kEntryLog2;
    const int gs = sg.gs;
    const int ngrp = gs >= 128 ? 1 : 128 / gs;
    const int grp0 = (t * 128) / gs;
    // rows past the last LUT row reuse it (scripts/palettized_modules.py:155-156 upstream)
    const int grp0c = min(grp0, sg.lut_rows - 1);
    build_tables<B>(lds, jb.lut + ((size_t)grp0c << B), min(ngrp, sg.lut_rows - grp0c), jb.es, tid);

    const int es = jb.es;
    const int slot_mask = (1 << (es - EL)) - 1;
    uint32_t lane_off[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int row_local = (u >> 1) * 64 + v * 16;
        int q = gs >= 128 ? 0 : row_local / gs;
        q = min(q, sg.lut_rows - 1 - grp0c);
        lane_off[v] = (uint32_t)(q * (E << es) + ((L & slot_mask) << EL));
    }
    __syncthreads();

    // ---- K loop ---------------------------------------------------------------
    float acc[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) acc[a] = 0.0f;
    const uint32_t *xs32 = (const uint32_t *)(lds + p.lds_x);
    const int xi = (L & 3) * 8 + ((L >> 2) & 3);   // kt*8 + i
    const bool perm = (es == 8);
    for (int gb = 0; gb < p.gs_tiles; gb += kPrefetch) {
#pragma unroll
        for (int i = 0; i < kPrefetch; ++i) {
            const int g = gb + i;
            if (g < p.gs_tiles) {                   // uniform
                uint32_t w[B];
#pragma unroll
                for (int j = 0; j < B; ++j) w[j] = q[i][j];
                if (g + kPrefetch < p.gs_tiles)
                    load_quarter<B>(q[i], qbase + (size_t)(g + kPrefetch) * (1024 * B));
                const uint32_t xa = xs32[g * 32 + xi];
                const uint32_t xb = xs32[g * 32 + xi + 4];
                if (B != 3 && perm)
                    consume_tile<B, BF16, (B != 3)>(w, xa, xb, lds, lane_off, es, acc);
                else
                    consume_tile<B, BF16, false>(w, xa, xb, lds, lane_off, es, acc);
            }
        }
    }

    // ---- fold the 16 lanes that share a row -----------------------------------
#pragma unroll
    for (int a = 0; a < 8; ++a) acc[a] = row16_sum(acc[a]);
    float *red = (float *)(lds + p.lds_red);        // [128] row sums of this workgroup
    if ((L & 15) == 0) {
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            const int row = (u >> 1) * 64 + (a >> 1) * 16 + (a & 1) * 8 + 4 * (u & 1) + (L >> 4);
            red[row] = acc[a];
        }
    }
    __syncthreads();

    // ---- publish, take a ticket, let the last arrival finish the tile ---------
    int *flag = (int *)(lds + p.lds_xb + kGemvMaxRank * 4);
    if (!direct) {
        if (tid < 128)
            p.P[(size_t)(jb.slot0 + s) * p.p_stride + sg.n0 + t * 128 + tid] = red[tid];
        __threadfence();
        __syncthreads();
        if (tid == 0) {
            const int old = atomicAdd(p.tickets + sg.ticket0 + t, 1);
            *flag = (old == sg.arrivals - 1);
        }
        __syncthreads();
        if (!*flag) return;
        __threadfence();
    }

    // residual coefficients x . resB[r], folded over the splits in fixed order
    const int nseg_out = p.silu_mul ? 2 : 1;
    float yv[2] = {0.0f, 0.0f};
#pragma unroll
    for (int so = 0; so < 2; ++so) {
        if (so >= nseg_out) break;                 // uniform
        const GemvSeg &og = p.silu_mul ? (so == 0 ? p.seg[0] : p.seg[1]) : sg;
        if (og.R > 0 && !direct) {
            __syncthreads();
            for (int r = tid; r < og.R; r += kGemvThreads) {
                float c = 0.0f;
                for (int sp = 0; sp < p.split; ++sp)
                    c += __hip_atomic_load(p.P + (size_t)sp * p.p_stride + og.r0 + r,
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                xB[r] = c;
            }
            __syncthreads();
        }
        if (tid < 128) {
            const int n = t * 128 + tid;
            float y = fold_row(p, og, n, !direct, red[tid]);
            if (og.R > 0) {
                const uint16_t *ra = og.resA + (size_t)n * og.R;
                for (int r = 0; r < og.R; ++r)
                    y = fmaf(xB[r], p.act_bf16 ? bf2f(ra[r]) : h2f(ra[r]), y);
            }
            if (og.bias) y += p.act_bf16 ? bf2f(og.bias[n]) : h2f(og.bias[n]);
            yv[so] = y;
        }
    }
    if (tid < 128) {
        const int n = t * 128 + tid;
        float y = yv[0];
        uint16_t *out = sg.out;
        if (p.silu_mul) {
            y = (yv[0] / (1.0f + expf(-yv[0]))) * yv[1];
            out = p.seg[0].out;
        }
        out[n] = round_act(y, p.act_bf16);
    }
    if (!direct && tid == 0) {
        __hip_atomic_store(p.tickets + sg.ticket0 + t, 0, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <bool BF16>
__global__ void __launch_bounds__(kGemvThreads) gemv_kernel(const GemvParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    // Pick this workgroup's job and weight with static indices only, so that the
    // kernel arguments stay in scalar registers.
    GemvJob jb = p.job[0];
#pragma unroll
    for (int j = 1; j < kGemvMaxJobs; ++j)
        if (j < p.njobs && (int)blockIdx.x >= p.job[j].tile0) jb = p.job[j];
    GemvSeg sg = p.seg[0];
#pragma unroll
    for (int i = 1; i < kGemvMaxSegs; ++i)
        if (jb.seg == i) sg = p.seg[i];
    switch (jb.bits) {
        case 4: gemv_body<4, BF16>(p, jb, sg, lds); break;
        case 3: gemv_body<3, BF16>(p, jb, sg, lds); break;
        case 2: gemv_body<2, BF16>(p, jb, sg, lds); break;
        default: gemv_body<1, BF16>(p, jb, sg, lds); break;
    }
}

}  // namespace flute
