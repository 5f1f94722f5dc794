// Launchers of the M = 1 LUT GEMV family: single weight, merged gate/up with
// SiLU*mul, several weights sharing one input, and the two-launch MLP block.
#include "gemv_kernel.h"
#include "gemv4_kernel.h"
#include "host_common.h"

#include <atomic>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace flute {

namespace {

// Residual coefficients: xb[r] = sum_k x[k] * resB[r][k] in fp32, one workgroup
// per residual row, x taken as given (already rotated).  A thread-strided sum
// followed by a fixed-order tree: deterministic.
__global__ void __launch_bounds__(256) residual_coeff_kernel(const uint16_t *x,
                                                             const uint16_t *resB, float *xb,
                                                             int K, int act_bf16) {
    __shared__ float part[256];
    const uint16_t *row = resB + (size_t)blockIdx.x * K;
    float s = 0.0f;
    for (int k = threadIdx.x; k < K; k += 256) {
        const float a = act_bf16 ? bf2f(x[k]) : h2f(x[k]);
        const float b = act_bf16 ? bf2f(row[k]) : h2f(row[k]);
        s = fmaf(a, b, s);
    }
    part[threadIdx.x] = s;
    __syncthreads();
    for (int step = 128; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) part[threadIdx.x] += part[threadIdx.x + step];
        __syncthreads();
    }
    if (threadIdx.x == 0) xb[blockIdx.x] = part[0];
}

int entries_log2(int bits) { return bits == 3 ? 6 : 8; }
int entry_bytes_log2(int bits) { return bits >= 3 ? 2 : (bits == 2 ? 3 : 4); }

struct Plan {
    GemvParams p;
    int pair;               // 10 * b1 + b2 when the widths are a pair the lean kernel serves with two tables, else 0
    bool k_group;           // the LUT is grouped along K (single weight, lean kernel only)
    size_t lds_bytes;
    int grid_x;
    int threads;
    int total_tickets;
    size_t p_floats;        // partial sums
    size_t xb_floats;       // residual coefficients
    size_t xrot_halves;     // pre-rotated inputs of weights that carry a residual
    bool lut_bf16;
    // pre-kernels: residual coefficients (and the rotation they need)
    struct Pre {
        const uint16_t *resB;
        const float *signs, *awq;
        int R, seg;
        int share;              // index of an earlier entry with the same rotation, or -1
        size_t xb_off, xrot_off;
    } pre[kGemvMaxSegs];
    int npre;
    int rot_block;
};

// Shape of the launch for `rows` output rows over G tiles of K.  A workgroup
// owns `rw` rows.  The library's own policy splits K only where a workgroup's K range
// would be very long over few rows: the exchange between workgroups (partial sums
// written through, a ticket, the last arrival reading them back) is three memory round
// trips, and up to K = 24576 the unsplit launch measured faster for every narrow shape
// (N = 128...3072; e.g. N = 1024, K = 4096: 4.5 us against 5.9 / 10.4 / 11.4 us split
// 2 / 4 / 8 ways; N = 512, K = 24576: 7.7 against 8.2 / 11.5).  From K = 32768 on, four
// ways win up to 512 rows and two ways up to 1024 (K = 32768: N = 128 6.8 against
// 8.7 us, N = 512 7.5 against 9.0, N = 1024 8.3 against 9.2; K = 65536: N = 512 8.8
// against 19.0, N = 1024 12.8 against 20.9); 2048 rows and more stay unsplit (11.0
// against 14.3 us).  A caller's explicit split is honoured.
void choose_shape(int rows, int G, int split_req, int *rw, int *split, int *waves,
                  bool may_split = true) {
    int best_rw = tuning().gemv_rw;
    if (best_rw != 8 && best_rw != 16 && best_rw != 32) {
        // The narrowest slices whose grid is still resident at once (three four-wavefront
        // workgroups per CU): a second round of workgroups costs far more than wider
        // slices do (8192 rows at K = 4096: 512 sixteen-row workgroups 7.3 us, 1024
        // eight-row ones 13.2 us; 16384 rows: 11.3 us with 32 rows against 15.3 with 16).
        best_rw = 32;
        for (int cand : {8, 16}) {
            if (rows / cand <= 3 * kNumCU) { best_rw = cand; break; }
        }
        // A grid of exactly one or two 16-row workgroups per CU, unsplit, measured best
        // where K is long enough to give each of them eight wavefronts (4096 rows at
        // K = 12288: 256 workgroups, 8.5 us against 9.2 us for 512 eight-row ones and
        // 9.5 us for 768 with a three-way K split).
        if (rows % (16 * kNumCU) == 0 && rows / (16 * kNumCU) <= 2 && G / 2 >= 64) {
            best_rw = 16;
        }
    }
    int sp = split_req;
    if (sp > 0) {
        // a wavefront load spans 32/rw tiles of K: widen the slices until the K
        // range of one split is a whole number of loads
        while (G % sp == 0 && (G / sp) % (32 / best_rw) != 0 && best_rw < 32) best_rw *= 2;
    } else {
        sp = 1;
        // (not with a rotation fused into the prologue: its blocks would have to fit the slices)
        if (may_split && G >= 512 && rows <= 512 && G % 4 == 0) sp = 4;
        else if (may_split && G >= 512 && rows <= 1024 && G % 2 == 0) sp = 2;
        while ((G / sp) % (32 / best_rw) != 0 && best_rw < 32) best_rw *= 2;
    }
    *rw = best_rw;
    *split = sp;
    int wv = tuning().gemv_waves;
    if (wv != 1 && wv != 2 && wv != 4 && wv != 8) {
        // Eight wavefronts when each still has two loads or more and the grid is at most
        // one workgroup per CU, or two per CU of eight-row workgroups with a long K range
        // (measured: 384 eight-row workgroups at K >= 8192 gain 2-10 % from eight, 512
        // sixteen- or 32-row ones lose 3-8 %).  Otherwise four, fewer for very short K.
        const int units = (G / sp) / (32 / best_rw);
        const long wgs = (long)(rows / best_rw) * sp;
        const bool eight = units >= 16 && (wgs <= kNumCU || (wgs <= 2 * kNumCU && units >= 32 &&
                                                             best_rw == 8));
        wv = eight ? 8 : (units >= 4 ? 4 : (units >= 2 ? 2 : 1));
    }
    *waves = wv;
}

// Fill a launch plan for `count` weights that share x.  silu_mul couples
// weights 0 and 1 into one output.
flute_status make_plan(const flute_linear *segs, int count, const void *x, void *const *outs,
                       int act_dtype, int split, int silu_mul, const char *who, Plan *plan) {
    FLUTE_REQUIRE(count >= 1 && count <= kGemvMaxSegs, FLUTE_ERR_INVALID,
                  "%s: 1..%d weights per launch (got %d)", who, kGemvMaxSegs, count);
    FLUTE_REQUIRE(x != nullptr, FLUTE_ERR_INVALID, "%s: x is NULL", who);
    FLUTE_REQUIRE(((uintptr_t)x & 15) == 0, FLUTE_ERR_INVALID,
                  "%s: x must be 16-byte aligned (the kernels read it 16 bytes at a time)", who);
    FLUTE_REQUIRE(act_dtype == FLUTE_F16 || act_dtype == FLUTE_BF16, FLUTE_ERR_INVALID,
                  "%s: activations must be float16 or bfloat16", who);
    for (int i = 0; i < count; ++i) {
        flute_status st = validate_linear(&segs[i], count == 1 && !silu_mul ? kModeKGroupOk : 0, who);
        if (st != FLUTE_OK) return st;
        FLUTE_REQUIRE(outs[i] != nullptr, FLUTE_ERR_INVALID, "%s: output %d is NULL", who, i);
        FLUTE_REQUIRE(((uintptr_t)outs[i] & 1) == 0, FLUTE_ERR_INVALID,
                      "%s: output %d must be 2-byte aligned", who, i);
        FLUTE_REQUIRE(segs[i].K == segs[0].K, FLUTE_ERR_INVALID,
                      "%s: all weights of one launch must share K (%d vs %d)", who, segs[i].K,
                      segs[0].K);
        FLUTE_REQUIRE(segs[i].lut_dtype == segs[0].lut_dtype, FLUTE_ERR_UNSUPPORTED,
                      "%s: all weights of one launch must share the LUT dtype", who);
        FLUTE_REQUIRE(segs[i].rot_block == segs[0].rot_block, FLUTE_ERR_UNSUPPORTED,
                      "%s: all weights of one launch must share the rotation block", who);
    }
    const bool lut_bf16 = segs[0].lut_dtype == FLUTE_BF16;
    FLUTE_REQUIRE(!(lut_bf16 && act_dtype == FLUTE_F16), FLUTE_ERR_UNSUPPORTED,
                  "%s: a bfloat16 LUT with float16 activations is not served (the pair product "
                  "runs in the LUT's type and float16 does not convert to bfloat16 exactly)",
                  who);
    if (silu_mul) {
        FLUTE_REQUIRE(count == 2 && segs[0].N == segs[1].N, FLUTE_ERR_INVALID,
                      "%s: gate and up must agree in N (%d vs %d)", who, segs[0].N,
                      count == 2 ? segs[1].N : -1);
    }
    const int K = segs[0].K;
    const int G = K / 64;
    FLUTE_REQUIRE(split <= 0 || G % split == 0, FLUTE_ERR_INVALID,
                  "%s: split %d must divide K/64 = %d", who, split, G);

    const int split_in = split;
    GemvParams &p = plan->p;
    std::memset(&p, 0, sizeof(p));
    int rows = 0;
    for (int i = 0; i < (silu_mul ? 1 : count); ++i) rows += segs[i].N;
    int rw, waves;
    bool rotated = false;
    for (int i = 0; i < count; ++i) rotated |= segs[i].signs != nullptr;
    // (the library's own K split was measured on single weights only: merged gate/up launches
    // split when the caller asks for it)
    choose_shape(rows, G, split, &rw, &split, &waves, !rotated && !silu_mul);
    const bool k_group = segs[0].k_group != 0;
    if (k_group) {
        // Only the lean kernel serves this form: four or eight wavefronts, each with an even
        // number (two at least) of loads of 32 / rw tiles.  The workgroup stages its LUT rows in
        // LDS, 64 bytes per (row, K group), at most kKGroupPieces 16-byte pieces per thread, whole
        // K groups per split.  The shape chosen above is kept where it fits; else wider slices or
        // another wavefront count; else, where the library chooses the split, a larger one.
        auto ok = [&](int sp, int rw_, int wv) {
            if (G % sp || (G / sp) % 2 || (G / sp) % (32 / rw_)) return false;
            const int units = (G / sp) / (32 / rw_);
            if (!(wv == 4 || (wv == 8 && rw_ <= 16)) || units % wv) return false;
            const int u = units / wv;
            return u >= 2 && u % 2 == 0 &&
                   (long)rw_ * (G / sp / 2) * 2 <= (long)kKGroupPieces * wv * 64;
        };
        auto settle = [&](int sp) {
            if (ok(sp, rw, waves)) return true;
            for (int r = rw; r <= 32; r *= 2)
                for (int wv : {4, 8})
                    if (ok(sp, r, wv)) {
                        rw = r;
                        waves = wv;
                        return true;
                    }
            return false;
        };
        bool done = settle(split);
        for (int sp = split * 2; !done && split_in <= 0 && sp <= G / 2 && G % sp == 0; sp *= 2) {
            choose_shape(rows, G, sp, &rw, &split, &waves, false);
            done = settle(split);
        }
        FLUTE_REQUIRE(done, FLUTE_ERR_UNSUPPORTED,
                      "%s: K=%d at split %d does not divide into the loads of the kernel that serves "
                      "a LUT grouped along K (K/split must be a multiple of 512 whose LUT rows fit a "
                      "workgroup's staging); try another split", who, K, split);
    }
    FLUTE_REQUIRE((G / split) % (32 / rw) == 0, FLUTE_ERR_UNSUPPORTED,
                  "%s: K/64/split = %d is not a whole number of wavefront loads", who, G / split);
    const int gs_tiles = G / split;
    const int kc = gs_tiles * 64;
    const int spt = 128 / rw;

    bool any_fused_rot = false;
    const int fht_block = segs[0].rot_block;
    plan->npre = 0;
    plan->rot_block = fht_block;
    size_t xb_off = 0, xrot_off = 0;
    int n0 = 0, col = 0, ticket = 0;
    size_t tab_bytes = 0;
    // LDS: tables/scratch | x slice | row sums.  The table stride is the largest
    // that still lets the whole grid be resident at once (one round of
    // workgroups), since a second round repeats the start-up latency.
    int budget = tuning().gemv_table_log2;
    if (budget < 12 || budget > 17) {
        long wgs = 0;
        for (int i = 0; i < (silu_mul ? 1 : count); ++i) wgs += (long)(segs[i].N / rw) * split;
        long per_cu = (wgs + kNumCU - 1) / kNumCU;
        // The lean all-4-bit kernel needs the full 32 KB table and is built for three
        // workgroups per CU; grids of many rounds gain more from it than from a fourth
        // resident workgroup with a half-size table in the general kernel (4096 -> 248320:
        // 104 us against 127 us).
        bool lean = true;
        for (int i = 0; i < count; ++i)
            lean &= segs[i].b1 == 4 && (segs[i].b2 == 0 || segs[i].b2 == 4) && segs[i].group_size >= 128;
        if (per_cu > (lean ? 3 : 4)) per_cu = lean ? 3 : 4;
        if (per_cu < 1) per_cu = 1;
        const long fixed = kc * 2 + 4096;
        budget = 14;
        for (int cand = 15; cand >= 14; --cand)
            if (((1L << cand) + fixed) * per_cu <= kLdsPerCU) { budget = cand; break; }
    }
    for (int i = 0; i < count; ++i) {
        const flute_linear &w = segs[i];
        GemvSeg &sg = p.seg[i];
        sg.resA = (const uint16_t *)w.resA;
        sg.bias = (const uint16_t *)w.bias;
        sg.out = (uint16_t *)outs[i];
        sg.N = w.N;
        sg.R = w.R;
        sg.gs = k_group ? 128 : w.group_size;       // (a LUT grouped along K: group_size is not read)
        sg.lut_rows = w.lut_rows;
        sg.nstreams = w.b2 > 0 ? 2 : 1;
        sg.n0 = n0;
        sg.col0 = (silu_mul && i == 1) ? 0 : col;
        sg.ticket0 = (silu_mul && i == 1) ? 0 : ticket;
        n0 += w.N;
        if (!(silu_mul && i == 1)) {
            col += (w.N / 128) * spt;
            ticket += (w.N / 128) * spt;
        }
        // Rotating inside the GEMV makes every workgroup transform the whole row itself
        // (about 5 us of VALU work per CU at K = 4096); a separate rotation launch in
        // front measured slower still (a dependent launch costs more than that), so it
        // stays an opt-in.
        const bool prerotate = w.signs != nullptr && w.R == 0 &&
                               tuning().gemv_prerotate != 0;
        if (w.R > 0 || prerotate) {
            // the residual needs x . resB[r] before any row can finish: computed by a
            // small kernel in front, on the rotated input when the weight is rotated
            Plan::Pre &pre = plan->pre[plan->npre++];
            pre.resB = (const uint16_t *)w.resB;
            pre.signs = w.signs;
            pre.awq = w.awq;
            pre.R = w.R;
            pre.seg = i;
            pre.xb_off = xb_off;
            pre.share = -1;
            for (int j = 0; j + 1 < plan->npre && w.signs; ++j)
                if (plan->pre[j].signs == w.signs && plan->pre[j].awq == w.awq) pre.share = j;
            pre.xrot_off = pre.share >= 0 ? plan->pre[pre.share].xrot_off : xrot_off;
            xb_off += (size_t)((w.R + 3) & ~3);
            if (w.signs && pre.share < 0) xrot_off += (size_t)K;
            sg.signs = nullptr;                     // the kernel reads the pre-rotated row
            sg.awq = nullptr;
        } else {
            sg.signs = w.signs;
            sg.awq = w.awq;
            any_fused_rot |= w.signs != nullptr;
        }
        const int ngrp_log2 = k_group || w.group_size >= 128 ? 0 : ilog2(128 / w.group_size);
        for (int st = 0; st < sg.nstreams; ++st) {
            GemvStream &gs = sg.st[st];
            gs.q = (const uint8_t *)(st ? w.q2 : w.q1);
            gs.lut = (const uint16_t *)(st ? w.lut2 : w.lut1);
            gs.bits = st ? w.b2 : w.b1;
            int es = budget - entries_log2(gs.bits) - ngrp_log2;
            if (es > 7) es = 7;             // 32 replicas cover the 32 LDS banks
            if (es < entry_bytes_log2(gs.bits)) es = entry_bytes_log2(gs.bits);
            if (k_group) es = 7;            // (no table: the lean kernel's LUT rows, sized below)
            gs.es = es;
            const size_t tb = k_group ? (size_t)(kc / 128) * (rw * 64 + (rw / 8) * 64)
                                      : ((size_t)1 << (entries_log2(gs.bits) + es)) << ngrp_log2;
            if (tb > tab_bytes) tab_bytes = tb;
        }
    }
    size_t scratch = 0;
    if (fht_block > 0) {
        bool any_rot = false;
        for (int i = 0; i < count; ++i) any_rot |= segs[i].signs != nullptr;
        FLUTE_REQUIRE(any_rot, FLUTE_ERR_INVALID, "%s: a rotation block needs rotation signs", who);
        FLUTE_REQUIRE(is_pow2(fht_block) && fht_block >= 32 && fht_block <= 16384 &&
                          K % fht_block == 0,
                      FLUTE_ERR_INVALID,
                      "%s: rotation block must be a power of two in [32, 16384] dividing K", who);
        FLUTE_REQUIRE(kc % fht_block == 0, FLUTE_ERR_UNSUPPORTED,
                      "%s: K slice %d of split %d is not a whole number of %d-column rotation "
                      "blocks",
                      who, kc, split, fht_block);
        if (any_fused_rot) scratch = (size_t)kc * 4;
    } else if (any_fused_rot) {
        scratch = (size_t)make_segments(K, 0).len[0] * 4;
    }
    p.fht_block = fht_block;
    p.nsegs = count;
    p.K = K;
    p.split = split;
    p.gs_tiles = gs_tiles;
    p.lpg_log2 = ilog2(2 * rw);
    p.p_stride = (n0 + 31) & ~31;
    p.silu_mul = silu_mul;
    p.act_bf16 = act_dtype == FLUTE_BF16;
    p.x = (const uint16_t *)x;

    // Mixed widths (and 3 + 3 bits) in the lean kernel: both tables of a weight stand side by
    // side (4^b entries of 128 bytes each).  Decided here because it sets the table region;
    // the launcher may still send the launch to the general kernel, which needs less.
    plan->pair = 0;
    plan->k_group = k_group;
    if (!k_group) {
        int b1 = segs[0].b1, b2 = 0;
        bool ok = true;
        for (int i = 0; i < count; ++i) {
            ok &= segs[i].b1 == b1 && segs[i].group_size >= 128;
            if (segs[i].b2 > 0) {
                if (b2 == 0) b2 = segs[i].b2;
                ok &= segs[i].b2 == b2;
            }
        }
        int code = 10 * b1 + b2;
        // a single narrow stream ((3, 0) is one of upstream's pairs): the two-table instantiation
        // of its width with the second table unused
        if (b2 == 0 && b1 < 4) {
            b2 = b1 == 3 ? 3 : (b1 == 2 ? 3 : 4);
            code = 10 * b1 + b2;
        }
        if (ok && (code == 41 || code == 14 || code == 33 || code == 24 || code == 23)) {
            plan->pair = code;
            // (4^b entries of 128 bytes; a 1-bit stream's nibble table: 16 entries of 256 bytes)
            auto tab = [](int b) { return b == 1 ? (size_t)16 * 256 : ((size_t)1 << (2 * b)) * 128; };
            const size_t both = tab(b1) + tab(b2);
            if (both > tab_bytes) tab_bytes = both;
            // (4, 1) where every weight has both streams: the kernel walks the 1-bit stream first
            // (the sum of the two streams does not depend on their order beyond fp32 rounding, and
            // the order is fixed, so results stay deterministic).  With the narrow stream in front
            // all of its loads go out in the prologue: 4096 -> 12288 measured 9.7 us against 11.1 us.
            bool all_two = true;
            for (int i = 0; i < count; ++i) all_two &= segs[i].b2 > 0;
            if (code == 41 && all_two) {
                for (int i = 0; i < count; ++i) std::swap(p.seg[i].st[0], p.seg[i].st[1]);
                plan->pair = 14;
            }
        }
    }
    size_t region0 = tab_bytes > scratch ? tab_bytes : scratch;
    region0 = (region0 + 255) & ~(size_t)255;
    p.lds_x = (int)region0;
    p.lds_red = p.lds_x + ((kc * 2 + 15) & ~15);
    // row sums [2][8][32], the ticket flag (16 bytes), then one word per wavefront for the
    // row maximum of a bfloat16 slice (not the row-sum area: a merged launch restages for its
    // second output while the first output's sums are still waiting to be folded)
    plan->lds_bytes = (size_t)p.lds_red + kGemvRedBytes + 16 + 8 * 4;
    FLUTE_REQUIRE(plan->lds_bytes <= (size_t)kLdsPerCU, FLUTE_ERR_UNSUPPORTED,
                  "%s: K=%d at split %d needs %zu B of LDS (limit %d)", who, K, split,
                  plan->lds_bytes, kLdsPerCU);
    plan->grid_x = col;
    plan->threads = waves * 64;
    plan->total_tickets = ticket;
    plan->p_floats = split > 1 ? (size_t)split * p.p_stride : 0;
    plan->xb_floats = xb_off;
    plan->xrot_halves = xrot_off;
    plan->lut_bf16 = lut_bf16;
    return FLUTE_OK;
}

template <bool BF16, int BFIX>
flute_status launch_typed(Plan &plan, hipStream_t stream) {
    static std::atomic<bool> attr_done{false};   // threads may race to the first call: the call is idempotent
    if (!attr_done) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)gemv_kernel<BF16, BFIX>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)kLdsPerCU));
        attr_done = true;
    }
    dim3 grid(plan.grid_x, plan.p.split);
    hipLaunchKernelGGL((gemv_kernel<BF16, BFIX>), grid, dim3(plan.threads), plan.lds_bytes, stream,
                       plan.p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}

template <int LPGL, int NW, int PF, bool BF16, bool WALK>
flute_status launch_fast4_grid(const Plan &plan, int gx, hipStream_t stream) {
    static std::atomic<bool> attr_done{false};   // threads may race to the first call: the call is idempotent
    if (!attr_done) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)gemv4_kernel<LPGL, NW, PF, BF16, WALK>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)kLdsPerCU));
        attr_done = true;
    }
    dim3 grid(gx, plan.p.split);
    hipLaunchKernelGGL((gemv4_kernel<LPGL, NW, PF, BF16, WALK>), grid, dim3(NW * 64), plan.lds_bytes,
                       stream, plan.p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}

template <int LPGL, int NW, int PF, bool BF16>
flute_status launch_fast4(Plan &plan, hipStream_t stream) {
    // A grid of several rounds of workgroups: as many workgroups as are resident at once walk
    // over the row slices instead, which stages the activations once per workgroup and lets a
    // slice's first loads travel under the previous slice's last products.
    int gx = plan.grid_x;
    plan.p.slices = 0;
    if constexpr (NW == 4) {                     // (eight-wavefront workgroups serve short grids only)
        // three workgroups per CU is what the kernel's registers allow (3 wavefronts per SIMD)
        const int per_cu = tuning().gemv4_walk >= 0 ? (tuning().gemv4_walk < 3 ? tuning().gemv4_walk : 3) : 3;
        const int resident = per_cu * kNumCU;
        if (per_cu > 0 && plan.p.split == 1 && (plan.p.nsegs == 1 || plan.p.silu_mul) &&
            plan.lds_bytes * per_cu <= (size_t)kLdsPerCU && gx > resident) {
            plan.p.slices = gx;
            plan.p.xcd_runs = tuning().gemv_xcd && resident % 8 == 0;
            return launch_fast4_grid<LPGL, NW, PF, BF16, true>(plan, resident, stream);
        }
    }
    return launch_fast4_grid<LPGL, NW, PF, BF16, false>(plan, gx, stream);
}

// Loads a lane keeps in flight in the lean kernel: 4 when that divides the loads of a
// wavefront, else 2; 0 when the launch does not fit the kernel (the wavefronts would get
// different or odd numbers of loads: two loads feed one matrix product).
int pick_prefetch(const Plan &plan, int nw) {
    const int gpi = 64 >> plan.p.lpg_log2;
    if (plan.p.gs_tiles % gpi) return 0;
    const int units = plan.p.gs_tiles / gpi;
    if (units % nw) return 0;
    const int u = units / nw;
    if (u < 2 || (u & 1)) return 0;
    const int pf = tuning().gemv4_pf;
    if ((pf == 2 || pf == 4) && u % pf == 0) return pf;
    return u % 4 == 0 ? 4 : 2;
}

template <int LPGL, int NW, bool BF16>
flute_status launch_fast4_pf(Plan &plan, hipStream_t stream) {
    switch (pick_prefetch(plan, NW)) {
        case 2: return launch_fast4<LPGL, NW, 2, BF16>(plan, stream);
        default: return launch_fast4<LPGL, NW, 4, BF16>(plan, stream);
    }
}

template <int LPGL, bool BF16>
flute_status launch_fast4_shape(Plan &plan, int nw, hipStream_t stream) {
    return nw == 4 ? launch_fast4_pf<LPGL, 4, BF16>(plan, stream)
                   : launch_fast4_pf<LPGL, 8, BF16>(plan, stream);
}

template <bool BF16>
flute_status launch_width(Plan &plan, hipStream_t stream) {
    // one width for the whole launch -> the instantiation specialised for it
    int bits = plan.p.seg[0].st[0].bits;
    int es = plan.p.seg[0].st[0].es;
    bool one_group = true;
    for (int i = 0; i < plan.p.nsegs; ++i) {
        one_group &= plan.p.seg[i].gs >= 128;
        for (int st = 0; st < plan.p.seg[i].nstreams; ++st) {
            if (plan.p.seg[i].st[st].bits != bits) bits = 0;
            if (plan.p.seg[i].st[st].es != es) es = 0;
        }
    }
    const int nw = plan.threads / 64;
    // (a contiguous run of row slices per XCD: every weight's slices must come in eights)
    plan.p.xcd_runs = tuning().gemv_xcd != 0;
    for (int i = 0; i < plan.p.nsegs; ++i)
        if (((plan.p.seg[i].N >> 7) * (256 >> plan.p.lpg_log2)) % 8 != 0) plan.p.xcd_runs = 0;
    // the lean kernel stages the activations once: gate and up must share input and rotation
    const bool one_input = !plan.p.silu_mul ||
                           (plan.p.seg[0].xsrc == plan.p.seg[1].xsrc &&
                            plan.p.seg[0].signs == plan.p.seg[1].signs &&
                            plan.p.seg[0].awq == plan.p.seg[1].awq);
    // the lean kernel reads LUT rows through the scalar cache: dword-aligned LUTs only
    bool luts_aligned = true;
    for (int i = 0; i < plan.p.nsegs; ++i)
        for (int st = 0; st < plan.p.seg[i].nstreams; ++st)
            luts_aligned &= ((uintptr_t)plan.p.seg[i].st[st].lut & 3) == 0;
    if (plan.k_group) {
        // only the lean kernel knows this form: no general-kernel route
        const int pf = pick_prefetch(plan, nw);
        FLUTE_REQUIRE(pf != 0 && (nw == 4 || (nw == 8 && plan.p.lpg_log2 <= 5)), FLUTE_ERR_UNSUPPORTED,
                      "flute_gemv: K=%d at split %d with %d-row workgroups of %d wavefronts does not "
                      "divide into the loads of the kernel that serves a LUT grouped along K; try "
                      "another split", plan.p.K, plan.p.split, 1 << (plan.p.lpg_log2 - 1), nw);
        plan.p.slices = 0;
        return launch_gemv_kgroup(plan.p, plan.grid_x, nw, pf, plan.lds_bytes, BF16, stream);
    }
    if (bits == 4 && one_group && one_input && es == 7 && (nw == 4 || nw == 8) && luts_aligned &&
        pick_prefetch(plan, nw) != 0 && tuning().gemv_no_fast == 0) {
        switch (plan.p.lpg_log2) {
            case 4: return launch_fast4_shape<4, BF16>(plan, nw, stream);
            case 5: return launch_fast4_shape<5, BF16>(plan, nw, stream);
            default: return launch_fast4_shape<6, BF16>(plan, nw, stream);
        }
    }
    if (plan.pair && one_group && one_input && es == 7 && luts_aligned &&
        (nw == 4 || (nw == 8 && plan.p.lpg_log2 <= 5)) && pick_prefetch(plan, nw) != 0 &&
        tuning().gemv_no_fast == 0) {
        int pf = pick_prefetch(plan, nw);
        // a 1-bit stream with loads that come in eights: the deep ring (launch_pair's pf 8)
        const int u = (plan.p.gs_tiles / (64 >> plan.p.lpg_log2)) / nw;
        if (pf == 4 && plan.pair == 14 && u % 8 == 0 && tuning().gemv4_pf == 0) pf = 8;
        plan.p.slices = 0;
        return (plan.pair == 41 || plan.pair == 14)
                   ? launch_gemv_pair_1bit(plan.p, plan.pair, plan.grid_x, nw, pf, plan.lds_bytes, BF16, stream)
                   : launch_gemv_pair_wide(plan.p, plan.pair, plan.grid_x, nw, pf, plan.lds_bytes, BF16, stream);
    }
    switch (bits) {
        case 4: return launch_typed<BF16, 4>(plan, stream);
        case 3: return launch_typed<BF16, 3>(plan, stream);
        case 2: return launch_typed<BF16, 2>(plan, stream);
        case 1: return launch_typed<BF16, 1>(plan, stream);
        default: break;
    }
    // mixed widths: the pairs deployed artifacts hold ((1,4) x45, (4,1) x24, (2,3) x3, (2,4) x6
    // in upstream's census, flute_extended/__init__.py:226-233) have instantiations of their own
    int b1 = plan.p.seg[0].st[0].bits, b2 = 0;
    bool pair = true;
    for (int i = 0; i < plan.p.nsegs; ++i) {
        pair &= plan.p.seg[i].st[0].bits == b1;
        if (plan.p.seg[i].nstreams == 2) {
            if (b2 == 0) b2 = plan.p.seg[i].st[1].bits;
            pair &= plan.p.seg[i].st[1].bits == b2;
        }
    }
    if (pair) {
        switch (10 * b1 + b2) {
            case 14: return launch_typed<BF16, 14>(plan, stream);
            case 41: return launch_typed<BF16, 41>(plan, stream);
            case 23: return launch_typed<BF16, 23>(plan, stream);
            case 24: return launch_typed<BF16, 24>(plan, stream);
            default: break;
        }
    }
    return launch_typed<BF16, 0>(plan, stream);
}

// Scratch memory a launch needs beyond its operands: partial sums of a K split, tickets,
// residual coefficients, pre-rotated inputs.
struct ScratchNeed {
    size_t floats, ints;
};
ScratchNeed scratch_need(const Plan &plan) {
    if (!(plan.p_floats || plan.npre)) return {0, 0};
    const size_t xb_pad = (plan.xb_floats + 3) & ~(size_t)3;
    return {plan.p_floats + xb_pad + (plan.xrot_halves + 1) / 2 + 64, (size_t)plan.total_tickets + 1};
}

// fixed_base/fixed_tickets: caller-provided scratch (the allocation-free entry point);
// null = the library's per-device workspace, grown on demand.
flute_status launch(Plan &plan, int act_dtype, hipStream_t stream, float *fixed_base = nullptr,
                    int *fixed_tickets = nullptr) {
    if (plan.p_floats || plan.npre) {
        const size_t xb_pad = (plan.xb_floats + 3) & ~(size_t)3;
        const ScratchNeed need = scratch_need(plan);
        float *base = fixed_base;
        int *tickets = fixed_tickets;
        flute_status st = FLUTE_OK;
        if (!base) st = get_workspace(need.floats, need.ints, stream, &base, &tickets);
        if (st != FLUTE_OK) return st;
        plan.p.P = base;
        plan.p.tickets = tickets;
        float *xb_base = base + plan.p_floats;
        uint16_t *xrot_base = (uint16_t *)(xb_base + xb_pad);
        for (int i = 0; i < plan.npre; ++i) {
            const Plan::Pre &pre = plan.pre[i];
            const uint16_t *xin = plan.p.x;
            if (pre.signs) {
                uint16_t *xr = xrot_base + pre.xrot_off;
                if (pre.share < 0) {
                    st = flute_fht(plan.p.x, pre.signs, pre.awq, xr, 1, plan.p.K, act_dtype, 0,
                                   plan.rot_block, stream);
                    if (st != FLUTE_OK) return st;
                }
                xin = xr;
                plan.p.seg[pre.seg].xsrc = xr;
            }
            if (pre.R > 0) {
                float *xb = xb_base + pre.xb_off;
                hipLaunchKernelGGL(residual_coeff_kernel, dim3(pre.R), dim3(256), 0, stream, xin,
                                   pre.resB, xb, plan.p.K, plan.p.act_bf16);
                FLUTE_HIP_CHECK(hipGetLastError());
                plan.p.seg[pre.seg].xb = xb;
            }
        }
    }
    const flute_status st = plan.lut_bf16 ? launch_width<true>(plan, stream) : launch_width<false>(plan, stream);
    if ((plan.p_floats || plan.npre) && !fixed_base) workspace_done(stream);
    return st;
}

// ---- the allocation-free variant's scratch ------------------------------------------
// One fixed array per device, part of the code object: held from the time the library is
// loaded on a device until the process ends.  Layout: [tickets: kNoAllocTickets ints]
// [partial sums, residual coefficients, pre-rotated input: the rest as floats].
constexpr size_t kNoAllocBytes = (size_t)2 << 20;
constexpr size_t kNoAllocTickets = 4096;
constexpr size_t kNoAllocFloats = (kNoAllocBytes - kNoAllocTickets * sizeof(int)) / sizeof(float);
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kNoAllocBytes];

__global__ void zero_ints_kernel(int *dst, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = 0;
}

static std::mutex g_scratch_mu;
static unsigned char *g_scratch_ptr[kMaxDevices] = {};

// Device address of this device's copy of the array (the array's name is a host-side
// stand-in, not a device address): resolved once per device, with that device current.
flute_status noalloc_scratch(unsigned char **out, hipStream_t stream) {
    int dev = 0;
    FLUTE_HIP_CHECK(hipGetDevice(&dev));
    FLUTE_REQUIRE(dev >= 0 && dev < kMaxDevices, FLUTE_ERR_UNSUPPORTED,
                  "flute_gemv_noalloc: device ordinal %d beyond %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> guard(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        // resolving the symbol may load the code object: not something to do inside a capture
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        FLUTE_HIP_CHECK(hipStreamIsCapturing(stream, &cap));
        FLUTE_REQUIRE(cap == hipStreamCaptureStatusNone, FLUTE_ERR_INVALID,
                      "flute_gemv_noalloc: the first call on device %d that needs the scratch array "
                      "resolves its address and must not be under stream capture; make one such "
                      "call outside the capture first", dev);
        unsigned char *ptr = nullptr;
        FLUTE_HIP_CHECK(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        FLUTE_REQUIRE(ptr != nullptr, FLUTE_ERR_HIP,
                      "flute_gemv_noalloc: the scratch array has no address on device %d", dev);
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return FLUTE_OK;
}

}  // namespace

}  // namespace flute

using namespace flute;

extern "C" {

flute_status flute_gemv(const flute_linear *w, const void *x, void *y, int act_dtype, int split,
                        void *stream) {
    Plan plan;
    void *outs[1] = {y};
    flute_status st = make_plan(w, 1, x, outs, act_dtype, split, 0, "flute_gemv", &plan);
    if (st != FLUTE_OK) return st;
    return launch(plan, act_dtype, (hipStream_t)stream);
}

flute_status flute_gemv_noalloc(const flute_linear *w, const void *x, void *y, int act_dtype,
                                int split, void *stream) {
    Plan plan;
    void *outs[1] = {y};
    flute_status st = make_plan(w, 1, x, outs, act_dtype, split, 0, "flute_gemv_noalloc", &plan);
    if (st != FLUTE_OK) return st;
    const ScratchNeed need = scratch_need(plan);
    FLUTE_REQUIRE(need.floats <= kNoAllocFloats && need.ints <= kNoAllocTickets,
                  FLUTE_ERR_UNSUPPORTED,
                  "flute_gemv_noalloc: this launch needs %zu B of scratch and %zu tickets; the fixed "
                  "array holds %zu B and %zu tickets (N=%d, K=%d, R=%d, split=%d). Use flute_gemv, "
                  "or a smaller split",
                  need.floats * sizeof(float), need.ints, kNoAllocFloats * sizeof(float),
                  kNoAllocTickets, w->N, w->K, w->R, plan.p.split);
    if (need.floats == 0) return launch(plan, act_dtype, (hipStream_t)stream);
    unsigned char *ptr = nullptr;
    st = noalloc_scratch(&ptr, (hipStream_t)stream);
    if (st != FLUTE_OK) return st;
    int *tickets = (int *)ptr;
    float *base = (float *)(ptr + kNoAllocTickets * sizeof(int));
    if (plan.p.split > 1) {
        // the array keeps the last call's contents: tickets must start at zero (a fill
        // kernel, not a memset node, so that the call can be captured into a graph)
        const int n = (int)need.ints;
        hipLaunchKernelGGL(zero_ints_kernel, dim3((n + 255) / 256), dim3(256), 0,
                           (hipStream_t)stream, tickets, n);
        FLUTE_HIP_CHECK(hipGetLastError());
    }
    return launch(plan, act_dtype, (hipStream_t)stream, base, tickets);
}

flute_status flute_gemv_mlp(const flute_linear *gate, const flute_linear *up, const void *x,
                            void *h, int act_dtype, int split, void *stream) {
    FLUTE_REQUIRE(gate && up, FLUTE_ERR_INVALID, "flute_gemv_mlp: gate/up descriptor is NULL");
    flute_linear segs[2] = {*gate, *up};
    void *outs[2] = {h, h};
    Plan plan;
    flute_status st = make_plan(segs, 2, x, outs, act_dtype, split, 1, "flute_gemv_mlp", &plan);
    if (st != FLUTE_OK) return st;
    return launch(plan, act_dtype, (hipStream_t)stream);
}

flute_status flute_gemv_multi(const flute_linear *segs, int count, const void *x,
                              void *const *outs, int act_dtype, int split, void *stream) {
    FLUTE_REQUIRE(segs && outs, FLUTE_ERR_INVALID, "flute_gemv_multi: NULL argument");
    Plan plan;
    flute_status st =
        make_plan(segs, count, x, outs, act_dtype, split, 0, "flute_gemv_multi", &plan);
    if (st != FLUTE_OK) return st;
    return launch(plan, act_dtype, (hipStream_t)stream);
}

flute_status flute_mlp_block(const flute_linear *gate, const flute_linear *up,
                             const flute_linear *down, const void *x, void *h, void *y,
                             int act_dtype, void *stream) {
    FLUTE_REQUIRE(gate && up && down, FLUTE_ERR_INVALID, "flute_mlp_block: NULL descriptor");
    FLUTE_REQUIRE(down->K == gate->N, FLUTE_ERR_INVALID,
                  "flute_mlp_block: down K (%d) must equal gate/up N (%d)", down->K, gate->N);
    flute_status st = flute_gemv_mlp(gate, up, x, h, act_dtype, 0, stream);
    if (st != FLUTE_OK) return st;
    return flute_gemv(down, h, y, act_dtype, 0, stream);
}

int flute_pick_split(int N, int K) {
    if (N <= 0 || K <= 0 || N % 128 || K % 64) return 1;
    int rw, split, waves;
    choose_shape(N, K / 64, 0, &rw, &split, &waves);
    return split;
}

int64_t flute_gemv_lds_bytes(const flute_linear *w, int split) {
    Plan plan;
    alignas(16) char dummy_x[16] = {}, dummy_y[16] = {};    // never dereferenced
    void *outs[1] = {dummy_y};
    if (make_plan(w, 1, dummy_x, outs, (w && w->lut_dtype == FLUTE_BF16) ? FLUTE_BF16 : FLUTE_F16,
                  split, 0, "flute_gemv_lds_bytes", &plan) != FLUTE_OK)
        return 0;
    return (int64_t)plan.lds_bytes;
}

}  // extern "C"

#ifdef FLUTE_STAMPS
// Instrumented builds only: where the lean kernel writes its phase times (NULL switches them off).
extern "C" int flute_debug_gemv_stamps(void *buf) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_gemv_stamps), &buf, sizeof(buf));
}
#endif
