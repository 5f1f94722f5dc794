// Launchers of the M = 1 LUT GEMV family: single weight, merged gate/up with
// SiLU*mul, several weights sharing one input, and the two-launch MLP block.
#include "gemv_kernel.h"
#include "host_common.h"

#include <cmath>
#include <cstdlib>
#include <cstring>

namespace flute {

namespace {

int env_int(const char *name, int fallback) {
    const char *e = std::getenv(name);
    if (!e || !*e) return fallback;
    return std::atoi(e);
}

// log2 of the LDS bytes one workgroup may spend on lookup tables.
int table_budget_log2() {
    int v = env_int("FLUTE_GEMV_TABLE_LOG2", 16);
    if (v < 12) v = 12;
    if (v > 17) v = 17;
    return v;
}

int entries_log2(int bits) { return bits == 3 ? 6 : 8; }
int entry_bytes_log2(int bits) { return bits >= 3 ? 2 : (bits == 2 ? 3 : 4); }

struct Plan {
    GemvParams p;
    size_t lds_bytes;
    int grid_x;
    int total_tickets;
    size_t ws_floats;
    bool lut_bf16;
};

// Fill a launch plan for `count` weights that share x.  silu_mul couples
// weights 0 and 1 into one output.
flute_status make_plan(const flute_linear *segs, int count, const void *x, void *const *outs,
                       int act_dtype, int split, int silu_mul, int fht_block, const char *who,
                       Plan *plan) {
    FLUTE_REQUIRE(count >= 1 && count <= kGemvMaxSegs, FLUTE_ERR_INVALID,
                  "%s: 1..%d weights per launch (got %d)", who, kGemvMaxSegs, count);
    FLUTE_REQUIRE(x != nullptr, FLUTE_ERR_INVALID, "%s: x is NULL", who);
    FLUTE_REQUIRE(act_dtype == FLUTE_F16 || act_dtype == FLUTE_BF16, FLUTE_ERR_INVALID,
                  "%s: activations must be float16 or bfloat16", who);
    for (int i = 0; i < count; ++i) {
        flute_status st = validate_linear(&segs[i], 0, who);
        if (st != FLUTE_OK) return st;
        FLUTE_REQUIRE(outs[i] != nullptr, FLUTE_ERR_INVALID, "%s: output %d is NULL", who, i);
        FLUTE_REQUIRE(segs[i].K == segs[0].K, FLUTE_ERR_INVALID,
                      "%s: all weights of one launch must share K (%d vs %d)", who, segs[i].K,
                      segs[0].K);
        FLUTE_REQUIRE(segs[i].lut_dtype == segs[0].lut_dtype, FLUTE_ERR_UNSUPPORTED,
                      "%s: all weights of one launch must share the LUT dtype", who);
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

    GemvParams &p = plan->p;
    std::memset(&p, 0, sizeof(p));
    int tiles = 0;
    for (int i = 0; i < count; ++i)
        tiles += (segs[i].N / 128) * (segs[i].b2 > 0 ? 2 : 1);
    if (split <= 0) split = pick_split_tiles(tiles, G);
    FLUTE_REQUIRE(split >= 1 && G % split == 0, FLUTE_ERR_INVALID,
                  "%s: split %d must divide K/64 = %d", who, split, G);
    const int gs_tiles = G / split;
    const int kc = gs_tiles * 64;

    bool any_rot = false;
    for (int i = 0; i < count; ++i) any_rot |= segs[i].signs != nullptr;
    size_t scratch = 0;
    if (fht_block > 0) {
        FLUTE_REQUIRE(any_rot, FLUTE_ERR_INVALID, "%s: a rotation block needs rotation signs", who);
        FLUTE_REQUIRE(is_pow2(fht_block) && fht_block >= 32 && fht_block <= 16384 &&
                          K % fht_block == 0,
                      FLUTE_ERR_INVALID,
                      "%s: rotation block must be a power of two in [32, 16384] dividing K", who);
        FLUTE_REQUIRE(kc % fht_block == 0, FLUTE_ERR_UNSUPPORTED,
                      "%s: K slice %d of split %d is not a whole number of %d-column rotation "
                      "blocks",
                      who, kc, split, fht_block);
        scratch = (size_t)kc * 4;
    } else if (any_rot) {
        scratch = (size_t)make_segments(K, 0).len[0] * 4;
    }
    p.fht_block = fht_block;

    const int budget = table_budget_log2();
    size_t tab_bytes = 0;
    int njobs = 0, col = 0, n0 = 0, r0 = 0, ticket = 0;
    int ntot = 0;
    for (int i = 0; i < count; ++i) ntot += segs[i].N;
    for (int i = 0; i < count; ++i) {
        const flute_linear &w = segs[i];
        GemvSeg &sg = p.seg[i];
        sg.resB = (const uint16_t *)w.resB;
        sg.resA = (const uint16_t *)w.resA;
        sg.bias = (const uint16_t *)w.bias;
        sg.signs = w.signs;
        sg.awq = w.awq;
        sg.out = (uint16_t *)outs[i];
        sg.N = w.N;
        sg.R = w.R;
        sg.gs = w.group_size;
        sg.lut_rows = w.lut_rows;
        const int nstreams = w.b2 > 0 ? 2 : 1;
        sg.nslots = nstreams * split;
        sg.arrivals = sg.nslots;
        sg.n0 = n0;
        sg.r0 = ntot + r0;
        sg.ticket0 = (silu_mul && i == 1) ? p.seg[0].ticket0 : ticket;
        n0 += w.N;
        r0 += w.R;
        if (!(silu_mul && i == 1)) ticket += w.N / 128;
        const int ngrp_log2 = w.group_size >= 128 ? 0 : ilog2(128 / w.group_size);
        for (int st = 0; st < nstreams; ++st) {
            GemvJob &jb = p.job[njobs++];
            jb.q = (const uint8_t *)(st ? w.q2 : w.q1);
            jb.lut = (const uint16_t *)(st ? w.lut2 : w.lut1);
            jb.bits = st ? w.b2 : w.b1;
            jb.seg = i;
            jb.tile0 = col;
            jb.ntiles = w.N / 128;
            jb.slot0 = st * split;
            int es = budget - entries_log2(jb.bits) - ngrp_log2;
            if (es > 8) es = 8;
            if (es < entry_bytes_log2(jb.bits)) es = entry_bytes_log2(jb.bits);
            jb.es = es;
            const size_t tb = ((size_t)1 << (entries_log2(jb.bits) + es)) << ngrp_log2;
            if (tb > tab_bytes) tab_bytes = tb;
            col += jb.ntiles;
        }
    }
    if (silu_mul) {
        const int total = p.seg[0].nslots + p.seg[1].nslots;
        p.seg[0].arrivals = p.seg[1].arrivals = total;
    }
    p.njobs = njobs;
    p.K = K;
    p.split = split;
    p.gs_tiles = gs_tiles;
    p.p_stride = (ntot + r0 + 31) & ~31;
    p.silu_mul = silu_mul;
    p.act_bf16 = act_dtype == FLUTE_BF16;
    p.x = (const uint16_t *)x;

    size_t region0 = tab_bytes > scratch ? tab_bytes : scratch;
    region0 = (region0 + 255) & ~(size_t)255;
    p.lds_x = (int)region0;
    p.lds_red = p.lds_x + ((kc * 2 + 15) & ~15);
    p.lds_xb = p.lds_red + 128 * 4;
    plan->lds_bytes = (size_t)p.lds_xb + kGemvMaxRank * 4 + 16;
    FLUTE_REQUIRE(plan->lds_bytes <= (size_t)kLdsPerCU, FLUTE_ERR_UNSUPPORTED,
                  "%s: K=%d at split %d needs %zu B of LDS (limit %d)", who, K, split,
                  plan->lds_bytes, kLdsPerCU);
    plan->grid_x = col;
    plan->total_tickets = ticket;
    int max_slots = 0;
    for (int i = 0; i < count; ++i)
        if (p.seg[i].nslots > max_slots) max_slots = p.seg[i].nslots;
    plan->ws_floats = (size_t)max_slots * p.p_stride;
    plan->lut_bf16 = lut_bf16;
    return FLUTE_OK;
}

template <bool BF16>
flute_status launch_typed(Plan &plan, hipStream_t stream) {
    static size_t attr_bytes = 0;
    if (plan.lds_bytes > attr_bytes) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)gemv_kernel<BF16>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)kLdsPerCU));
        attr_bytes = kLdsPerCU;
    }
    dim3 grid(plan.grid_x, plan.p.split);
    hipLaunchKernelGGL(gemv_kernel<BF16>, grid, dim3(kGemvThreads), plan.lds_bytes, stream, plan.p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}

flute_status launch(Plan &plan, hipStream_t stream) {
    bool need_ws = false;
    for (int i = 0; i < kGemvMaxSegs; ++i) need_ws |= plan.p.seg[i].arrivals > 1;
    if (need_ws) {
        flute_status st = get_workspace(plan.ws_floats, (size_t)plan.total_tickets, stream,
                                        &plan.p.P, &plan.p.tickets);
        if (st != FLUTE_OK) return st;
    }
    return plan.lut_bf16 ? launch_typed<true>(plan, stream) : launch_typed<false>(plan, stream);
}

}  // namespace

}  // namespace flute

using namespace flute;

extern "C" {

flute_status flute_gemv(const flute_linear *w, const void *x, void *y, int act_dtype, int split,
                        void *stream) {
    Plan plan;
    void *outs[1] = {y};
    flute_status st = make_plan(w, 1, x, outs, act_dtype, split, 0,
                                (w && w->signs) ? w->rot_block : 0, "flute_gemv", &plan);
    if (st != FLUTE_OK) return st;
    return launch(plan, (hipStream_t)stream);
}

flute_status flute_gemv_mlp(const flute_linear *gate, const flute_linear *up, const void *x,
                            void *h, int act_dtype, int split, void *stream) {
    FLUTE_REQUIRE(gate && up, FLUTE_ERR_INVALID, "flute_gemv_mlp: gate/up descriptor is NULL");
    flute_linear segs[2] = {*gate, *up};
    void *outs[2] = {h, h};
    Plan plan;
    flute_status st = make_plan(segs, 2, x, outs, act_dtype, split, 1, 0, "flute_gemv_mlp", &plan);
    if (st != FLUTE_OK) return st;
    return launch(plan, (hipStream_t)stream);
}

flute_status flute_gemv_multi(const flute_linear *segs, int count, const void *x,
                              void *const *outs, int act_dtype, int split, void *stream) {
    FLUTE_REQUIRE(segs && outs, FLUTE_ERR_INVALID, "flute_gemv_multi: NULL argument");
    Plan plan;
    flute_status st =
        make_plan(segs, count, x, outs, act_dtype, split, 0, 0, "flute_gemv_multi", &plan);
    if (st != FLUTE_OK) return st;
    return launch(plan, (hipStream_t)stream);
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
    return pick_split_tiles(N / 128, K / 64);
}

int64_t flute_gemv_lds_bytes(const flute_linear *w, int split) {
    Plan plan;
    char dummy_x = 0, dummy_y = 0;
    void *outs[1] = {&dummy_y};
    if (make_plan(w, 1, &dummy_x, outs, FLUTE_F16 + (w && w->lut_dtype == FLUTE_BF16), split, 0, 0,
                  "flute_gemv_lds_bytes", &plan) != FLUTE_OK)
        return 0;
    return (int64_t)plan.lds_bytes;
}

}  // extern "C"
