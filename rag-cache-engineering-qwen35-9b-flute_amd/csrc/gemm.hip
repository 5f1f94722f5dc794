// Host side of the small-M / prefill LUT GEMM: shape policy, workspace layout,
// pre-passes (activation permutation, residual coefficients) and the launch.
#include <stdlib.h>

#include "gemm_kernel.h"
#include "host_common.h"

#include <atomic>

namespace flute {

namespace {

struct GemmShape {
    int mb, kw, mw;       // 16-row blocks per wavefront, k ways, m ways
    int wg_per_cu;        // workgroups the policy expects to be resident per CU
};

// Rows of A per workgroup.  One or two 16-row blocks per wavefront with eight k ways (the
// launch is then a weight stream, like the GEMV) as long as one workgroup per 16 (32) rows
// and tile fits the device in one round and the indices are not re-read too often: every
// chunk of rows streams its tile again, and beyond about 64 MB (100 MB) of index traffic
// the next shape wins.  Measured: M = 32, 4096 -> 12288: 18.0 us with 16 rows, 24.6 us
// with 64; M = 64: 21.5 us with 32 rows, 26.0 us with 64; M = 256, 4096 -> 4096: 23.8 us
// with 32 rows, 29.0 us with 64; M = 96, 12288 -> 4096: 31.6 us with 32 rows, 37.8 us
// with 16, 34.7 us with 64.  Otherwise four blocks per wavefront: 64 rows per workgroup
// with eight k ways while that fits the device in one round, else 128 rows (two m groups,
// four k ways); further rows go to gridDim.y.  The tables plus staging take most of a
// CU's LDS, so one workgroup per CU is resident.  FLUTE_GEMM_ROWS = 16, 32, 64 or 128
// forces the shape (a tuning and test knob, like FLUTE_GEMV_RW).
GemmShape choose_gemm_shape(int M, int tiles, int64_t index_bytes) {
    {
        const int v = tuning().gemm_rows;
        if (v == 16) return {1, 8, 1, 1};
        if (v == 32) return {2, 8, 1, 1};
        if (v == 64) return {4, 8, 1, 1};
        if (v == 128) return {4, 4, 2, 1};
    }
    if (M <= 16) return {1, 8, 1, 1};
    const int chunks16 = (M + 15) / 16, chunks32 = (M + 31) / 32;
    if ((int64_t)tiles * chunks16 <= kNumCU && chunks16 * index_bytes <= (int64_t)64 << 20)
        return {1, 8, 1, 1};
    if ((int64_t)tiles * chunks32 <= kNumCU && chunks32 * index_bytes <= (int64_t)100 << 20)
        return {2, 8, 1, 1};
    const int chunks64 = (M + 63) / 64;
    if ((int64_t)tiles * chunks64 <= kNumCU) return {4, 8, 1, 1};
    return {4, 4, 2, 1};
}

template <int MB, int KW, int MW, bool BF16, int B1, bool PERM = false, bool DIRECT = false,
          bool LEAN = false>
flute_status launch_gemm(const GemmParams &p, dim3 grid, int lds, hipStream_t stream) {
    static std::atomic<bool> attr_done{false};   // threads may race to the first call: the call is idempotent
    if (!attr_done) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute((const void *)gemm_kernel<MB, KW, MW, BF16, B1, PERM, DIRECT, LEAN>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)kLdsPerCU));
        attr_done = true;
    }
    hipLaunchKernelGGL((gemm_kernel<MB, KW, MW, BF16, B1, PERM, DIRECT, LEAN>), grid, dim3(64 * KW * MW), lds,
                       stream, p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}

template <int MB, int KW, int MW, bool BF16>
flute_status launch_gemm_bits(const GemmParams &p, dim3 grid, int lds, hipStream_t stream) {
    if (p.nstreams == 1) {
        switch (p.bits[0]) {
            case 4:
                if constexpr (MB == 1) {
                    if (p.rep_log2[0] == 6 && p.A8)
                        return launch_gemm<MB, KW, MW, BF16, 4, true, true>(p, grid, lds, stream);
                }
                if constexpr (MB == 4) {
                    if (p.rep_log2[0] == 6 && p.lean)
                        return launch_gemm<MB, KW, MW, BF16, 4, true, false, true>(p, grid, lds, stream);
                }
                if (p.rep_log2[0] == 6) return launch_gemm<MB, KW, MW, BF16, 4, true>(p, grid, lds, stream);
                return launch_gemm<MB, KW, MW, BF16, 4>(p, grid, lds, stream);
            case 3: return launch_gemm<MB, KW, MW, BF16, 3>(p, grid, lds, stream);
            case 2: return launch_gemm<MB, KW, MW, BF16, 2>(p, grid, lds, stream);
            default: return launch_gemm<MB, KW, MW, BF16, 1>(p, grid, lds, stream);
        }
    }
    if constexpr (MB == 1) {
        return launch_gemm<MB, KW, MW, BF16, 0>(p, grid, lds, stream);
    } else {
        set_error("flute_gemm: two streams at this size run as one launch per stream");
        return FLUTE_ERR_UNSUPPORTED;
    }
}

template <bool BF16>
flute_status launch_gemm_shape(const GemmShape &s, const GemmParams &p, dim3 grid, int lds,
                               hipStream_t stream) {
    if (s.mb == 1) return launch_gemm_bits<1, 8, 1, BF16>(p, grid, lds, stream);
    if (s.mb == 2) return launch_gemm_bits<2, 8, 1, BF16>(p, grid, lds, stream);
    if (s.mw == 1) return launch_gemm_bits<4, 8, 1, BF16>(p, grid, lds, stream);
    return launch_gemm_bits<4, 4, 2, BF16>(p, grid, lds, stream);
}


// LDS plan of one launch: pair tables (+ staging on the fast path), sized against the
// reduction tree and the totals tile that reuse the same memory afterwards.
// A single 4-bit stream with at most two LUT groups per 128-row tile gets 64-lane
// replication (256 bytes per entry, 64 KB per group, first table at LDS offset 0: the
// layout the one-instruction address needs).  Everything else: as much replication as
// the budget allows, 32 lanes at most.
int plan_lds(GemmParams &p, const GemmShape &shape) {
    const int ngrp = p.gs >= 128 ? 1 : 128 / p.gs;
    const bool perm = p.nstreams == 1 && p.bits[0] == 4 && ngrp <= 2 &&
                      !tuning().gemm_no_perm;
    const int table_budget = (shape.mb == 1 ? 64 : 96) * 1024 / p.nstreams;
    int lds_tables = 0;
    for (int s = 0; s < p.nstreams; ++s) {
        const int entries = ngrp << (2 * p.bits[s]);
        int rl = 5;
        while (rl > 0 && (entries << rl) * 4 > table_budget) --rl;
        if (perm) rl = 6;
        p.rep_log2[s] = rl;
        p.tab_off[s] = lds_tables;
        lds_tables += (entries << rl) * 4;
    }
    p.lean = 0;
    if (perm) {                                  // per-wavefront tile staging behind the tables
        // four blocks per wavefront and one LUT group per tile: the lean loop, whose tiles go
        // straight into two staging buffers per wavefront
        p.lean = shape.mb == 4 && ngrp == 1 && !tuning().gemm_no_lean;
        p.stage_off = lds_tables;
        lds_tables += shape.kw * shape.mw * (p.lean ? 8192 : 4096);
        if (p.lean) {                            // one progress word per wavefront
            p.prog_off = lds_tables;
            lds_tables += 64;
            p.balance = !tuning().gemm_no_balance;
        }
    }
    const int slot_bytes = shape.mb * 8 * 64 * 16;
    const int lds_reduce = (shape.kw / 2) * shape.mw * slot_bytes;
    const int lds_tile = shape.mw * shape.mb * 16 * 132 * 4 + 16;   // totals tile + ticket flag
    int lds = lds_tables > lds_reduce ? lds_tables : lds_reduce;
    if (lds_tile > lds) lds = lds_tile;
    // the hand-overs between the k ways: eight 16 KB areas, then eight of 8 KB behind the totals tile
    if (p.scatter && lds < 17 * 4096 + 8 * 8192) lds = 17 * 4096 + 8 * 8192;
    return lds;
}

}  // namespace

}  // namespace flute

using namespace flute;

extern "C" flute_status flute_gemm(const flute_linear *w, const void *A, void *C, int M,
                                   int64_t lda, int64_t ldc, int act_dtype, void *stream_) {
    flute_status st = validate_linear(w, 1, "flute_gemm");
    if (st != FLUTE_OK) return st;
    FLUTE_REQUIRE(act_dtype == FLUTE_F16 || act_dtype == FLUTE_BF16, FLUTE_ERR_INVALID,
                  "flute_gemm: activations must be float16 or bfloat16");
    FLUTE_REQUIRE(M >= 0, FLUTE_ERR_INVALID, "flute_gemm: M must be >= 0 (got %d)", M);
    if (M == 0) return FLUTE_OK;
    FLUTE_REQUIRE(A != nullptr && C != nullptr, FLUTE_ERR_INVALID,
                  "flute_gemm: A and C must not be NULL");
    FLUTE_REQUIRE(lda >= w->K && ldc >= w->N, FLUTE_ERR_INVALID,
                  "flute_gemm: row strides must cover a row (lda=%lld < K=%d or ldc=%lld < N=%d)",
                  (long long)lda, w->K, (long long)ldc, w->N);
    FLUTE_REQUIRE(((uintptr_t)A & 1) == 0 && ((uintptr_t)C & 1) == 0, FLUTE_ERR_INVALID,
                  "flute_gemm: A and C must be 2-byte aligned");
    FLUTE_REQUIRE(w->R == 0 || (int64_t)M * w->R <= 16384, FLUTE_ERR_UNSUPPORTED,
                  "flute_gemm: the fused residual serves M*R <= 16384 (got M=%d, R=%d); add "
                  "(A @ resB^T) @ resA^T outside for larger products",
                  M, w->R);
    hipStream_t stream = (hipStream_t)stream_;

    GemmShape shape = choose_gemm_shape(M, w->N / 128, w->q1_bytes + (w->b2 > 0 ? w->q2_bytes : 0));
    GemmParams p = {};
    p.nstreams = w->b2 > 0 ? 2 : 1;
    p.q[0] = (const uint8_t *)w->q1;
    p.q[1] = (const uint8_t *)w->q2;
    p.lut[0] = (const uint16_t *)w->lut1;
    p.lut[1] = (const uint16_t *)w->lut2;
    p.bits[0] = w->b1;
    p.bits[1] = w->b2;
    p.M = M;
    p.N = w->N;
    p.K = w->K;
    p.G = w->K / 64;
    p.gs = w->group_size;
    p.lut_rows = w->lut_rows;
    p.R = w->R;
    p.resA = (const uint16_t *)w->resA;
    p.bias = (const uint16_t *)w->bias;
    p.C = C;
    p.ldc = ldc;
    p.out_bf16 = act_dtype == FLUTE_BF16;
    p.vec_store = (ldc % 8 == 0) && (((uintptr_t)C & 15) == 0);
    p.mblk_total = (M + 15) / 16;

    // ---- grid and K split --------------------------------------------------------
    const int tiles = w->N / 128;
    const int mchunks = (p.mblk_total + shape.mb * shape.mw - 1) / (shape.mb * shape.mw);
    const int64_t units = (int64_t)tiles * mchunks;
    p.mblk_pad = mchunks * shape.mb * shape.mw;
    const int64_t cap = (int64_t)kNumCU * shape.wg_per_cu;
    // K is split until the grid reaches one workgroup per CU, while every wavefront keeps
    // two tiles or more; with four blocks of rows per wavefront at most four ways, because
    // the workgroup that arrives last reads every 32 KB partial tile of its unit back
    // (measured at M = 64: 12288 -> 4096 29.7 us four ways, 36.4 us eight ways; 4096 -> 4096
    // 21.8 us four ways, 23.0 us two ways, 24.6 us eight ways).
    const int max_split = shape.mb == 1 ? 64 : 4;
    int ksplit = 1;
    while (units * ksplit * 2 <= cap && ksplit * 2 <= max_split &&
           p.G / (ksplit * 2) >= shape.kw * 2)
        ksplit *= 2;
    {
        const int v = tuning().gemm_ksplit;
        if (v >= 1 && v <= p.G) ksplit = v;
    }
    p.gper = (p.G + ksplit - 1) / ksplit;
    ksplit = (p.G + p.gper - 1) / p.gper;
    p.ksplit = ksplit;
    // Four blocks per wavefront and K ranges that start on a multiple of the k ways: the image is
    // written in the order the k ways want their blocks and they hand blocks to each other
    // instead of reducing through a tree (gemm_kernel.h; FLUTE_GEMM_NO_HANDOVER keeps the tree).
    p.scatter = 0;
    if (shape.mb == 4 && shape.kw * shape.mw == 8 && p.gper % shape.kw == 0 && !tuning().gemm_no_handover)
        p.scatter = shape.kw == 4 ? 1 : 2;
    const int block_xor = p.scatter;
    FLUTE_REQUIRE(mchunks <= 65535 && ksplit <= 65535, FLUTE_ERR_UNSUPPORTED,
                  "flute_gemm: M=%d exceeds the grid", M);

    // ---- workspace: [partial images][xb][Ap] -----------------------------------------
    const size_t image = (size_t)shape.mw * shape.mb * 8 * 64 * 4;
    const int zparts = ksplit * ((p.nstreams == 2 && shape.mb > 1) ? 2 : 1);
    const size_t p_floats = zparts > 1 ? (size_t)zparts * units * image : 0;
    const size_t xb_floats = ((size_t)M * w->R + 3) & ~(size_t)3;
    const size_t ap_floats = (size_t)p.G * 2 * p.mblk_pad * 64 * 4;
    const size_t rot_floats = w->signs ? ((size_t)M * w->K / 2 + 4) & ~(size_t)3 : 0;
    // bfloat16 activations presented as float16 operands: one power-of-two scale per row
    const bool scale_rows = act_dtype == FLUTE_BF16 && w->lut_dtype == FLUTE_F16;
    const size_t shift_floats = scale_rows ? ((size_t)M + 3) & ~(size_t)3 : 0;
    float *base = nullptr;
    int *tickets = nullptr;
    st = get_workspace(p_floats + xb_floats + ap_floats + rot_floats + shift_floats + 64, (size_t)units + 1, stream, &base,
                       &tickets);
    if (st != FLUTE_OK) return st;
    p.P = base;
    p.tickets = tickets;
    float *xb = base + p_floats;
    u4_t *Ap = (u4_t *)(xb + xb_floats);
    p.Ap = Ap;
    // One block of rows per wavefront on the single-stream 4-bit fast path: the kernel reads
    // A itself (16-byte pieces of a row, put into operand order in registers), so the
    // pre-pass launch is dropped.  Needs 16-byte aligned rows.
    {
        const int ngrp = w->group_size >= 128 ? 1 : 128 / w->group_size;
        const bool fast = p.nstreams == 1 && w->b1 == 4 && ngrp <= 2 &&
                          !tuning().gemm_no_perm;
        if (shape.mb == 1 && fast && !w->signs && ((uintptr_t)A & 15) == 0 && lda % 8 == 0 &&
            !tuning().gemm_no_direct) {
            p.A8 = (const u4_t *)A;
            p.lda8 = lda / 8;
            p.a_bf16 = act_dtype == FLUTE_BF16;
        }
    }
    int *rowshift = scale_rows
        ? (int *)(base + p_floats + xb_floats + ap_floats + rot_floats) : nullptr;
    auto launch_rowshift = [&](const void *rows, int64_t ld) -> flute_status {
        hipLaunchKernelGGL(gemm_rowshift_kernel, dim3(M), dim3(256), 0, stream,
                           (const uint16_t *)rows, ld, w->K, rowshift);
        FLUTE_HIP_CHECK(hipGetLastError());
        p.rowshift = rowshift;
        return FLUTE_OK;
    };
    if (p.A8) {
        // nothing to prepare but the row scales
        if (scale_rows) {
            st = launch_rowshift(A, lda);
            if (st != FLUTE_OK) return st;
        }
    } else if (w->signs && w->R == 0 && !scale_rows) {
        // the rotation writes the operand image itself: one launch instead of two
        FhtOperandOut image_out = {(uint32_t *)Ap, p.mblk_pad, (int)(w->lut_dtype == FLUTE_BF16), block_xor};
        st = fht_launch(A, lda, w->signs, w->awq, nullptr, 0, M, w->K, act_dtype, 0, w->rot_block,
                        stream, &image_out);
        if (st != FLUTE_OK) return st;
    } else {
        if (w->signs) {
            // the residual coefficients and the row scales need the rotated rows as rows:
            // rotated copy first, then the ordinary pre-pass on it
            void *Arot = (void *)(Ap + (size_t)p.G * 2 * p.mblk_pad * 64);
            st = fht_launch(A, lda, w->signs, w->awq, Arot, w->K, M, w->K, act_dtype, 0,
                            w->rot_block, stream, nullptr);
            if (st != FLUTE_OK) return st;
            A = Arot;
            lda = w->K;
        }
        if (scale_rows) {
            st = launch_rowshift(A, lda);
            if (st != FLUTE_OK) return st;
        }
        const int64_t total = (int64_t)p.G * 2 * p.mblk_pad * 64;
        const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
        if (((uintptr_t)A & 15) == 0 && lda % 8 == 0) {
            // 16-byte aligned rows: one coalesced 16-byte load per thread and a transpose
            // inside each quad (M = 256, K = 4096: 2.2 us against 5.2 us for the gathers)
            hipLaunchKernelGGL(gemm_prep_quad_kernel, dim3(blocks), dim3(256), 0, stream,
                               (const uint16_t *)A, Ap, M, lda, p.G, p.mblk_pad,
                               (int)(act_dtype == FLUTE_BF16), (int)(w->lut_dtype == FLUTE_BF16),
                               rowshift, (const uint32_t *)w->lut1,
                               (int)(((size_t)w->lut_rows << w->b1) * 2 / 64), block_xor);
        } else {
            hipLaunchKernelGGL(gemm_prep_kernel, dim3(blocks), dim3(256), 0, stream,
                               (const uint16_t *)A, Ap, M, lda, p.G, p.mblk_pad,
                               (int)(act_dtype == FLUTE_BF16), (int)(w->lut_dtype == FLUTE_BF16),
                               (int)((((uintptr_t)A & 3) == 0) && (lda % 2 == 0)), rowshift, block_xor);
        }
        FLUTE_HIP_CHECK(hipGetLastError());
    }
    if (w->R > 0) {
        hipLaunchKernelGGL(gemm_coeff_kernel, dim3(w->R, M), dim3(256), 0, stream,
                           (const uint16_t *)A, lda, (const uint16_t *)w->resB, xb, w->K, w->R,
                           p.out_bf16);
        FLUTE_HIP_CHECK(hipGetLastError());
        p.xb = xb;
    }

    // Two streams with four blocks per wavefront: one launch per stream through the
    // single-stream kernels (the two-stream kernel does not fit the register file at
    // that size); both write partial tiles and the last workgroup of the second launch
    // folds everything, exactly as a K split does.
    const bool per_stream = p.nstreams == 2 && shape.mb > 1;
    const int passes = per_stream ? 2 : 1;
    const dim3 grid(tiles, mchunks, ksplit);
    for (int pass = 0; pass < passes; ++pass) {
        GemmParams q = p;
        if (per_stream) {
            q.nstreams = 1;
            q.q[0] = p.q[pass];
            q.lut[0] = p.lut[pass];
            q.bits[0] = p.bits[pass];
        }
        q.z_base = pass * ksplit;
        q.ztotal = passes * ksplit;
        const int lds = plan_lds(q, shape);
        FLUTE_REQUIRE(lds <= kLdsPerCU, FLUTE_ERR_UNSUPPORTED,
                      "flute_gemm: %d bytes of LDS exceed the %d of one CU", lds, kLdsPerCU);
        st = w->lut_dtype == FLUTE_BF16 ? launch_gemm_shape<true>(shape, q, grid, lds, stream)
                                        : launch_gemm_shape<false>(shape, q, grid, lds, stream);
        if (st != FLUTE_OK) return st;
    }
    workspace_done(stream);
    return FLUTE_OK;
}

#ifdef FLUTE_STAMPS
// Instrumented builds only: where the kernels write their phase times (NULL switches them off).
extern "C" int flute_debug_stamps(void *buf) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(flute::g_gemm_stamps), &buf, sizeof(buf));
}
#endif
