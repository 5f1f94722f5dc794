// Host-side helpers shared by the launchers: validation, split policy and the
// per-device split-K workspace.
#pragma once

#include "common.h"

namespace flute {

// Shape/size/alignment contract of one weight (no device access).
// mode: 0 = GEMV, 1 = GEMM / dequant; | kModeKGroupOk where the entry point serves a LUT
// grouped along K (flute_linear.k_group).
constexpr int kModeKGroupOk = 0x100;
flute_status validate_linear(const flute_linear *w, int mode, const char *who);

// Split-K workspace of the current device: `floats` fp32 partial sums and
// `ints` zero-initialised tickets.  Grows geometrically, never shrinks; the
// tickets are zeroed once at allocation and every kernel leaves them at zero.
// One workspace per device: launches that use it must be ordered on one stream
// (the same contract as upstream include/flute/gemv_host.h:31-38).
// When the buffers must grow while `stream` is being captured into a graph the call is
// refused (FLUTE_ERR_INVALID): an allocation and the clearing of fresh tickets cannot be
// part of a capture.  Warm the shape up outside the capture first.
flute_status get_workspace(size_t floats, size_t ints, hipStream_t stream, float **P,
                           int **tickets);
// Called by an entry point after the last launch that uses the workspace: once the workspace
// has been used from two streams, records the event the next stream's call waits on.
void workspace_done(hipStream_t stream);

// What get_workspace does for a request, as pure host arithmetic: 0 = the buffers are
// large enough, 1 = they grow, 2 = growth refused because the stream is capturing.
int workspace_decision(size_t have_floats, size_t need_floats, size_t have_ints, size_t need_ints,
                       bool capturing);

// Tuning and test knobs of the launchers, read from the environment once per process
// (flute_reload_tuning re-reads them): FLUTE_GEMV_RW, FLUTE_GEMV_WAVES,
// FLUTE_GEMV_TABLE_LOG2, FLUTE_GEMV_PREROTATE, FLUTE_GEMV4_PF, FLUTE_GEMV_NO_FAST,
// FLUTE_GEMV4_WALK, FLUTE_GEMV_XCD, FLUTE_GEMM_ROWS, FLUTE_GEMM_NO_PERM, FLUTE_GEMM_KSPLIT,
// FLUTE_GEMM_NO_DIRECT, FLUTE_GEMM_NO_LEAN, FLUTE_GEMM_NO_BALANCE, FLUTE_GEMM_NO_HANDOVER,
// FLUTE_FHT_STEPS.  Unset or empty = 0, except fht_steps and
// gemv4_walk = -1 (the launcher's own choice) and gemv_xcd = 1 (0: workgroup b of the lean GEMV takes
// row slice b instead of a contiguous run of slices per XCD).
struct Tuning {
    int gemv_rw, gemv_waves, gemv_table_log2, gemv_prerotate, gemv4_pf, gemv_no_fast, gemv4_walk, gemv_xcd;
    int gemm_rows, gemm_no_perm, gemm_ksplit, gemm_no_direct, gemm_no_lean, gemm_no_balance, gemm_no_handover;
    int fht_steps;
};
const Tuning &tuning();

// The Walsh-Hadamard rotation of flute_fht with row strides, and optionally with its
// output written in the operand order of the LUT GEMM (the image the GEMM's activation
// pre-pass would produce from the rotated rows, padding rows zeroed) instead of as rows.
struct FhtOperandOut {
    uint32_t *ap;       // Ap[g][j][m / 16][lane][4 dwords]
    int mblk_pad;       // 16-row blocks the image holds per half tile
    int lut_bf16;       // 16-bit type of the image
    int block_xor;      // the mode of image_block_xor (common.h) the image is written with
};
flute_status fht_launch(const void *x, int64_t ldx, const float *signs, const float *awq, void *out,
                        int64_t ldo, int M, int K, int dtype, int adjoint, int block,
                        hipStream_t stream, const FhtOperandOut *operand);

inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
inline int ilog2(int v) { return 31 - __builtin_clz((unsigned)v); }

}  // namespace flute
