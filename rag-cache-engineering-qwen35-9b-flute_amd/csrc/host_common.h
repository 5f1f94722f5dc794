// Host-side helpers shared by the launchers: validation, split policy and the
// per-device split-K workspace.
#pragma once

#include "common.h"

namespace flute {

// Shape/size/alignment contract of one weight (no device access).
// mode: 0 = GEMV, 1 = GEMM / dequant.
flute_status validate_linear(const flute_linear *w, int mode, const char *who);

// K-split the GEMV launchers use for `tiles` 128-row workgroup columns over
// G = K/64 tiles of K.

// Split-K workspace of the current device: `floats` fp32 partial sums and
// `ints` zero-initialised tickets.  Grows geometrically, never shrinks; the
// tickets are zeroed once at allocation and every kernel leaves them at zero.
// One workspace per device: launches that use it must be ordered on one stream
// (the same contract as upstream include/flute/gemv_host.h:31-38).
flute_status get_workspace(size_t floats, size_t ints, hipStream_t stream, float **P,
                           int **tickets);

inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
inline int ilog2(int v) { return 31 - __builtin_clz((unsigned)v); }

}  // namespace flute
