// Launch of the lean GEMV kernel's two-table instantiations (mixed width pairs and single
// narrow streams).  Included by the translation units that hold them (gemv_pairs_*.hip): the
// instantiations are many, and two units compile side by side.
#pragma once

#include <atomic>

#include "host_common.h"
#include "gemv_kernel.h"
#include "gemv4_kernel.h"

namespace flute {

namespace {

// The lean kernel with two resident tables (mixed widths); no walking grid.  Eight wavefronts
// come with 8- or 16-row slices only (choose_shape).
template <int LPGL, int NW, int PF, bool BF16, int BA, int BB, bool DEEP = false>
flute_status launch_pair_grid(const GemvParams &p, int grid_x, size_t lds_bytes, hipStream_t stream) {
    static std::atomic<bool> attr_done{false};
    if (!attr_done) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute(
            (const void *)gemv4_kernel<LPGL, NW, PF, BF16, false, BA, BB, false, DEEP>,
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsPerCU));
        attr_done = true;
    }
    dim3 grid(grid_x, p.split);
    hipLaunchKernelGGL((gemv4_kernel<LPGL, NW, PF, BF16, false, BA, BB, false, DEEP>), grid, dim3(NW * 64),
                       lds_bytes, stream, p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}
// pf: 2 or 4; 8 = four with the deep ring for the 1-bit stream of the pair (a wavefront's loads
// are then a multiple of eight)
template <bool BF16, int BA, int BB>
flute_status launch_pair(const GemvParams &p, int grid_x, int nw, int pf, size_t lds_bytes, hipStream_t stream) {
    constexpr bool NARROW = BA == 1;                 // the deep ring: for a 1-bit stream in front
    switch (nw * 100 + p.lpg_log2 * 10 + pf) {
        case 442: return launch_pair_grid<4, 4, 2, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 444: return launch_pair_grid<4, 4, 4, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 452: return launch_pair_grid<5, 4, 2, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 454: return launch_pair_grid<5, 4, 4, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 462: return launch_pair_grid<6, 4, 2, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 464: return launch_pair_grid<6, 4, 4, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 842: return launch_pair_grid<4, 8, 2, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 844: return launch_pair_grid<4, 8, 4, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 852: return launch_pair_grid<5, 8, 2, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        case 854: return launch_pair_grid<5, 8, 4, BF16, BA, BB>(p, grid_x, lds_bytes, stream);
        default: break;
    }
    if constexpr (NARROW) {
        switch (nw * 100 + p.lpg_log2 * 10 + pf) {
            case 448: return launch_pair_grid<4, 4, 4, BF16, BA, BB, true>(p, grid_x, lds_bytes, stream);
            case 458: return launch_pair_grid<5, 4, 4, BF16, BA, BB, true>(p, grid_x, lds_bytes, stream);
            case 468: return launch_pair_grid<6, 4, 4, BF16, BA, BB, true>(p, grid_x, lds_bytes, stream);
            case 848: return launch_pair_grid<4, 8, 4, BF16, BA, BB, true>(p, grid_x, lds_bytes, stream);
            case 858: return launch_pair_grid<5, 8, 4, BF16, BA, BB, true>(p, grid_x, lds_bytes, stream);
            default: break;
        }
    }
    return FLUTE_ERR_UNSUPPORTED;                    // (not reached: the caller checks the shape)
}


}  // namespace

}  // namespace flute
