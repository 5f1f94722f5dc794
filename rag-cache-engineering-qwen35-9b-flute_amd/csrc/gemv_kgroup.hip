// The lean GEMV kernel for a LUT grouped along K (flute_linear.k_group = 128): its
// instantiations and their launch, apart from the other GEMV kernels so that the two
// translation units compile side by side.
#include <atomic>

#include "host_common.h"
#include "gemv_kernel.h"
#include "gemv4_kernel.h"

namespace flute {

namespace {

template <int LPGL, int NW, int PF, bool BF16>
flute_status launch_grid(const GemvParams &p, int grid_x, size_t lds_bytes, hipStream_t stream) {
    static std::atomic<bool> attr_done{false};   // threads may race to the first call: the call is idempotent
    if (!attr_done) {
        FLUTE_HIP_CHECK(hipFuncSetAttribute(
            (const void *)gemv4_kernel<LPGL, NW, PF, BF16, false, 4, 4, true>,
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsPerCU));
        attr_done = true;
    }
    hipLaunchKernelGGL((gemv4_kernel<LPGL, NW, PF, BF16, false, 4, 4, true>), dim3(grid_x, p.split),
                       dim3(NW * 64), lds_bytes, stream, p);
    FLUTE_HIP_CHECK(hipGetLastError());
    return FLUTE_OK;
}

template <bool BF16>
flute_status launch_shape(const GemvParams &p, int grid_x, int nw, int pf, size_t lds_bytes,
                          hipStream_t stream) {
    switch (nw * 100 + p.lpg_log2 * 10 + pf) {
        case 442: return launch_grid<4, 4, 2, BF16>(p, grid_x, lds_bytes, stream);
        case 444: return launch_grid<4, 4, 4, BF16>(p, grid_x, lds_bytes, stream);
        case 452: return launch_grid<5, 4, 2, BF16>(p, grid_x, lds_bytes, stream);
        case 454: return launch_grid<5, 4, 4, BF16>(p, grid_x, lds_bytes, stream);
        case 462: return launch_grid<6, 4, 2, BF16>(p, grid_x, lds_bytes, stream);
        case 464: return launch_grid<6, 4, 4, BF16>(p, grid_x, lds_bytes, stream);
        case 842: return launch_grid<4, 8, 2, BF16>(p, grid_x, lds_bytes, stream);
        case 844: return launch_grid<4, 8, 4, BF16>(p, grid_x, lds_bytes, stream);
        case 852: return launch_grid<5, 8, 2, BF16>(p, grid_x, lds_bytes, stream);
        case 854: return launch_grid<5, 8, 4, BF16>(p, grid_x, lds_bytes, stream);
        default: break;
    }
    FLUTE_REQUIRE(false, FLUTE_ERR_UNSUPPORTED,
                  "flute_gemv: no kernel for a LUT grouped along K with %d wavefronts, %d-row "
                  "workgroups and %d loads in flight", nw, 1 << (p.lpg_log2 - 1), pf);
}

}  // namespace

flute_status launch_gemv_kgroup(const GemvParams &p, int grid_x, int nw, int pf, size_t lds_bytes,
                                bool lut_bf16, hipStream_t stream) {
    return lut_bf16 ? launch_shape<true>(p, grid_x, nw, pf, lds_bytes, stream)
                    : launch_shape<false>(p, grid_x, nw, pf, lds_bytes, stream);
}

}  // namespace flute
