// Two-table instantiations of the lean GEMV kernel without a 1-bit stream: (3, 3), (2, 4), (2, 3).
#include "gemv_pair_launch.h"

namespace flute {

flute_status launch_gemv_pair_wide(const GemvParams &p, int pair, int grid_x, int nw, int pf,
                                   size_t lds_bytes, bool lut_bf16, hipStream_t stream) {
    switch (pair) {
        case 24:
            return lut_bf16 ? launch_pair<true, 2, 4>(p, grid_x, nw, pf, lds_bytes, stream)
                            : launch_pair<false, 2, 4>(p, grid_x, nw, pf, lds_bytes, stream);
        case 23:
            return lut_bf16 ? launch_pair<true, 2, 3>(p, grid_x, nw, pf, lds_bytes, stream)
                            : launch_pair<false, 2, 3>(p, grid_x, nw, pf, lds_bytes, stream);
        default:
            return lut_bf16 ? launch_pair<true, 3, 3>(p, grid_x, nw, pf, lds_bytes, stream)
                            : launch_pair<false, 3, 3>(p, grid_x, nw, pf, lds_bytes, stream);
    }
}

}  // namespace flute
