// Two-table instantiations of the lean GEMV kernel with a 1-bit stream: (4, 1) and (1, 4).
#include "gemv_pair_launch.h"

namespace flute {

flute_status launch_gemv_pair_1bit(const GemvParams &p, int pair, int grid_x, int nw, int pf,
                                   size_t lds_bytes, bool lut_bf16, hipStream_t stream) {
    if (pair == 41)
        return lut_bf16 ? launch_pair<true, 4, 1>(p, grid_x, nw, pf, lds_bytes, stream)
                        : launch_pair<false, 4, 1>(p, grid_x, nw, pf, lds_bytes, stream);
    return lut_bf16 ? launch_pair<true, 1, 4>(p, grid_x, nw, pf, lds_bytes, stream)
                    : launch_pair<false, 1, 4>(p, grid_x, nw, pf, lds_bytes, stream);
}

}  // namespace flute
