// Small-M / prefill LUT GEMM (placeholder entry until the MFMA kernel lands in
// this file): refuses loudly.
#include "host_common.h"

using namespace flute;

extern "C" flute_status flute_gemm(const flute_linear *w, const void *A, void *C, int M,
                                   int64_t lda, int64_t ldc, int act_dtype, void *stream) {
    (void)A; (void)C; (void)M; (void)lda; (void)ldc; (void)act_dtype; (void)stream;
    flute_status st = validate_linear(w, 1, "flute_gemm");
    if (st != FLUTE_OK) return st;
    set_error("flute_gemm: not built yet");
    return FLUTE_ERR_UNSUPPORTED;
}
