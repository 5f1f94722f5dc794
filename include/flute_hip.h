/*
 * flute_hip.h — C ABI of the MI355X (gfx950) idxN LUT-palettized linear layer.
 *
 * One shared library, libflute_hip.so, plain pointers and sizes, no framework
 * types.  Every pointer named "device" must be memory of the current HIP
 * device; `stream` is a hipStream_t passed as void* (NULL = the null stream).
 * Launches are asynchronous: no entry point synchronises or copies to the host.
 *
 * Each entry point names the upstream interface it replaces (paths relative to
 * the upstream tree's src/flute_extended/).  Upstream exposes these through
 * pybind11 with torch::Tensor arguments (src/bindings.cpp:230-546); here the
 * same operands arrive as raw pointers plus the sizes upstream derives from
 * the tensors.
 *
 * Error model: every function returns FLUTE_OK or one of the FLUTE_ERR_* codes;
 * the message of the last failure on the calling thread is available from
 * flute_last_error().  All argument validation happens before the device is
 * touched, so the refusal paths can be exercised on a machine without a GPU.
 * There is no fallback of any kind: a shape or dtype the kernels do not serve
 * is refused with FLUTE_ERR_UNSUPPORTED.
 */
#ifndef FLUTE_HIP_H
#define FLUTE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum flute_status {
    FLUTE_OK = 0,
    FLUTE_ERR_INVALID = 1,      /* contract violation (shape, size, alignment, NULL) */
    FLUTE_ERR_UNSUPPORTED = 2,  /* valid but outside what the kernels serve          */
    FLUTE_ERR_HIP = 3,          /* a HIP runtime call failed                          */
    FLUTE_ERR_NOMEM = 4         /* workspace allocation failed                        */
} flute_status;

typedef enum flute_dtype {
    FLUTE_F16 = 0,
    FLUTE_BF16 = 1,
    FLUTE_F32 = 2,
    FLUTE_U8 = 3           /* index blobs; only in flute_tensor records */
} flute_dtype;

/*
 * One palettized weight, as the upstream kernel entries receive it
 * (src/kernel_gemv.cu:322-333, src/kernel_gemv_splitk.cu:813-830):
 *
 *   W[n, k] = lut1[n / group_size][idx1[n, k]]  (+ the same for stream 2)
 *   y       = x W^T + (x resB^T) resA^T + bias
 *
 * q1/q2   idxN blobs (flute_extended/idxN.py:37-55), N*K*b/8 bytes, 16-byte aligned
 * lut1/2  [ceil(N/group_size), 2^b] in lut_dtype, contiguous
 * b2 == 0 means "single stream" and q2/lut2 are ignored
 * resB    (R, K), resA (N, R), bias (N,) in the ACTIVATION dtype, or NULL / R = 0
 * Arithmetic type: the products run in lut_dtype, so that the dequantised weight is the
 * LUT entry exactly.  bfloat16 activations with a float16 LUT are scaled by a power of
 * two per staged row (exact) on their way into the kernel and the row sums are scaled
 * back, so activations beyond float16's range (|x| > 65504, |x| < 6e-8) give the same
 * result as fp32 arithmetic on x.float().  A row that holds an infinity or a NaN is not
 * scaled (there is no finite maximum to scale by): its finite values beyond float16's range
 * saturate, so the outputs of such a row are unspecified (they may be NaN where fp32
 * arithmetic gives an infinity).  float16 activations with a bfloat16 LUT are
 * refused (FLUTE_ERR_UNSUPPORTED): that conversion is not exact.
 * signs   (K,) fp32 +-1: when non-NULL the input is rotated first, x <- x @ T
 *         (fht.py:19-35); awq (K,) fp32 then selects ((x*s) @ T) / s
 */
typedef struct flute_linear {
    const void *q1;
    const void *lut1;
    const void *q2;
    const void *lut2;
    const void *resB;
    const void *resA;
    const void *bias;
    const float *signs;
    const float *awq;
    int64_t q1_bytes;
    int64_t q2_bytes;
    int32_t lut_rows;      /* rows of lut1 (and of lut2): must equal ceil(N/group_size) */
    int32_t N;
    int32_t K;
    int32_t R;
    int32_t b1;
    int32_t b2;
    int32_t group_size;
    int32_t lut_dtype;     /* FLUTE_F16 or FLUTE_BF16 */
    int32_t rot_block;     /* 0: rotation over the descending power-of-two segments of K
                              (upstream's transform); > 0: equal blocks of this many
                              columns, each normalised by 1/sqrt(rot_block) */
    int32_t k_group;       /* 0: the LUT is grouped along N (every upstream artifact).
                              128: the LUT is grouped along K, one row of 16 values per
                              (output row, 128-wide K group): lut1 is [N, K/128, 16],
                              lut_rows = N * K/128, W[n, k] = lut1[n][k / 128][idx[n, k]].
                              No upstream kernel or artifact has this form; it needs
                              b1 = 4, b2 = 0, K % 128 == 0 and a 16-byte aligned lut1;
                              group_size is not read.  Served by flute_gemv,
                              flute_gemv_noalloc and flute_dequant; every other entry
                              point refuses it.  (The field takes what were four bytes of
                              padding at the end of the structure: its size is unchanged,
                              and a caller that zero-initialises the structure gets 0.) */
} flute_linear;

/* Library identity and diagnostics. */
int flute_abi_version(void);
const char *flute_last_error(void);
/* Name of the code-object architecture the kernels were built for ("gfx950"). */
const char *flute_target_arch(void);

/*
 * M = 1 LUT GEMV:  y[1, N] = linear(x[1, K]).
 * Replaces qgemm_gemv_stream, qgemm_gemv_fht_stream, qgemm_gemv_splitk_stream
 * and qgemm_gemv_splitk_fht_stream (src/bindings.cpp:277-354): rotation is
 * selected by w->signs, the K split by `split` (0 = library policy,
 * flute_pick_split; otherwise 1 <= split, split must divide K/64).
 * x and y are act_dtype (FLUTE_F16 or FLUTE_BF16).  Deterministic: partial
 * sums are folded in a fixed order, so repeated calls are bit identical.
 */
flute_status flute_gemv(const flute_linear *w, const void *x, void *y,
                        int act_dtype, int split, void *stream);

/*
 * flute_gemv for callers that cannot allocate (code under HIP graph capture, serving
 * loops and harnesses that forbid hipMalloc).  No counterpart upstream.  Same operands,
 * same kernels and bit-identical results; what flute_gemv takes from the library's
 * growing workspace (partial sums and tickets of a K split, residual coefficients, the
 * pre-rotated input of a rotated weight with a residual) lives in a fixed 2 MiB array
 * that is part of the code object: each device the library runs on holds its own copy
 * until the process ends.  The call allocates nothing and frees nothing.  A launch whose
 * scratch exceeds the array (more than 520192 floats or 4096 tickets: roughly
 * split * (N + R) + R + K/2 floats, N/8 tickets) is refused with FLUTE_ERR_UNSUPPORTED.
 * Every call on a device shares that device's array: calls that overlap on one device
 * (two streams, or a replaying graph next to eager calls) race; order them.
 */
flute_status flute_gemv_noalloc(const flute_linear *w, const void *x, void *y,
                                int act_dtype, int split, void *stream);

/*
 * Merged gate+up GEMV with the SiLU*mul epilogue, M = 1:
 *   h[n] = silu(gate(x)[n]) * up(x)[n],   silu(v) = v / (1 + exp(-v)), fp32,
 * one rounding to act_dtype.  Replaces qgemm_gemv_mlp (src/bindings.cpp:378-384,
 * src/kernel_gemv_mlp.cu:536-691).  gate and up must agree in N and K; all
 * other fields may differ.
 */
flute_status flute_gemv_mlp(const flute_linear *gate, const flute_linear *up,
                            const void *x, void *h, int act_dtype, int split,
                            void *stream);

/*
 * Several weights sharing one input row, one launch (the QKV merge):
 * outs[i][1, N_i] = linear_i(x).  Replaces qgemm_gemv_multi
 * (src/bindings.cpp:368-373, src/kernel_gemv_multi.cu).  1 <= count <= 4, all K
 * equal.
 */
flute_status flute_gemv_multi(const flute_linear *segs, int count, const void *x,
                              void *const *outs, int act_dtype, int split,
                              void *stream);

/*
 * The whole decode MLP block for one token, two dependent launches on `stream`
 * (merged gate+up with SiLU*mul, then down):  y = down( silu(gate(x)) * up(x) ).  h is caller-provided scratch
 * of gate->N elements in act_dtype.  Mirrors FusedPalettizedMLP.forward at
 * M = 1 (scripts/palettized_modules.py:1673-1682).
 */
flute_status flute_mlp_block(const flute_linear *gate, const flute_linear *up,
                             const flute_linear *down, const void *x, void *h,
                             void *y, int act_dtype, void *stream);

/*
 * Small-M / prefill LUT GEMM:  C[M, N] = A[M, K] @ W^T (+ stream 2, residual,
 * bias), fp32 accumulate on MFMA, one rounding to act_dtype.  Replaces
 * qgemm_per_group_lut / qgemm_cutlass_streaming (src/bindings.cpp:231-251,
 * src/kernel_streaming.cu:2297-2443) and qgemm_dual_stream
 * (src/bindings.cpp:257-270).  The MFMA operand type follows lut_dtype, so the
 * dequantised tile is exactly the LUT entry; A is converted to that type if it
 * differs.  lda = row stride of A in elements (>= K), ldc likewise for C.
 * When w->signs is set the rows of A are rotated first (a flute_fht pass into the
 * library workspace), as the M = 1 entry does in its prologue.  The fused residual
 * serves M * R <= 16384; larger products are refused with FLUTE_ERR_UNSUPPORTED.
 */
flute_status flute_gemm(const flute_linear *w, const void *A, void *C, int M,
                        int64_t lda, int64_t ldc, int act_dtype, void *stream);

/*
 * Scalar differential twin of the LUT GEMM:  C[M, N] = A[M, K] @ W^T for one stream, one
 * thread per output, every weight decoded from its bit position and looked up in the LUT
 * in global memory, fp32 sum in ascending k, one rounding.  Shares no code with
 * flute_gemm.  Replaces qgemm_debug_simple (src/bindings.cpp:243,
 * src/kernel_debug_simple.cu:94-267).  layout 0: q holds the LOGICAL packed rows
 * [N, K*bits/8], LSB-first along k (upstream's twin consumes this layout); layout 1: q is
 * the idxN blob, so the twin and flute_gemm can read the same bytes.  Slow by design.
 */
flute_status flute_gemm_debug_simple(const void *q, int64_t q_bytes, int layout,
                                     const void *lut, int lut_rows, int lut_dtype, int bits,
                                     int group_size, int N, int K, const void *A, void *C,
                                     int M, int64_t lda, int64_t ldc, int act_dtype,
                                     void *stream);

/*
 * Dequantise one stream to a dense row-major [N, K] matrix in lut_dtype,
 * through the same tile decoder the GEMM uses.  which = 1 or 2.  Serves the
 * bit-exact tile check that upstream runs against dequantize_reference
 * (test_flute.py:172-223) and the role of its scalar differential twin
 * (src/kernel_debug_simple.cu).
 */
flute_status flute_dequant(const flute_linear *w, int which, void *W_out,
                           void *stream);

/*
 * Walsh-Hadamard rotation of M rows of length K (fht.py:19-35):
 *   adjoint == 0:  out = x @ T      = ((x @ H) * s) / sqrt(b) per segment
 *   adjoint != 0:  out = x @ T^T    = ((x * s) @ H) / sqrt(b) per segment
 *   awq != NULL (forward only): out = ((x * awq) @ T) / awq, fp32, true division
 * Segments are the descending powers of two of K when block == 0, or equal
 * blocks of `block` columns (a power of two dividing K) otherwise.  out == x is
 * allowed.  dtype is FLUTE_F16, FLUTE_BF16 or FLUTE_F32 for both x and out.
 * Replaces fht_forward, fht_backward, fht_inplace_ and fht_forward_awq
 * (src/bindings.cpp:386-399, src/kernel_fht.cu:335-397).
 * Contract: K % 32 == 0, 32 <= K <= 65504, every segment <= 16384
 * (fht.py:381-390).
 */
flute_status flute_fht(const void *x, const float *signs, const float *awq,
                       void *out, int M, int K, int dtype, int adjoint, int block,
                       void *stream);

/*
 * Embedding rows out of a palettized table:  out[i, :] = row ids[i] of the table, in
 * lut_dtype.  Replaces PalettizedEmbedding.forward (scripts/palettized_modules.py:
 * 1998-2015, 2298-2335), which upstream runs as torch gathers: stream 1 and stream 2
 * are added in the LUT's 16-bit type (stream 1 first), the residual resA[n, :] @ resB
 * (both in lut_dtype here) is added in fp32, a rotated (tied) table is un-rotated with
 * the adjoint transform when w->signs is set, and the row is rounded once.
 * ids: `count` int64 on the device; an id outside [0, N) yields a row of zeros (the
 * Python mirror refuses such ids before the launch).  No bias, no awq.
 */
flute_status flute_embedding(const flute_linear *w, const int64_t *ids, int64_t count,
                             void *out, void *stream);

/*
 * The K-split the library would choose for an (N, K) GEMV without a fused rotation on this
 * device (the MI355X counterpart of gemv_pick_split, src/gemv_host.cpp:29-38; the numbers
 * are this device's, not the A10G's).  Up to K = 24576 the unsplit launch measured fastest
 * for every N, so the answer is 1; from K = 32768 it is 4 for N <= 512 and 2 for N <= 1024
 * (N = 512, K = 32768: 7.5 us against 9.0 us unsplit).  Callers that pass an explicit split
 * to flute_gemv still get it.  Pure host arithmetic: usable without a GPU.
 */
int flute_pick_split(int N, int K);

/* LDS bytes one GEMV workgroup needs for this weight (0 when the weight is
 * refused); the host-side gates mirror it (flute_extended/__init__.py:643-665). */
int64_t flute_gemv_lds_bytes(const flute_linear *w, int split);

/*
 * The argument checks of a binding, once.  Upstream's bindings check the tensors they are handed
 * (dtype, rank, shape against K and the blob's byte count, contiguity, device) before they build
 * a launch (src/bindings.cpp:230-546, src/kernel_gemv.cu:379-474); so must any binding of this
 * library, and these two calls do it for them: the binding records what it knows about each
 * tensor in a flute_tensor (no tensor type crosses the boundary) and gets back either the filled
 * flute_linear and N, or FLUTE_ERR_INVALID with the message upstream's check would raise in
 * flute_last_error().  "Absent" operands follow upstream's convention: an empty tensor
 * (numel = 0); signs and awq are absent when `present` is 0.  Both bindings in this repository
 * (flute_extended/_C.py over ctypes and csrc/torch_binding.cpp) call them, so the checks, their
 * order and their messages exist in one place.  Pure host code: usable without a GPU.
 */
typedef struct flute_tensor {
    const void *data;        /* address of element 0 (device memory for a GPU tensor) */
    const char *dtype_name;  /* how the binding prints the dtype ("torch.float64"), or NULL */
    int64_t numel;
    int64_t size[4];         /* the first min(ndim, 4) sizes */
    int32_t ndim;
    int32_t dtype;           /* FLUTE_F16 / FLUTE_BF16 / FLUTE_F32 / FLUTE_U8, -1 for any other */
    int32_t contiguous;
    int32_t device;          /* ordinal of the GPU that holds it, -1 for host memory */
    int32_t present;         /* 0: no such operand was passed (None) */
    int32_t reserved;
} flute_tensor;

typedef struct flute_operands {
    flute_tensor A, indices, lut, indices2, lut2, resB, resA, bias, signs, awq;
    int64_t K;
    int32_t b1, b2, group_size, rot_block;
    int32_t max_rank;        /* largest residual rank the entry point accepts */
    uint32_t gs_allowed;     /* bit i set: group size 2^i is accepted by the entry point */
} flute_operands;

/* A must be a contiguous 2-D float16/bfloat16 [M, K] with K % 64 == 0 (and M == 1 if need_m1). */
flute_status flute_check_input(const char *who, const flute_tensor *A, int need_m1);
/* Every check of one weight's operands; on success *out is ready for the launch entry points
 * (data pointers as given: re-align misaligned blobs before the call) and *N_out is N. */
flute_status flute_describe_linear(const char *who, const flute_operands *ops, flute_linear *out,
                                   int64_t *N_out);

/* Validate a weight descriptor exactly as the launchers do, without touching
 * the device.  mode: 0 = GEMV (accepts k_group = 128), 1 = GEMM (refuses it). */
flute_status flute_validate(const flute_linear *w, int mode);

/* Release the per-device split-K workspaces (also done at process exit).
 * The workspace (partial sums and tickets of a K split, residual coefficients, a pre-rotated
 * input, the GEMM's operand image) is one per device, shared by every stream (upstream's
 * has a single-stream contract, src/gemv_host.h:31-38).  A call on another stream than the
 * previous user's is ordered behind it with an event, so eager work on two streams stays
 * correct (and serialised); what remains the caller's to order: calls issued at the same
 * moment from two host threads, and streams under capture (no event is inserted there).
 * A call that needs it to grow while its stream is capturing is refused (FLUTE_ERR_INVALID). */
void flute_release_workspaces(void);

/*
 * The launchers read their tuning and test knobs (FLUTE_GEMV_RW, FLUTE_GEMV_WAVES,
 * FLUTE_GEMV_TABLE_LOG2, FLUTE_GEMV_PREROTATE, FLUTE_GEMV4_PF, FLUTE_GEMV_NO_FAST,
 * FLUTE_GEMV4_WALK, FLUTE_GEMM_ROWS, FLUTE_GEMM_NO_PERM, FLUTE_GEMM_KSPLIT,
 * FLUTE_GEMM_NO_DIRECT, FLUTE_GEMM_NO_LEAN, FLUTE_FHT_STEPS) from the environment once per
 * process; this
 * re-reads them.
 */
void flute_reload_tuning(void);

/*
 * What a workspace request does, as pure host arithmetic (usable without a GPU):
 * 0 = the buffers held are large enough, 1 = they grow (hipMalloc), 2 = refused with
 * FLUTE_ERR_INVALID because the stream is being captured into a graph and the buffers
 * would have to grow.  Sizes in elements.
 */
int flute_workspace_decision(int64_t have_floats, int64_t need_floats, int64_t have_ints,
                             int64_t need_ints, int capturing);

/*
 * No upstream counterpart.  The library's own helper that rebuilds a 64-bit address from two
 * 32-bit halves delivered as signed ints (the kernels move wavefront-uniform pointers into
 * scalar registers that way), callable on the host so that it can be checked without a GPU:
 * returns (uint32)lo | (uint32)hi << 32 for every bit pattern, bit 31 of either half included.
 */
uint64_t flute_join_address_halves(int32_t lo, int32_t hi);

/*
 * No upstream counterpart; a measurement aid, not part of the layer.  Reads `bytes` of device
 * memory once and discards them: `workgroups` workgroups of 256 threads, 16-byte non-temporal
 * loads, `loads_in_flight` (2, 4 or 8) per thread, the load pattern of the M = 1 kernel without
 * its table, lookups and sums.  Timed on the bytes of one weight it shows what a single launch of
 * that size can reach on the device.  sink: 4 bytes of device memory (practically never
 * written).
 */
flute_status flute_read_probe(const void *src, int64_t bytes, int workgroups,
                              int loads_in_flight, void *sink, void *stream);

/*
 * No upstream counterpart.  Sixteen hex digits of the SHA-256 over the sources the library was
 * built from (csrc sources and this header, in the Makefile's order), so that a harness that
 * loads a library by path can tell whether it is the tree's current build.
 */
const char *flute_build_id(void);

#ifdef __cplusplus
}
#endif
#endif /* FLUTE_HIP_H */
