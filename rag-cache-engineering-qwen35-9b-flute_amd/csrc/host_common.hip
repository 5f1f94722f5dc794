// Validation, split policy, workspace and the small identity entry points.
#include "host_common.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <atomic>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace flute {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

static bool aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

flute_status validate_linear(const flute_linear *w, int mode, const char *who) {
    FLUTE_REQUIRE(w != nullptr, FLUTE_ERR_INVALID, "%s: weight descriptor is NULL", who);
    FLUTE_REQUIRE(w->b1 >= 1 && w->b1 <= 4, FLUTE_ERR_INVALID,
                  "%s: bitwidth must be 1, 2, 3 or 4 (got %d)", who, w->b1);
    FLUTE_REQUIRE(w->b2 >= 0 && w->b2 <= 4, FLUTE_ERR_INVALID,
                  "%s: bitwidth2 must be 0 (single stream) or 1..4 (got %d)", who, w->b2);
    FLUTE_REQUIRE(w->K > 0 && w->K % 64 == 0, FLUTE_ERR_INVALID,
                  "%s: K must be a positive multiple of 64, the idxN blob's 64-k tiles (got K=%d)",
                  who, w->K);
    FLUTE_REQUIRE(w->N > 0 && w->N % 128 == 0, FLUTE_ERR_INVALID,
                  "%s: the idxN layout requires N %% 128 == 0 (got N=%d)", who, w->N);
    const int gs = w->group_size;
    FLUTE_REQUIRE(is_pow2(gs) && gs >= 16 && gs <= 2048, FLUTE_ERR_INVALID,
                  "%s: group_size must be one of 16/32/64/128/256/512/1024/2048 (got %d)", who, gs);
    FLUTE_REQUIRE(w->lut_dtype == FLUTE_F16 || w->lut_dtype == FLUTE_BF16, FLUTE_ERR_INVALID,
                  "%s: lut dtype must be float16 or bfloat16", who);
    FLUTE_REQUIRE(w->q1 != nullptr && w->lut1 != nullptr, FLUTE_ERR_INVALID,
                  "%s: stream-1 indices/lut must not be NULL", who);
    const int64_t want1 = (int64_t)w->N * w->K * w->b1 / 8;
    FLUTE_REQUIRE(w->q1_bytes == want1, FLUTE_ERR_INVALID,
                  "%s: stream-1 byte count %lld is not N*K*%d/8 = %lld (N=%d, K=%d)", who,
                  (long long)w->q1_bytes, w->b1, (long long)want1, w->N, w->K);
    FLUTE_REQUIRE(aligned(w->q1, 16), FLUTE_ERR_INVALID,
                  "%s: stream-1 indices must be 16-byte aligned", who);
    FLUTE_REQUIRE(aligned(w->lut1, 2), FLUTE_ERR_INVALID, "%s: lut misaligned", who);
    if (w->k_group != 0) {
        // the LUT grouped along K: [N, K/128, 16]
        FLUTE_REQUIRE((mode & kModeKGroupOk) != 0, FLUTE_ERR_UNSUPPORTED,
                      "%s: a LUT grouped along K (k_group = %d) is served by flute_gemv, "
                      "flute_gemv_noalloc and flute_dequant only", who, w->k_group);
        FLUTE_REQUIRE(w->k_group == 128, FLUTE_ERR_INVALID,
                      "%s: k_group must be 0 (LUT grouped along N) or 128 (got %d)", who, w->k_group);
        FLUTE_REQUIRE(w->b1 == 4 && w->b2 == 0, FLUTE_ERR_UNSUPPORTED,
                      "%s: a LUT grouped along K has one 4-bit stream (got b1=%d, b2=%d)", who, w->b1,
                      w->b2);
        FLUTE_REQUIRE(w->K % 128 == 0, FLUTE_ERR_INVALID,
                      "%s: a LUT grouped along K needs K %% 128 == 0 (got K=%d)", who, w->K);
        const int64_t krows = (int64_t)w->N * (w->K / 128);
        FLUTE_REQUIRE(krows <= INT32_MAX && w->lut_rows == (int32_t)krows, FLUTE_ERR_INVALID,
                      "%s: a LUT grouped along K must be [N, K/128, 16] = %lld rows (got %d)", who,
                      (long long)krows, w->lut_rows);
        FLUTE_REQUIRE(aligned(w->lut1, 16), FLUTE_ERR_INVALID,
                      "%s: a LUT grouped along K must be 16-byte aligned (read 16 bytes at a time)", who);
    } else {
        const int rows = (w->N + gs - 1) / gs;
        FLUTE_REQUIRE(w->lut_rows == rows, FLUTE_ERR_INVALID,
                      "%s: lut must be [ceil(N/group_size), 2^bitwidth] = [%d, %d] (got %d rows)", who,
                      rows, 1 << w->b1, w->lut_rows);
    }
    if (w->b2 > 0) {
        FLUTE_REQUIRE(w->q2 != nullptr && w->lut2 != nullptr, FLUTE_ERR_INVALID,
                      "%s: a second stream needs both indices2 and lut2", who);
        const int64_t want2 = (int64_t)w->N * w->K * w->b2 / 8;
        FLUTE_REQUIRE(w->q2_bytes == want2, FLUTE_ERR_INVALID,
                      "%s: stream-2 byte count %lld != N*K*%d/8 = %lld", who,
                      (long long)w->q2_bytes, w->b2, (long long)want2);
        FLUTE_REQUIRE(aligned(w->q2, 16), FLUTE_ERR_INVALID,
                      "%s: stream-2 indices must be 16-byte aligned", who);
    }
    // Operands the kernels read element by element still have to sit on an element boundary
    // (16-bit values on 2 bytes, fp32 on 4): an odd address is refused here rather than met
    // by a load in the kernel.
    FLUTE_REQUIRE(w->b2 == 0 || aligned(w->lut2, 2), FLUTE_ERR_INVALID, "%s: lut2 misaligned", who);
    FLUTE_REQUIRE(aligned(w->resA, 2) && aligned(w->resB, 2), FLUTE_ERR_INVALID,
                  "%s: resA and resB must be 2-byte aligned", who);
    FLUTE_REQUIRE(aligned(w->bias, 2), FLUTE_ERR_INVALID, "%s: bias must be 2-byte aligned", who);
    FLUTE_REQUIRE(aligned(w->signs, 4) && aligned(w->awq, 4), FLUTE_ERR_INVALID,
                  "%s: rotation signs and awq scale are fp32 and must be 4-byte aligned", who);
    FLUTE_REQUIRE((w->resA != nullptr) == (w->resB != nullptr), FLUTE_ERR_INVALID,
                  "%s: resB and resA must be supplied together", who);
    FLUTE_REQUIRE((w->resA != nullptr) == (w->R > 0), FLUTE_ERR_INVALID,
                  "%s: residual rank %d does not match the residual pointers", who, w->R);
    FLUTE_REQUIRE(w->R >= 0 && w->R <= 256, FLUTE_ERR_INVALID,
                  "%s: residual rank must be 0..256 (got R=%d)", who, w->R);
    FLUTE_REQUIRE(w->awq == nullptr || w->signs != nullptr, FLUTE_ERR_INVALID,
                  "%s: awq scale only exists as a companion to the rotation signs", who);
    if (w->signs != nullptr) {
        FLUTE_REQUIRE(w->K % 32 == 0 && w->K >= 32 && w->K <= 65504, FLUTE_ERR_INVALID,
                      "%s: rotation needs K %% 32 == 0 and 32 <= K <= 65504 (got %d)", who, w->K);
        (void)mode;
        const Segs sg = make_segments(w->K, w->rot_block);
        FLUTE_REQUIRE(sg.len[0] <= 16384, FLUTE_ERR_UNSUPPORTED,
                      "%s: rotation segment %d exceeds 16384 columns", who, sg.len[0]);
    }
    return FLUTE_OK;
}

struct Workspace {
    float *P = nullptr;
    int *tickets = nullptr;
    size_t floats = 0;
    size_t ints = 0;
    // The stream of the last call that took the workspace (compared, never dereferenced: the
    // caller may have destroyed it since), and the event that call recorded behind its launches
    // for a call on another stream to wait on.  Events are only recorded once a second stream
    // has been seen (`shared`), so single-stream use pays nothing.
    hipStream_t last_stream = nullptr;
    bool used = false;
    bool shared = false;
    bool recorded = false;
    hipEvent_t handover = nullptr;
};

static std::mutex g_ws_mu;
static std::unordered_map<int, Workspace> g_ws;
static std::vector<void *> g_retired;   // outgrown buffers, freed at release

int workspace_decision(size_t have_floats, size_t need_floats, size_t have_ints, size_t need_ints,
                       bool capturing) {
    if (have_floats >= need_floats && have_ints >= need_ints) return 0;
    return capturing ? 2 : 1;
}

flute_status get_workspace(size_t floats, size_t ints, hipStream_t stream, float **P,
                           int **tickets) {
    int dev = 0;
    FLUTE_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> guard(g_ws_mu);
    Workspace &ws = g_ws[dev];
    if (ws.floats < floats || ws.ints < ints) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        FLUTE_HIP_CHECK(hipStreamIsCapturing(stream, &cap));
        if (workspace_decision(ws.floats, floats, ws.ints, ints,
                               cap != hipStreamCaptureStatusNone) == 2) {
            set_error("workspace: this call needs %zu B of partial sums and %zu tickets, more than the "
                      "%zu B / %zu held, and the stream is being captured: an allocation cannot be "
                      "part of a graph. Run the same call once outside the capture first",
                      floats * sizeof(float), ints, ws.floats * sizeof(float), ws.ints);
            return FLUTE_ERR_INVALID;
        }
    }
    if (ws.floats < floats) {
        size_t want = ws.floats ? ws.floats : (size_t)1 << 20;
        while (want < floats) want *= 2;
        float *fresh = nullptr;
        if (hipMalloc((void **)&fresh, want * sizeof(float)) != hipSuccess) {
            set_error("split-K workspace: hipMalloc of %zu bytes failed", want * sizeof(float));
            return FLUTE_ERR_NOMEM;
        }
        if (ws.P) g_retired.push_back(ws.P);       // kernels in flight may still read it
        ws.P = fresh;
        ws.floats = want;
    }
    if (ws.ints < ints) {
        size_t want = ws.ints ? ws.ints : (size_t)1 << 14;
        while (want < ints) want *= 2;
        int *fresh = nullptr;
        if (hipMalloc((void **)&fresh, want * sizeof(int)) != hipSuccess) {
            set_error("split-K workspace: hipMalloc of %zu bytes failed", want * sizeof(int));
            return FLUTE_ERR_NOMEM;
        }
        FLUTE_HIP_CHECK(hipMemsetAsync(fresh, 0, want * sizeof(int), stream));
        if (ws.tickets) g_retired.push_back(ws.tickets);
        ws.tickets = fresh;
        ws.ints = want;
    }
    // One workspace serves every stream of the device.  A call on another stream than the last
    // one is ordered behind it: it waits on the event the earlier call recorded at its end
    // (workspace_done).  The earlier stream's handle is not touched (it may be gone).  The first
    // change of stream finds no event yet and waits for the device once.  Calls that really
    // overlap (two host threads at once) and streams under capture (an event recorded outside
    // a capture cannot join it) remain the caller's to order.
    if (ws.used && ws.last_stream != stream) {
        hipStreamCaptureStatus mine = hipStreamCaptureStatusNone;
        FLUTE_HIP_CHECK(hipStreamIsCapturing(stream, &mine));
        if (mine == hipStreamCaptureStatusNone) {
            if (ws.recorded)
                FLUTE_HIP_CHECK(hipStreamWaitEvent(stream, ws.handover, 0));
            else
                FLUTE_HIP_CHECK(hipDeviceSynchronize());
        }
        ws.shared = true;
    }
    ws.last_stream = stream;
    ws.used = true;
    *P = ws.P;
    *tickets = ws.tickets;
    return FLUTE_OK;
}

void workspace_done(hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> guard(g_ws_mu);
    auto it = g_ws.find(dev);
    if (it == g_ws.end() || !it->second.shared) return;
    Workspace &ws = it->second;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
        ws.recorded = false;       // nothing a later stream could wait on: it synchronises instead
        return;
    }
    if (!ws.handover && hipEventCreateWithFlags(&ws.handover, hipEventDisableTiming) != hipSuccess) {
        ws.handover = nullptr;
        ws.recorded = false;
        return;
    }
    ws.recorded = hipEventRecord(ws.handover, stream) == hipSuccess;
}

static Tuning g_tuning;
static std::atomic<bool> g_tuning_ready{false};
static std::mutex g_tuning_mu;

static int env_or(const char *name, int fallback) {
    const char *e = std::getenv(name);
    if (!e || !*e) return fallback;
    return std::atoi(e);
}

static void read_tuning() {
    Tuning t;
    t.gemv_rw = env_or("FLUTE_GEMV_RW", 0);
    t.gemv_waves = env_or("FLUTE_GEMV_WAVES", 0);
    t.gemv_table_log2 = env_or("FLUTE_GEMV_TABLE_LOG2", 0);
    t.gemv_prerotate = env_or("FLUTE_GEMV_PREROTATE", 0);
    t.gemv4_pf = env_or("FLUTE_GEMV4_PF", 0);
    t.gemv_no_fast = env_or("FLUTE_GEMV_NO_FAST", 0);
    t.gemv4_walk = env_or("FLUTE_GEMV4_WALK", -1);
    t.gemv_xcd = env_or("FLUTE_GEMV_XCD", 1);
    t.gemm_rows = env_or("FLUTE_GEMM_ROWS", 0);
    t.gemm_no_perm = std::getenv("FLUTE_GEMM_NO_PERM") != nullptr;
    t.gemm_ksplit = env_or("FLUTE_GEMM_KSPLIT", 0);
    t.gemm_no_direct = std::getenv("FLUTE_GEMM_NO_DIRECT") != nullptr;
    t.gemm_no_lean = std::getenv("FLUTE_GEMM_NO_LEAN") != nullptr;
    t.gemm_no_balance = std::getenv("FLUTE_GEMM_NO_BALANCE") != nullptr;
    t.gemm_no_handover = std::getenv("FLUTE_GEMM_NO_HANDOVER") != nullptr;
    t.fht_steps = env_or("FLUTE_FHT_STEPS", -1);
    g_tuning = t;
}

const Tuning &tuning() {
    if (!g_tuning_ready.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> guard(g_tuning_mu);
        if (!g_tuning_ready.load(std::memory_order_relaxed)) {
            read_tuning();
            g_tuning_ready.store(true, std::memory_order_release);
        }
    }
    return g_tuning;
}

}  // namespace flute

extern "C" {

int flute_abi_version(void) { return 2; }

const char *flute_last_error(void) { return flute::g_error; }

const char *flute_target_arch(void) { return "gfx950"; }

flute_status flute_validate(const flute_linear *w, int mode) {
    // (mode 0, the GEMV, serves a LUT grouped along K; the GEMM does not)
    return flute::validate_linear(w, mode == 0 ? flute::kModeKGroupOk : (mode & 0xff), "flute_validate");
}

void flute_reload_tuning(void) {
    std::lock_guard<std::mutex> guard(flute::g_tuning_mu);
    flute::read_tuning();
    flute::g_tuning_ready.store(true, std::memory_order_release);
}

int flute_workspace_decision(int64_t have_floats, int64_t need_floats, int64_t have_ints,
                             int64_t need_ints, int capturing) {
    return flute::workspace_decision((size_t)have_floats, (size_t)need_floats, (size_t)have_ints,
                                     (size_t)need_ints, capturing != 0);
}

void flute_release_workspaces(void) {
    std::lock_guard<std::mutex> guard(flute::g_ws_mu);
    for (auto &kv : flute::g_ws) {
        if (kv.second.P) (void)hipFree(kv.second.P);
        if (kv.second.tickets) (void)hipFree(kv.second.tickets);
        if (kv.second.handover) (void)hipEventDestroy(kv.second.handover);
    }
    flute::g_ws.clear();
    for (void *p : flute::g_retired) (void)hipFree(p);
    flute::g_retired.clear();
}

}  // extern "C"

extern "C" uint64_t flute_join_address_halves(int32_t lo, int32_t hi) {
    return flute::join_address_halves(lo, hi);
}

#ifndef FLUTE_BUILD_ID
#define FLUTE_BUILD_ID "unknown"
#endif
extern "C" const char *flute_build_id(void) { return FLUTE_BUILD_ID; }
