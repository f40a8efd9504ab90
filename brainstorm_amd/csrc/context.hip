// Library lifecycle, error state and stream timers.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "common.h"

namespace bship {

static Context g_ctx;
static std::mutex g_ctx_mutex;
static thread_local char t_error[512] = {0};

Context& ctx() { return g_ctx; }

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_error, sizeof(t_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    return set_error(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return check_hip(e, what);
    if (g_ctx.debug_sync && !graph_recording()) return check_hip(hipStreamSynchronize(g_ctx.stream), what);
    return 0;
}

void graph_release_all();  // graph.hip
void pool_release_all();   // pool.hip
void rng_release();        // rng.hip
void gemm_release();       // gemm.hip
int reduce_scratch_init(int device);   // reduce.hip

}  // namespace bship

using namespace bship;

extern "C" {

int bship_version(void) { return BSHIP_VERSION; }

const char* bship_last_error(void) { return t_error; }

int bship_init(int device) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    if (g_ctx.inited) {
        if (g_ctx.device == device) return 0;
        return set_error(BSHIP_ERR_UNSUPPORTED,
                         "bship_init: already initialised on device %d (asked for %d); "
                         "call bship_shutdown() first", g_ctx.device, device);
    }
    int count = 0;
    BSHIP_HIP(hipGetDeviceCount(&count));
    if (device < 0 || device >= count)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "bship_init: device %d not in [0,%d)",
                         device, count);
    BSHIP_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    BSHIP_HIP(hipGetDeviceProperties(&prop, device));
    g_ctx.num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    snprintf(g_ctx.name, sizeof(g_ctx.name), "%s (%s)", prop.name, prop.gcnArchName);
    // One stream at the default priority; every kernel and copy goes here in call order.
    BSHIP_HIP(hipStreamCreateWithFlags(&g_ctx.stream, hipStreamNonBlocking));
    {
        // device address of the static partial-sum buffer of bship_sum_noalloc_f32, once per device
        int st = reduce_scratch_init(device);
        if (st != 0) {
            (void)hipStreamDestroy(g_ctx.stream);
            g_ctx.stream = nullptr;
            return st;
        }
    }
    const char* dbg = getenv("BSHIP_DEBUG_SYNC");
    g_ctx.debug_sync = dbg && dbg[0] && dbg[0] != '0';
    const char* bpc = getenv("BSHIP_BLOCKS_PER_CU");
    if (bpc && atoi(bpc) > 0 && atoi(bpc) <= 64) g_ctx.blocks_per_cu = atoi(bpc);
    const char* cpc = getenv("BSHIP_COLSUM_BLOCKS_PER_CU");
    if (cpc && atoi(cpc) > 0 && atoi(cpc) <= 64) g_ctx.colsum_blocks_per_cu = atoi(cpc);
    const char* wtm = getenv("BSHIP_WRITE_THROUGH_MIN");
    if (wtm && wtm[0]) g_ctx.write_through_min = static_cast<size_t>(strtoull(wtm, nullptr, 10));
    const char* stm = getenv("BSHIP_STORE_THROUGH_MIN");
    if (stm && stm[0]) g_ctx.store_through_min = static_cast<size_t>(strtoull(stm, nullptr, 10));
    const char* stx = getenv("BSHIP_STORE_THROUGH_MAX");
    if (stx && stx[0]) g_ctx.store_through_max = static_cast<size_t>(strtoull(stx, nullptr, 10));
    const char* smk = getenv("BSHIP_SM_CHUNK_KB");
    if (smk && smk[0]) g_ctx.softmax_run_bytes = static_cast<size_t>(strtoull(smk, nullptr, 10)) << 10;
    const char* erk = getenv("BSHIP_EW_RUN_KB");
    if (erk && erk[0]) g_ctx.ew_run_bytes = static_cast<size_t>(strtoull(erk, nullptr, 10)) << 10;
    const char* csm = getenv("BSHIP_COL2IM_STREAM_MIN");
    if (csm && csm[0]) g_ctx.col2im_stream_min_images_per_cu = static_cast<int64_t>(strtoll(csm, nullptr, 10));
    g_ctx.device = device;
    g_ctx.inited = true;
    return 0;
}

int bship_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    if (!g_ctx.inited) return 0;
    (void)window_flush();
    (void)flush_deferred_fills();
    g_window_on.store(0);
    graph_release_all();
    (void)hipStreamSynchronize(g_ctx.stream);
    gemm_release();
    rng_release();
    pool_release_all();
    for (hipEvent_t e : g_ctx.events)
        if (e) (void)hipEventDestroy(e);
    (void)hipStreamDestroy(g_ctx.stream);
    g_ctx = Context();
    return 0;
}

int bship_sync(void) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    BSHIP_HIP(hipStreamSynchronize(g_ctx.stream));
    return 0;
}

int bship_device_info(char* name_host, size_t name_len, int* compute_units) {
    BSHIP_REQUIRE_INIT();
    if (name_host && name_len) {
        strncpy(name_host, g_ctx.name, name_len - 1);
        name_host[name_len - 1] = 0;
    }
    if (compute_units) *compute_units = g_ctx.num_cus;
    return 0;
}

int bship_event_record(int slot) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(slot >= 0 && slot < BSHIP_MAX_EVENTS);
    BSHIP_REQUIRE_EAGER();
    if (!g_ctx.events[slot]) BSHIP_HIP(hipEventCreate(&g_ctx.events[slot]));
    BSHIP_HIP(hipEventRecord(g_ctx.events[slot], g_ctx.stream));
    return 0;
}

int bship_event_elapsed_ms(int start_slot, int stop_slot, float* ms_host) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_PTR(ms_host);
    BSHIP_REQUIRE_EAGER();
    BSHIP_REQUIRE_DIM(start_slot >= 0 && start_slot < BSHIP_MAX_EVENTS);
    BSHIP_REQUIRE_DIM(stop_slot >= 0 && stop_slot < BSHIP_MAX_EVENTS);
    if (!g_ctx.events[start_slot] || !g_ctx.events[stop_slot])
        return set_error(BSHIP_ERR_BAD_DIMENSION, "bship_event_elapsed_ms: slot never recorded");
    BSHIP_HIP(hipEventSynchronize(g_ctx.events[stop_slot]));
    BSHIP_HIP(hipEventElapsedTime(ms_host, g_ctx.events[start_slot], g_ctx.events[stop_slot]));
    return 0;
}

}  // extern "C"
