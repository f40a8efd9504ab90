// The fusing window behind the public entry points (matcher and patterns: window_core.h).
//
// Operations enter through window_push() from the entry points that take part (elementwise,
// matrix-vector, fill, dense sums, softmax, one-hot, gather, dense masks). What the matcher lets go
// is enqueued through the same public entry points, with t_window_emitting set so that they
// launch instead of coming back; a complete sequence is enqueued through the fused entry point
// that computes it. One mutex serialises the queue; the reference drives a handler from one
// thread (two threads on one stream have no order to preserve anyway).
#include <mutex>

#include "window.h"
#include "window_sink.h"

namespace bship {

std::atomic<int> g_window_on{0};
std::atomic<int> g_window_held{0};
thread_local bool t_window_emitting = false;

namespace {

using namespace window;

std::mutex g_window_mutex;
Matcher g_matcher;

struct Emitting {
    Emitting() { t_window_emitting = true; }
    ~Emitting() { t_window_emitting = false; }
};

}  // namespace

int window_push(const window::Rec& r) {
    std::lock_guard<std::mutex> lock(g_window_mutex);
    Emitting guard;
    DeviceSink sink;
    const int st = g_matcher.push(r, sink);
    g_window_held.store(g_matcher.held(), std::memory_order_relaxed);
    return st;
}

void window_other_work() {
    // an entry point that does not go through the window is about to enqueue something: it may write the arrays
    // that the packed copy of the last backward step's gate deltas mirrors (mode "stacked")
    std::lock_guard<std::mutex> lock(g_window_mutex);
    window::packed_deltas().forget();
}

int window_flush() {
    std::lock_guard<std::mutex> lock(g_window_mutex);
    Emitting guard;
    DeviceSink sink;
    const int st = g_matcher.flush(sink);
    g_window_held.store(g_matcher.held(), std::memory_order_relaxed);
    return st;
}

int window_note_free(const void* p, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_window_mutex);
    Emitting guard;
    DeviceSink sink;
    const int st = g_matcher.note_free(p, bytes, sink);
    g_window_held.store(g_matcher.held(), std::memory_order_relaxed);
    return st;
}

int window_before_product(const void* const* rd, const size_t* rd_len, int nrd, const void* const* wr,
                          const size_t* wr_len, int nwr) {
    std::lock_guard<std::mutex> lock(g_window_mutex);
    if (g_matcher.held() == 0) return 0;
    if (g_matcher.independent(reinterpret_cast<const char* const*>(rd), rd_len, nrd,
                              reinterpret_cast<const char* const*>(wr), wr_len, nwr)) {
        g_matcher.count_overtaken();
        return 0;
    }
    Emitting guard;
    DeviceSink sink;
    const int st = g_matcher.flush(sink);
    g_window_held.store(g_matcher.held(), std::memory_order_relaxed);
    return st;
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_fusing_set(int mode) {
    BSHIP_REQUIRE_INIT();          // what is held is enqueued before the mode changes
    BSHIP_REQUIRE_DIM(mode >= 0 && mode <= 2);
    std::lock_guard<std::mutex> lock(g_window_mutex);
    g_matcher.set_stacked(mode == 2);
    if (mode != 2) window::packed_deltas().release();
    g_window_on.store(mode, std::memory_order_relaxed);
    return 0;
}

int bship_fusing_get(int* on_host) {
    BSHIP_REQUIRE_PTR(on_host);
    *on_host = g_window_on.load(std::memory_order_relaxed);
    return 0;
}

int bship_fusing_flush(void) {
    BSHIP_REQUIRE_INIT();
    return 0;
}

int bship_fusing_stats(unsigned long long* calls, unsigned long long* unfused, unsigned long long* fused_calls,
                       unsigned long long* fused_launches, unsigned long long* overtaken, int reset) {
    std::lock_guard<std::mutex> lock(g_window_mutex);
    const window::Stats& s = g_matcher.stats();
    if (calls) *calls = s.calls;
    if (unfused) *unfused = s.unfused;
    if (fused_calls) *fused_calls = s.fused_calls;
    if (fused_launches) *fused_launches = s.fused;
    if (overtaken) *overtaken = s.overtaken;
    if (reset) g_matcher.reset_stats();
    return 0;
}

}  // extern "C"
