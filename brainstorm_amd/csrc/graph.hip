// Recorded steps: a sequence of library calls captured once into a HIP graph and replayed with
// one launch. The workloads this serves issue dozens of small kernels per training step (an MLP
// step is ~70 launches of 2-15 us each), so the host, not the device, sets their pace; a replay
// costs one launch.
//
// Recording uses stream capture of the library's one stream in relaxed mode (pool allocations
// may reach hipMalloc). What a recorded step may contain: every compute entry point, device-to-
// device copies, bship_malloc / bship_free. What it may not: anything that waits for the device
// or touches host memory (bship_sync, bship_h2d, bship_d2h, timers, bship_isfinite_f32,
// bship_fill_gaussian_f32, generator seeding and read-back) - those return BSHIP_ERR_UNSUPPORTED
// while recording. No memset nodes are recorded: the library clears memory with fill kernels.
//
// Memory: pool blocks handed out during the recording are the graph's for its lifetime (pool.hip),
// so temporaries of the recorded calls keep their addresses and are not handed to anyone else.
// Dropout masks: see "masks of recorded steps" in rng.hip.
#include <map>
#include <mutex>

#include "common.h"

namespace bship {

namespace {
struct GraphRec {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};
std::mutex g_graph_mutex;
std::map<int, GraphRec> g_graphs;
int g_next_graph = 1;
std::atomic<int> g_recording{0};   // read by every entry point without the mutex

void destroy_rec(int id, GraphRec& rec) {
    if (rec.exec) (void)hipGraphExecDestroy(rec.exec);
    if (rec.graph) (void)hipGraphDestroy(rec.graph);
    rng_graph_destroyed(id);
    pool_graph_destroyed(id);
}
}  // namespace

bool graph_recording() { return g_recording != 0; }

void graph_release_all() {
    std::lock_guard<std::mutex> lock(g_graph_mutex);
    if (g_recording) {
        hipGraph_t g = nullptr;
        (void)hipStreamEndCapture(ctx().stream, &g);
        if (g) (void)hipGraphDestroy(g);
        pool_graph_end();
        g_recording = 0;
    }
    (void)hipStreamSynchronize(ctx().stream);
    for (auto& kv : g_graphs) destroy_rec(kv.first, kv.second);
    g_graphs.clear();
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_graph_begin(void) {
    BSHIP_REQUIRE_INIT();
    std::lock_guard<std::mutex> lock(g_graph_mutex);
    if (g_recording)
        return set_error(BSHIP_ERR_UNSUPPORTED, "bship_graph_begin: a step is already being recorded");
    const int id = g_next_graph++;
    int st = rng_graph_begin(id);
    if (st != 0) return st;
    st = check_hip(hipStreamBeginCapture(ctx().stream, hipStreamCaptureModeRelaxed), "hipStreamBeginCapture");
    if (st != 0) { rng_graph_destroyed(id); return st; }
    pool_graph_begin(id);
    g_recording = id;
    return 0;
}

int bship_graph_end(int* graph_id) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_PTR(graph_id);
    std::lock_guard<std::mutex> lock(g_graph_mutex);
    if (!g_recording)
        return set_error(BSHIP_ERR_UNSUPPORTED, "bship_graph_end: no step is being recorded");
    const int id = g_recording.load();
    GraphRec rec;
    int st = rng_graph_end(id);
    const hipError_t e = hipStreamEndCapture(ctx().stream, &rec.graph);
    pool_graph_end();
    g_recording = 0;
    if (st == 0) st = check_hip(e, "hipStreamEndCapture");
    if (st == 0 && !rec.graph) st = set_error(BSHIP_ERR_UNSUPPORTED, "bship_graph_end: the recording is empty");
    if (st == 0) st = check_hip(hipGraphInstantiate(&rec.exec, rec.graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    if (st != 0) {
        (void)hipGetLastError();
        destroy_rec(id, rec);
        return st;
    }
    g_graphs[id] = rec;
    *graph_id = id;
    return 0;
}

int bship_graph_launch(int graph_id) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    std::lock_guard<std::mutex> lock(g_graph_mutex);
    auto it = g_graphs.find(graph_id);
    if (it == g_graphs.end())
        return set_error(BSHIP_ERR_BAD_DIMENSION, "bship_graph_launch: no recorded step %d", graph_id);
    int st = rng_graph_before_launch(graph_id);
    if (st != 0) return st;
    st = check_hip(hipGraphLaunch(it->second.exec, ctx().stream), "hipGraphLaunch");
    return st != 0 ? st : rng_graph_after_launch(graph_id);
}

int bship_graph_destroy(int graph_id) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    std::lock_guard<std::mutex> lock(g_graph_mutex);
    auto it = g_graphs.find(graph_id);
    if (it == g_graphs.end())
        return set_error(BSHIP_ERR_BAD_DIMENSION, "bship_graph_destroy: no recorded step %d", graph_id);
    BSHIP_HIP(hipStreamSynchronize(ctx().stream));    // a replay may still be running
    destroy_rec(graph_id, it->second);
    g_graphs.erase(it);
    return 0;
}

}  // extern "C"
