// Caching device-memory pool, host<->device copies, copy_to and fill.
//
// The pool never returns memory to the driver while the library is in use:
// freed blocks go to a per-size free list and are handed out again. Because
// every kernel runs on the one library stream, a block that is reused is
// touched by its new owner only after all work of the previous owner.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.h"
#include "window.h"

namespace bship {

namespace {
std::mutex g_pool_mutex;
std::map<size_t, std::vector<void*>> g_free;       // rounded size -> cached blocks
std::unordered_map<void*, size_t> g_live;          // handed-out block -> rounded size
size_t g_in_use = 0, g_cached = 0, g_device_allocs = 0;
int g_recording_graph = 0;                          // graph whose step is being recorded, or 0
std::unordered_map<void*, int> g_graph_owner;      // block handed out during a recording -> graph
struct Parked { size_t size; int graph; };
std::unordered_map<void*, Parked> g_parked;        // such blocks after their owner freed them

size_t round_size(size_t n) {
    size_t q = n < (64u << 10) ? 256 : (n < (1u << 20) ? 4096 : (2u << 20));
    return (n + q - 1) / q * q;
}

size_t pool_limit() {
    const char* s = getenv("BSHIP_POOL_LIMIT_BYTES");
    return s && s[0] ? static_cast<size_t>(strtoull(s, nullptr, 10)) : 0;
}

void trim_locked() {
    for (auto& kv : g_free)
        for (void* p : kv.second) (void)hipFree(p);
    g_free.clear();
    g_cached = 0;
}
}  // namespace

// Pinned host memory for small read-backs (bship_d2h).
constexpr size_t kBounceBytes = 64u << 10;
static void* g_bounce = nullptr;
static void* g_bounce_dev = nullptr;
static std::mutex g_bounce_mutex;
static unsigned g_bounce_seq = 0;              // number of the last polled read-back (behind the buffer)
static bool g_bounce_failed = false;           // coherent pinned memory could not be had: ordinary copies

int pool_alloc_raw(size_t nbytes, void** out) {
    *out = nullptr;
    if (nbytes == 0) return 0;
    size_t sz = round_size(nbytes);
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    auto it = g_free.find(sz);
    if (it != g_free.end() && !it->second.empty()) {
        *out = it->second.back();
        it->second.pop_back();
        g_cached -= sz;
    } else {
        size_t limit = pool_limit();
        if (g_recording_graph && limit && g_in_use + g_cached + sz > limit)
            return set_error(BSHIP_ERR_OUT_OF_MEMORY, "pool limit of %zu bytes reached while a step is being recorded", limit);
        if (limit && g_in_use + g_cached + sz > limit) {
            // Give cached blocks back before refusing.
            (void)hipStreamSynchronize(ctx().stream);
            trim_locked();
            if (g_in_use + sz > limit)
                return set_error(BSHIP_ERR_OUT_OF_MEMORY,
                                 "pool limit of %zu bytes reached (in use %zu, asked %zu)",
                                 limit, g_in_use, sz);
        }
        hipError_t e = hipMalloc(out, sz);
        if (e != hipSuccess && g_recording_graph) {
            (void)hipGetLastError();
            *out = nullptr;
            return set_error(BSHIP_ERR_OUT_OF_MEMORY, "hipMalloc of %zu bytes failed while a step is being recorded: %s",
                             sz, hipGetErrorString(e));
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            (void)hipStreamSynchronize(ctx().stream);
            trim_locked();
            e = hipMalloc(out, sz);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                *out = nullptr;
                return set_error(BSHIP_ERR_OUT_OF_MEMORY,
                                 "hipMalloc of %zu bytes failed: %s (in use %zu)", sz,
                                 hipGetErrorString(e), g_in_use);
            }
        }
        ++g_device_allocs;
    }
    g_live[*out] = sz;
    g_in_use += sz;
    if (g_recording_graph) g_graph_owner[*out] = g_recording_graph;
    return 0;
}

int pool_free_raw(void* p) {
    if (!p) return 0;
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    auto it = g_live.find(p);
    if (it == g_live.end())
        return set_error(BSHIP_ERR_BAD_POINTER, "bship_free: %p was not allocated by the pool", p);
    size_t sz = it->second;
    g_live.erase(it);
    auto owner = g_graph_owner.find(p);
    if (owner != g_graph_owner.end()) {
        // a recorded step uses this block on every replay: keep it out of circulation
        g_parked[p] = Parked{sz, owner->second};
        g_graph_owner.erase(owner);
        return 0;
    }
    g_in_use -= sz;
    g_free[sz].push_back(p);
    g_cached += sz;
    return 0;
}

void pool_graph_begin(int id) {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    g_recording_graph = id;
}

void pool_graph_end() {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    g_recording_graph = 0;
}

void pool_graph_destroyed(int id) {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    for (auto it = g_parked.begin(); it != g_parked.end();) {
        if (it->second.graph == id) {
            g_in_use -= it->second.size;
            g_free[it->second.size].push_back(it->first);
            g_cached += it->second.size;
            it = g_parked.erase(it);
        } else {
            ++it;
        }
    }
    for (auto it = g_graph_owner.begin(); it != g_graph_owner.end();)
        it = it->second == id ? g_graph_owner.erase(it) : std::next(it);
}

void pool_release_all() {
    {
        std::lock_guard<std::mutex> block(g_bounce_mutex);
        if (g_bounce) (void)hipHostFree(g_bounce);
        g_bounce = g_bounce_dev = nullptr;
        g_bounce_failed = false;
    }
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    trim_locked();
    for (auto& kv : g_live) (void)hipFree(kv.first);
    g_live.clear();
    for (auto& kv : g_parked) (void)hipFree(kv.first);
    g_parked.clear();
    g_graph_owner.clear();
    g_recording_graph = 0;
    g_in_use = 0;
    g_device_allocs = 0;
}

// ------------------------------- kernels ----------------------------------

// One workgroup per tile of kBlock*4 floats, one 128-bit access per lane.
constexpr size_t kCopyTile = static_cast<size_t>(kBlock) * 4;

// WT: write-through stores (large arrays); otherwise AL selects the aligned non-temporal store.
template <bool AL, bool WT>
__global__ __launch_bounds__(kBlock) void fill_kernel(float* __restrict__ p, float val, size_t n) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) * 4;
    if (i + 4 <= n) {
        const f4 vv = {val, val, val, val};
        if constexpr (WT) vstore_writeonly<4>(p + i, vv);
        else vstore<4, AL>(p + i, vv);
    } else {
        for (size_t j = i; j < n; ++j) p[j] = val;
    }
}

template <bool AL>
__global__ __launch_bounds__(kBlock) void copy_kernel(const float* __restrict__ s,
                                                      float* __restrict__ d, size_t n, bool through) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) * 4;
    if (i + 4 <= n) {
        vstore<4, AL>(d + i, vload<4, AL>(s + i), through);
    } else {
        for (size_t j = i; j < n; ++j) d[j] = s[j];
    }
}

// dst(rows, cols) with row pitch ld_dst = src(rows, cols) with row pitch ld_src; pitches in
// elements. 2^L lanes share a row (the power of two that covers its 128-bit accesses, 256 at
// most), so a workgroup covers 2^(8-L) rows x one tile of 2^L accesses. Rows of a pitched view
// start anywhere: the accesses promise 4-byte alignment only.
__global__ __launch_bounds__(kBlock) void copy2d_kernel(const float* __restrict__ src, int64_t ld_src,
                                                        float* __restrict__ dst, int64_t ld_dst, int64_t rows,
                                                        int64_t cols, unsigned tiles_per_row, int L, bool through) {
    const int64_t row = (static_cast<int64_t>(blockIdx.x / tiles_per_row) << (8 - L)) + (threadIdx.x >> L);
    const int64_t c = ((static_cast<int64_t>(blockIdx.x % tiles_per_row) << L) + (threadIdx.x & ((1u << L) - 1))) * 4;
    if (row >= rows || c >= cols) return;
    const float* s = src + row * ld_src + c;
    float* d = dst + row * ld_dst + c;
    if (c + 4 <= cols) {
        vstore<4, false>(d, vload<4, false>(s), through);
    } else {
        for (int64_t j = 0; c + j < cols; ++j) d[j] = s[j];
    }
}

// Copy of up to kBlock*4 floats by one workgroup (to or from pinned host memory), followed by a
// sequence number the host polls for: the copy is complete and visible before the number is.
__global__ __launch_bounds__(kBlock) void readback_kernel(const float* __restrict__ src, float* dst, size_t n,
                                                          unsigned* flag, unsigned seq) {
    for (size_t i = threadIdx.x; i < n; i += kBlock) dst[i] = src[i];
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) {
        __atomic_store_n(flag, seq, __ATOMIC_RELEASE);
    }
}

int launch_fill(float* p, float val, size_t n) {
    if (n == 0) return 0;
    const size_t tiles = (n + kCopyTile - 1) / kCopyTile;
    if (tiles > 0x7fffffffu) return set_error(BSHIP_ERR_BAD_DIMENSION, "fill: %zu elements exceed one launch", n);
    const dim3 grid(static_cast<unsigned>(tiles));
    if (n >= ctx().write_through_min)
        hipLaunchKernelGGL((fill_kernel<false, true>), grid, dim3(kBlock), 0, ctx().stream, p, val, n);
    else if (aligned16(p))
        hipLaunchKernelGGL((fill_kernel<true, false>), grid, dim3(kBlock), 0, ctx().stream, p, val, n);
    else
        hipLaunchKernelGGL((fill_kernel<false, false>), grid, dim3(kBlock), 0, ctx().stream, p, val, n);
    return check_launch("fill_kernel");
}

// ------------------------------ deferred fills ------------------------------
// A training step clears a dozen small buffers in a row (BufferManager.clear_backward_buffers,
// buffers.py:147-150: one fill per backward-only hub), each a launch of a few microseconds that
// costs more to issue than to run. Fills of up to kDeferredFillMax elements are therefore only
// noted; the next entry point of any kind (BSHIP_REQUIRE_INIT), or a full list, enqueues all
// noted fills as ONE launch (grid.y = fill). Fills that overlap a noted one are enqueued in
// order: the noted ones go first.
constexpr int kMaxDeferredFills = 16;
constexpr size_t kDeferredFillMax = size_t(1) << 18;      // 1 MiB
struct DeferredFill { float* p; size_t n; float val; };
struct DeferredFills { DeferredFill f[kMaxDeferredFills]; };
static DeferredFills g_deferred;
std::atomic<int> g_deferred_fill_count{0};
static std::mutex g_deferred_mutex;

__global__ __launch_bounds__(kBlock) void multi_fill_kernel(DeferredFills d) {
    const DeferredFill f = d.f[blockIdx.y];
    const size_t i = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) * 4;
    if (i >= f.n) return;
    if (i + 4 <= f.n && (reinterpret_cast<uintptr_t>(f.p + i) & 15u) == 0) {
        *reinterpret_cast<f4*>(f.p + i) = f4{f.val, f.val, f.val, f.val};
    } else {
        for (size_t j = i; j < f.n && j < i + 4; ++j) f.p[j] = f.val;
    }
}

static int flush_deferred_locked() {
    if (g_deferred_fill_count == 0) return 0;
    size_t most = 0;
    const int count = g_deferred_fill_count.load();
    for (int k = 0; k < count; ++k) most = g_deferred.f[k].n > most ? g_deferred.f[k].n : most;
    const dim3 grid(static_cast<unsigned>((most + kCopyTile - 1) / kCopyTile), static_cast<unsigned>(count));
    g_deferred_fill_count = 0;
    hipLaunchKernelGGL(multi_fill_kernel, grid, dim3(kBlock), 0, ctx().stream, g_deferred);
    return check_launch("multi_fill_kernel");
}

int flush_deferred_fills() {
    std::lock_guard<std::mutex> lock(g_deferred_mutex);
    return flush_deferred_locked();
}

// Notes mem[0:n] = val for the next flush (n <= kDeferredFillMax).
static int defer_fill(float* mem, float val, size_t n) {
    std::lock_guard<std::mutex> lock(g_deferred_mutex);
    bool overlaps = false;
    for (int k = 0, count = g_deferred_fill_count.load(); k < count; ++k) {
        const DeferredFill& f = g_deferred.f[k];
        overlaps = overlaps || (mem < f.p + f.n && f.p < mem + n);
    }
    if (overlaps || g_deferred_fill_count == kMaxDeferredFills) {
        int st = flush_deferred_locked();
        if (st != 0) return st;
    }
    const int slot = g_deferred_fill_count.load();
    g_deferred.f[slot] = DeferredFill{mem, n, val};
    g_deferred_fill_count = slot + 1;
    return 0;
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_malloc(size_t nbytes, void** out) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_PTR(out);
    int st = pool_alloc_raw(nbytes, out);
    if (st != 0 || *out == nullptr) return st;
    // Blocks are rounded to a multiple of 256 bytes, so clearing whole floats covers nbytes. Small
    // blocks (a layer's vector-sized temporaries) are cleared with the noted fills: every launch
    // enqueues those first.
    const size_t n = (nbytes + 3) / 4;
    if (n <= kDeferredFillMax) return defer_fill(static_cast<float*>(*out), 0.0f, n);
    return launch_fill(static_cast<float*>(*out), 0.0f, n);
}

int bship_malloc_scratch(size_t nbytes, void** out) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_PTR(out);
    return pool_alloc_raw(nbytes, out);
}

int bship_free(void* p) {
    BSHIP_REQUIRE_INIT_NO_FLUSH();
    // Operations that the fusing window holds may still name this block: they are enqueued before
    // anything a later owner does (bship_malloc enqueues what is held first), and a layer's
    // sequence that only waits for its temporaries to be dropped is completed by this very call.
    if (p && g_window_held.load(std::memory_order_relaxed) != 0 && !t_window_emitting) {
        size_t bytes = 0;
        {
            std::lock_guard<std::mutex> lock(g_pool_mutex);
            auto it = g_live.find(p);
            if (it != g_live.end()) bytes = it->second;
        }
        if (bytes) {
            int st = window_note_free(p, bytes);
            if (st != 0) { (void)pool_free_raw(p); return st; }
        }
    }
    return pool_free_raw(p);
}

int bship_pool_trim(void) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    BSHIP_HIP(hipStreamSynchronize(ctx().stream));
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    trim_locked();
    return 0;
}

int bship_pool_stats(size_t* bytes_in_use, size_t* bytes_cached, size_t* device_allocations) {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    if (bytes_in_use) *bytes_in_use = g_in_use;
    if (bytes_cached) *bytes_cached = g_cached;
    if (device_allocations) *device_allocations = g_device_allocs;
    return 0;
}

// Pinned host memory for small transfers, allocated on first use (the caller holds g_bounce_mutex).
// Coherent (fine-grained) memory, asked for explicitly: the host polls a sequence number that a
// running kernel writes behind its data, which needs the kernel's system-scope release to be visible
// to the host while the kernel runs; with the default flag that depends on the environment. If such
// memory cannot be had, small transfers take the runtime's ordinary copies.
static bool bounce_ready() {
    if (g_bounce) return true;
    if (g_bounce_failed) return false;
    if (hipHostMalloc(&g_bounce, kBounceBytes + 64, hipHostMallocCoherent | hipHostMallocMapped) != hipSuccess ||
        hipHostGetDevicePointer(&g_bounce_dev, g_bounce, 0) != hipSuccess) {
        (void)hipGetLastError();
        if (g_bounce) (void)hipHostFree(g_bounce);
        g_bounce = g_bounce_dev = nullptr;
        g_bounce_failed = true;
        return false;
    }
    memset(static_cast<char*>(g_bounce) + kBounceBytes, 0, 64);
    return true;
}

// One workgroup copies n floats between the pinned buffer and device memory and then writes a
// sequence number behind the buffer; the host polls for it instead of waiting for the stream
// (after 1 ms without an answer it waits the usual way).
static int bounce_copy_and_wait(const float* src, float* dst, size_t n) {
    unsigned* flag_host = reinterpret_cast<unsigned*>(static_cast<char*>(g_bounce) + kBounceBytes);
    unsigned* flag_dev = reinterpret_cast<unsigned*>(static_cast<char*>(g_bounce_dev) + kBounceBytes);
    const unsigned seq = ++g_bounce_seq;
    hipLaunchKernelGGL(readback_kernel, dim3(1), dim3(kBlock), 0, ctx().stream, src, dst, n, flag_dev, seq);
    int st = check_launch("small transfer");
    if (st != 0) return st;
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(1);
    bool seen = false;
    for (int spin = 0; !seen; ++spin) {
        seen = __atomic_load_n(flag_host, __ATOMIC_ACQUIRE) == seq;
        if (!seen && (spin & 63) == 63 && std::chrono::steady_clock::now() > deadline) break;
    }
    if (!seen) BSHIP_HIP(hipStreamSynchronize(ctx().stream));
    return 0;
}

int bship_h2d(void* dst, const void* src_host, size_t nbytes) {
    BSHIP_REQUIRE_INIT();
    if (nbytes == 0) return 0;
    BSHIP_REQUIRE_PTR(dst);
    BSHIP_REQUIRE_PTR(src_host);
    BSHIP_REQUIRE_EAGER();
    if (nbytes <= kCopyTile * 4 && ((reinterpret_cast<uintptr_t>(dst) | nbytes) & 3u) == 0) {
        // small uploads (a batch of labels, a scalar): through pinned memory and one workgroup,
        // 8 us instead of 14 us through the runtime's copy from pageable memory
        std::lock_guard<std::mutex> lock(g_bounce_mutex);
        if (bounce_ready()) {
            memcpy(g_bounce, src_host, nbytes);
            return bounce_copy_and_wait(static_cast<const float*>(g_bounce_dev), static_cast<float*>(dst), nbytes / 4);
        }
    }
    BSHIP_HIP(hipMemcpyAsync(dst, src_host, nbytes, hipMemcpyHostToDevice, ctx().stream));
    BSHIP_HIP(hipStreamSynchronize(ctx().stream));
    return 0;
}

int bship_d2h(void* dst_host, const void* src, size_t nbytes) {
    BSHIP_REQUIRE_INIT();
    if (nbytes == 0) return 0;
    BSHIP_REQUIRE_PTR(dst_host);
    BSHIP_REQUIRE_PTR(src);
    BSHIP_REQUIRE_EAGER();
    if (nbytes <= kBounceBytes && ((reinterpret_cast<uintptr_t>(src) | nbytes) & 3u) == 0) {
        // Small read-backs (the loss after every training step, trainer.py:100; flags): a kernel writes
        // the values into pinned host memory and the caller's buffer is filled from there. Measured
        // for one float: 8.5 us (polled) / 12.8 us instead of 21.8 us through the runtime's copy to
        // pageable memory.
        std::lock_guard<std::mutex> lock(g_bounce_mutex);
        if (bounce_ready()) {
            const size_t n = nbytes / 4;
            if (nbytes <= kCopyTile * 4) {
                int st = bounce_copy_and_wait(static_cast<const float*>(src), static_cast<float*>(g_bounce_dev), n);
                if (st != 0) return st;
            } else {
                hipLaunchKernelGGL(copy_kernel<false>, dim3(static_cast<unsigned>((n + kCopyTile - 1) / kCopyTile)),
                                   dim3(kBlock), 0, ctx().stream, static_cast<const float*>(src),
                                   static_cast<float*>(g_bounce_dev), n, false);
                int st = check_launch("read-back");
                if (st != 0) return st;
                BSHIP_HIP(hipStreamSynchronize(ctx().stream));
            }
            memcpy(dst_host, g_bounce, nbytes);
            return 0;
        }
    }
    BSHIP_HIP(hipMemcpyAsync(dst_host, src, nbytes, hipMemcpyDeviceToHost, ctx().stream));
    BSHIP_HIP(hipStreamSynchronize(ctx().stream));
    return 0;
}

int bship_d2d(void* dst, const void* src, size_t nbytes) {
    BSHIP_REQUIRE_INIT_NO_FLUSH();
    if (nbytes == 0 || dst == src) return 0;
    BSHIP_REQUIRE_PTR(dst);
    BSHIP_REQUIRE_PTR(src);
    uintptr_t bits = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | nbytes;
    // a copy opens an LSTM layer's backward time step (lstm_layer.py:175): held in mode "stacked"
    if ((bits & 3u) == 0 && g_window_on.load(std::memory_order_relaxed) == 2 && window_takes())
        return window_push(window::rec_copy(src, dst, nbytes / 4));
    BSHIP_FLUSH_PENDING();
    if (bits & 3u) {  // not float-granular: let the runtime copy bytes
        BSHIP_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, ctx().stream));
        return 0;
    }
    const size_t n = nbytes / 4;
    const size_t tiles = (n + kCopyTile - 1) / kCopyTile;
    if (tiles > 0x7fffffffu) return set_error(BSHIP_ERR_BAD_DIMENSION, "copy: %zu bytes exceed one launch", nbytes);
    const dim3 grid(static_cast<unsigned>(tiles));
    const float* s = static_cast<const float*>(src);
    float* d = static_cast<float*>(dst);
    if (aligned16(s) && aligned16(d))
        hipLaunchKernelGGL(copy_kernel<true>, grid, dim3(kBlock), 0, ctx().stream, s, d, n, store_through(n));
    else
        hipLaunchKernelGGL(copy_kernel<false>, grid, dim3(kBlock), 0, ctx().stream, s, d, n, store_through(n));
    return check_launch("copy_kernel");
}

int bship_copy2d_f32(float* dst, int64_t ld_dst, const float* src, int64_t ld_src, int64_t rows,
                     int64_t cols) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(rows >= 0 && cols >= 0);
    if (rows == 0 || cols == 0) return 0;
    BSHIP_REQUIRE_PTR(dst);
    BSHIP_REQUIRE_PTR(src);
    BSHIP_REQUIRE_F32_ALIGNED(dst);
    BSHIP_REQUIRE_F32_ALIGNED(src);
    BSHIP_REQUIRE_DIM(ld_dst >= cols && ld_src >= cols);
    if (ld_dst == cols && ld_src == cols) return bship_d2d(dst, src, static_cast<size_t>(rows * cols) * 4);
    int L = 0;
    while (L < 8 && (int64_t(4) << L) < cols) ++L;
    const int64_t tiles_per_row = ceil_div(cols, int64_t(4) << L);
    const int64_t row_groups = ceil_div(rows, int64_t(1) << (8 - L));
    BSHIP_REQUIRE_DIM(tiles_per_row * row_groups <= 0x7fffffff);
    hipLaunchKernelGGL(copy2d_kernel, dim3(static_cast<unsigned>(tiles_per_row * row_groups)), dim3(kBlock), 0,
                       ctx().stream, src, ld_src, dst, ld_dst, rows, cols, static_cast<unsigned>(tiles_per_row), L,
                       store_through(static_cast<size_t>(rows) * static_cast<size_t>(cols)));
    return check_launch("copy2d");
}

int bship_fill_f32(float* mem, float val, size_t n) {
    BSHIP_REQUIRE_INIT_NO_FLUSH();
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(mem);
    BSHIP_REQUIRE_F32_ALIGNED(mem);
    // fills are part of layers' sequences (highway_layer.py:64, softmax_ce_layer.py:83): with the
    // fusing window on they pass through it and come back here when it lets them go
    if (window_takes()) return window_push(window::rec_fill(mem, val, n));
    if (n <= kDeferredFillMax) return defer_fill(mem, val, n);
    int st = flush_deferred_fills();
    return st != 0 ? st : launch_fill(mem, val, n);
}

}  // extern "C"
