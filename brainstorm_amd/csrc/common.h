// Shared plumbing of libbship: library context (device, stream), error
// reporting, launch-shape helpers and the 128-bit vector types used by every
// streaming kernel. gfx950 only: wavefronts are 64 lanes wide.
#pragma once

#include <atomic>

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/bship.h"

namespace bship {

constexpr int kWave = 64;      // lanes per wavefront on CDNA
constexpr int kBlock = 256;    // default workgroup: 4 wavefronts

struct Context {
    bool inited = false;
    int device = -1;
    int num_cus = 256;
    hipStream_t stream = nullptr;
    hipEvent_t events[BSHIP_MAX_EVENTS] = {nullptr};   // created on first use
    bool debug_sync = false;   // BSHIP_DEBUG_SYNC=1: sync + check after every launch
    int blocks_per_cu = 8;     // streaming kernels launch num_cus*blocks_per_cu blocks
    int colsum_blocks_per_cu = 3;   // column sums: row bands are chosen to reach this many workgroups per CU (measured optimum)
    size_t write_through_min = size_t(1) << 22;   // elements from which write-only kernels store write-through
    // kernels that read and write store write-through when their output has between these many elements
    // (BSHIP_STORE_THROUGH_MIN, BSHIP_STORE_THROUGH_MAX): at least 1 MB, at most the 256 MB of the last-level cache
    size_t store_through_min = size_t(1) << 18, store_through_max = size_t(1) << 26;
    size_t softmax_run_bytes = size_t(512) << 10;  // softmax rows a multiple of 64 KiB apart: bytes of adjacent rows that an XCD takes in one run (BSHIP_SM_CHUNK_KB)
    size_t ew_run_bytes = size_t(512) << 10;      // elementwise kernels with two inputs: bytes per stream that an XCD takes in one run (BSHIP_EW_RUN_KB)
    int64_t col2im_stream_min_images_per_cu = 1;  // col2im: the streaming kernel takes batches of at least this many images per compute unit, 0: never (BSHIP_COL2IM_STREAM_MIN)
    char name[256] = {0};
};

Context& ctx();
static inline bool store_through(size_t out_elements) {
    return out_elements >= ctx().store_through_min && out_elements <= ctx().store_through_max;
}

// The dispatcher deals consecutive workgroups of a 1-D grid to the 8 XCDs in turn. With run > 1
// the tiles are renumbered so that each XCD takes runs of `run` adjacent tiles instead of every
// eighth tile; the tiles beyond the last whole group of 8 runs keep their numbers.
__device__ __forceinline__ unsigned xcd_run_tile(unsigned run) {
    unsigned tile = blockIdx.x;
    if (run > 1) {
        const unsigned group = 8 * run;
        if (tile < gridDim.x / group * group) tile = (tile % 8) * run + (tile / 8) % run + tile / group * group;
    }
    return tile;
}

// Records a formatted message for bship_last_error() and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// 0 if e == hipSuccess, else records "<what>: <hip error string>" and returns e.
int check_hip(hipError_t e, const char* what);
// To be called right after a kernel launch.
int check_launch(const char* what);

// Small fills are collected and enqueued together as one launch (pool.hip); every entry point
// first enqueues what has been collected, so the order of effects is the order of the calls.
int flush_deferred_fills();
extern std::atomic<int> g_deferred_fill_count;   // read without the list's lock: 0 means nothing to do

// The fusing window (window.hip, window_core.h) holds back operations that may turn out to be the
// beginning of a layer's sequence. Entry points that take part hand their call to window_push()
// while window_takes(); every other entry point first enqueues what is held (BSHIP_REQUIRE_INIT),
// so the order of effects stays the order of the calls. While the window itself enqueues kernels
// through the public entry points, t_window_emitting keeps them from coming back to it.
extern std::atomic<int> g_window_on;       // bship_fusing_set: 0 off, 1 on (same bits), 2 products of an LSTM step stacked as well
extern std::atomic<int> g_window_held;     // operations held right now
extern thread_local bool t_window_emitting;
int window_flush();
void window_other_work();
static inline bool window_takes() {
    return g_window_on.load(std::memory_order_relaxed) != 0 && !t_window_emitting;
}
// For code that holds one of the library's own locks while it calls public entry points: those calls
// must not go for the window's lock (the window takes that lock first and the other one inside when it
// enqueues a held operation). What the window held was enqueued by the outer entry point already.
struct WindowBypass {
    bool before;
    WindowBypass() : before(t_window_emitting) { t_window_emitting = true; }
    ~WindowBypass() { t_window_emitting = before; }
};

#define BSHIP_REQUIRE_INIT_NO_FLUSH()                                            \
    do {                                                                         \
        if (!::bship::ctx().inited)                                              \
            return ::bship::set_error(BSHIP_ERR_NOT_INITIALIZED,                 \
                                      "%s: bship_init() has not been called",    \
                                      __func__);                                 \
    } while (0)

// What earlier calls left behind goes first. Noted fills are older than anything the window holds
// (with the window on, a fill is noted only when the window lets it go), and the entry points
// through which the window enqueues held operations start with this same macro, so the fills
// still go first.
#define BSHIP_FLUSH_PENDING()                                                    \
    do {                                                                         \
        if (::bship::g_window_on.load(std::memory_order_relaxed) == 2 &&         \
            !::bship::t_window_emitting)                                         \
            ::bship::window_other_work();                                        \
        if (::bship::g_window_held.load(std::memory_order_relaxed) != 0 &&       \
            !::bship::t_window_emitting) {                                       \
            int flush_st_ = ::bship::window_flush();                             \
            if (flush_st_ != 0) return flush_st_;                                \
        }                                                                        \
        if (::bship::g_deferred_fill_count.load(std::memory_order_relaxed) != 0) { \
            int flush_st_ = ::bship::flush_deferred_fills();                     \
            if (flush_st_ != 0) return flush_st_;                                \
        }                                                                        \
    } while (0)

#define BSHIP_REQUIRE_INIT()                                                     \
    do {                                                                         \
        BSHIP_REQUIRE_INIT_NO_FLUSH();                                           \
        BSHIP_FLUSH_PENDING();                                                   \
    } while (0)

#define BSHIP_REQUIRE_PTR(p)                                                     \
    do {                                                                         \
        if ((p) == nullptr)                                                      \
            return ::bship::set_error(BSHIP_ERR_NULL_POINTER,                    \
                                      "%s: argument '%s' is NULL", __func__, #p);\
    } while (0)

#define BSHIP_REQUIRE_F32_ALIGNED(p)                                             \
    do {                                                                         \
        if ((reinterpret_cast<uintptr_t>(p) & 3u) != 0)                          \
            return ::bship::set_error(BSHIP_ERR_BAD_POINTER,                     \
                                      "%s: argument '%s' is not 4-byte aligned", \
                                      __func__, #p);                             \
    } while (0)

#define BSHIP_REQUIRE_DIM(cond)                                                  \
    do {                                                                         \
        if (!(cond))                                                             \
            return ::bship::set_error(BSHIP_ERR_BAD_DIMENSION,                   \
                                      "%s: requirement '%s' violated", __func__, \
                                      #cond);                                    \
    } while (0)

#define BSHIP_HIP(call)                                                          \
    do {                                                                         \
        int _st = ::bship::check_hip((call), #call);                             \
        if (_st != 0) return _st;                                                \
    } while (0)

// 128-bit vectors. f4 promises 16-byte alignment; f4u only 4-byte alignment --
// the compiler still emits one global_load_dwordx4 for it (the memory system
// accepts dword-aligned wide accesses), so views that start at an odd element
// of the flat buffer keep wide transactions. The alignment of f4u lives in the
// typedef, not in the type, so it must not be passed as a template argument:
// kernels are parameterised by <W, AL> and go through vload/vstore below.
typedef float f4 __attribute__((ext_vector_type(4)));
typedef f4 f4u __attribute__((aligned(4)));

template <int W> struct VecT { typedef float type; };
template <> struct VecT<4> { typedef f4 type; };

// Streaming (non-temporal) load/store of W floats starting at p.
template <int W, bool AL>
__device__ __forceinline__ typename VecT<W>::type vload(const float* p) {
    if constexpr (W == 1) return __builtin_nontemporal_load(p);
    else if constexpr (AL) return __builtin_nontemporal_load(reinterpret_cast<const f4*>(p));
    else return __builtin_nontemporal_load(reinterpret_cast<const f4u*>(p));
}
template <int W, bool AL>
__device__ __forceinline__ void vstore(float* p, typename VecT<W>::type v) {
    if constexpr (W == 1) __builtin_nontemporal_store(v, p);
    else if constexpr (AL) __builtin_nontemporal_store(v, reinterpret_cast<f4*>(p));
    else __builtin_nontemporal_store(v, reinterpret_cast<f4u*>(p));
}

// Store for kernels that write without reading (large fills, one-hot rows): a
// system-scope write-through store. Measured on MI355X for a pure 1 GiB write
// stream: 7.08 TB/s against 6.73 TB/s for the non-temporal store and 6.91 TB/s
// for a plain one; for kernels that also read, the non-temporal store is the
// faster one. Needs only 4-byte alignment.
template <int W>
__device__ __forceinline__ void vstore_writeonly(float* p, typename VecT<W>::type v) {
    if constexpr (W == 1) asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    // s_nop 1: two wait states before anything may overwrite the four data registers (gfx950 reads the
    // data of a store of more than 64 bits after issue; the compiler keeps that distance for its own
    // stores, but does not know that this statement is one)
    else asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
// Context::write_through_min is the element count from which write-only kernels use it (16 MB; lowering it
// to 1 MB changed none of the network workloads' step times).

// Store of a kernel that reads as well: write-through when `through`, non-temporal otherwise. Outputs of
// Context::store_through_min to store_through_max elements go through (store_through above): the
// write-through store hands the data to the memory side at once, where the last-level cache takes an
// output of up to its 256 MB (measured in the operation sweep on 8192 x 8192 tensors: elementwise kernels
// 0.83 -> 0.91 of the HBM peak, matrix-vector kernels 0.77 -> 0.88, copies 0.78 -> 0.87, softmax 0.75 ->
// 0.84). An output of 1 GB does not fit there and the whole sweep on 16384 x 16384 tensors is 1 % slower
// with such stores; a kernel that writes a small array ends sooner when its stores may stay in the L2 (a
// training step of a small network is a chain of such kernels).
template <int W, bool AL>
__device__ __forceinline__ void vstore(float* p, typename VecT<W>::type v, bool through) {
    if (through) vstore_writeonly<W>(p, v);
    else vstore<W, AL>(p, v);
}

static inline bool aligned16(const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Number of workgroups for a grid-stride streaming kernel over `tiles` tiles.
static inline unsigned stream_grid(int64_t tiles) {
    const Context& c = ctx();
    int64_t cap = static_cast<int64_t>(c.num_cus) * c.blocks_per_cu;
    int64_t g = tiles < cap ? tiles : cap;
    return static_cast<unsigned>(g < 1 ? 1 : g);
}

// Scratch from the pool without zero-fill (internal partial-result buffers).
int pool_alloc_raw(size_t nbytes, void** out);
int pool_free_raw(void* p);

// ---- recorded steps (graph.hip) ----
// True while bship_graph_begin() ... bship_graph_end() records the library's stream. Calls that
// wait for the device or move data to or from host memory are refused then (BSHIP_REQUIRE_EAGER).
bool graph_recording();
// Pool blocks handed out while graph `id` is recorded belong to it: when their owner frees them
// they are parked, not reused, until the graph is destroyed (its kernels keep writing to them).
void pool_graph_begin(int id);
void pool_graph_end();
void pool_graph_destroyed(int id);

// rng.hip: dropout masks of a recorded step (see "masks of recorded steps" there)
int rng_graph_begin(int id);
int rng_graph_end(int id);
int rng_graph_before_launch(int id);
int rng_graph_after_launch(int id);
void rng_graph_destroyed(int id);

#define BSHIP_REQUIRE_EAGER()                                                                    \
    do {                                                                                         \
        if (::bship::graph_recording())                                                          \
            return ::bship::set_error(BSHIP_ERR_UNSUPPORTED,                                     \
                                      "%s: not possible while a step is being recorded "         \
                                      "(bship_graph_begin)", __func__);                          \
    } while (0)
// Enqueues mem[0:n] = val.
int launch_fill(float* mem, float val, size_t n);

// n / d for 32-bit unsigned n by multiply and shift (Granlund-Montgomery, rounded-up
// multiplier): with l = ceil(log2 d) and m = floor(2^32 (2^l - d) / d) + 1,
// n / d = (mulhi(m, n) + n) >> l for every 32-bit n.
struct FastDiv {
    uint32_t d, magic, shift;
    FastDiv() : d(1), magic(1), shift(0) {}
    explicit FastDiv(uint32_t dd) : d(dd) {
        shift = 0;
        while ((uint64_t(1) << shift) < dd) ++shift;
        magic = static_cast<uint32_t>(((uint64_t(1) << 32) * ((uint64_t(1) << shift) - dd)) / dd + 1);
    }
    __device__ __forceinline__ uint32_t div(uint32_t n) const {
        return static_cast<uint32_t>((static_cast<uint64_t>(__umulhi(n, magic)) + n) >> shift);
    }
    __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
        q = div(n);
        r = n - q * d;
    }
};

// ---- loads that complete in order: waiting by count ----
// Waits until at most N of this wavefront's vector memory operations are outstanding.
template <int N>
__device__ __forceinline__ void wait_until_outstanding() {
    static_assert(N >= 0 && N < 64, "the counter has 6 bits");
    // vmcnt: bits 3:0 and 15:14; expcnt (6:4) and lgkmcnt (11:8) at their maximum: not waited for
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
    asm volatile("" ::: "memory");
}

// ---- integer labels stored as float32 (device) ----
// Column selected by label v in a row of K columns: truncated toward zero like astype(int32);
// labels in [-K, -1] count from the end, as NumPy's indexing does (numpy_handler.py:101, 203).
// Anything else (beyond [-K, K), NaN, infinities) selects no column: -1. NumPy raises IndexError
// there; a kernel cannot, so such a row gets no one-hot entry and gathers 0.
__device__ __forceinline__ int64_t label_column(float v, int64_t K) {
    if (!(v > -2147483648.0f && v < 2147483648.0f)) return -1;
    int64_t j = static_cast<int64_t>(static_cast<int>(v));
    if (j < 0) j += K;
    return (j >= 0 && j < K) ? j : -1;
}

// ---- wavefront reductions (device) ----
// All 64 lanes must be active. Four DPP steps (lane^1, lane^2, mirror inside 8 lanes, mirror inside
// a row of 16) leave every lane of a row with the row's result without touching LDS (a shuffle is a
// ds_bpermute through the LDS crossbar, ~100 cycles each, six in a butterfly); the four row results
// are read out as scalars and combined, so every lane returns the same value.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    const int x = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(x, x, CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
constexpr int kDppXor1 = 0xB1;          // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;          // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;   // row_half_mirror
constexpr int kDppMirror = 0x140;       // row_mirror

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    v += dpp_move<kDppMirror>(v);
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<kDppXor1>(v));
    v = fmaxf(v, dpp_move<kDppXor2>(v));
    v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_move<kDppMirror>(v));
    return fmaxf(fmaxf(read_lane(v, 0), read_lane(v, 16)), fmaxf(read_lane(v, 32), read_lane(v, 48)));
}

}  // namespace bship
