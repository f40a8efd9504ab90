// Device-resident MT19937 that reproduces numpy.random.RandomState bit for bit.
//
// The reference draws dropout masks from the handler's RandomState
// (numpy_handler.py 199-200: rnd.uniform(size) < p). To give the same masks
// the generator state (624 words + position + the cached gaussian of the legacy
// polar method) lives in device memory and one workgroup advances it. Nothing
// is copied to the host, so mask generation stays asynchronous.
//
// The generator is treated as one linear stream of raw words r[0], r[1], ...:
// the 624 words of the current block are r[0..623] and every later word follows
// from
//     r[n] = r[n-227] ^ T(r[n-624], r[n-623]),     T = the MT19937 twist
// (the block-wise regeneration of the MT19937 reference code, unrolled). Words
// closer than 227 apart are independent, so a step of 227 lanes would do; but
// each step costs an LDS round trip and a workgroup barrier, which is what the
// serial kernel's time consists of. Two properties shorten it:
//  * T is linear over GF(2) (its OR joins disjoint bit fields), so substituting
//    the recurrence into itself twice collapses into ONE twist,
//        r[n] = r[n-681] ^ T(r[n-624]^r[n-851]^r[n-1078], r[n-623]^r[n-850]^r[n-1077]),
//    in which every operand is at least 623 words old: one step produces 623
//    consecutive words (2.7 times fewer steps) for the price of 4 more XORs;
//  * the serial kernel only EXTENDS THE STREAM and stores raw words; tempering,
//    pairing into 53-bit doubles and the compare with p run afterwards in an
//    ordinary data-parallel kernel over the whole device.
// Measured on MI355X: 0.72 ns per double (a 100x1200 dropout mask in 0.09 ms).
// History of the serial part: block-wise three-phase twist 2.25 ns per double;
// 227-word steps with the conversion in the same workgroup 1.48; 623-word steps
// with register-cached operands and separate conversion wavefronts 1.31; raw
// words only 1.15; all LDS reads of a step issued together 0.85; one twist 0.72.
// A minimal LDS-read / write / barrier step of such a workgroup costs 0.13 us,
// which bounds the single-stream design near 0.4 ns per double. (A variant in
// which ONE wavefront generates 10 words per lane without any barrier was
// measured at 4.4 ns per double: a whole step's arithmetic on a single SIMD.)
#include <cstdlib>
#include <type_traits>
#include <deque>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "common.h"
#include "window.h"
#include "mt_jump.h"

namespace bship {

constexpr int kMtN = 624;
constexpr int kMtM = 397;

struct RngState {
    uint32_t key[kMtN];
    int32_t pos;          // next unread word of key; kMtN means "regenerate first"
    int32_t has_gauss;    // legacy_gauss cache flag
    double gauss;         // cached second variate of the polar method
};

// Generators. Every handler object has its own random stream (numpy_handler.py:21: `self.rnd`), so
// the library keeps any number of generators (MT19937 state + the optional fast stream's state, in
// device memory) and ONE of them selected: g_state / g_fast_state below are the selected generator's,
// and the look-ahead queue, the mask slots of a primed recorded step and the pattern history always
// belong to it. Selecting another generator (bship_rng_select, a cheap no-op when it is selected
// already) first gives up what was drawn ahead, so each generator's stream is exactly the
// sequential one whatever the interleaving. Generator 0 exists from the start.
static RngState* g_state = nullptr;   // device memory; the selected generator's
static std::mutex g_rng_mutex;
static int g_current_generator = 0;
static int select_generator_locked(int id);      // caller holds g_rng_mutex

__device__ __forceinline__ uint32_t mt_twist(uint32_t u, uint32_t v) {
    const uint32_t y = (u & 0x80000000u) | (v & 0x7fffffffu);
    return (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
}

__device__ __forceinline__ uint32_t mt_temper(uint32_t y) {
    y ^= (y >> 11);
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= (y >> 18);
    return y;
}

// Workgroup barrier that orders LDS traffic only. __syncthreads() also waits for
// the wavefront's outstanding GLOBAL stores (the raw words being written), which
// would put a memory round trip into the serial chain.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

constexpr int kLag = kMtN - kMtM;             // 227
constexpr int kWide = kMtN - 1;               // 623 words per wide step
constexpr int kWideHistory = kMtN + 2 * kLag; // 1078: oldest word a wide step reads is n-1078

constexpr int kRawThreads = 640;              // lanes 0..622 generate one word per wide step
static_assert(kRawThreads >= kWide && kRawThreads % kWave == 0, "generator lanes cover a step");

// raw[0..nw) = the next nw words of the stream r[pos0 .. pos0+nw); state left as numpy leaves it.
//
// LDS holds the last kWin = 2048 words twice: word n lives in slots (n mod kWin) and
// (n mod kWin) + kWin. A step reads words n-1078 .. n-623 relative to its own word; starting
// from slot (have mod kWin) + kWin - 1078 + lane all of them sit at fixed positive distances,
// never wrap, and are addressed by the constant offsets of the LDS instructions (no index
// arithmetic per load). The 623 slots a step writes and the 1078 it reads are disjoint modulo
// kWin (623 + 1078 <= 2048), so one barrier per step still suffices.
constexpr int kWin = 2048;
static_assert(kWide + kWideHistory <= kWin, "a step's reads and writes must not alias");

// `win` is the workgroup's LDS window (2 * kWin words), `key` the 624-word block to start from (position
// pos0 in it is the first word wanted), `st_out` (may be null) receives the state afterwards.
__device__ __forceinline__ void mt_generate(uint32_t* win, const uint32_t* key, size_t pos0, size_t nw,
                                            uint32_t* __restrict__ raw, RngState* st_out) {
    const unsigned t = threadIdx.x;
    for (unsigned i = t; i < kMtN; i += kRawThreads) {
        const uint32_t v = key[i];
        win[i] = v;
        win[i + kWin] = v;
    }
    __syncthreads();
    const size_t end_word = pos0 + nw;
    const size_t gen_end = (end_word + kMtN - 1) / kMtN * kMtN;
    for (size_t i = pos0 + t; i < kMtN && i < end_word; i += kRawThreads) raw[i - pos0] = win[i];
    size_t have = kMtN;
    unsigned hm = kMtN;                                   // have mod kWin
    // raw slot of word `have` (uniform; lane t adds t); words at or beyond end_word are not stored
    uint32_t* out = raw + (kMtN - pos0);
    // One step: lanes below `step` compute word have + t (all LDS reads are issued together),
    // store it twice into the window and once into raw, then everybody meets at the barrier.
    auto advance = [&](auto wide_tag) {
        constexpr bool wide = decltype(wide_tag)::value;
        constexpr unsigned step = wide ? kWide : kLag;
        if (t < step) {
            // slot of word (have + t - kWideHistory), in the upper copy
            const uint32_t* p = win + (hm + kWin - kWideHistory) + t;
            uint32_t v;
            if constexpr (wide) {
                const uint32_t a2 = p[0], b2 = p[1];
                const uint32_t a1 = p[kWideHistory - kMtN - kLag], b1 = p[kWideHistory - kMtN - kLag + 1];
                const uint32_t c = p[kWideHistory - 3 * kLag];
                const uint32_t a0 = p[kWideHistory - kMtN], b0 = p[kWideHistory - kMtN + 1];
                // the twist is linear over GF(2) (its OR joins disjoint bit fields), so the three
                // twists of the wide step are one twist of the XORed operands
                v = c ^ mt_twist(a0 ^ a1 ^ a2, b0 ^ b1 ^ b2);
            } else {
                v = p[kWideHistory - kLag] ^ mt_twist(p[kWideHistory - kMtN], p[kWideHistory - kMtN + 1]);
            }
            const unsigned x = (hm + t) & (kWin - 1);
            win[x] = v;
            win[x + kWin] = v;
            const size_t rest = end_word > have ? end_word - have : 0;       // uniform
            if (t < (rest < step ? static_cast<unsigned>(rest) : step)) out[t] = v;
        }
        have += step;
        hm = (hm + step) & (kWin - 1);
        out += step;
        lds_barrier();
    };
    while (have < gen_end && have < kWideHistory) advance(std::false_type());    // two plain steps
    while (have < gen_end) advance(std::true_type());
    __syncthreads();
    if (st_out != nullptr) {
        const size_t block0 = gen_end - kMtN;
        for (unsigned i = t; i < kMtN; i += kRawThreads) st_out->key[i] = win[(block0 + i) & (kWin - 1)];
        if (t == 0) st_out->pos = static_cast<int32_t>(end_word - block0);
    }
}

__global__ __launch_bounds__(kRawThreads) void mt_raw_kernel(RngState* st, uint32_t* __restrict__ raw,
                                                             size_t nw, RngState* before) {
    __shared__ uint32_t win[2 * kWin];
    const unsigned t = threadIdx.x;
    const size_t pos0 = static_cast<size_t>(st->pos);
    if (before != nullptr) {
        for (unsigned i = t; i < kMtN; i += kRawThreads) before->key[i] = st->key[i];
        if (t == 0) before->pos = static_cast<int32_t>(pos0);
    }
    mt_generate(win, st->key, pos0, nw, raw, st);
}

// ------------------------------ parallel draws ------------------------------
// A long draw is cut into segments of a whole number of 624-word blocks. The key block each segment
// starts from is computed from the current one by jump-ahead (mt_jump.h): with w[0..] the stream
// that starts at the current key block and g the polynomial of the distance d,
//     block d words ahead [j] = XOR over { i : g_i = 1 } of w[i + j],     j = 0 .. 623,
// so one workgroup first writes the "history" w[0 .. 19938 + 624), a grid then forms all the
// segments' blocks from it (each workgroup a slice of the coefficients, combined with atomic XOR:
// exact and order-free), and the segments are generated side by side, one workgroup each. The last
// segment leaves the state exactly as the sequential generator would.
constexpr int kJumpBits = 19938;                      // coefficients of a jump polynomial (mtjump::kPolyBits)
constexpr int kHistWords = kJumpBits + kMtN;          // stream words the combination reads
constexpr int kJumpChunk = 256;                       // coefficients per workgroup
constexpr int kJumpChunks = (kJumpBits + kJumpChunk - 1) / kJumpChunk;
static_assert(kJumpChunks * kJumpChunk == kMtN * 32, "a polynomial is stored as 624 words");

// hist[0 .. kHistWords) = the stream from the start of the current key block; seeds[0] = the
// current state, seeds[1 .. nseg) cleared for the combination; *before = the current key and pos.
__global__ __launch_bounds__(kRawThreads) void mt_history_kernel(const RngState* st, uint32_t* __restrict__ hist,
                                                                 RngState* seeds, int nseg, RngState* before) {
    __shared__ uint32_t win[2 * kWin];
    const unsigned t = threadIdx.x;
    for (unsigned i = t; i < kMtN; i += kRawThreads) {
        const uint32_t v = st->key[i];
        seeds[0].key[i] = v;
        if (before != nullptr) before->key[i] = v;
        for (int s = 1; s < nseg; ++s) seeds[s].key[i] = 0u;
    }
    if (t == 0) {
        seeds[0].pos = st->pos;
        if (before != nullptr) before->pos = st->pos;
    }
    mt_generate(win, st->key, 0, kHistWords, hist, nullptr);
}

// seeds[blockIdx.y + 1].key ^= the part of the combination that coefficients
// [blockIdx.x * kJumpChunk, +kJumpChunk) of polynomial blockIdx.y contribute.
__global__ __launch_bounds__(kRawThreads) void mt_jump_kernel(const uint32_t* __restrict__ polys,
                                                              const uint32_t* __restrict__ hist, RngState* seeds) {
    __shared__ uint32_t h[kJumpChunk + kMtN];
    const unsigned t = threadIdx.x;
    const int i0 = blockIdx.x * kJumpChunk;
    for (int i = t; i < kJumpChunk + kMtN; i += kRawThreads) h[i] = i0 + i < kHistWords ? hist[i0 + i] : 0u;
    __syncthreads();
    if (t >= kMtN) return;
    const uint32_t* g = polys + static_cast<size_t>(blockIdx.y) * kMtN + i0 / 32;
    uint32_t acc = 0;
#pragma unroll
    for (int wd = 0; wd < kJumpChunk / 32; ++wd) {
        const uint32_t bits = g[wd];                      // the same for every lane
#pragma unroll
        for (int b = 0; b < 32; ++b) acc ^= h[wd * 32 + b + t] & (0u - ((bits >> b) & 1u));
    }
    if (acc != 0u) atomicXor(&seeds[blockIdx.y + 1].key[t], acc);
}

// Segment blockIdx.x: seg_words words (the last one: what is left of nw) from seeds[blockIdx.x], all
// starting at position seeds[0].pos of their block; the last segment writes the state to *st.
__global__ __launch_bounds__(kRawThreads) void mt_segments_kernel(const RngState* seeds, RngState* st,
                                                                  uint32_t* __restrict__ raw, size_t nw,
                                                                  size_t seg_words) {
    __shared__ uint32_t win[2 * kWin];
    const size_t first = static_cast<size_t>(blockIdx.x) * seg_words;
    const bool last = blockIdx.x + 1 == gridDim.x;
    mt_generate(win, seeds[blockIdx.x].key, static_cast<size_t>(seeds[0].pos), last ? nw - first : seg_words,
                raw + first, last ? st : nullptr);
}

__device__ __forceinline__ uint64_t raw_to_k53(const uint32_t* __restrict__ raw, size_t i) {
    const uint32_t w0 = mt_temper(raw[2 * i]), w1 = mt_temper(raw[2 * i + 1]);
    return (static_cast<uint64_t>(w0 >> 5) << 26) | static_cast<uint64_t>(w1 >> 6);
}
// Element i of the mask goes to row i / cols, column i % cols of a matrix whose rows lie ld elements
// apart (ld == cols: the dense mask).
__global__ __launch_bounds__(kBlock) void raw_to_mask_kernel(const uint32_t* __restrict__ raw,
                                                             float* __restrict__ mask, size_t n, double p,
                                                             size_t cols, size_t ld) {
    uint64_t threshold;
    if (!(p > 0.0)) threshold = 0;
    else if (p >= 1.0) threshold = ~static_cast<uint64_t>(0);
    else threshold = static_cast<uint64_t>(ceil(p * 9007199254740992.0));
    const size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= n) return;
    size_t at = i;
    if (ld != cols) {
        const size_t row = i / cols;
        at = row * ld + (i - row * cols);
    }
    mask[at] = raw_to_k53(raw, i) < threshold ? 1.0f : 0.0f;
}
__global__ __launch_bounds__(kBlock) void raw_to_doubles_kernel(const uint32_t* __restrict__ raw,
                                                                double* __restrict__ u, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < n) u[i] = static_cast<double>(raw_to_k53(raw, i)) * (1.0 / 9007199254740992.0);
}

// Legacy polar method (RandomState.standard_normal): trial t uses doubles
// u[2t], u[2t+1]; x1 = 2u0-1, x2 = 2u1-1, r2 = x1^2+x2^2; rejected if r2 >= 1 or
// r2 == 0; an accepted trial yields f*x2 first and caches f*x1 for the next
// call, f = sqrt(-2 ln(r2) / r2). One workgroup scans the trials in order and
// compacts the accepted ones with a prefix sum, so output k comes from the
// same trial as in the sequential algorithm.
// result[0] = number of trials consumed, result[1] = outputs written.
__global__ __launch_bounds__(kBlock) void gauss_polar_kernel(RngState* st, const double* __restrict__ u,
                                                             size_t trials, float* __restrict__ out,
                                                             size_t n, size_t start, double mean,
                                                             double stdv, unsigned long long* result) {
    __shared__ unsigned int counts[kBlock];
    __shared__ size_t used_s;
    size_t produced = start;          // outputs already written (from the cache or earlier chunks)
    size_t t0 = 0;
    if (threadIdx.x == 0) { used_s = 0; }
    __syncthreads();
    while (t0 < trials && produced < n) {
        const size_t t = t0 + threadIdx.x;
        double x1 = 0.0, x2 = 0.0, r2 = 2.0;
        if (t < trials) {
            x1 = 2.0 * u[2 * t] - 1.0;
            x2 = 2.0 * u[2 * t + 1] - 1.0;
            r2 = x1 * x1 + x2 * x2;
        }
        const bool acc = (t < trials) && !(r2 >= 1.0 || r2 == 0.0);
        counts[threadIdx.x] = acc ? 1u : 0u;
        __syncthreads();
        // inclusive scan over the workgroup (Hillis-Steele; 8 steps)
        for (int off = 1; off < kBlock; off <<= 1) {
            unsigned int v = counts[threadIdx.x];
            if (threadIdx.x >= static_cast<unsigned>(off)) v += counts[threadIdx.x - off];
            __syncthreads();
            counts[threadIdx.x] = v;
            __syncthreads();
        }
        const unsigned int incl = counts[threadIdx.x];
        const unsigned int total = counts[kBlock - 1];
        if (acc) {
            const size_t k = produced + 2 * static_cast<size_t>(incl - 1);   // index of first output
            if (k < n) {
                const double f = sqrt(-2.0 * log(r2) / r2);
                out[k] = static_cast<float>(stdv * (f * x2) + mean);
                if (k + 1 < n) {
                    out[k + 1] = static_cast<float>(stdv * (f * x1) + mean);
                } else {
                    // the last output is the first of its pair: cache the second
                    st->gauss = f * x1;
                    st->has_gauss = 1;
                }
                // the trial that produced output n-1 or n-2 is the last one consumed
                if (k + 2 >= n) used_s = t + 1;
            }
        }
        __syncthreads();
        produced += 2 * static_cast<size_t>(total);
        t0 += kBlock;
    }
    if (threadIdx.x == 0) {
        const bool complete = produced >= n;
        result[0] = complete ? used_s : trials;
        result[1] = complete ? n : produced;
    }
}

// Emits the cached gaussian (if any) as output 0 and clears the cache flag.
__global__ void gauss_cache_kernel(RngState* st, float* out, size_t n, double mean, double stdv,
                                   unsigned long long* result) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        unsigned long long start = 0;
        if (n > 0 && st->has_gauss) {
            out[0] = static_cast<float>(stdv * st->gauss + mean);
            st->has_gauss = 0;
            st->gauss = 0.0;
            start = 1;
        }
        result[2] = start;
    }
}

// Copies the word stream position only (key and pos); the gaussian cache is left alone.
__global__ void rng_copy_state_kernel(const RngState* src, RngState* dst) {
    for (int i = threadIdx.x; i < kMtN; i += blockDim.x) dst->key[i] = src->key[i];
    if (threadIdx.x == 0) { dst->pos = src->pos; }
}

static int rng_ensure_state() {
    if (g_state) return 0;
    void* p = nullptr;
    int st = pool_alloc_raw(sizeof(RngState), &p);
    if (st != 0) return st;
    g_state = static_cast<RngState*>(p);
    return 0;
}

// ------------------------------ mask prefetch ------------------------------
// A mask costs a fixed sequential time on ONE compute unit and depends on
// nothing but the stream position, while a training loop asks for the same
// masks, in the same order, every step. Once the recent requests (n, p) repeat
// with some period P, the next P masks (a "round") are drawn ahead of time on a
// second stream into staging buffers, overlapping the step's other kernels: one
// draw of the round's words (the masks are consecutive in the stream; long
// enough, the draw is cut into parallel segments) and one kernel that turns them
// into the P masks. A matching request then is a wait on an event plus a device
// copy. Two rounds alternate: when the first mask of a round is asked for, the
// draw of the following round is enqueued, so it has the whole step to finish.
// A round keeps the stream position from before its draw, so any request that
// does not match the prediction (or any other use of the generator) rewinds to
// that position and re-draws the words of the masks already handed out: the
// generator is exactly where a purely sequential one would be, and results never
// depend on whether a request was served from a round.
struct MaskPrefetch {
    size_t n;
    double p;
    float* staging;
    float* next;           // slots of a recorded step: the mask after the one in staging
    uint32_t* raw;         // the 2n raw words of the draw (scratch of the entry's own)
    RngState* before;      // key and pos before this mask was drawn
    hipEvent_t ready;      // second stream: the mask is in staging
    hipEvent_t consumed;   // main stream: staging has been copied out
};
static std::vector<std::pair<size_t, double>> g_history;
static hipStream_t g_side = nullptr;
static hipEvent_t g_join = nullptr;          // orders one stream behind the other
constexpr size_t kMaxPeriod = 16;
static size_t g_min_period = 1;              // raised after a wrong guess, see prefetch_flush()
constexpr size_t kMaxPrefetchFloats = size_t(1) << 26;   // per period: 256 MiB of staging at most

// ---- plan of a parallel draw ----
// Cost model (measured): forming one segment's start block costs about 1 us of the whole device
// (19938 x 624 AND-XOR pairs), generating a segment 0.13 us per 623 words on one compute unit, so
// the time 1.05 P + 0.13 nw / (623 P) is least for P = sqrt(nw / 5000) segments.
constexpr int kMaxSegments = 64;
constexpr int kMinSegments = 4;                 // below (61 000 words), the sequential kernel is as fast
constexpr size_t kEagerJumpMinWords = size_t(1) << 20;
struct JumpPolys { uint32_t* dev; int count; };
constexpr size_t kMaxJumpTables = 256;          // distinct segment lengths kept (up to 160 KB of device memory each)
static std::vector<uint32_t*> g_jump_retired;          // replaced tables, freed at shutdown
static std::map<size_t, JumpPolys> g_jump_polys;      // words per segment -> polynomials of 1, 2, ... segments ahead
static uint32_t* g_hist = nullptr;                    // kHistWords words
static RngState* g_seeds = nullptr;                   // kMaxSegments states
// The generator's scratch (g_hist, g_seeds) is used like g_state itself: by one stream at a time,
// in an order fixed by events; the polynomials are written once and then only read.

static bool jump_enabled() {
    static const bool on = [] {
        const char* e = getenv("BSHIP_RNG_JUMP");
        return !(e && e[0] == '0');
    }();
    return on;
}

struct JumpPlan { int segments; size_t seg_words; const uint32_t* polys; };

// Segments and words per segment for a draw of nw words, or false for "draw sequentially".
static bool jump_shape(size_t nw, bool for_replay, int* segments, size_t* seg_words) {
    if (!jump_enabled()) return false;
    // A training step of small layers that is issued call by call is paced by the host: there the
    // two extra launches cost more than the shorter draw saves (MLP 784-1200-1200-10: 0.35 -> 0.45 ms
    // per step), so only long draws are cut up. Next to the replay of a recorded step the host is
    // idle and the draw is what the step waits for: there every draw long enough is cut up.
    if (!for_replay && nw < kEagerJumpMinWords) return false;
    int target = static_cast<int>(sqrt(static_cast<double>(nw) / 5000.0) + 0.5);
    if (target < kMinSegments) return false;
    if (target > kMaxSegments) target = kMaxSegments;
    const size_t blocks = static_cast<size_t>(ceil_div(static_cast<int64_t>(nw), static_cast<int64_t>(kMtN) * target));
    *seg_words = blocks * kMtN;
    *segments = static_cast<int>((nw + *seg_words - 1) / *seg_words);
    return *segments >= 2;
}

// The polynomials of 1 ... count segments of seg_words ahead, on the device; computed (tens of
// milliseconds on the host) and uploaded on first use. Not while a step is being recorded: the
// upload is a blocking copy, which invalidates a recording. Null: not available.
static const uint32_t* jump_polys(size_t seg_words, int count) {
    auto it = g_jump_polys.find(seg_words);
    if (it != g_jump_polys.end() && it->second.count >= count) return it->second.dev;
    if (graph_recording()) return nullptr;
    if (it == g_jump_polys.end() && g_jump_polys.size() >= kMaxJumpTables) return nullptr;   // draw sequentially
    if (!g_hist && hipMalloc(reinterpret_cast<void**>(&g_hist), kHistWords * sizeof(uint32_t)) != hipSuccess) {
        (void)hipGetLastError(); g_hist = nullptr; return nullptr;
    }
    if (!g_seeds && hipMalloc(reinterpret_cast<void**>(&g_seeds), kMaxSegments * sizeof(RngState)) != hipSuccess) {
        (void)hipGetLastError(); g_seeds = nullptr; return nullptr;
    }
    std::vector<uint32_t> host;
    if (!mtjump::jump_polynomials(seg_words, count, host)) return nullptr;
    uint32_t* dev = nullptr;
    // memory of its own, not a pool block: a pool block may still be read by kernels in flight,
    // and this copy does not wait for the library's streams
    if (hipMalloc(reinterpret_cast<void**>(&dev), host.size() * sizeof(uint32_t)) != hipSuccess) {
        (void)hipGetLastError(); return nullptr;
    }
    if (hipMemcpy(dev, host.data(), host.size() * sizeof(uint32_t), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError(); (void)hipFree(dev); return nullptr;
    }
    if (it != g_jump_polys.end()) {
        // a shorter table of the same length may be in use by kernels in flight or recorded steps: keep it
        g_jump_retired.push_back(it->second.dev);
        it->second = JumpPolys{dev, count};
    } else {
        g_jump_polys.emplace(seg_words, JumpPolys{dev, count});
    }
    return dev;
}

// Decides whether a draw of nw words is cut into segments. Any failure means "draw sequentially".
static bool jump_plan(size_t nw, bool for_replay, JumpPlan* plan) {
    if (!jump_shape(nw, for_replay, &plan->segments, &plan->seg_words)) return false;
    plan->polys = jump_polys(plan->seg_words, plan->segments - 1);
    return plan->polys != nullptr;
}

// Enqueues raw[0 .. nw) = the next nw words of the stream on `stream`, *before = the state before.
// for_replay: the words are masks of a recorded step (the draw overlaps the replay: see jump_shape).
static void launch_raw_words(hipStream_t stream, uint32_t* raw, size_t nw, RngState* before, bool for_replay = false) {
    JumpPlan plan;
    if (!jump_plan(nw, for_replay, &plan)) {
        hipLaunchKernelGGL(mt_raw_kernel, dim3(1), dim3(kRawThreads), 0, stream, g_state, raw, nw, before);
        return;
    }
    hipLaunchKernelGGL(mt_history_kernel, dim3(1), dim3(kRawThreads), 0, stream, g_state, g_hist, g_seeds,
                       plan.segments, before);
    hipLaunchKernelGGL(mt_jump_kernel, dim3(kJumpChunks, plan.segments - 1), dim3(kRawThreads), 0, stream,
                       plan.polys, g_hist, g_seeds);
    hipLaunchKernelGGL(mt_segments_kernel, dim3(plan.segments), dim3(kRawThreads), 0, stream, g_seeds, g_state, raw,
                       nw, plan.seg_words);
}

// Enqueues mask[0..n) = (next n doubles of the stream < p) on `stream`; raw is scratch for 2n words.
// The mask is a matrix of `cols` columns whose rows lie `ld` elements apart (0: dense).
static void launch_mask(hipStream_t stream, float* mask, size_t n, double p, RngState* before, uint32_t* raw,
                        size_t cols = 0, size_t ld = 0) {
    launch_raw_words(stream, raw, 2 * n, before);
    if (cols == 0) cols = ld = n;
    hipLaunchKernelGGL(raw_to_mask_kernel, dim3(static_cast<unsigned>(ceil_div(static_cast<int64_t>(n), kBlock))),
                       dim3(kBlock), 0, stream, raw, mask, n, p, cols, ld);
}

// Enqueues u[0..n) = the next n doubles of the stream on the main stream (raw: scratch for 2n words).
static void launch_doubles(double* u, size_t n, uint32_t* raw) {
    launch_raw_words(ctx().stream, raw, 2 * n, nullptr);
    hipLaunchKernelGGL(raw_to_doubles_kernel, dim3(static_cast<unsigned>(ceil_div(static_cast<int64_t>(n), kBlock))),
                       dim3(kBlock), 0, ctx().stream, raw, u, n);
}

static bool prefetch_enabled() {
    static const bool on = [] {
        const char* e = getenv("BSHIP_RNG_PREFETCH");
        return !(e && e[0] == '0');
    }();
    return on;
}

static void free_entry(MaskPrefetch& e) {
    if (e.staging) pool_free_raw(e.staging);
    if (e.next) pool_free_raw(e.next);
    if (e.raw) pool_free_raw(e.raw);
    if (e.before) pool_free_raw(e.before);
    if (e.ready) (void)hipEventDestroy(e.ready);
    if (e.consumed) (void)hipEventDestroy(e.consumed);
    e = MaskPrefetch();
}

// Makes `later` wait for everything enqueued on `earlier` so far.
static int order_streams(hipStream_t earlier, hipStream_t later) {
    if (!g_join) BSHIP_HIP(hipEventCreateWithFlags(&g_join, hipEventDisableTiming));
    BSHIP_HIP(hipEventRecord(g_join, earlier));
    BSHIP_HIP(hipStreamWaitEvent(later, g_join, 0));
    return 0;
}

// Gives up everything drawn ahead and puts the generator back to its sequential position (defined
// behind the masks of recorded steps, whose helpers the look-ahead shares).
static int prefetch_flush(bool restore_position, bool wrong_guess = false);
static void prefetch_maybe_start();

// --------------------------- masks of recorded steps ---------------------------
// A recorded step (bship_graph_begin ... bship_graph_end) replays the same kernels with the same
// arguments, so its masks cannot be served by the queue above, and drawing them inline would put
// their time on the step's critical path. Instead every mask request of the recording gets a slot
// of its own (two mask buffers, generator snapshot), and the recorded graph only READS the slots'
// `staging` buffers: it contains no generator kernel at all. Each replay (bship_graph_launch) then
// issues, next to the graph and on the second stream, ONE draw of the raw words of all slots'
// following masks (they are consecutive in the stream; long enough, the draw is cut into parallel
// segments) and one kernel that turns them into the slots' `next` buffers, and behind the graph one
// kernel that copies next -> staging. So replay r consumes what replay r-1 (or the priming below) drew, the
// random stream is used exactly as by eager execution, and the draws overlap the whole step as
// ordinary work of a second stream. (Drawing inside the graph, on a captured branch, was measured
// first: the graph executor ran a branch forked where the mask is consumed partly, and a branch
// forked at the root entirely, in series with the main chain.) Before the first replay, and after
// any other use of the generator, the slots are "primed": their masks are drawn eagerly in order.
// Any eager use of the generator first "unprimes": it puts the generator back to the snapshot taken
// before the pending, not yet consumed masks.
struct GraphMasks {
    int generator = 0;             // the generator selected while the step was recorded: its replays draw from it
    std::vector<MaskPrefetch> slots;
    uint32_t* raw = nullptr;       // the raw words of one round of all slots' masks: they are consecutive in the
    size_t words = 0;              // stream, so a round is ONE draw (a parallel one, if long enough)
    bool primed = false;
};
static std::map<int, GraphMasks> g_graph_masks;
static int g_recording_masks = 0;      // graph being recorded, or 0
static int g_primed_graph = 0;         // graph whose slots hold drawn, unconsumed masks, or 0
static hipEvent_t g_before_graph = nullptr;   // main stream, right before a replay's graph

// The pending masks of the primed graph are given up: the generator returns to the position before them.
static int graph_masks_unprime() {
    if (g_primed_graph == 0) return 0;
    GraphMasks& gm = g_graph_masks[g_primed_graph];
    g_primed_graph = 0;
    gm.primed = false;
    if (gm.slots.empty()) return 0;
    hipLaunchKernelGGL(rng_copy_state_kernel, dim3(1), dim3(kBlock), 0, ctx().stream, gm.slots.front().before, g_state);
    return check_launch("random stream rewind");
}

static int ensure_side_stream() {
    if (!g_side) BSHIP_HIP(hipStreamCreateWithFlags(&g_side, hipStreamNonBlocking));
    if (!g_join) BSHIP_HIP(hipEventCreateWithFlags(&g_join, hipEventDisableTiming));
    if (!g_before_graph) BSHIP_HIP(hipEventCreateWithFlags(&g_before_graph, hipEventDisableTiming));
    return 0;
}

// A mask request while recording: a new slot, handed back like a queue hit.
static int graph_mask_slot(size_t n, double p, MaskPrefetch* hit) {
    MaskPrefetch e = MaskPrefetch();
    e.n = n;
    e.p = p;
    void* a = nullptr;
    void* a2 = nullptr;
    void* b = nullptr;
    int st = pool_alloc_raw(n * sizeof(float), &a);
    e.staging = static_cast<float*>(a);
    if (st == 0) st = pool_alloc_raw(n * sizeof(float), &a2);
    e.next = static_cast<float*>(a2);
    if (st == 0) st = pool_alloc_raw(sizeof(RngState), &b);
    e.before = static_cast<RngState*>(b);
    if (st != 0) { free_entry(e); return st; }
    *hit = e;
    return 0;
}

// The recorded main stream has enqueued its read of the slot's staging buffer: the slot joins the recording.
static int graph_mask_redraw(MaskPrefetch& e) {
    g_graph_masks[g_recording_masks].slots.push_back(e);
    return 0;
}

// masks of up to kMaxSlotCopies slots from their parts of one raw draw, in one launch (grid.y = slot)
constexpr int kMaxSlotCopies = 16;
struct SlotMasks { const uint32_t* raw[kMaxSlotCopies]; float* mask[kMaxSlotCopies]; size_t n[kMaxSlotCopies]; double p[kMaxSlotCopies]; };
__global__ __launch_bounds__(kBlock) void raw_to_masks_kernel(SlotMasks c) {
    const size_t n = c.n[blockIdx.y];
    const size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= n) return;
    const double p = c.p[blockIdx.y];
    uint64_t threshold;
    if (!(p > 0.0)) threshold = 0;
    else if (p >= 1.0) threshold = ~static_cast<uint64_t>(0);
    else threshold = static_cast<uint64_t>(ceil(p * 9007199254740992.0));
    c.mask[blockIdx.y][i] = raw_to_k53(c.raw[blockIdx.y], i) < threshold ? 1.0f : 0.0f;
}

// One round of the slots' masks, drawn on `stream` into their `next` (or `staging`) buffers; the first
// slot's snapshot receives the generator state from before the round.
static int launch_graph_masks(hipStream_t stream, GraphMasks& gm, bool into_next) {
    launch_raw_words(stream, gm.raw, gm.words, gm.slots.front().before, true);
    size_t offset = 0;
    for (size_t first = 0; first < gm.slots.size(); first += kMaxSlotCopies) {
        SlotMasks c = SlotMasks();
        size_t most = 0;
        const size_t count = gm.slots.size() - first < static_cast<size_t>(kMaxSlotCopies) ? gm.slots.size() - first : kMaxSlotCopies;
        for (size_t k = 0; k < count; ++k) {
            const MaskPrefetch& e = gm.slots[first + k];
            c.raw[k] = gm.raw + offset;
            c.mask[k] = into_next ? e.next : e.staging;
            c.n[k] = e.n;
            c.p[k] = e.p;
            offset += 2 * e.n;
            most = e.n > most ? e.n : most;
        }
        hipLaunchKernelGGL(raw_to_masks_kernel, dim3(static_cast<unsigned>(ceil_div(static_cast<int64_t>(most), kBlock)),
                                                     static_cast<unsigned>(count)), dim3(kBlock), 0, stream, c);
    }
    return check_launch("masks of a recorded step");
}

// next -> staging for up to kMaxSlotCopies slots in one launch (grid.y = slot)
struct SlotCopies { const float* src[kMaxSlotCopies]; float* dst[kMaxSlotCopies]; size_t n[kMaxSlotCopies]; };
__global__ __launch_bounds__(kBlock) void slot_copy_kernel(SlotCopies c) {
    const float* src = c.src[blockIdx.y];
    float* dst = c.dst[blockIdx.y];
    const size_t n = c.n[blockIdx.y];
    const size_t i = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) * 4;
    if (i >= n) return;
    if (i + 4 <= n) {                              // pool blocks: 256-byte aligned
        *reinterpret_cast<f4*>(dst + i) = *reinterpret_cast<const f4*>(src + i);
    } else {
        for (size_t j = i; j < n; ++j) dst[j] = src[j];
    }
}


// ------------------------------ look-ahead rounds ------------------------------
struct Round {
    GraphMasks gm;                    // the round's masks: slots (n, p, staging), raw words, snapshot in slots.front().before
    hipEvent_t ready = nullptr;       // second stream: the masks are in the slots' staging buffers
    hipEvent_t consumed = nullptr;    // main stream: the round's last mask has been read
    bool drawn = false;               // the draw is enqueued and not yet used up
    bool read = false;                // `consumed` has been recorded
};
static Round g_round[2];
static int g_round_cur = 0;           // the round being handed out
static size_t g_round_cursor = 0;     // its next slot
static bool g_lookahead = false;

static void free_round(Round& r) {
    for (MaskPrefetch& e : r.gm.slots) free_entry(e);
    if (r.gm.raw) pool_free_raw(r.gm.raw);
    if (r.ready) (void)hipEventDestroy(r.ready);
    if (r.consumed) (void)hipEventDestroy(r.consumed);
    r = Round();
}

// Enqueues the draw of round r on the second stream, which owns the generator while rounds are in use.
static int draw_round(Round& r) {
    if (r.read) BSHIP_HIP(hipStreamWaitEvent(g_side, r.consumed, 0));    // its buffers were read on the main stream
    int st = launch_graph_masks(g_side, r.gm, false);
    if (st != 0) return st;
    BSHIP_HIP(hipEventRecord(r.ready, g_side));
    r.drawn = true;
    return 0;
}

static int prefetch_flush(bool restore_position, bool wrong_guess) {
    g_history.clear();
    if (!g_lookahead) return 0;
    Round& cur = g_round[g_round_cur];
    // "A B B" looks like period 1 after its second B: when a guess turns out wrong, only
    // longer periods are tried next (any multiple of the true period serves as well)
    const size_t period = cur.gm.slots.size();
    if (wrong_guess) g_min_period = period + 1 > kMaxPeriod ? 1 : period + 1;
    int st = order_streams(g_side, ctx().stream);
    if (st == 0 && restore_position && cur.drawn) {
        hipLaunchKernelGGL(rng_copy_state_kernel, dim3(1), dim3(kBlock), 0, ctx().stream,
                           cur.gm.slots.front().before, g_state);
        st = check_launch("random stream rewind");
        size_t used = 0;
        for (size_t k = 0; k < g_round_cursor; ++k) used += 2 * cur.gm.slots[k].n;
        if (st == 0 && used > 0) {
            // the masks already handed out: their words again (into the round's own buffer, which
            // nobody reads any more), so that the generator stands right behind them
            hipLaunchKernelGGL(mt_raw_kernel, dim3(1), dim3(kRawThreads), 0, ctx().stream, g_state, cur.gm.raw,
                               used, static_cast<RngState*>(nullptr));
            st = check_launch("random stream rewind");
        }
    }
    // the blocks go back to the pool; their next owners run on the main stream, which is
    // ordered behind the second stream now
    free_round(g_round[0]);
    free_round(g_round[1]);
    g_lookahead = false;
    g_round_cur = 0;
    g_round_cursor = 0;
    return st;
}

// After a mask was drawn directly: if the recent requests repeat with period P, set up two
// rounds of P masks and draw the first. Failures here only mean "no look-ahead".
static void prefetch_maybe_start() {
    const size_t h = g_history.size();
    size_t period = 0;
    for (size_t P = g_min_period; P <= kMaxPeriod && 2 * P <= h; ++P) {
        bool same = true;
        for (size_t k = 0; k < P && same; ++k) same = g_history[h - 1 - k] == g_history[h - 1 - k - P];
        if (same) { period = P; break; }
    }
    if (h > 4 * kMaxPeriod) g_history.erase(g_history.begin(), g_history.begin() + (h - 2 * kMaxPeriod));
    if (period == 0) return;
    size_t total = 0;
    for (size_t k = 0; k < period; ++k) total += g_history[g_history.size() - period + k].first;
    if (2 * total > kMaxPrefetchFloats) return;
    if (ensure_side_stream() != 0) { (void)hipGetLastError(); return; }
    const std::vector<std::pair<size_t, double>> next(g_history.end() - period, g_history.end());
    bool ok = true;
    for (Round& r : g_round) {
        r = Round();
        for (const auto& req : next) {
            MaskPrefetch e = MaskPrefetch();
            e.n = req.first;
            e.p = req.second;
            void* a = nullptr;
            ok = ok && pool_alloc_raw(e.n * sizeof(float), &a) == 0;
            e.staging = static_cast<float*>(a);
            r.gm.slots.push_back(e);
            r.gm.words += 2 * e.n;
        }
        void* b = nullptr;
        void* w = nullptr;
        ok = ok && pool_alloc_raw(sizeof(RngState), &b) == 0;
        r.gm.slots.front().before = static_cast<RngState*>(b);
        ok = ok && pool_alloc_raw(r.gm.words * sizeof(uint32_t), &w) == 0;
        r.gm.raw = static_cast<uint32_t*>(w);
        ok = ok && hipEventCreateWithFlags(&r.ready, hipEventDisableTiming) == hipSuccess;
        ok = ok && hipEventCreateWithFlags(&r.consumed, hipEventDisableTiming) == hipSuccess;
    }
    // fresh pool blocks may still be in use by earlier main-stream work, and the generator passes
    // to the second stream: both are ordered here
    ok = ok && order_streams(ctx().stream, g_side) == 0;
    if (ok) {
        g_lookahead = true;          // from here on the second stream has run the generator ahead
        g_round_cur = 0;
        g_round_cursor = 0;
        ok = draw_round(g_round[0]) == 0;
        if (!ok) (void)prefetch_flush(g_round[0].drawn);
        return;
    }
    (void)hipGetLastError();
    free_round(g_round[0]);
    free_round(g_round[1]);
}

int rng_graph_begin(int id) {
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    int st = ensure_side_stream();
    if (st == 0 && g_state) st = prefetch_flush(true);
    if (st == 0 && g_state) st = graph_masks_unprime();
    if (st != 0) return st;
    g_recording_masks = id;
    g_graph_masks[id] = GraphMasks();
    g_graph_masks[id].generator = g_current_generator;
    return 0;
}

// The recording is complete: one buffer for the raw words of a round of its masks (a block of the recording's own).
int rng_graph_end(int id) {
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    g_recording_masks = 0;
    auto it = g_graph_masks.find(id);
    if (it == g_graph_masks.end() || it->second.slots.empty()) return 0;
    GraphMasks& gm = it->second;
    gm.words = 0;
    for (const MaskPrefetch& e : gm.slots) gm.words += 2 * e.n;
    void* r = nullptr;
    int st = pool_alloc_raw(gm.words * sizeof(uint32_t), &r);
    gm.raw = static_cast<uint32_t*>(r);
    return st;
}

int rng_graph_before_launch(int id) {
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    auto it = g_graph_masks.find(id);
    if (it == g_graph_masks.end() || it->second.slots.empty()) return 0;
    {
        int st = select_generator_locked(it->second.generator);
        if (st != 0) return st;
    }
    if (g_primed_graph != id) {
        int st = prefetch_flush(true);
        if (st == 0) st = graph_masks_unprime();
        if (st != 0) return st;
        st = launch_graph_masks(ctx().stream, it->second, false);
        if (st != 0) return st;
        it->second.primed = true;
        g_primed_graph = id;
    }
    return check_hip(hipEventRecord(g_before_graph, ctx().stream), "hipEventRecord");
}

// The graph of recording `id` has just been enqueued on the main stream: next to it, the second
// stream draws the masks of the replay after this one; behind it, they move into place.
static int draw_next_round(GraphMasks& gm) {
    std::vector<MaskPrefetch>& slots = gm.slots;
    // the second stream starts behind everything that preceded the graph on the main stream: the
    // priming draws, or the previous replay's copy out of the `next` buffers
    BSHIP_HIP(hipStreamWaitEvent(g_side, g_before_graph, 0));
    int st = launch_graph_masks(g_side, gm, true);
    if (st != 0) return st;
    st = order_streams(g_side, ctx().stream);
    for (size_t first = 0; st == 0 && first < slots.size(); first += kMaxSlotCopies) {
        SlotCopies c = SlotCopies();
        size_t most = 0;
        const size_t count = slots.size() - first < static_cast<size_t>(kMaxSlotCopies) ? slots.size() - first : kMaxSlotCopies;
        for (size_t k = 0; k < count; ++k) {
            c.src[k] = slots[first + k].next;
            c.dst[k] = slots[first + k].staging;
            c.n[k] = slots[first + k].n;
            most = c.n[k] > most ? c.n[k] : most;
        }
        const size_t tiles = (most + static_cast<size_t>(kBlock) * 4 - 1) / (static_cast<size_t>(kBlock) * 4);
        hipLaunchKernelGGL(slot_copy_kernel, dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(count)),
                           dim3(kBlock), 0, ctx().stream, c);
        st = check_launch("masks of the next replay, move into place");
    }
    return st;
}

int rng_graph_after_launch(int id) {
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    auto it = g_graph_masks.find(id);
    if (it == g_graph_masks.end() || it->second.slots.empty()) return 0;
    const int st = draw_next_round(it->second);
    if (st != 0) {
        // the staging buffers were not refilled: the next replay must not consume them again
        it->second.primed = false;
        if (g_primed_graph == id) g_primed_graph = 0;
    }
    return st;
}

void rng_graph_destroyed(int id) {
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    auto it = g_graph_masks.find(id);
    if (it == g_graph_masks.end()) return;
    if (g_primed_graph == id) (void)graph_masks_unprime();
    for (MaskPrefetch& e : it->second.slots) free_entry(e);
    if (it->second.raw) pool_free_raw(it->second.raw);
    g_graph_masks.erase(it);
}

// Serves a mask request: either hands back a drawn mask (*is_hit; the caller reads hit->staging on
// the main stream and then calls mask_end, or mask_abort if it could not), or draws the mask into
// `mask` directly.
static int mask_begin(float* mask, size_t n, double p, MaskPrefetch* hit, bool* is_hit, size_t cols = 0,
                      size_t ld = 0) {
    *is_hit = false;
    if (g_recording_masks) {
        *is_hit = true;
        return graph_mask_slot(n, p, hit);
    }
    int ust = graph_masks_unprime();
    if (ust != 0) return ust;
    if (g_lookahead) {
        Round& cur = g_round[g_round_cur];
        const MaskPrefetch& e = cur.gm.slots[g_round_cursor];
        if (e.n == n && e.p == p) {
            if (g_round_cursor == 0) {
                BSHIP_HIP(hipStreamWaitEvent(ctx().stream, cur.ready, 0));
                // the round after this one: drawn while this one is handed out
                int st = draw_round(g_round[g_round_cur ^ 1]);
                if (st != 0) { (void)prefetch_flush(true); return st; }
            }
            *hit = e;
            *is_hit = true;
            return 0;
        }
        int st = prefetch_flush(true, true);
        if (st != 0) return st;
    }
    void* raw = nullptr;
    int st = pool_alloc_raw(2 * n * sizeof(uint32_t), &raw);
    if (st != 0) return st;
    launch_mask(ctx().stream, mask, n, p, nullptr, static_cast<uint32_t*>(raw), cols, ld);
    st = check_launch("generate_probability_mask");
    pool_free_raw(raw);               // its next owner runs on this stream, after the two kernels
    if (st == 0 && prefetch_enabled()) {
        g_history.emplace_back(n, p);
        prefetch_maybe_start();
    }
    return st;
}

// The main stream has enqueued its read of the mask handed out by mask_begin.
static int mask_end(MaskPrefetch& e) {
    if (g_recording_masks) return graph_mask_redraw(e);
    Round& cur = g_round[g_round_cur];
    if (++g_round_cursor < cur.gm.slots.size()) return 0;
    // the round is used up: its buffers may be drawn into again once this read has run
    g_round_cursor = 0;
    cur.drawn = false;
    hipError_t err = hipEventRecord(cur.consumed, ctx().stream);
    cur.read = true;
    g_round_cur ^= 1;
    if (err != hipSuccess) {
        (void)prefetch_flush(true);
        return check_hip(err, "hipEventRecord");
    }
    return 0;
}

// The read of the mask handed out by mask_begin could not be enqueued.
static void mask_abort(MaskPrefetch& e) {
    if (g_recording_masks) free_entry(e);      // a slot of its own, not yet part of the recording
    // a round's slot stays where it is: the next request is served from it again
}

// Dropout forward (dropout_layer.py:41-45) behind the mask: mask = src (the mask as drawn),
// out = in * mask, out = scale * out.
template <bool AL>
__global__ __launch_bounds__(kBlock) void dropout_apply_kernel(const float* src, float* mask, const float* in,
                                                               float* out, float scale, size_t n) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) * 4;
    if (i >= n) return;
    if (i + 4 <= n) {
        const f4 m = vload<4, AL>(src + i);
        const f4 x = vload<4, AL>(in + i);
        if (src != mask) vstore<4, AL>(mask + i, m);
        f4 o;
#pragma unroll
        for (int k = 0; k < 4; ++k) { const float t = x[k] * m[k]; o[k] = scale * t; }
        vstore<4, AL>(out + i, o);
    } else {
        for (size_t j = i; j < n; ++j) {
            const float m = src[j];
            const float t = in[j] * m;
            mask[j] = m;
            out[j] = scale * t;
        }
    }
}

// ------------------------------ fast random stream ------------------------------
// Optional and NOT NumPy's stream: masks from the Philox4x32-10 counter-based generator
// (Salmon et al., SC'11). Every group of four mask elements is one generator block, a pure
// function of (key, block number), so a mask is one fully parallel streaming launch instead of
// the sequential MT19937 walk (0.08 ms per 100x1200 mask, the floor of an MLP step). The state
// (64-bit key and block counter) lives in device memory and is advanced by a one-lane kernel
// behind the mask kernel, so recorded steps draw fresh masks on every replay.
struct FastRngState {
    unsigned long long key;
    unsigned long long next_block;
};
static FastRngState* g_fast_state = nullptr;      // the selected generator's

struct Generator { RngState* state = nullptr; FastRngState* fast = nullptr; };
static std::map<int, Generator> g_generators = {{0, Generator()}};   // states of the generators NOT selected are kept here
static int g_next_generator = 1;

static int select_generator_locked(int id) {
    if (id == g_current_generator) return 0;
    if (g_generators.find(id) == g_generators.end())
        return set_error(BSHIP_ERR_BAD_DIMENSION, "random generator %d does not exist", id);
    if (g_recording_masks)
        return set_error(BSHIP_ERR_UNSUPPORTED, "another random generator cannot be selected while a step is being recorded");
    // what was drawn ahead belongs to the generator selected so far: back to its sequential position
    int st = g_state ? prefetch_flush(true) : 0;
    if (st == 0) st = graph_masks_unprime();
    if (st != 0) return st;
    g_min_period = 1;
    g_generators[g_current_generator] = Generator{g_state, g_fast_state};
    g_state = g_generators[id].state;
    g_fast_state = g_generators[id].fast;
    g_current_generator = id;
    return 0;
}

__device__ __forceinline__ void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c[0]), lo0 = 0xD2511F53u * c[0];
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c[2]), lo1 = 0xCD9E8D57u * c[2];
        const uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
        c[0] = n0; c[1] = lo1; c[2] = n2; c[3] = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

// mask[4b..4b+3] = (word j of block next_block + b) < threshold; with `in`: out = scale * (in * mask)
// as dropout_apply_kernel does. threshold in [0, 2^32].
template <bool APPLY>
__global__ __launch_bounds__(kBlock) void philox_mask_kernel(const FastRngState* st, float* mask, size_t n,
                                                             unsigned long long threshold, const float* in,
                                                             float* out, float scale) {
    const size_t b = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    const size_t i = b * 4;
    if (i >= n) return;
    const unsigned long long block = st->next_block + b;
    uint32_t c[4] = {static_cast<uint32_t>(block), static_cast<uint32_t>(block >> 32), 0u, 0u};
    philox4x32_10(c, static_cast<uint32_t>(st->key), static_cast<uint32_t>(st->key >> 32));
    float m[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) m[j] = c[j] < threshold ? 1.0f : 0.0f;
    const bool whole = i + 4 <= n;
    if (whole && (reinterpret_cast<uintptr_t>(mask + i) & 15u) == 0 &&
        (!APPLY || ((reinterpret_cast<uintptr_t>(in + i) | reinterpret_cast<uintptr_t>(out + i)) & 15u) == 0)) {
        const f4 mv = {m[0], m[1], m[2], m[3]};
        if (APPLY) {
            const f4 x = *reinterpret_cast<const f4*>(in + i);
            f4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) { const float t = x[j] * m[j]; o[j] = scale * t; }
            *reinterpret_cast<f4*>(out + i) = o;
        }
        *reinterpret_cast<f4*>(mask + i) = mv;
    } else {
        for (int j = 0; j < 4 && i + j < n; ++j) {
            if (APPLY) { const float t = in[i + j] * m[j]; out[i + j] = scale * t; }
            mask[i + j] = m[j];
        }
    }
}

__global__ void philox_advance_kernel(FastRngState* st, unsigned long long blocks) {
    st->next_block += blocks;
}

static unsigned long long mask_threshold(double p) {
    double t = floor(p * 4294967296.0);
    if (!(t > 0.0)) t = 0.0;
    if (t > 4294967296.0) t = 4294967296.0;
    return static_cast<unsigned long long>(t);
}

static int launch_fast_mask(const float* in, float* mask, float* out, size_t n, double p, float scale) {
    const size_t blocks = (n + 3) / 4;
    const size_t groups = (blocks + kBlock - 1) / kBlock;
    if (groups > 0x7fffffffu) return set_error(BSHIP_ERR_BAD_DIMENSION, "mask: %zu elements exceed one launch", n);
    const dim3 grid(static_cast<unsigned>(groups));
    if (in)
        hipLaunchKernelGGL(philox_mask_kernel<true>, grid, dim3(kBlock), 0, ctx().stream, g_fast_state, mask, n,
                           mask_threshold(p), in, out, scale);
    else
        hipLaunchKernelGGL(philox_mask_kernel<false>, grid, dim3(kBlock), 0, ctx().stream, g_fast_state, mask, n,
                           mask_threshold(p), static_cast<const float*>(nullptr), static_cast<float*>(nullptr), 1.0f);
    hipLaunchKernelGGL(philox_advance_kernel, dim3(1), dim3(1), 0, ctx().stream, g_fast_state,
                       static_cast<unsigned long long>(blocks));
    return check_launch("fast mask");
}

void rng_release() {
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (g_side) (void)hipStreamSynchronize(g_side);
    free_round(g_round[0]);
    free_round(g_round[1]);
    g_lookahead = false;
    g_round_cur = 0;
    g_round_cursor = 0;
    for (auto& kv : g_graph_masks) {
        for (MaskPrefetch& e : kv.second.slots) free_entry(e);
        if (kv.second.raw) pool_free_raw(kv.second.raw);
    }
    g_graph_masks.clear();
    g_primed_graph = 0;
    g_recording_masks = 0;
    g_history.clear();
    g_min_period = 1;
    if (g_join) { (void)hipEventDestroy(g_join); g_join = nullptr; }
    if (g_before_graph) { (void)hipEventDestroy(g_before_graph); g_before_graph = nullptr; }

    if (g_side) { (void)hipStreamDestroy(g_side); g_side = nullptr; }
    g_generators[g_current_generator] = Generator{g_state, g_fast_state};
    for (auto& kv : g_generators) {
        if (kv.second.state) pool_free_raw(kv.second.state);
        if (kv.second.fast) pool_free_raw(kv.second.fast);
    }
    g_generators.clear();
    g_generators[0] = Generator();
    g_current_generator = 0;
    g_next_generator = 1;
    g_state = nullptr;
    g_fast_state = nullptr;
    for (auto& kv : g_jump_polys) (void)hipFree(kv.second.dev);
    g_jump_polys.clear();
    for (uint32_t* p : g_jump_retired) (void)hipFree(p);
    g_jump_retired.clear();
    if (g_hist) { (void)hipFree(g_hist); g_hist = nullptr; }
    if (g_seeds) { (void)hipFree(g_seeds); g_seeds = nullptr; }
}

}  // namespace bship

using namespace bship;

// The drawing and state operations. generator >= 0: that generator is selected first, under the same
// lock as the operation itself, so that two handlers used from two threads cannot come between
// another handler's selection and its draw; generator < 0: the generator selected last.
static int rng_seed_impl(int generator, uint32_t seed) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    int st = rng_ensure_state();
    if (st == 0) st = prefetch_flush(false);
    if (st == 0) st = graph_masks_unprime();
    if (st != 0) return st;
    // init_genrand of the MT19937 reference code, as used by RandomState(int)
    RngState h;
    h.key[0] = seed;
    for (int i = 1; i < kMtN; ++i)
        h.key[i] = 1812433253u * (h.key[i - 1] ^ (h.key[i - 1] >> 30)) + static_cast<uint32_t>(i);
    h.pos = kMtN;
    h.has_gauss = 0;
    h.gauss = 0.0;
    return bship_h2d(g_state, &h, sizeof(RngState));
}

static int rng_get_state_impl(int generator, uint32_t* key_host, int* pos_host, int* has_gauss_host, double* gauss_host) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_state) return set_error(BSHIP_ERR_NOT_INITIALIZED, "bship_rng_get_state: bship_rng_seed() has not been called");
    RngState h;
    int st = prefetch_flush(true);
    if (st == 0) st = graph_masks_unprime();
    if (st == 0) st = bship_d2h(&h, g_state, sizeof(RngState));
    if (st != 0) return st;
    if (key_host) for (int i = 0; i < kMtN; ++i) key_host[i] = h.key[i];
    if (pos_host) *pos_host = h.pos;
    if (has_gauss_host) *has_gauss_host = h.has_gauss;
    if (gauss_host) *gauss_host = h.gauss;
    return 0;
}

static int prob_mask_pitched_f32_impl(int generator, float* mask, int64_t ld_mask, int64_t rows, int64_t cols, double p) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(rows >= 0 && cols >= 0 && ld_mask >= cols);
    const size_t n = static_cast<size_t>(rows) * static_cast<size_t>(cols);
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(mask);
    BSHIP_REQUIRE_F32_ALIGNED(mask);
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_state) return set_error(BSHIP_ERR_NOT_INITIALIZED, "%s: bship_rng_seed() has not been called", "bship_prob_mask_pitched_f32");
    MaskPrefetch hit;
    bool is_hit = false;
    int st = mask_begin(mask, n, p, &hit, &is_hit, static_cast<size_t>(cols), static_cast<size_t>(ld_mask));
    if (st != 0 || !is_hit) return st;
    st = bship_copy2d_f32(mask, ld_mask, hit.staging, cols, rows, cols);
    if (st != 0) { mask_abort(hit); return st; }
    return mask_end(hit);
}

static int dropout_fwd_f32_impl(int generator, const float* in, float* mask, float* out, size_t n, double keep_probability,
                          float scale) {
    BSHIP_REQUIRE_INIT();
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(mask);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(in);
    BSHIP_REQUIRE_F32_ALIGNED(mask);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    const size_t tiles = (n + static_cast<size_t>(kBlock) * 4 - 1) / (static_cast<size_t>(kBlock) * 4);
    if (tiles > 0x7fffffffu) return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: %zu elements exceed one launch", "bship_dropout_fwd_f32", n);
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_state) return set_error(BSHIP_ERR_NOT_INITIALIZED, "bship_dropout_fwd_f32: bship_rng_seed() has not been called");
    MaskPrefetch hit;
    bool is_hit = false;
    int st = mask_begin(mask, n, keep_probability, &hit, &is_hit);
    if (st != 0) return st;
    const float* src = is_hit ? hit.staging : mask;
    const dim3 grid(static_cast<unsigned>(tiles)), blk(kBlock);
    if (aligned16(src) && aligned16(mask) && aligned16(in) && aligned16(out))
        hipLaunchKernelGGL(dropout_apply_kernel<true>, grid, blk, 0, ctx().stream, src, mask, in, out, scale, n);
    else
        hipLaunchKernelGGL(dropout_apply_kernel<false>, grid, blk, 0, ctx().stream, src, mask, in, out, scale, n);
    st = check_launch("dropout_forward");
    if (is_hit) {
        if (st != 0) { mask_abort(hit); return st; }
        st = mask_end(hit);
    }
    return st;
}

static int fill_gaussian_f32_impl(int generator, float* out, size_t n, double mean, double stdv) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_state) return set_error(BSHIP_ERR_NOT_INITIALIZED, "bship_fill_gaussian_f32: bship_rng_seed() has not been called");
    hipStream_t s = ctx().stream;
    int st = prefetch_flush(true);
    if (st == 0) st = graph_masks_unprime();
    if (st != 0) return st;
    // device scalars: [0] trials consumed, [1] outputs written, [2] outputs taken from the cache
    void* rp = nullptr;
    st = pool_alloc_raw(3 * sizeof(unsigned long long), &rp);
    if (st != 0) return st;
    unsigned long long* result = static_cast<unsigned long long*>(rp);
    void* snap_p = nullptr;
    st = pool_alloc_raw(sizeof(RngState), &snap_p);
    if (st != 0) { pool_free_raw(rp); return st; }
    RngState* snap = static_cast<RngState*>(snap_p);

    hipLaunchKernelGGL(gauss_cache_kernel, dim3(1), dim3(64), 0, s, g_state, out, n, mean, stdv, result);
    st = check_launch("fill_gaussian cache");
    unsigned long long host_res[3] = {0, 0, 0};
    if (st == 0) st = bship_d2h(host_res, result, sizeof(host_res));
    size_t produced = static_cast<size_t>(host_res[2]);
    while (st == 0 && produced < n) {
        // Acceptance rate is pi/4; draw a generous batch of trials, then rewind the
        // generator to exactly the number of trials the sequential algorithm consumes.
        const size_t need = (n - produced + 1) / 2;
        const size_t trials = need + need / 2 + 1024;
        void* up = nullptr;
        st = pool_alloc_raw(2 * trials * sizeof(double), &up);
        if (st != 0) break;
        double* u = static_cast<double*>(up);
        void* rawp = nullptr;
        st = pool_alloc_raw(4 * trials * sizeof(uint32_t), &rawp);
        if (st != 0) { pool_free_raw(up); break; }
        uint32_t* raw = static_cast<uint32_t*>(rawp);
        hipLaunchKernelGGL(rng_copy_state_kernel, dim3(1), dim3(kBlock), 0, s, g_state, snap);
        launch_doubles(u, 2 * trials, raw);
        hipLaunchKernelGGL(gauss_polar_kernel, dim3(1), dim3(kBlock), 0, s, g_state, u, trials, out, n,
                           produced, mean, stdv, result);
        st = check_launch("fill_gaussian");
        if (st == 0) st = bship_d2h(host_res, result, sizeof(host_res));
        if (st == 0) {
            const size_t used = static_cast<size_t>(host_res[0]);
            produced = static_cast<size_t>(host_res[1]);
            if (used < trials) {
                // rewind: restore the snapshot and skip exactly 2*used doubles
                hipLaunchKernelGGL(rng_copy_state_kernel, dim3(1), dim3(kBlock), 0, s, snap, g_state);
                if (used > 0)      // only the position matters: the words go to the scratch again
                    hipLaunchKernelGGL(mt_raw_kernel, dim3(1), dim3(kRawThreads), 0, s, g_state, raw, 4 * used,
                                       static_cast<RngState*>(nullptr));
                st = check_launch("fill_gaussian rewind");
            }
        }
        pool_free_raw(rawp);
        pool_free_raw(up);
    }
    pool_free_raw(snap_p);
    pool_free_raw(rp);
    if (st == 0) st = bship_sync();
    return st;
}

static int fast_rng_seed_impl(int generator, unsigned long long seed) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_fast_state) {
        void* p = nullptr;
        int st = pool_alloc_raw(sizeof(FastRngState), &p);
        if (st != 0) return st;
        g_fast_state = static_cast<FastRngState*>(p);
    }
    const FastRngState h = {seed, 0ull};
    return bship_h2d(g_fast_state, &h, sizeof(h));
}

static int fast_rng_get_state_impl(int generator, unsigned long long* seed_host, unsigned long long* next_block_host) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_fast_state) return set_error(BSHIP_ERR_NOT_INITIALIZED, "bship_fast_rng_get_state: bship_fast_rng_seed() has not been called");
    FastRngState h;
    int st = bship_d2h(&h, g_fast_state, sizeof(h));
    if (st != 0) return st;
    if (seed_host) *seed_host = h.key;
    if (next_block_host) *next_block_host = h.next_block;
    return 0;
}

static int prob_mask_fast_f32_impl(int generator, float* mask, size_t n, double p) {
    BSHIP_REQUIRE_INIT();
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(mask);
    BSHIP_REQUIRE_F32_ALIGNED(mask);
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_fast_state) return set_error(BSHIP_ERR_NOT_INITIALIZED, "bship_prob_mask_fast_f32: bship_fast_rng_seed() has not been called");
    return launch_fast_mask(nullptr, mask, nullptr, n, p, 1.0f);
}

static int dropout_fwd_fast_f32_impl(int generator, const float* in, float* mask, float* out, size_t n, double keep_probability,
                               float scale) {
    BSHIP_REQUIRE_INIT();
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(mask);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(in);
    BSHIP_REQUIRE_F32_ALIGNED(mask);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator >= 0) {
        int sel_st = select_generator_locked(generator);
        if (sel_st != 0) return sel_st;
    }
    if (!g_fast_state) return set_error(BSHIP_ERR_NOT_INITIALIZED, "bship_dropout_fwd_fast_f32: bship_fast_rng_seed() has not been called");
    return launch_fast_mask(in, mask, out, n, keep_probability, scale);
}

extern "C" {

int bship_rng_create(int* generator_id) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_PTR(generator_id);
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    *generator_id = g_next_generator++;
    g_generators[*generator_id] = Generator();
    return 0;
}

int bship_rng_select(int generator_id) {
    BSHIP_REQUIRE_INIT_NO_FLUSH();
    {
        std::lock_guard<std::mutex> lock(g_rng_mutex);
        if (generator_id == g_current_generator) return 0;
    }
    BSHIP_FLUSH_PENDING();       // masks that the fusing window holds are drawn from the generator selected so far
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    return select_generator_locked(generator_id);
}

int bship_rng_destroy(int generator_id) {
    BSHIP_REQUIRE_INIT();
    std::lock_guard<std::mutex> lock(g_rng_mutex);
    WindowBypass bypass;      // entry points called from here neither flush nor feed the fusing window (lock order)
    if (generator_id == 0) return set_error(BSHIP_ERR_BAD_DIMENSION, "bship_rng_destroy: generator 0 is the library's own");
    if (g_generators.find(generator_id) == g_generators.end())
        return set_error(BSHIP_ERR_BAD_DIMENSION, "bship_rng_destroy: generator %d does not exist", generator_id);
    if (generator_id == g_current_generator) {
        int st = select_generator_locked(0);
        if (st != 0) return st;
    }
    // the blocks' next owners run on the library's stream, behind every kernel that used them
    const Generator g = g_generators[generator_id];
    if (g.state) pool_free_raw(g.state);
    if (g.fast) pool_free_raw(g.fast);
    g_generators.erase(generator_id);
    return 0;
}

int bship_rng_seed(uint32_t seed) { return rng_seed_impl(-1, seed); }

int bship_rng_seed_on(int generator, uint32_t seed) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return rng_seed_impl(generator, seed);
}

int bship_rng_get_state(uint32_t* key_host, int* pos_host, int* has_gauss_host, double* gauss_host) { return rng_get_state_impl(-1, key_host, pos_host, has_gauss_host, gauss_host); }

int bship_rng_get_state_on(int generator, uint32_t* key_host, int* pos_host, int* has_gauss_host, double* gauss_host) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return rng_get_state_impl(generator, key_host, pos_host, has_gauss_host, gauss_host);
}

// A dense mask may be the first call of a dropout layer's sequence (dropout_layer.py:41-45): it goes
// through the fusing window. generator < 0: the generator selected when the mask is drawn
// (bship_rng_select enqueues what the window holds before it selects another one).
static int dense_mask(int generator, float* mask, size_t n, double p, bool fast) {
    if (window_takes()) {
        BSHIP_REQUIRE_INIT_NO_FLUSH();
        if (n == 0) return 0;
        BSHIP_REQUIRE_PTR(mask);
        BSHIP_REQUIRE_F32_ALIGNED(mask);
        return window_push(window::rec_mask(mask, n, p, generator, fast));
    }
    if (fast) return prob_mask_fast_f32_impl(generator, mask, n, p);
    return prob_mask_pitched_f32_impl(generator, mask, static_cast<int64_t>(n), 1, static_cast<int64_t>(n), p);
}

int bship_prob_mask_f32(float* mask, size_t n, double p) { return dense_mask(-1, mask, n, p, false); }

int bship_prob_mask_on_f32(int generator, float* mask, size_t n, double p) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return dense_mask(generator, mask, n, p, false);
}

int bship_prob_mask_pitched_f32(float* mask, int64_t ld_mask, int64_t rows, int64_t cols, double p) { return prob_mask_pitched_f32_impl(-1, mask, ld_mask, rows, cols, p); }

int bship_prob_mask_pitched_on_f32(int generator, float* mask, int64_t ld_mask, int64_t rows, int64_t cols, double p) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return prob_mask_pitched_f32_impl(generator, mask, ld_mask, rows, cols, p);
}

int bship_dropout_fwd_f32(const float* in, float* mask, float* out, size_t n, double keep_probability,
                          float scale) { return dropout_fwd_f32_impl(-1, in, mask, out, n, keep_probability, scale); }

int bship_dropout_fwd_on_f32(int generator, const float* in, float* mask, float* out, size_t n, double keep_probability,
                          float scale) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return dropout_fwd_f32_impl(generator, in, mask, out, n, keep_probability, scale);
}

int bship_fill_gaussian_f32(float* out, size_t n, double mean, double stdv) { return fill_gaussian_f32_impl(-1, out, n, mean, stdv); }

int bship_fill_gaussian_on_f32(int generator, float* out, size_t n, double mean, double stdv) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return fill_gaussian_f32_impl(generator, out, n, mean, stdv);
}

int bship_fast_rng_seed(unsigned long long seed) { return fast_rng_seed_impl(-1, seed); }

int bship_fast_rng_seed_on(int generator, unsigned long long seed) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return fast_rng_seed_impl(generator, seed);
}

int bship_fast_rng_get_state(unsigned long long* seed_host, unsigned long long* next_block_host) { return fast_rng_get_state_impl(-1, seed_host, next_block_host); }

int bship_fast_rng_get_state_on(int generator, unsigned long long* seed_host, unsigned long long* next_block_host) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return fast_rng_get_state_impl(generator, seed_host, next_block_host);
}

int bship_prob_mask_fast_f32(float* mask, size_t n, double p) { return dense_mask(-1, mask, n, p, true); }

int bship_prob_mask_fast_on_f32(int generator, float* mask, size_t n, double p) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return dense_mask(generator, mask, n, p, true);
}

int bship_dropout_fwd_fast_f32(const float* in, float* mask, float* out, size_t n, double keep_probability,
                               float scale) { return dropout_fwd_fast_f32_impl(-1, in, mask, out, n, keep_probability, scale); }

int bship_dropout_fwd_fast_on_f32(int generator, const float* in, float* mask, float* out, size_t n, double keep_probability,
                               float scale) {
    BSHIP_REQUIRE_DIM(generator >= 0);
    return dropout_fwd_fast_f32_impl(generator, in, mask, out, n, keep_probability, scale);
}

}  // extern "C"
