// Convolutions whose filters are thin (kh * kw * channels <= 128: the first layer of an image network,
// 5 x 5 x 3 = 75) without the col matrix.
//
// conv2d_forward_batch / conv2d_backward_batch (numpy_handler.py:110-171) build, per image, the matrix
// of all filter windows (_cpuop.pyx:251-309) and multiply it with the weights: for 100 images of 32 x 32 x 3
// that matrix is 30 MB, written and read three times per training step for products of 0.5 GFLOP each. Here
// a workgroup stages the rows of ONE image that a band of output rows looks at in LDS once (a few KB), and
// the matrix cores read the windows straight out of that copy: v_mfma_f32_16x16x4f32 takes A[l % 16][l / 16]
// and B[l / 16][l % 16] from lane l, so "row i of the col matrix at column k" is just the LDS word at
// pixel_offset(i) + window_offset(k), two additions on per-lane constants.
//
//   forward   out[p][f]  = sum_k col[p][k] W[f][k] + bias[f]       tiles: 16 pixels x 16 filters, k in steps of 4
//   weights   dW[f][k]   = sum_p dy[p][f] col[p][k]                tiles: 16 filters x 16 window entries, p in steps
//             db[f]      = sum_p dy[p][f]                          of 4; column K of the same tiles is a column of ones
//   inputs    dcol[p][k] = sum_f dy[p][f] W[f][k]  into LDS,       tiles: 16 pixels x 16 window entries, f in steps of 4
//             dx[y][x][c] += the kh * kw entries of dcol that window (y, x, c) lies in
//
// Sums inside a product are float32 accumulations of the matrix cores in k order (forward), pixel order
// (weights) and filter order (inputs); the handler's bar for products is 1e-5 relative to the result's scale,
// as for the hipBLASLt path. Nothing depends on which workgroup finishes first: the weights' deltas are
// per-workgroup partial sums in a scratch buffer that a second kernel adds in workgroup order, and every element
// of the inputs' deltas is summed by one thread in a fixed order. With finite operands, that is: where a tile has
// fewer than 16 pixels the spare rows are multiplied by zero, which an infinity in the image turns into NaN
// (is_fully_finite reports either).
//
// Taken for stride 1, any padding, kh * kw * c <= 128 (127 backward: the bias takes a window entry), filters a
// multiple of 16 up to 64, and images whose band fits the LDS; everything else returns BSHIP_ERR_UNSUPPORTED
// with nothing launched and the caller takes the im2col path.
#include "common.h"

#include <algorithm>
#include <cmath>
#include <mutex>

namespace bship {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kThinMaxK = 128;
constexpr int kThinMaxF = 64;
constexpr int kThinThreads = 256;

struct ThinGeom {
    int h, w, c, f, kh, kw, pad;
    int oh, ow;
    int K;            // kh * kw * c
    int rows;         // output rows per band
    int bands;        // bands per image
    int bw;           // columns of the staged band: w + 2 * pad
    int br;           // rows of the staged band: rows + kh - 1
    FastDiv by_band_row, by_c, by_ow, by_K, by_window_row;      // divisions by bw * c, c, ow, K, kw * c
};

// window entry k = (ky * kw + kx) * c + ch lies this many floats behind a pixel's first window entry in the band
__device__ __forceinline__ int window_offset(const ThinGeom& g, int k) {
    uint32_t ky, rest;
    g.by_window_row.divmod(static_cast<uint32_t>(k), ky, rest);
    return static_cast<int>(ky) * g.bw * g.c + static_cast<int>(rest);            // kx * c + ch = rest
}

// Global loads of a staging loop are requested kStageAhead per lane before the first is used: a loop of
// dependent load-store pairs would pay a memory round trip per iteration.
constexpr int kStageAhead = 8;
constexpr int kStageChunk = kThinThreads * kStageAhead;

// Elements [c0, c0 + kStageChunk) of the band: the image rows [y0 - pad, y0 - pad + br) x all columns, zero beyond
// the image.
__device__ __forceinline__ void band_chunk_load(const FastDiv& by_band_row, const FastDiv& by_c, int pad, int h, int w, int c,
                                                const float* __restrict__ src, int y0, int c0, int total,
                                                float (&v)[kStageAhead]) {
#pragma unroll
    for (int u = 0; u < kStageAhead; ++u) {
        const int i = c0 + threadIdx.x + u * kThinThreads;
        uint32_t by, rest, bx, ch;
        by_band_row.divmod(static_cast<uint32_t>(i < total ? i : 0), by, rest);
        by_c.divmod(rest, bx, ch);
        const int y = y0 - pad + static_cast<int>(by), x = static_cast<int>(bx) - pad;
        const bool inside = i < total && y >= 0 && y < h && x >= 0 && x < w;
        const int64_t at = inside ? (static_cast<int64_t>(y) * w + x) * c + ch : 0;
        const float loaded = src[at];                  // element 0 of the image for the lanes with nothing to fetch
        v[u] = inside ? loaded : 0.0f;
    }
}

__device__ __forceinline__ void chunk_store(float* dst, int c0, int total, const float (&v)[kStageAhead]) {
#pragma unroll
    for (int u = 0; u < kStageAhead; ++u) {
        const int i = c0 + threadIdx.x + u * kThinThreads;
        if (i < total) dst[i] = v[u];
    }
}

__device__ __forceinline__ void flat_chunk_load(const float* __restrict__ src, int c0, int total, float (&v)[kStageAhead]) {
#pragma unroll
    for (int u = 0; u < kStageAhead; ++u) {
        const int i = c0 + threadIdx.x + u * kThinThreads;
        v[u] = src[i < total ? i : 0];
    }
}

// ------------------------------------------------------------------ forward
// LDS: band | window offsets (K4) | weights transposed wt[k][f] with a row pitch of f + 1 (zero rows from K on)
constexpr int kFwdTogether = 4;      // pixel tiles a wavefront works on at once: independent accumulation chains

// T pixel tiles pt0, pt0 + pstride, ... against one tile of 16 filters. Per step the lane needs its weight
// wt[4 s + q4][filter] and the offset of window entry 4 s + q4; both come from LDS one step ahead of the
// products that use them (the offset two steps ahead, since the image value's address needs it), and the reads
// of a step are requested before the products of the step before are issued. Only the last step can hold
// entries from K on (their weights are zero); there the lane reads the pixel's first entry and replaces it by
// zero, so that an infinity in the image stays out of windows it is not in. (Reading four steps ahead, or
// computing the offsets instead of reading them, was measured slower: the loop is bound by the instructions
// issued per product, not by the LDS latency.)
template <int T>
__device__ __forceinline__ void fwd_tiles(const ThinGeom& g, const float* band, const int* kq, const float* wcol, int wpitch,
                                          int steps, bool beyond, int pt0, int pstride, int pixels, int m, int q4,
                                          float bias_f, float* __restrict__ out_col) {
    int base[T];
    v4f acc[T];
#pragma unroll
    for (int u = 0; u < T; ++u) {
        // rows of a tile beyond the band's pixels are computed from pixel 0's windows and never stored
        int p = (pt0 + u * pstride) * 16 + m;
        p = p < pixels ? p : 0;
        uint32_t py, px;
        g.by_ow.divmod(static_cast<uint32_t>(p), py, px);
        base[u] = static_cast<int>(py * g.bw + px) * g.c;
        acc[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
    float a_next[T];
    float b_next = wcol[0];
    int k_after = kq[4 * min(1, steps - 1)];
    {
        const int k_first = kq[0];
#pragma unroll
        for (int u = 0; u < T; ++u) a_next[u] = band[base[u] + k_first];
    }
    for (int s = 0; s < steps; ++s) {
        float a_now[T];
        const bool drop = beyond && s == steps - 1;
#pragma unroll
        for (int u = 0; u < T; ++u) a_now[u] = drop ? 0.0f : a_next[u];
        const float b_now = b_next;
        const int k_next = k_after;
        __builtin_amdgcn_sched_barrier(0);
        b_next = wcol[min(s + 1, steps - 1) * 4 * wpitch];
        k_after = kq[4 * min(s + 2, steps - 1)];
#pragma unroll
        for (int u = 0; u < T; ++u) a_next[u] = band[base[u] + k_next];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < T; ++u) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_now[u], b_now, acc[u], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
    // component q: pixel tile * 16 + 4 * (lane / 16) + q, filter ft * 16 + lane % 16
#pragma unroll
    for (int u = 0; u < T; ++u) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int pq = (pt0 + u * pstride) * 16 + 4 * q4 + q;
            if (pq < pixels) out_col[static_cast<int64_t>(pq) * g.f] = acc[u][q] + bias_f;
        }
    }
}

__global__ __launch_bounds__(kThinThreads) void conv_thin_fwd_kernel(ThinGeom g, const float* __restrict__ in,
                                                                     int64_t in_pitch, const float* __restrict__ W,
                                                                     const float* __restrict__ bias, float* __restrict__ out) {
    extern __shared__ float lds[];
    const int K4 = (g.K + 3) & ~3;
    const int wpitch = g.f + 1;
    const int band_floats = g.br * g.bw * g.c;
    float* band = lds;
    int* koff_all = reinterpret_cast<int*>(lds + band_floats);
    float* wt = lds + band_floats + K4;
    const int64_t img = blockIdx.x / g.bands;
    const int y0 = static_cast<int>(blockIdx.x % g.bands) * g.rows;
    const float* src = in + img * in_pitch;
    const int w_floats = g.f * g.K;
    // the band and the weights (W is (f, K): read in order, stored transposed) are requested together
    for (int c = 0; c < max(band_floats, w_floats); c += kStageChunk) {
        float bv[kStageAhead], wv[kStageAhead];
        if (c < band_floats) band_chunk_load(g.by_band_row, g.by_c, g.pad, g.h, g.w, g.c, src, y0, c, band_floats, bv);
        if (c < w_floats) flat_chunk_load(W, c, w_floats, wv);
        if (c < band_floats) chunk_store(band, c, band_floats, bv);
        if (c < w_floats) {
#pragma unroll
            for (int u = 0; u < kStageAhead; ++u) {
                const int i = c + threadIdx.x + u * kThinThreads;
                uint32_t f, k;
                g.by_K.divmod(static_cast<uint32_t>(i), f, k);
                if (i < w_floats) wt[k * wpitch + f] = wv[u];
            }
        }
    }
    // the window offsets of all k < K4 (0 for the entries from K on): one division per entry and workgroup
    for (int k = threadIdx.x; k < K4; k += kThinThreads) koff_all[k] = k < g.K ? window_offset(g, k) : 0;
    for (int i = threadIdx.x; i < (K4 - g.K) * g.f; i += kThinThreads) wt[(g.K + i / g.f) * wpitch + i % g.f] = 0.0f;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 15, q4 = lane >> 4;
    const int ftiles = g.f / 16;
    const int ft = wave % ftiles;
    const int band_rows = min(g.rows, g.oh - y0);
    const int pixels = band_rows * g.ow;
    const int ptiles = (pixels + 15) / 16;
    const int steps = K4 / 4;
    const float* wcol = wt + q4 * wpitch + ft * 16 + m;
    const int* kq = koff_all + q4;
    const bool beyond = 4 * (steps - 1) + q4 >= g.K;
    const float bias_f = bias[ft * 16 + m];
    float* out_col = out + ((img * g.oh + y0) * g.ow) * static_cast<int64_t>(g.f) + ft * 16 + m;
    const int pstride = 4 / ftiles;                 // wavefronts that share a filter tile deal the pixel tiles among them
    int pt0 = wave / ftiles;
    for (; pt0 + (kFwdTogether - 1) * pstride < ptiles; pt0 += pstride * kFwdTogether)
        fwd_tiles<kFwdTogether>(g, band, kq, wcol, wpitch, steps, beyond, pt0, pstride, pixels, m, q4, bias_f, out_col);
    const int left = pt0 < ptiles ? (ptiles - pt0 + pstride - 1) / pstride : 0;     // the same for the whole wavefront
    if (left == 3) fwd_tiles<3>(g, band, kq, wcol, wpitch, steps, beyond, pt0, pstride, pixels, m, q4, bias_f, out_col);
    if (left == 2) fwd_tiles<2>(g, band, kq, wcol, wpitch, steps, beyond, pt0, pstride, pixels, m, q4, bias_f, out_col);
    if (left == 1) fwd_tiles<1>(g, band, kq, wcol, wpitch, steps, beyond, pt0, pstride, pixels, m, q4, bias_f, out_col);
}

// Output rows per band: the candidate with the lowest estimate of the launch's time, in units of one tile's
// products. Workgroups on one compute unit share its matrix cores, so a launch takes the workgroups a compute
// unit gets times a band's tiles per wavefront - but never less than `alone` times those tiles, what one
// wavefront per SIMD needs when nothing else covers its LDS latency - plus a set-up (staging is a memory round
// trip) and a share of it per further workgroup on the unit. `tiles_per_pixel_tile`: work per 16 pixels of a
// band, in forward tiles; four wavefronts share a band's tiles; `halo`: rows a band works on beyond its own.
// The constants are fitted to sweeps over the rows at batch sizes 100 and 2048.
static int thin_rows(int64_t n, int extent, int ow, int max_rows, double tiles_per_pixel_tile, int halo = 0) {
    const double alone = 2.5, setup = 2.5, setup_share = 1.0;
    const int64_t cus = ctx().num_cus;
    int best = 1;
    double best_cost = 0.0;
    for (int rows = 1; rows <= max_rows; ++rows) {
        const int64_t bands = (extent + rows - 1) / rows;
        const int64_t rounds = (n * bands + cus - 1) / cus;
        const int64_t ptiles = (static_cast<int64_t>(rows + halo) * ow + 15) / 16;
        const double per_wave = std::ceil(static_cast<double>(ptiles) * tiles_per_pixel_tile / 4.0);
        const double cost = std::max(static_cast<double>(rounds) * per_wave, alone * per_wave) +
                            setup + setup_share * static_cast<double>(rounds);
        if (rows == 1 || cost < best_cost) { best = rows; best_cost = cost; }
    }
    return best;
}

static bool thin_geometry(ThinGeom& g, int64_t n, int h, int w, int c, int f, int kh, int kw, int pad, int sh, int sw,
                          size_t fixed_lds_floats, double tiles_per_pixel_tile, size_t* lds_bytes) {
    if (sh != 1 || sw != 1 || n < 1 || h < 1 || w < 1 || c < 1 || kh < 1 || kw < 1 || pad < 0) return false;
    const int64_t K = static_cast<int64_t>(kh) * kw * c;
    if (K > kThinMaxK || f < 16 || f > kThinMaxF || f % 16 != 0) return false;
    g.h = h; g.w = w; g.c = c; g.f = f; g.kh = kh; g.kw = kw; g.pad = pad;
    g.oh = h + 2 * pad - kh + 1;
    g.ow = w + 2 * pad - kw + 1;
    if (g.oh < 1 || g.ow < 1 || g.ow > 4096) return false;
    g.K = static_cast<int>(K);
    g.bw = w + 2 * pad;
    const size_t budget = 60 * 1024 / sizeof(float);
    int max_rows = g.oh;
    while (max_rows > 1 && static_cast<size_t>(max_rows + kh - 1) * g.bw * c + fixed_lds_floats > budget) --max_rows;
    int rows = thin_rows(n, g.oh, g.ow, max_rows, tiles_per_pixel_tile);
    g.rows = rows;
    g.bands = (g.oh + rows - 1) / rows;
    g.br = rows + kh - 1;
    g.by_band_row = FastDiv(static_cast<uint32_t>(g.bw * c));
    g.by_c = FastDiv(static_cast<uint32_t>(c));
    g.by_ow = FastDiv(static_cast<uint32_t>(g.ow));
    g.by_K = FastDiv(static_cast<uint32_t>(g.K));
    g.by_window_row = FastDiv(static_cast<uint32_t>(kw * c));
    *lds_bytes = (static_cast<size_t>(g.br) * g.bw * c + fixed_lds_floats) * sizeof(float);
    return *lds_bytes <= 64 * 1024 && n * g.bands <= 0x7fffffff;
}

// ------------------------------------------------------------------ backward
// Both backward kernels work on out_deltas a chunk of whole rows at a time (about 64 pixels): 256 threads copy
// the chunk into LDS (requested a chunk ahead, into registers), the four wavefronts take its tiles.
struct ThinBackGeom {
    int h, w, c, f, kh, kw, pad, oh, ow, K;
    int rows, bands;        // rows per band: of the inputs (their deltas), of the outputs (the weights' deltas)
    int chunk_rows;         // rows of out_deltas per chunk
    int chunk_px;           // their pixels, rounded up to whole tiles of 16
    int margin, owp;        // dcol: zero pixels either side of a row of out_deltas (kw - 1 - pad), and a row with them
    int wp, dp, fp;         // LDS row pitches in floats: weights, dcol, the chunk of out_deltas
    int bw, br;             // staged band of the inputs (the weights' deltas): columns, rows
    FastDiv by_f, by_wc, by_c, by_ow, by_band_row;
};

constexpr int kDyRegs = 16;          // floats of a chunk per thread: chunk_px * f <= kDyRegs * kThinThreads

__device__ __forceinline__ void dy_chunk_load(const float* __restrict__ src, int count, float (&v)[kDyRegs]) {
#pragma unroll
    for (int u = 0; u < kDyRegs; ++u) {
        const int i = threadIdx.x + u * kThinThreads;
        if (u * kThinThreads < count) v[u] = src[i < count ? i : 0];
    }
}

__device__ __forceinline__ void dy_chunk_store(const ThinBackGeom& g, float* dyb, int count, const float (&v)[kDyRegs]) {
    if (kThinThreads % g.f == 0) {           // 16, 32 or 64 filters: a thread's elements lie 256 / f pixels apart
        uint32_t px, ff;
        g.by_f.divmod(threadIdx.x, px, ff);
        float* to = dyb + px * g.fp + ff;
        const int step = (kThinThreads / g.f) * g.fp;
#pragma unroll
        for (int u = 0; u < kDyRegs; ++u) {
            if (static_cast<int>(threadIdx.x) + u * kThinThreads < count) to[u * step] = v[u];
        }
        return;
    }
#pragma unroll
    for (int u = 0; u < kDyRegs; ++u) {
        const int i = threadIdx.x + u * kThinThreads;
        if (i < count) {
            uint32_t px, ff;
            g.by_f.divmod(static_cast<uint32_t>(i), px, ff);
            dyb[px * g.fp + ff] = v[u];
        }
    }
}

// in_deltas += col2im(out_deltas x W). A workgroup owns the rows [y0, y0 + rows) of one image's in_deltas and
// walks over the rows of out_deltas that reach them (kh - 1 more than it owns: neighbouring bands compute those
// again). Per chunk: dcol[pixel][k] = sum_f out_deltas[pixel][f] W[f][k] on the matrix cores into LDS (a tile is
// 16 pixels x 16 window entries, f in steps of 4; the KT tiles of one pixel tile share the out_deltas operand),
// then every element of in_deltas the chunk reaches adds its entries of dcol - out_deltas rows ascending, kx
// ascending - to its sum in LDS; one thread per element, so no atomics and the same order every time.
template <int KT>
__global__ __launch_bounds__(kThinThreads) void conv_thin_dx_kernel(ThinBackGeom g, const float* __restrict__ W,
                                                                    const float* __restrict__ dy,
                                                                    float* __restrict__ din, int64_t din_pitch) {
    extern __shared__ float lds[];
    constexpr int KW = KT * 16;
    float* wl = lds;                               // W as (f, wp), zero from K on
    float* dyb = wl + g.f * g.wp;                  // the chunk (chunk_px, fp)
    float* dcol = dyb + g.chunk_px * g.fp;         // (chunk_rows, owp, dp): rows of out_deltas between zero pixels
    float* dxb = dcol + g.chunk_rows * g.owp * g.dp;   // the band's sums (rows, w * c)
    float* zeros = dxb + g.rows * g.w * g.c;           // what a row of out_deltas outside an element's windows reads
    const int wc = g.w * g.c;
    const int64_t img = blockIdx.x / g.bands;
    const int y0 = static_cast<int>(blockIdx.x % g.bands) * g.rows;
    const int band_rows = min(g.rows, g.h - y0);
    const int oy_lo = max(0, y0 + g.pad - (g.kh - 1));
    const int oy_hi = min(g.oh, y0 + band_rows + g.pad);        // rows [oy_lo, oy_hi) of out_deltas reach this band
    const float* dy_img = dy + img * g.oh * g.ow * static_cast<int64_t>(g.f);
    float ahead[kDyRegs];
    int ahead_count = oy_lo < oy_hi ? min(g.chunk_rows, oy_hi - oy_lo) * g.ow * g.f : 0;
    dy_chunk_load(dy_img + static_cast<int64_t>(oy_lo) * g.ow * g.f, ahead_count, ahead);
    const int w_items = g.f * KW;
    for (int c0 = 0; c0 < w_items; c0 += kStageChunk) {
        float v[kStageAhead];
#pragma unroll
        for (int u = 0; u < kStageAhead; ++u) {
            const int i = c0 + threadIdx.x + u * kThinThreads;
            const int fi = i / KW, k = i % KW;
            const bool ok = i < w_items && k < g.K;
            const float loaded = W[ok ? fi * g.K + k : 0];
            v[u] = ok ? loaded : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kStageAhead; ++u) {
            const int i = c0 + threadIdx.x + u * kThinThreads;
            if (i < w_items) wl[(i / KW) * g.wp + i % KW] = v[u];
        }
    }
    for (int i = threadIdx.x; i < band_rows * wc; i += kThinThreads) dxb[i] = 0.0f;
    const int zero_floats = (g.kw - 1) * (g.dp - g.c) + 1;
    for (int i = threadIdx.x; i < zero_floats; i += kThinThreads) zeros[i] = 0.0f;
    // the zero pixels either side of dcol's rows: windows that hang over the edge of out_deltas read them
    for (int i = threadIdx.x; i < g.chunk_rows * 2 * g.margin * g.dp; i += kThinThreads) {
        const int col = i % g.dp, slot = i / g.dp;
        const int r = slot / (2 * g.margin), side = slot % (2 * g.margin);
        dcol[(r * g.owp + (side < g.margin ? side : g.ow + side)) * g.dp + col] = 0.0f;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 15, q4 = lane >> 4;
    const int steps = g.f / 4;
    for (int oy0 = oy_lo; oy0 < oy_hi; oy0 += g.chunk_rows) {
        const int rows_c = min(g.chunk_rows, oy_hi - oy0);
        dy_chunk_store(g, dyb, ahead_count, ahead);
        __syncthreads();                            // the chunk (and, the first time, the weights) are in LDS
        const int oy_next = oy0 + g.chunk_rows;
        ahead_count = oy_next < oy_hi ? min(g.chunk_rows, oy_hi - oy_next) * g.ow * g.f : 0;
        dy_chunk_load(dy_img + static_cast<int64_t>(oy_next < oy_hi ? oy_next : oy_lo) * g.ow * g.f, ahead_count, ahead);
        const int ptiles = (rows_c * g.ow + 15) / 16;
        for (int pt = wave; pt < ptiles; pt += 4) {
            v4f acc[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) acc[kt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            // Rows of the tile beyond the chunk's pixels hold whatever LDS held: their products are not kept.
            // f is a multiple of 16, so steps come in groups of four: a group's operands (4 values of
            // out_deltas, 4 x KT weights) are read from LDS while the 4 x KT products of the group before are
            // issued.
            const float* ap = dyb + (pt * 16 + m) * g.fp + q4;
            const float* bp = wl + q4 * g.wp + m;
            float a_next[4], b_next[4][KT];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                a_next[j] = ap[4 * j];
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) b_next[j][kt] = bp[j * 4 * g.wp + kt * 16];
            }
#pragma unroll 2
            for (int s0 = 0; s0 < steps; s0 += 4) {
                float a_now[4], b_now[4][KT];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    a_now[j] = a_next[j];
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) b_now[j][kt] = b_next[j][kt];
                }
                __builtin_amdgcn_sched_barrier(0);
                const int sn = s0 + 4 < steps ? s0 + 4 : s0;       // the last group reads itself again
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    a_next[j] = ap[4 * (sn + j)];
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) b_next[j][kt] = bp[(sn + j) * 4 * g.wp + kt * 16];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt)
                        acc[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_now[j], b_now[j][kt], acc[kt], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            // component q: pixel pt * 16 + 4 * (lane / 16) + q, window entry kt * 16 + lane % 16
            uint32_t r, ox;
            g.by_ow.divmod(static_cast<uint32_t>(pt * 16 + 4 * q4), r, ox);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (pt * 16 + 4 * q4 + q < rows_c * g.ow) {
                    float* to = dcol + (r * g.owp + ox + g.margin) * g.dp + m;
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) to[kt * 16] = acc[kt][q];
                }
                if (++ox == static_cast<uint32_t>(g.ow)) {       // the next pixel starts a row of out_deltas
                    ox = 0;
                    ++r;
                }
            }
        }
        __syncthreads();                            // dcol is complete, nobody reads the chunk any more
        const int reach = (rows_c + g.kh - 1) * wc;         // rows oy0 - pad ... of in_deltas, whole rows
        for (int i = threadIdx.x; i < reach; i += kThinThreads) {
            uint32_t t, e, x, ch;
            g.by_wc.divmod(static_cast<uint32_t>(i), t, e);
            const int y = oy0 - g.pad + static_cast<int>(t);
            if (y < y0 || y >= y0 + band_rows) continue;
            g.by_c.divmod(e, x, ch);
            float sum = 0.0f;
            // entry (ky, kx, ch) of pixel (r, x + pad - kx): from kx to kx + 1 one pixel back and one entry on
            const float* at = dcol + (static_cast<int>(x) + g.pad + g.margin) * g.dp + ch;
            const int next = g.c - g.dp;
            // kx in fours: four reads under way before the first is added. A row of out_deltas whose windows
            // do not hold this element's row reads zeros instead, so the loops are the same for every lane.
            const float* zero_at = zeros + (g.kw - 1) * (g.dp - g.c);
            for (int r = 0; r < rows_c; ++r) {
                const int ky = static_cast<int>(t) - r;
                const float* p = ky >= 0 && ky < g.kh ? at + (r * g.owp) * g.dp + ky * g.kw * g.c : zero_at;
                int kx = 0;
                for (; kx + 4 <= g.kw; kx += 4) {
                    const float v0 = p[kx * next], v1 = p[(kx + 1) * next], v2 = p[(kx + 2) * next], v3 = p[(kx + 3) * next];
                    sum += v0;
                    sum += v1;
                    sum += v2;
                    sum += v3;
                }
                for (; kx < g.kw; ++kx) sum += p[kx * next];
            }
            dxb[(y - y0) * wc + static_cast<int>(e)] += sum;
        }
        // the next chunk's copy into LDS waits for nobody: its readers passed the barrier above; dcol is
        // written again only after the next barrier
    }
    __syncthreads();
    float* dst = din + img * din_pitch + static_cast<int64_t>(y0) * wc;
    for (int i = threadIdx.x; i < band_rows * wc; i += kThinThreads) dst[i] += dxb[i];
}

// Partial sums of weight_deltas[f][k] = sum_pixels out_deltas[pixel][f] col[pixel][k] and, in column K,
// bias_deltas[f] = sum_pixels out_deltas[pixel][f] (a window entry that is always one). A workgroup walks over
// bands of images (unit = image x band of output rows; unit, unit + gridDim.x, ...), keeps its sums in the
// accumulators throughout and writes them once: partial[workgroup][f][KT * 16]. Tiles are 16 filters x 16
// window entries, pixels in steps of 4. A wavefront owns all FT x KT tiles and every fourth step: per step it
// reads FT values of out_deltas and KT of the image for FT x KT products, which keeps the matrix cores busier
// than the reads and the address arithmetic keep the issue slots.
template <int KT, int FT>
__global__ __launch_bounds__(kThinThreads) void conv_thin_dw_kernel(ThinBackGeom g, const float* __restrict__ in,
                                                                    int64_t in_pitch, const float* __restrict__ dy,
                                                                    float* __restrict__ partial, int64_t units) {
    extern __shared__ float lds[];
    constexpr int KW = KT * 16;
    const int band_floats = g.br * g.bw * g.c;
    float* band = lds;
    float* dyb = lds + band_floats;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 15, q4 = lane >> 4;
    int koff[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        const int k = kt * 16 + m;
        koff[kt] = k < g.K ? (k / (g.kw * g.c)) * g.bw * g.c + k % (g.kw * g.c) : 0;
    }
    const bool one = (KT - 1) * 16 + m == g.K, none = (KT - 1) * 16 + m > g.K;      // in the last tile of entries
    v4f acc[FT][KT];
#pragma unroll
    for (int ft = 0; ft < FT; ++ft) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) acc[ft][kt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
    for (int64_t unit = blockIdx.x; unit < units; unit += gridDim.x) {
        const int64_t img = unit / g.bands;
        const int y0 = static_cast<int>(unit % g.bands) * g.rows;
        const int band_rows = min(g.rows, g.oh - y0);
        const float* dy_band = dy + (img * g.oh + y0) * g.ow * static_cast<int64_t>(g.f);
        float ahead[kDyRegs];
        int ahead_count = min(g.chunk_rows, band_rows) * g.ow * g.f;
        dy_chunk_load(dy_band, ahead_count, ahead);
        __syncthreads();                            // the previous unit's readers are done with the band
        const float* src = in + img * in_pitch;
        for (int c0 = 0; c0 < band_floats; c0 += kStageChunk) {
            float v[kStageAhead];
            band_chunk_load(g.by_band_row, g.by_c, g.pad, g.h, g.w, g.c, src, y0, c0, band_floats, v);
            chunk_store(band, c0, band_floats, v);
        }
        for (int r0 = 0; r0 < band_rows; r0 += g.chunk_rows) {
            const int rows_c = min(g.chunk_rows, band_rows - r0);
            dy_chunk_store(g, dyb, ahead_count, ahead);
            __syncthreads();                        // the chunk (and, the first time, the band) are in LDS
            const int r_next = r0 + g.chunk_rows;
            ahead_count = r_next < band_rows ? min(g.chunk_rows, band_rows - r_next) * g.ow * g.f : 0;
            dy_chunk_load(dy_band + static_cast<int64_t>(r_next < band_rows ? r_next : 0) * g.ow * g.f, ahead_count, ahead);
            const int px_c = rows_c * g.ow;
            const int steps = (px_c + 3) / 4;
            if (wave < steps) {
                // Steps go in pairs: a pair's operands are read from LDS while the 2 x FT x KT products of the
                // pair before are issued. A step past the end reads pixel 0 and multiplies by zero, like the
                // pixels past the chunk in the last step.
                auto read_step = [&](int s, float (&a)[FT], float (&b)[KT]) {
                    const int p = 4 * s + q4;
                    const bool valid = p < px_c;
                    uint32_t py, px;
                    g.by_ow.divmod(static_cast<uint32_t>(valid ? p : 0), py, px);
                    const float* from = dyb + (valid ? p : 0) * g.fp + m;
#pragma unroll
                    for (int ft = 0; ft < FT; ++ft) {
                        const float a_read = from[ft * 16];
                        a[ft] = valid ? a_read : 0.0f;
                    }
                    const float* at = band + (static_cast<int>(r0 + py) * g.bw + static_cast<int>(px)) * g.c;
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) b[kt] = at[koff[kt]];
                    b[KT - 1] = one ? 1.0f : (none ? 0.0f : b[KT - 1]);
                };
                float a_next[2][FT], b_next[2][KT];
                read_step(wave, a_next[0], b_next[0]);
                read_step(wave + 4, a_next[1], b_next[1]);
                for (int s = wave; s < steps; s += 8) {
                    float a_now[2][FT], b_now[2][KT];
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
#pragma unroll
                        for (int ft = 0; ft < FT; ++ft) a_now[j][ft] = a_next[j][ft];
#pragma unroll
                        for (int kt = 0; kt < KT; ++kt) b_now[j][kt] = b_next[j][kt];
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    read_step(s + 8, a_next[0], b_next[0]);
                    read_step(s + 12, a_next[1], b_next[1]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
#pragma unroll
                        for (int ft = 0; ft < FT; ++ft) {
#pragma unroll
                            for (int kt = 0; kt < KT; ++kt)
                                acc[ft][kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_now[j][ft], b_now[j][kt], acc[ft][kt], 0, 0, 0);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __syncthreads();                        // before the next chunk replaces this one
        }
    }
    // The four wavefronts' sums are added in wavefront order: red[tile][component q][lane]
    float* red = lds;
    for (int w = 0; w < 4; ++w) {
        __syncthreads();
        if (wave == w) {
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float* at = red + ((ft * KT + kt) * 4 + q) * 64 + lane;
                        *at = w == 0 ? acc[ft][kt][q] : *at + acc[ft][kt][q];
                    }
                }
            }
        }
    }
    __syncthreads();
    float* mine = partial + static_cast<int64_t>(blockIdx.x) * g.f * KW;
    for (int i = threadIdx.x; i < FT * KT * 256; i += kThinThreads) {
        // component q of lane l of tile (ft, kt): filter ft * 16 + 4 * (l / 16) + q, window entry kt * 16 + l % 16
        const int l = i & 63, q = (i >> 6) & 3, tile = i >> 8;
        const int kt = tile % KT, ft = tile / KT;
        mine[(ft * 16 + 4 * (l >> 4) + q) * KW + kt * 16 + (l & 15)] = red[i];
    }
}

// weight_deltas[f][k] and bias_deltas[f] (column K) = the sum over the `count` partial results, in their order:
// sixteen threads per output add a sixteenth of them each, the first of the sixteen adds those sums in order.
__global__ __launch_bounds__(256) void conv_thin_dw_sum_kernel(const float* __restrict__ partial, int count, int f, int KW,
                                                               int K, float* __restrict__ dW, float* __restrict__ db) {
    __shared__ float part[16][17];
    const int o_local = threadIdx.x & 15, seg = threadIdx.x >> 4;
    const int o = blockIdx.x * 16 + o_local;
    const int total = f * KW;
    const int per = (count + 15) / 16;
    float sum = 0.0f;
    if (o < total) {
        const int hi = min(count, (seg + 1) * per);
        for (int i0 = seg * per; i0 < hi; i0 += 8) {       // eight loads under way before the first is added
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[static_cast<int64_t>(min(i0 + u, hi - 1)) * total + o];
#pragma unroll
            for (int u = 0; u < 8; ++u) sum += i0 + u < hi ? v[u] : 0.0f;
        }
    }
    part[seg][o_local] = sum;
    __syncthreads();
    if (seg == 0 && o < total) {
        float all = 0.0f;
#pragma unroll
        for (int s = 0; s < 16; ++s) all += part[s][o_local];
        const int fi = o / KW, k = o % KW;
        if (k < K) dW[fi * K + k] = all;
        else if (k == K) db[fi] = all;
    }
}

static void thin_back_chunk(ThinBackGeom& g, int rows) {
    g.chunk_rows = rows;
    g.chunk_px = (rows * g.ow + 15) & ~15;
}

// What both backward kernels share: sizes, the chunk, the LDS pitches (chosen so that the wavefront's reads of
// each array fall into distinct banks: the 16 lanes of a quarter read consecutive words, the quarters lie 16, 2
// or c words apart modulo 32).
static bool thin_back_geometry(ThinBackGeom& g, int64_t n, int h, int w, int c, int f, int kh, int kw, int pad, int sh,
                               int sw, int KT, bool for_weights) {
    if (sh != 1 || sw != 1 || n < 1 || h < 1 || w < 1 || c < 1 || kh < 1 || kw < 1 || pad < 0) return false;
    const int64_t K = static_cast<int64_t>(kh) * kw * c;
    if (K > kThinMaxK || KT < 1 || KT > 8 || f < 16 || f > kThinMaxF || f % 16 != 0) return false;
    g.h = h; g.w = w; g.c = c; g.f = f; g.kh = kh; g.kw = kw; g.pad = pad;
    g.oh = h + 2 * pad - kh + 1;
    g.ow = w + 2 * pad - kw + 1;
    if (g.oh < 1 || g.ow < 1) return false;
    g.K = static_cast<int>(K);
    g.margin = std::max(0, kw - 1 - pad);
    g.owp = g.ow + 2 * g.margin;
    thin_back_chunk(g, std::max(1, 64 / g.ow));
    if (static_cast<int64_t>(g.chunk_rows) * g.ow * f > kDyRegs * kThinThreads) return false;
    const int KW = KT * 16;
    g.wp = KW % 32 == 16 ? KW : KW + 16;
    g.dp = KW + ((c % 32) - (KW % 32) + 32) % 32;
    g.fp = for_weights ? (f % 32 == 16 ? f : f + 16) : f + 2;
    g.bw = w + 2 * pad;
    g.br = 0;               // set with the rows per band, for the weights' deltas
    g.rows = g.bands = 0;
    g.by_f = FastDiv(static_cast<uint32_t>(f));
    g.by_wc = FastDiv(static_cast<uint32_t>(w * c));
    g.by_c = FastDiv(static_cast<uint32_t>(c));
    g.by_ow = FastDiv(static_cast<uint32_t>(g.ow));
    g.by_band_row = FastDiv(static_cast<uint32_t>(g.bw * c));
    return true;
}

constexpr size_t kThinLdsFloats = 64 * 1024 / sizeof(float);

template <int KT>
static void launch_dx(const ThinBackGeom& g, int64_t n, size_t lds, const float* W, const float* dy, float* din,
                      int64_t din_pitch) {
    hipLaunchKernelGGL(conv_thin_dx_kernel<KT>, dim3(static_cast<unsigned>(n * g.bands)), dim3(kThinThreads), lds,
                       ctx().stream, g, W, dy, din, din_pitch);
}

// Workgroups of the weights' kernel that one compute unit holds at a time (registers and LDS decide): the
// launch has that many per unit at most, and each walks over the units that are left.
template <int KT, int FT>
static int dw_resident(size_t lds) {
    static std::mutex guard;
    static size_t asked_lds = ~size_t(0);
    static int answer = 1;
    std::lock_guard<std::mutex> lock(guard);
    if (lds != asked_lds) {                      // asked once per kernel and LDS size: the query is a driver call
        int blocks = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, conv_thin_dw_kernel<KT, FT>, kThinThreads, lds) != hipSuccess) {
            (void)hipGetLastError();
            blocks = 1;
        }
        answer = std::max(1, std::min(blocks, 4));
        asked_lds = lds;
    }
    return answer;
}

template <int KT>
static int dw_resident_for(int ftiles, size_t lds) {
    switch (ftiles) {
        case 1: return dw_resident<KT, 1>(lds);
        case 2: return dw_resident<KT, 2>(lds);
        case 3: return dw_resident<KT, 3>(lds);
        default: return dw_resident<KT, 4>(lds);
    }
}

template <int KT>
static void launch_dw(const ThinBackGeom& g, unsigned grid, size_t lds, const float* in, int64_t in_pitch, const float* dy,
                      float* partial, int64_t units) {
    const dim3 blocks(grid), threads(kThinThreads);
    switch (g.f / 16) {
        case 1: hipLaunchKernelGGL((conv_thin_dw_kernel<KT, 1>), blocks, threads, lds, ctx().stream, g, in, in_pitch, dy, partial, units); break;
        case 2: hipLaunchKernelGGL((conv_thin_dw_kernel<KT, 2>), blocks, threads, lds, ctx().stream, g, in, in_pitch, dy, partial, units); break;
        case 3: hipLaunchKernelGGL((conv_thin_dw_kernel<KT, 3>), blocks, threads, lds, ctx().stream, g, in, in_pitch, dy, partial, units); break;
        default: hipLaunchKernelGGL((conv_thin_dw_kernel<KT, 4>), blocks, threads, lds, ctx().stream, g, in, in_pitch, dy, partial, units); break;
    }
}

#define BSHIP_THIN_FOR_KT(kt, CALL)                                                     \
    switch (kt) {                                                                       \
        case 1: CALL(1); break; case 2: CALL(2); break; case 3: CALL(3); break;         \
        case 4: CALL(4); break; case 5: CALL(5); break; case 6: CALL(6); break;         \
        case 7: CALL(7); break; default: CALL(8); break;                                \
    }

}  // namespace bship

using namespace bship;

extern "C" {

int bship_conv2d_fwd_thin_f32(const float* in, int64_t in_pitch, const float* weights, const float* bias, float* out,
                              int64_t n, int h, int w, int c, int f, int kh, int kw, int pad, int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    ThinGeom g;
    size_t lds = 0;
    const int64_t K = static_cast<int64_t>(kh) * kw * c;
    if (!thin_geometry(g, n, h, w, c, f, kh, kw, pad, stride_h, stride_w,
                       static_cast<size_t>((K + 3) & ~int64_t(3)) * static_cast<size_t>(f > 0 ? f + 2 : 0), f / 16, &lds))
        return set_error(BSHIP_ERR_UNSUPPORTED, "%s: not a thin-filter convolution this kernel takes", __func__);
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(weights);
    BSHIP_REQUIRE_PTR(bias);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c);
    hipLaunchKernelGGL(conv_thin_fwd_kernel, dim3(static_cast<unsigned>(n * g.bands)), dim3(kThinThreads), lds,
                       ctx().stream, g, in, in_pitch, weights, bias, out);
    return check_launch("conv2d_forward_batch (thin filters)");
}

int bship_conv2d_bwd_thin_f32(const float* in, int64_t in_pitch, const float* weights, const float* out_deltas,
                              float* in_deltas, int64_t in_deltas_pitch, float* weight_deltas, float* bias_deltas,
                              int64_t n, int h, int w, int c, int f, int kh, int kw, int pad, int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    const int64_t K = static_cast<int64_t>(kh) * kw * c;
    const int kt_dx = static_cast<int>((K + 15) / 16), kt_dw = static_cast<int>((K + 16) / 16);
    ThinBackGeom gx, gw;
    bool ok = K >= 1 && thin_back_geometry(gx, n, h, w, c, f, kh, kw, pad, stride_h, stride_w, kt_dx, false) &&
              thin_back_geometry(gw, n, h, w, c, f, kh, kw, pad, stride_h, stride_w, kt_dw, true);
    size_t lds_x = 0, lds_w = 0;
    unsigned grid_w = 0;
    int64_t units = 0;
    if (ok) {
        // deltas of the inputs: bands of input rows, within what the LDS holds beside weights, chunk and dcol
        const size_t wc = static_cast<size_t>(w) * c;
        auto fixed_floats = [&]() {
            return static_cast<size_t>(f) * gx.wp + static_cast<size_t>(gx.chunk_px) * gx.fp +
                   static_cast<size_t>(gx.chunk_rows) * gx.owp * gx.dp + static_cast<size_t>(kw - 1) * (gx.dp - c) + 1;
        };
        // narrow images: fewer rows per chunk where their products (with the zero pixels either side) do not fit
        while (gx.chunk_rows > 1 && fixed_floats() + std::min<size_t>(h, 4) * wc > kThinLdsFloats)
            thin_back_chunk(gx, gx.chunk_rows - 1);
        const size_t fixed = fixed_floats();
        ok = fixed + wc <= kThinLdsFloats;
        if (ok) {
            const int max_rows = static_cast<int>(std::min<size_t>(h, (kThinLdsFloats - fixed) / wc));
            const double tile = kt_dx * (f / 4) / 19.0;
            gx.rows = thin_rows(n, h, gx.ow, max_rows, tile, kh - 1);
            gx.bands = (h + gx.rows - 1) / gx.rows;
            lds_x = (fixed + gx.rows * wc) * sizeof(float);
            ok = n * gx.bands <= 0x7fffffff;
        }
    }
    if (ok) {
        // deltas of the weights: bands of output rows; the LDS holds the band of the inputs and the chunk, and at
        // the end the sum of the four wavefronts' accumulators
        const size_t chunk = static_cast<size_t>(gw.chunk_px) * gw.fp, sums = static_cast<size_t>(f / 16) * kt_dw * 256;
        int max_rows = gw.oh;
        while (max_rows > 1 && static_cast<size_t>(max_rows + kh - 1) * gw.bw * c + chunk > kThinLdsFloats) --max_rows;
        ok = static_cast<size_t>(max_rows + kh - 1) * gw.bw * c + chunk <= kThinLdsFloats && sums <= kThinLdsFloats;
        if (ok) {
            const double tile = 4.0 * kt_dw * (f / 16) / 19.0;           // per 16 pixels: 4 steps of KT products per filter tile
            gw.rows = thin_rows(n, gw.oh, gw.ow, max_rows, tile);
            gw.bands = (gw.oh + gw.rows - 1) / gw.rows;
            gw.br = gw.rows + kh - 1;
            lds_w = std::max(static_cast<size_t>(gw.br) * gw.bw * c + chunk, sums) * sizeof(float);
            units = n * gw.bands;
            // as many workgroups as the device holds at a time, up to four per compute unit (beyond that the
            // partial sums cost more than the waiting units)
            int resident = 1;
#define BSHIP_THIN_RESIDENT(KT) resident = dw_resident_for<KT>(f / 16, lds_w)
            BSHIP_THIN_FOR_KT(kt_dw, BSHIP_THIN_RESIDENT)
#undef BSHIP_THIN_RESIDENT
            grid_w = static_cast<unsigned>(std::min<int64_t>(units, resident * static_cast<int64_t>(ctx().num_cus)));
        }
    }
    if (!ok) return set_error(BSHIP_ERR_UNSUPPORTED, "%s: not a thin-filter convolution these kernels take", __func__);
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(weights);
    BSHIP_REQUIRE_PTR(out_deltas);
    BSHIP_REQUIRE_PTR(in_deltas);
    BSHIP_REQUIRE_PTR(weight_deltas);
    BSHIP_REQUIRE_PTR(bias_deltas);
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c && in_deltas_pitch >= static_cast<int64_t>(h) * w * c);
    void* partial = nullptr;
    const int KW = kt_dw * 16;
    int st = pool_alloc_raw(static_cast<size_t>(grid_w) * f * KW * sizeof(float), &partial);
    if (st != 0) return st;
#define BSHIP_THIN_DW(KT) launch_dw<KT>(gw, grid_w, lds_w, in, in_pitch, out_deltas, static_cast<float*>(partial), units)
    BSHIP_THIN_FOR_KT(kt_dw, BSHIP_THIN_DW)
#undef BSHIP_THIN_DW
    st = check_launch("conv2d_backward_batch (thin filters, weights)");
    if (st == 0) {
        hipLaunchKernelGGL(conv_thin_dw_sum_kernel, dim3(static_cast<unsigned>((f * KW + 15) / 16)), dim3(256), 0, ctx().stream,
                           static_cast<const float*>(partial), static_cast<int>(grid_w), f, KW, static_cast<int>(K),
                           weight_deltas, bias_deltas);
        st = check_launch("conv2d_backward_batch (thin filters, sum)");
    }
    pool_free_raw(partial);                    // a later owner of the block runs after these launches
    if (st != 0) return st;
#define BSHIP_THIN_DX(KT) launch_dx<KT>(gx, n, lds_x, weights, out_deltas, in_deltas, in_deltas_pitch)
    BSHIP_THIN_FOR_KT(kt_dx, BSHIP_THIN_DX)
#undef BSHIP_THIN_DX
    return check_launch("conv2d_backward_batch (thin filters, inputs)");
}



}  // extern "C"
