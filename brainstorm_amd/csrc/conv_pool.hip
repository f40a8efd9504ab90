// NHWC image kernels: im2col / col2im for the convolution GEMMs and max /
// average pooling, forward and backward.
//
// Work is split per image (grid.y walks the images) and, inside an image, one
// lane handles W consecutive channels of one position (W = 4 when the channel
// count allows, so all accesses are 128-bit and neighbouring lanes touch
// neighbouring addresses). Positions are decoded from the lane's index with
// 32-bit multiply-shift divisions prepared on the host.
//
// The backward kernels are written in gather form (one lane per input position,
// visiting the output positions that cover it in row-major order): that is the
// order in which the reference's serial loops add their terms, so results are
// deterministic and match the reference bit for bit.
#pragma clang fp contract(off)

#include <cfloat>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>

#include "common.h"

namespace bship {

// A workgroup decodes its positions once and applies them to this many images.
#ifndef BSHIP_IMAGES_PER_WG
#define BSHIP_IMAGES_PER_WG 4
#endif
constexpr int kImagesPerWorkgroup = BSHIP_IMAGES_PER_WG;

struct ImgGeom {
    int h, w, c;          // input image
    int oh, ow;           // output positions
    int kh, kw;           // window / kernel
    int pad, sh, sw;
};

__host__ __device__ inline int imax(int a, int b) { return a > b ? a : b; }
__host__ __device__ inline int imin(int a, int b) { return a < b ? a : b; }

// Range [lo, hi) of output positions o with  o*stride - pad <= p < o*stride - pad + k.
__device__ __forceinline__ void cover_range(int p, int pad, const FastDiv& stride, int k, int n_out,
                                            int& lo, int& hi) {
    const int q = p + pad;                       // o*stride <= q < o*stride + k
    hi = imin(static_cast<int>(stride.div(static_cast<uint32_t>(q))) + 1, n_out);
    const int t = q - k + 1;                     // o*stride >= t
    lo = t <= 0 ? 0 : static_cast<int>(stride.div(static_cast<uint32_t>(t) + stride.d - 1));
}

// Cached (not streaming) accesses for what overlapping windows read again; operands that a kernel
// touches once (pooling outputs, the in_deltas a backward kernel updates) go through the
// non-temporal vload/vstore like the elementwise kernels' (max-pool backward 32x32x32: 149 -> 135 us).
template <int W, bool AL>
__device__ __forceinline__ typename VecT<W>::type img_load(const float* p) {
    if constexpr (W == 1) return *p;
    else if constexpr (AL) return *reinterpret_cast<const f4*>(p);
    else return *reinterpret_cast<const f4u*>(p);
}
template <int W, bool AL>
__device__ __forceinline__ void img_store(float* p, typename VecT<W>::type v) {
    if constexpr (W == 1) *p = v;
    else if constexpr (AL) *reinterpret_cast<f4*>(p) = v;
    else *reinterpret_cast<f4u*>(p) = v;
}
template <int W> __device__ __forceinline__ float& comp(typename VecT<W>::type& v, int j) {
    if constexpr (W == 1) return v;
    else return reinterpret_cast<float*>(&v)[j];
}
template <int W> __device__ __forceinline__ typename VecT<W>::type vsplat(float s) {
    if constexpr (W == 1) return s;
    else return f4{s, s, s, s};
}

// What every kernel gets: the geometry, the number of W-wide lanes of one image and the
// prepared divisors. cv = c / W channel vectors per position.
struct ImgPlan {
    ImgGeom g;
    uint32_t lanes_per_image;
    FastDiv d_cv, d_w, d_ow, d_kcv, d_kwcv, d_sh, d_sw;
    FastDiv d_pw;         // stride-aligned patches per image row (pooling backward)
    // elements from one image to the next: arrays shaped like the input (in, in_deltas), like the
    // output (out, out_deltas) and the argmax array. h*w*c / oh*ow*c for dense arrays; larger when
    // the array is a feature slice of a wider hub (each image is contiguous, images lie a pitch apart)
    int64_t in_pitch, out_pitch, aux_pitch;
    // launch shape: `tiles` workgroups cover one image, `groups` sets of images; see img_block
    uint32_t tiles, groups, per_xcd;
    bool in_order = false;   // tiles in dispatch order (kernels whose tiles share nothing)
    bool through = false;    // pooling backward: in_deltas stored write-through (outputs that fit the last-level cache)
    FastDiv d_tiles;
};

// Which (tile of an image, group of images) a workgroup of the 1-D grid works on. The hardware
// hands workgroups to the 8 XCDs round-robin by their number, and each XCD has an L2 of its own:
// with tile = blockIdx.x the neighbouring tiles of one image, whose windows overlap (a pooling
// output row is needed by the workgroups of three input rows), ran on different XCDs and each
// fetched the shared rows from HBM again (max-pool backward 32x32x32: 1.55x its algorithmic
// traffic). Here XCD x works through the x-th contiguous eighth of the (group, tile) sequence, so
// all tiles of an image group meet in one L2. The grid is 8 * per_xcd workgroups; numbers beyond
// the sequence's end have nothing to do. Kernels whose tiles share no cache lines (col2im with 32
// channels: every col element belongs to one input pixel, 128 bytes per pixel and col row) gain nothing
// from that and read faster as one front in dispatch order (measured 0.74 -> 0.76 of peak): in_order.
constexpr uint32_t kXcdCount = 8;
__device__ __forceinline__ bool img_block(const ImgPlan& pl, uint32_t& tile, uint32_t& group) {
    const uint32_t v = pl.in_order ? blockIdx.x : (blockIdx.x % kXcdCount) * pl.per_xcd + blockIdx.x / kXcdCount;
    if (v >= pl.tiles * pl.groups) return false;
    pl.d_tiles.divmod(v, group, tile);
    return true;
}

// col[(img, oy, ox), (ky, kx, ch)] = in[img, oy*sh-pad+ky, ox*sw-pad+kx, ch] or 0   (_cpuop 264-277)
// One lane per W channels of one (oy, ox, ky, kx); lanes_per_image = oh*ow*kh*kw*cv.
// WT: write-through stores for a col matrix too large to stay in the caches.
template <int W, bool AL, bool WT>
__device__ __forceinline__ void im2col_body(const float* __restrict__ in, float* __restrict__ col,
                                            int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t opix, r, oy, ox, ky, kxc, kx, chv;
    pl.d_kcv.divmod(p, opix, r);
    pl.d_ow.divmod(opix, oy, ox);
    pl.d_kwcv.divmod(r, ky, kxc);
    pl.d_cv.divmod(kxc, kx, chv);
    const int iy = static_cast<int>(oy) * g.sh - g.pad + static_cast<int>(ky);
    const int ix = static_cast<int>(ox) * g.sw - g.pad + static_cast<int>(kx);
    const bool inside = iy >= 0 && iy < g.h && ix >= 0 && ix < g.w;
    const int64_t in_off = (static_cast<int64_t>(iy) * g.w + ix) * g.c + chv * W;
    const int64_t in_img = pl.in_pitch;
    const int64_t col_img = static_cast<int64_t>(pl.lanes_per_image) * W;
    // kImagesPerWorkgroup images at a time: all loads first, then all stores
    for (int64_t img0 = static_cast<int64_t>(group) * kImagesPerWorkgroup; img0 < n;
         img0 += static_cast<int64_t>(pl.groups) * kImagesPerWorkgroup) {
        typename VecT<W>::type v[kImagesPerWorkgroup];
#pragma unroll
        for (int k = 0; k < kImagesPerWorkgroup; ++k) {
            v[k] = vsplat<W>(0.0f);
            if (inside && img0 + k < n) v[k] = img_load<W, AL>(in + (img0 + k) * in_img + in_off);
        }
#pragma unroll
        for (int k = 0; k < kImagesPerWorkgroup; ++k) {
            if (img0 + k < n) {
                float* q = col + (img0 + k) * col_img + static_cast<int64_t>(p) * W;
                if constexpr (WT) vstore_writeonly<W>(q, v[k]);
                else img_store<W, AL>(q, v[k]);
            }
        }
    }
}

// Channel counts that are not a multiple of 4 (RGB input): a lane still writes 4 consecutive
// col elements with one 128-bit store, gathering them with 4 scalar loads; each element is
// decoded on its own (they may lie in different kernel positions or output pixels). Needs
// oh*ow*kh*kw*c to be a multiple of 4; the plan's divisors are those of W = 1 and
// lanes_per_image counts the groups of 4.
template <bool WT>
__global__ __launch_bounds__(kBlock) void im2col_gather4(const float* __restrict__ in,
                                                         float* __restrict__ col, int64_t n, ImgPlan pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    int in_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t opix, r, oy, ox, ky, kxc, kx, ch;
        pl.d_kcv.divmod(p * 4 + j, opix, r);
        pl.d_ow.divmod(opix, oy, ox);
        pl.d_kwcv.divmod(r, ky, kxc);
        pl.d_cv.divmod(kxc, kx, ch);
        const int iy = static_cast<int>(oy) * g.sh - g.pad + static_cast<int>(ky);
        const int ix = static_cast<int>(ox) * g.sw - g.pad + static_cast<int>(kx);
        const bool inside = iy >= 0 && iy < g.h && ix >= 0 && ix < g.w;
        in_off[j] = inside ? (iy * g.w + ix) * g.c + static_cast<int>(ch) : -1;
    }
    const int64_t in_img = pl.in_pitch;
    const int64_t col_img = static_cast<int64_t>(pl.lanes_per_image) * 4;
    for (int64_t img0 = static_cast<int64_t>(group) * kImagesPerWorkgroup; img0 < n;
         img0 += static_cast<int64_t>(pl.groups) * kImagesPerWorkgroup) {
        f4 v[kImagesPerWorkgroup];
#pragma unroll
        for (int k = 0; k < kImagesPerWorkgroup; ++k) {
            const float* base = in + (img0 + k < n ? img0 + k : img0) * in_img;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[k][j] = in_off[j] >= 0 ? base[in_off[j]] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < kImagesPerWorkgroup; ++k) {
            if (img0 + k < n) {
                float* q = col + (img0 + k) * col_img + static_cast<int64_t>(p) * 4;
                if constexpr (WT) vstore_writeonly<4>(q, v[k]);
                else *reinterpret_cast<f4u*>(q) = v[k];
            }
        }
    }
}

template <int W, bool AL>
__global__ __launch_bounds__(kBlock) void im2col_cached(const float* __restrict__ in,
                                                        float* __restrict__ col, int64_t n, ImgPlan pl) {
    im2col_body<W, AL, false>(in, col, n, pl);
}
template <int W, bool AL>
__global__ __launch_bounds__(kBlock) void im2col_wt(const float* __restrict__ in, float* __restrict__ col,
                                                    int64_t n, ImgPlan pl) {
    im2col_body<W, AL, true>(in, col, n, pl);
}

// im2col through LDS. A workgroup produces one band of an image's col matrix: `band` consecutive
// floats (a multiple of 4), i.e. a few output rows. The image rows those output rows look at are
// staged once in LDS, zero-padded on all sides, so that every col element is an unconditional
// LDS read at (oy_rel*sh + ky) * wpc + ox*sw*c + (kx*c + ch); the band is then written with one
// 128-bit store per lane and iteration. Each input element is read from global memory once per
// band instead of once per col element, which leaves the vector memory path to the stores.
// Two LDS tiles alternate, so consecutive images of a workgroup need one barrier each.
struct BandPlan {
    ImgGeom g;
    uint32_t band;         // col floats per band
    uint32_t per_image;    // oh*ow*kh*kw*c
    int tile_rows;         // most image rows a band looks at
    int wpc;               // (w + 2*pad) * c : LDS row pitch
    int64_t in_pitch;      // elements from one input image to the next (h*w*c when dense)
    FastDiv d_k, d_ow, d_kwc, d_wpc, d_owk;
};

template <int W, bool WT>
__global__ __launch_bounds__(kBlock) void im2col_band(const float* __restrict__ in, float* __restrict__ col,
                                                      int64_t n, BandPlan pl) {
    extern __shared__ float band_tile[];
    const ImgGeom& g = pl.g;
    const int tid = static_cast<int>(threadIdx.x);
    const uint32_t first = blockIdx.x * pl.band;
    const uint32_t len = pl.per_image - first < pl.band ? pl.per_image - first : pl.band;
    const int oy_first = static_cast<int>(pl.d_owk.div(first));
    const int oy_last = static_cast<int>(pl.d_owk.div(first + len - 1));
    const int iy0 = oy_first * g.sh - g.pad;
    const int tile_len = ((oy_last - oy_first) * g.sh + g.kh) * pl.wpc;
    const int tile_cap = pl.tile_rows * pl.wpc;
    const int wc = g.w * g.c, padc = g.pad * g.c, swc = g.sw * g.c;
    const uint32_t kwc = static_cast<uint32_t>(g.kw * g.c);
    const int64_t in_img = pl.in_pitch;
    int buf = 0;
    for (int64_t img = blockIdx.y; img < n; img += gridDim.y) {
        float* t = band_tile + buf * tile_cap;
        const float* src = in + img * in_img;
        for (int e = tid * W; e < tile_len; e += kBlock * W) {
            uint32_t row, cx;
            pl.d_wpc.divmod(static_cast<uint32_t>(e), row, cx);
            const int iy = iy0 + static_cast<int>(row), xo = static_cast<int>(cx) - padc;
            const bool inside = iy >= 0 && iy < g.h && xo >= 0 && xo < wc;
            if constexpr (W == 4) {
                f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
                if (inside) v = *reinterpret_cast<const f4u*>(src + iy * wc + xo);
                *reinterpret_cast<f4*>(t + e) = v;
            } else {
                t[e] = inside ? src[iy * wc + xo] : 0.0f;
            }
        }
        __syncthreads();
        float* dst = col + img * static_cast<int64_t>(pl.per_image) + first;
        for (uint32_t s = static_cast<uint32_t>(tid) * 4; s < len; s += kBlock * 4) {
            uint32_t opix, kk, oy, ox, ky, r;
            pl.d_k.divmod(first + s, opix, kk);
            pl.d_ow.divmod(opix, oy, ox);
            pl.d_kwc.divmod(kk, ky, r);
            uint32_t oyr = oy - static_cast<uint32_t>(oy_first);
            f4 v;
            if constexpr (W == 4) {
                v = *reinterpret_cast<const f4*>(t + (oyr * g.sh + ky) * pl.wpc + ox * swc + r);
            } else {
                // the four elements may straddle kernel rows, output pixels and output rows
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[j] = t[(oyr * g.sh + ky) * pl.wpc + ox * swc + r];
                    if (++r == kwc) {
                        r = 0;
                        if (++ky == static_cast<uint32_t>(g.kh)) {
                            ky = 0;
                            if (++ox == static_cast<uint32_t>(g.ow)) { ox = 0; ++oyr; }
                        }
                    }
                }
            }
            if constexpr (WT) vstore_writeonly<4>(dst + s, v);
            else *reinterpret_cast<f4u*>(dst + s) = v;
        }
        buf ^= 1;
    }
}

// The same for channel counts that are not multiples of 4 (RGB input) when ow is: K = kh*kw*c floats
// per output pixel, so 4 neighbouring pixels of an output row are exactly K 128-bit stores. Where the 4
// floats of store number q of such a group lie relative to the group's first pixel (which pixel, kernel
// row, offset in the kernel row) depends on q alone: a table of K entries in LDS, filled once, replaces
// the per-store decoding of the general kernel above (which steps through its 4 elements with carries:
// 100 vector instructions per store, compute bound at 0.65 of peak for 32x32x3 images and 5x5 kernels).
// Lanes store in the same order as there: 256 consecutive 128-bit stores per iteration.
// Needs bands of whole output rows; the table lies behind the two tiles.
template <bool WT>
__global__ __launch_bounds__(kBlock) void im2col_band_groups(const float* __restrict__ in,
                                                             float* __restrict__ col, int64_t n, BandPlan pl,
                                                             FastDiv d_K, FastDiv d_groups_per_row) {
    extern __shared__ float band_tile[];
    const ImgGeom& g = pl.g;
    const int tid = static_cast<int>(threadIdx.x);
    const uint32_t first = blockIdx.x * pl.band;
    const uint32_t len = pl.per_image - first < pl.band ? pl.per_image - first : pl.band;
    const int oy_first = static_cast<int>(pl.d_owk.div(first));
    const int oy_last = static_cast<int>(pl.d_owk.div(first + len - 1));
    const int iy0 = oy_first * g.sh - g.pad;
    const int tile_len = ((oy_last - oy_first) * g.sh + g.kh) * pl.wpc;
    const int tile_cap = pl.tile_rows * pl.wpc;
    const int wc = g.w * g.c, padc = g.pad * g.c, swc = g.sw * g.c;
    const int K = g.kh * g.kw * g.c, kwc = g.kw * g.c;
    const int64_t in_img = pl.in_pitch;
    int4* table = reinterpret_cast<int4*>(band_tile + 2 * tile_cap);      // tile_cap is kept a multiple of 4
    for (int q = tid; q < K; q += kBlock) {
        int off[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int t = q * 4 + j;
            const int p = t / K, kk = t - p * K;
            const int ky = kk / kwc, r = kk - ky * kwc;
            off[j] = p * swc + ky * pl.wpc + r;
        }
        table[q] = make_int4(off[0], off[1], off[2], off[3]);
    }
    const uint32_t stores = len / 4;
    int buf = 0;
    for (int64_t img = blockIdx.y; img < n; img += gridDim.y) {
        float* t = band_tile + buf * tile_cap;
        const float* src = in + img * in_img;
        for (int e = tid; e < tile_len; e += kBlock) {
            uint32_t row, cx;
            pl.d_wpc.divmod(static_cast<uint32_t>(e), row, cx);
            const int iy = iy0 + static_cast<int>(row), xo = static_cast<int>(cx) - padc;
            const bool inside = iy >= 0 && iy < g.h && xo >= 0 && xo < wc;
            t[e] = inside ? src[iy * wc + xo] : 0.0f;
        }
        __syncthreads();                      // also: the table is complete
        float* dst = col + img * static_cast<int64_t>(pl.per_image) + first;
        for (uint32_t s = static_cast<uint32_t>(tid); s < stores; s += kBlock) {
            uint32_t G, q, row, gx;
            d_K.divmod(s, G, q);
            d_groups_per_row.divmod(G, row, gx);
            const float* base = t + row * (g.sh * pl.wpc) + gx * (4 * swc);
            const int4 off = table[q];
            const f4 v = {base[off.x], base[off.y], base[off.z], base[off.w]};
            if constexpr (WT) vstore_writeonly<4>(dst + s * 4, v);
            else *reinterpret_cast<f4u*>(dst + s * 4) = v;
        }
        buf ^= 1;
    }
}

// in_deltas[img, y, x, ch] += sum over covering (oy, ox), in scan order, of
// col[(img, oy, ox), (y - (oy*sh-pad), x - (ox*sw-pad), ch)]               (_cpuop 295-309)
// One lane per W channels of one input pixel; lanes_per_image = h*w*cv.
template <int W, bool AL>
__global__ __launch_bounds__(kBlock) void col2im_kernel(const float* __restrict__ col,
                                                        float* __restrict__ in_deltas, int64_t n,
                                                        ImgPlan pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t pix, chv, yy, xx;
    pl.d_cv.divmod(p, pix, chv);
    pl.d_w.divmod(pix, yy, xx);
    const int y = static_cast<int>(yy), x = static_cast<int>(xx);
    int oy0, oy1, ox0, ox1;
    cover_range(y, g.pad, pl.d_sh, g.kh, g.oh, oy0, oy1);
    cover_range(x, g.pad, pl.d_sw, g.kw, g.ow, ox0, ox1);
    const int64_t kc = static_cast<int64_t>(g.kh) * g.kw * g.c;
    const int64_t in_img = pl.in_pitch;
    const int64_t col_img = static_cast<int64_t>(g.oh) * g.ow * kc;
    for (int64_t img = group; img < n; img += pl.groups) {
        float* q = in_deltas + img * in_img + static_cast<int64_t>(p) * W;
        typename VecT<W>::type acc = img_load<W, AL>(q);
        const float* cimg = col + img * col_img + chv * W;
        for (int oy = oy0; oy < oy1; ++oy) {
            const int ky = y - (oy * g.sh - g.pad);
            for (int ox = ox0; ox < ox1; ++ox) {
                const int kx = x - (ox * g.sw - g.pad);
                acc += img_load<W, AL>(cimg + (static_cast<int64_t>(oy) * g.ow + ox) * kc +
                                       (ky * g.kw + kx) * g.c);
            }
        }
        img_store<W, AL>(q, acc);
    }
}

// The same for kh = kw = KS with stride 1, KS known at compile time: the covering positions are oy = y + pad -
// (KS-1) + a, ox = x + pad - (KS-1) + b for a, b in [0, KS), so the KS*KS terms of an element are loaded
// together (a term outside the col matrix reads a clamped address and is not added) and added in the same
// scan order. With the run-time loops above a lane waits for each of its up to 25 loads in turn, which at
// batch 100 (too few wavefronts to hide it) made the kernel 2.0 TB/s slow.
template <int W, bool AL, int KS>
__device__ __forceinline__ void col2im_ks_body(const float* __restrict__ col, float* __restrict__ in_deltas,
                                               int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t pix, chv, yy, xx;
    pl.d_cv.divmod(p, pix, chv);
    pl.d_w.divmod(pix, yy, xx);
    const int oy_first = static_cast<int>(yy) + g.pad - (KS - 1), ox_first = static_cast<int>(xx) + g.pad - (KS - 1);
    const int64_t kc = static_cast<int64_t>(KS) * KS * g.c;
    const int64_t col_img = static_cast<int64_t>(g.oh) * g.ow * kc;
    int off[KS * KS];
    bool ok[KS * KS];
#pragma unroll
    for (int a = 0; a < KS; ++a)
#pragma unroll
        for (int b = 0; b < KS; ++b) {
            const int oy = oy_first + a, ox = ox_first + b;
            const bool in = oy >= 0 && oy < g.oh && ox >= 0 && ox < g.ow;
            ok[a * KS + b] = in;
            // ky = KS-1-a, kx = KS-1-b
            off[a * KS + b] = in ? static_cast<int>((static_cast<int64_t>(oy) * g.ow + ox) * kc) +
                                       ((KS - 1 - a) * KS + (KS - 1 - b)) * g.c
                                 : 0;
        }
    for (int64_t img = group; img < n; img += pl.groups) {
        float* q = in_deltas + img * pl.in_pitch + static_cast<int64_t>(p) * W;
        const float* cimg = col + img * col_img + chv * W;
        typename VecT<W>::type v[KS * KS];
#pragma unroll
        for (int i = 0; i < KS * KS; ++i) v[i] = img_load<W, AL>(cimg + off[i]);
        typename VecT<W>::type acc = img_load<W, AL>(q);
#pragma unroll
        for (int i = 0; i < KS * KS; ++i)
            if (ok[i]) acc += v[i];
        img_store<W, AL>(q, acc);
    }
}
#define BSHIP_COL2IM_KS_KERNEL(name, KS)                                                                   \
    template <int W, bool AL>                                                                              \
    __global__ __launch_bounds__(kBlock) void name(const float* __restrict__ col,                          \
                                                   float* __restrict__ in_deltas, int64_t n, ImgPlan pl) { \
        col2im_ks_body<W, AL, KS>(col, in_deltas, n, pl);                                                  \
    }
BSHIP_COL2IM_KS_KERNEL(col2im_kernel_k3, 3)
BSHIP_COL2IM_KS_KERNEL(col2im_kernel_k5, 5)

// col2im through LDS, for narrow channel counts: there a lane's 4*c-byte pieces of the col
// matrix lie kh*kw*c floats apart and every cache line would be fetched several times.
// A workgroup walks down a band of image rows, `rows` of them per phase. The col rows (oy) that
// cover the rows of a phase are one contiguous range of the col matrix; they live in a ring of
// `ring` col rows in LDS (col row oy in slot oy mod ring). While the lanes gather the terms of
// the current phase from LDS (one lane per input element, same scan order as above), the col
// rows that the next phase adds are already on their way into registers; they replace the
// oldest slots after the phase. Inside a band every col element is therefore read once, with
// coalesced 128-bit loads; bands of one image overlap by the col rows that cover both.
// Bands of one image have the same workgroup index modulo 8 and follow each other, so with
// workgroups dealt round-robin to the 8 XCDs they meet in one L2.
// Needs ow*kh*kw*c (floats per col row) to be a multiple of 4.
constexpr int kCol2imThreads = 512;  // few workgroups fit a compute unit's LDS: make them large
constexpr int kCol2imPrefetch = 5;      // 128-bit loads in flight per lane
constexpr int kCol2imOutsPerLane = 2;   // image elements of one phase per lane, at most
constexpr uint32_t kXcds = 8;

struct Col2imBandPlan {
    ImgGeom g;
    int rows;              // image rows per phase
    int phases;            // phases per workgroup
    int bands;             // workgroups per image
    int ring;              // col rows held in LDS
    uint32_t owk;          // ow*kh*kw*c : floats per col row
    int64_t in_pitch;      // elements from one image of in_deltas to the next (h*w*c when dense)
    FastDiv d_bands, d_wc, d_w, d_sh, d_sw, d_ring, d_owk4;
};

// Copies col rows [lo, hi) of one image into their ring slots, kBatch loads in flight per lane.
template <int kBatch>
__device__ __forceinline__ void col2im_stage(const float* __restrict__ cimg, float* __restrict__ tile,
                                             int lo, int hi, const Col2imBandPlan& pl) {
    const int count4 = hi > lo ? (hi - lo) * static_cast<int>(pl.owk / 4) : 0;
    const float* src = cimg + static_cast<int64_t>(lo) * pl.owk;
    for (int q0 = static_cast<int>(threadIdx.x); q0 < count4; q0 += kCol2imThreads * kBatch) {
        f4 v[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int q = q0 + u * kCol2imThreads;
            if (q < count4) v[u] = vload<4, false>(src + static_cast<int64_t>(q) * 4);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int q = q0 + u * kCol2imThreads;
            if (q < count4) {
                uint32_t row, within;
                pl.d_owk4.divmod(static_cast<uint32_t>(q), row, within);
                const uint32_t slot = pl.d_ring.div(static_cast<uint32_t>(lo) + row);
                const uint32_t s = static_cast<uint32_t>(lo) + row - slot * pl.d_ring.d;
                *reinterpret_cast<f4*>(tile + s * pl.owk + within * 4) = v[u];
            }
        }
    }
}

// KS > 0: kh = kw = KS with stride 1, known at compile time: the KS*KS reads of an element are
// issued together (terms outside the col matrix read a clamped address and are not added).
template <int KS>
__global__ __launch_bounds__(kCol2imThreads) void col2im_band(const float* __restrict__ col,
                                                      float* __restrict__ in_deltas, int64_t n,
                                                      Col2imBandPlan pl) {
    extern __shared__ float band_tile[];
    const ImgGeom& g = pl.g;
    const uint32_t lane_group = blockIdx.x / kXcds, xcd = blockIdx.x % kXcds;
    uint32_t img_group, band;
    pl.d_bands.divmod(lane_group, img_group, band);
    const int64_t img = static_cast<int64_t>(img_group) * kXcds + xcd;
    if (img >= n) return;
    const int ybeg = static_cast<int>(band) * pl.rows * pl.phases;
    const int yend = imin(ybeg + pl.rows * pl.phases, g.h);
    const int kc = g.kh * g.kw * g.c, wc = g.w * g.c;
    const int pitch = static_cast<int>(pl.owk);
    const float* cimg = col + img * (static_cast<int64_t>(g.oh) * pl.owk);
    float* dimg = in_deltas + img * pl.in_pitch;
    // Lane index o of a phase -> image element: within an image row the lanes are ordered channel
    // first, then x, so that neighbouring lanes read LDS words kh*kw*c apart (an odd stride for
    // RGB images: no bank conflicts) rather than runs of c words with gaps.
    auto element_of = [&](int o) {
        uint32_t yr, rem, xx, ch;
        pl.d_wc.divmod(static_cast<uint32_t>(o), yr, rem);
        pl.d_w.divmod(rem, ch, xx);
        return static_cast<int>(yr * wc + xx * g.c + ch);
    };
    auto ring_slot = [&](int oy) {
        return static_cast<int>(static_cast<uint32_t>(oy) - pl.d_ring.div(static_cast<uint32_t>(oy)) * pl.d_ring.d);
    };

    // col rows of the first phase; a lane's image elements are o = lane + u*kCol2imThreads of the phase
    int p_lo, p_hi, unused;
    cover_range(ybeg, g.pad, pl.d_sh, g.kh, g.oh, p_lo, unused);
    cover_range(imin(ybeg + pl.rows, yend) - 1, g.pad, pl.d_sh, g.kh, g.oh, unused, p_hi);
    float init[kCol2imOutsPerLane];     // in_deltas before the update, loaded a phase ahead
    {
        const int outs = (imin(ybeg + pl.rows, yend) - ybeg) * wc;
        const float* drow = dimg + static_cast<int64_t>(ybeg) * wc;
#pragma unroll
        for (int u = 0; u < kCol2imOutsPerLane; ++u) {
            const int o = static_cast<int>(threadIdx.x) + u * kCol2imThreads;
            init[u] = o < outs ? drow[element_of(o)] : 0.0f;
        }
    }
    col2im_stage<8>(cimg, band_tile, p_lo, p_hi, pl);
    int have_hi = imax(p_hi, p_lo);     // col rows below have_hi have been loaded
    __syncthreads();

    for (int ya = ybeg; ya < yend; ya += pl.rows) {
        const int yb = imin(ya + pl.rows, yend);
        // what the next phase adds, into registers: col rows and the image rows' old values
        int n_lo = p_lo, n_hi = p_hi, new_lo = 0, count4 = 0;
        f4 pre[kCol2imPrefetch];
        float init_next[kCol2imOutsPerLane];
        if (yb < yend) {
            cover_range(yb, g.pad, pl.d_sh, g.kh, g.oh, n_lo, unused);
            cover_range(imin(yb + pl.rows, yend) - 1, g.pad, pl.d_sh, g.kh, g.oh, unused, n_hi);
            new_lo = imax(have_hi, n_lo);
            count4 = n_hi > new_lo ? (n_hi - new_lo) * static_cast<int>(pl.owk / 4) : 0;
            const float* src = cimg + static_cast<int64_t>(new_lo) * pl.owk;
#pragma unroll
            for (int u = 0; u < kCol2imPrefetch; ++u) {
                const int q = static_cast<int>(threadIdx.x) + u * kCol2imThreads;
                if (q < count4) pre[u] = vload<4, false>(src + static_cast<int64_t>(q) * 4);
            }
            const int outs_next = (imin(yb + pl.rows, yend) - yb) * wc;
            const float* drow_next = dimg + static_cast<int64_t>(yb) * wc;
#pragma unroll
            for (int u = 0; u < kCol2imOutsPerLane; ++u) {
                const int o = static_cast<int>(threadIdx.x) + u * kCol2imThreads;
                init_next[u] = o < outs_next ? drow_next[element_of(o)] : 0.0f;
            }
        }
        // this phase's image rows from LDS
        const int outs = (yb - ya) * wc;
        float* drow = dimg + static_cast<int64_t>(ya) * wc;
#pragma unroll
        for (int u = 0; u < kCol2imOutsPerLane; ++u) {
            const int o = static_cast<int>(threadIdx.x) + u * kCol2imThreads;
            if (o >= outs) break;
            uint32_t yr, rem, xx, ch;
            pl.d_wc.divmod(static_cast<uint32_t>(o), yr, rem);
            pl.d_w.divmod(rem, ch, xx);
            const int y = ya + static_cast<int>(yr), x = static_cast<int>(xx);
            float acc = init[u];
            if constexpr (KS > 0) {
                // oy = y + pad - ky ascends as ky descends; the same for ox
                float v[KS * KS];
#pragma unroll
                for (int a = 0; a < KS; ++a) {
                    const int ky = KS - 1 - a;
                    const int oy = imin(imax(y + g.pad - ky, p_lo), p_hi - 1);
                    const float* trow = band_tile + ring_slot(oy) * pitch + ky * KS * g.c + static_cast<int>(ch);
#pragma unroll
                    for (int b = 0; b < KS; ++b) {
                        const int kx = KS - 1 - b;
                        const int ox = imin(imax(x + g.pad - kx, 0), g.ow - 1);
                        v[a * KS + b] = trow[ox * kc + kx * g.c];
                    }
                }
#pragma unroll
                for (int a = 0; a < KS; ++a)
#pragma unroll
                    for (int b = 0; b < KS; ++b) {
                        const int oy = y + g.pad - (KS - 1 - a), ox = x + g.pad - (KS - 1 - b);
                        if (oy >= 0 && oy < g.oh && ox >= 0 && ox < g.ow) acc += v[a * KS + b];
                    }
            } else {
                int oy0, oy1, ox0, ox1;
                cover_range(y, g.pad, pl.d_sh, g.kh, g.oh, oy0, oy1);
                cover_range(x, g.pad, pl.d_sw, g.kw, g.ow, ox0, ox1);
                for (int oy = oy0; oy < oy1; ++oy) {
                    const int ky = y - (oy * g.sh - g.pad);
                    const float* trow = band_tile + ring_slot(oy) * pitch + ky * g.kw * g.c + ch;
                    for (int ox = ox0; ox < ox1; ++ox) {
                        const int kx = x - (ox * g.sw - g.pad);
                        acc += trow[ox * kc + kx * g.c];
                    }
                }
            }
            drow[yr * wc + xx * g.c + ch] = acc;
        }
        if (yb >= yend) break;
        __syncthreads();                 // every lane is done with the slots that are replaced now
#pragma unroll
        for (int u = 0; u < kCol2imPrefetch; ++u) {
            const int q = static_cast<int>(threadIdx.x) + u * kCol2imThreads;
            if (q < count4) {
                uint32_t row, within;
                pl.d_owk4.divmod(static_cast<uint32_t>(q), row, within);
                *reinterpret_cast<f4*>(band_tile + ring_slot(new_lo + static_cast<int>(row)) * pitch + within * 4) = pre[u];
            }
        }
#pragma unroll
        for (int u = 0; u < kCol2imOutsPerLane; ++u) init[u] = init_next[u];
        have_hi = imax(have_hi, n_hi);
        p_lo = n_lo;
        p_hi = n_hi;
        __syncthreads();
    }
}

// col2im for narrow channel counts and many images (KS x KS windows, stride 1, C channels, both known
// at compile time). The col matrix streams from memory straight into LDS (128-bit global loads with
// an LDS destination: no registers in between) and every col row is used up in the one phase after
// its arrival, so most of LDS holds data in flight.
//
// A workgroup takes whole images one after the other (image = workgroup index + i * workgroups). A
// phase is R consecutive col rows oy0 .. oy0+R-1 of one image. Their terms belong to the M = KS+R-1
// image rows oy0-pad .. oy0-pad+M-1; lane (s, x) of the first M*w lanes owns, during a phase, the
// pixel (y, x) of the one row with y = s (mod M) among them, and keeps the sums of its C channels in
// registers from the phase with the row's first col row (where they start from the old values:
// in_deltas is added to) to the phase with its last one (where they are stored). For each col row
// of the phase in turn, the lane adds the KS terms of its window row ky = y + pad - oy, kx descending:
// an element receives its terms with oy ascending, then ox ascending - the order of the serial loops
// (_cpuop 295-309).
//
// The other wavefronts request data: the col rows of a phase and the image rows that start in it go
// to the next slots of two rings in LDS, DEPTH phases before they are needed, as pieces of 1 KiB
// (one load instruction: 64 lanes x 16 bytes, LDS address = the wavefront's base + 16 * lane).
// Every requesting wavefront issues exactly PER load instructions per phase (pieces it has no use
// for become a 16-byte load into a spare slot). Loads complete in order, so when at most
// (DEPTH-1)*PER are outstanding, the wavefront's pieces of the current phase have arrived; then the
// workgroup's barrier. One barrier per phase; the slots that phase t + DEPTH fills are the ones
// phase t - 1 read.
// (A wavefront issues an instruction every four cycles at best and a phase lasts as long as its
// longest instruction stream, which is why requesting and adding run side by side in different
// wavefronts, and why the bookkeeping is additions on running counters.)
// Terms beyond the left and right image border are read from wherever their address falls (the
// ring has a guard in front and the old values behind) and not added.
// Needs ow*KS*KS*C and w*C to be multiples of 4, both operands 16-byte aligned, in_pitch % 4 == 0.
constexpr int kPieceFloats = 256;         // floats per load instruction of a wavefront

struct Col2imStreamPlan {
    int h, w, oh, ow, pad;
    int phases;            // phases per image
    int add_waves;         // adding wavefronts; the others request data
    int old_ring;          // image rows of old values held in LDS
    int old_image_step;    // what the ring position of image row "oy0 - pad" moves by from the last phase of an image to the first of the next, less R, modulo old_ring
    int guard;             // floats in front of the col ring
    int owk;               // ow*KS*KS*C : floats per col row
    int64_t in_pitch;      // elements from one image of in_deltas to the next
    FastDiv d_w;
};

template <int KS, int C, int R, int THREADS, int DEPTH, int PER>
__global__ __launch_bounds__(THREADS) void col2im_stream(const float* __restrict__ col,
                                                         float* __restrict__ in_deltas, int64_t n,
                                                         Col2imStreamPlan pl) {
    extern __shared__ float stream_lds[];
    constexpr int kWaves = THREADS / kWave;
    constexpr int KC = KS * KS * C;
    constexpr int M = KS + R - 1;                           // image rows a phase adds to
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWave);
    const int lane = static_cast<int>(threadIdx.x) & (kWave - 1);
    const int wc = pl.w * C, pitch = pl.owk;
    float* const tile = stream_lds + pl.guard;
    float* const old_area = tile + (DEPTH + 1) * R * pitch;
    const int my_images = static_cast<int>((n - blockIdx.x + gridDim.x - 1) / gridDim.x);
    const int total = my_images * pl.phases;                // the launcher keeps this below 2^31
    const int64_t col_image = static_cast<int64_t>(pl.oh) * pitch;
    const int64_t col_step = static_cast<int64_t>(gridDim.x) * col_image;
    const int64_t old_step = static_cast<int64_t>(gridDim.x) * pl.in_pitch;
    const int add_waves = pl.add_waves;

    if (wave >= add_waves) {
        // ---------------- requests ----------------
        const int req_wave = wave - add_waves, req_waves = kWaves - add_waves;
        const int row_pieces = (wc + kPieceFloats - 1) / kPieceFloats;
        float* const spare = old_area + pl.old_ring * wc;
        int req_phase = 0, req_slot = 0, req_old_slot = 0;
        const float* req_col = col + static_cast<int64_t>(blockIdx.x) * col_image;          // the image's col matrix
        const float* req_img = in_deltas + static_cast<int64_t>(blockIdx.x) * pl.in_pitch;  // the image's old values
        auto request = [&](bool real) {
            const int oy0 = req_phase * R;
            const int col_floats = imin(R, pl.oh - oy0) * pitch;
            const int col_pieces = (col_floats + kPieceFloats - 1) / kPieceFloats;
            // image rows whose first col row is in this phase
            const int y0 = oy0 == 0 ? 0 : oy0 + KS - 1 - pl.pad;
            const int rows = imax(imin(oy0 + R + KS - 1 - pl.pad, pl.h) - y0, 0);
            const int pieces = real ? col_pieces + rows * row_pieces : 0;
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                const int p = req_wave + k * req_waves;
                const float* src = col;
                float* dst = spare;
                int valid = 4;                 // floats left from this piece's start
                if (p < col_pieces && p < pieces) {
                    src = req_col + static_cast<int64_t>(oy0) * pitch + p * kPieceFloats;
                    dst = tile + req_slot * (R * pitch) + p * kPieceFloats;
                    valid = col_floats - p * kPieceFloats;
                } else if (p < pieces) {
                    const int q = p - col_pieces;
                    const int r = q / row_pieces, m = q - r * row_pieces;
                    int slot = req_old_slot + r;
                    if (slot >= pl.old_ring) slot -= pl.old_ring;
                    src = req_img + static_cast<int64_t>(y0 + r) * wc + m * kPieceFloats;
                    dst = old_area + slot * wc + m * kPieceFloats;
                    valid = wc - m * kPieceFloats;
                }
                if (lane * 4 < valid) __builtin_amdgcn_global_load_lds(src + lane * 4, dst, 16, 0, 2 /* non-temporal */);
            }
            if (!real) return;
            req_slot = req_slot == DEPTH ? 0 : req_slot + 1;
            req_old_slot += rows;
            if (req_old_slot >= pl.old_ring) req_old_slot -= pl.old_ring;
            if (++req_phase == pl.phases) {
                req_phase = 0;
                req_col += col_step;
                req_img += old_step;
            }
        };
        for (int d = 0; d < DEPTH; ++d) request(d < total);
        for (int t = 0; t < total; ++t) {
            wait_until_outstanding<(DEPTH - 1) * PER>();   // this wavefront's pieces of phase t are in LDS
            asm volatile("s_barrier" ::: "memory");        // everyone's are, and the adding wavefronts have left phase t - 1
            request(t + DEPTH < total);
        }
        wait_until_outstanding<0>();
        return;
    }

    // ---------------- additions ----------------
    // lane -> (s, x): the lane owns all C channels of its pixel (what it decides per window row - which
    // row, whether it has terms, first, last - it decides once for C sums); neighbouring lanes read LDS
    // words KS*KS*C apart (an odd stride for RGB images)
    uint32_t s_u, xx_u;
    pl.d_w.divmod(static_cast<uint32_t>(threadIdx.x), s_u, xx_u);
    const int s = static_cast<int>(s_u), xx = static_cast<int>(xx_u);
    const bool owner = s < M;
    const int eoff = xx * C;                               // within an image row
    // term (ky, kx) of element (y, x, ch) sits at  slot(oy)*pitch + (x+pad-kx)*KC + (ky*KS+kx)*C + ch
    //   = slot(oy)*pitch + ebase + ch + ky*KS*C + (KS-1-kx)*(KC-C)
    const int ebase = (xx + pl.pad) * KC - (KS - 1) * (KC - C);
    bool xok[KS];                                          // the terms with kx = KS-1-b exist
#pragma unroll
    for (int b = 0; b < KS; ++b) {
        const int ox = xx + pl.pad - (KS - 1 - b);
        xok[b] = ox >= 0 && ox < pl.ow;
    }
    const int m_start = (M - pl.pad % M) % M;
    float acc[C];
#pragma unroll
    for (int k = 0; k < C; ++k) acc[k] = 0.0f;
    int phase = 0, slot = 0;
    int mm = m_start;                      // (oy0 - pad) modulo M
    int old_pos = pl.old_ring - pl.pad;    // ring position of image row oy0 - pad (rows before the image have one too)
    float* img = in_deltas + static_cast<int64_t>(blockIdx.x) * pl.in_pitch;
    for (int t = 0; t < total; ++t) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // done reading phase t - 1
        asm volatile("s_barrier" ::: "memory");              // phase t is complete in LDS
        const int oy0 = phase * R;
        int d = s - mm;                                      // the lane's row is oy0 - pad + d
        if (d < 0) d += M;
        if (!owner) d = 0;                                   // lanes past the last pixel read where lane 0's row reads, and add nothing
        const int y = oy0 - pl.pad + d;
        const bool mine = owner && y >= 0 && y < pl.h;
        {
            // Everything below is selects rather than branches: a branch on a per-lane condition costs
            // several scalar instructions, and the scalar unit is shared by the whole compute unit.
            int pos = old_pos + d;
            if (pos >= pl.old_ring) pos -= pl.old_ring;
            float old_value[C];                                   // meaningful in the row's first phase
#pragma unroll
            for (int k = 0; k < C; ++k) old_value[k] = old_area[pos * wc + eoff + k];
            const float* tphase = tile + slot * (R * pitch) + ebase;
            float v[R][KS][C];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int ky = imin(imax(d - r, 0), KS - 1);      // clamped: the terms of a row without one are not added
                const float* trow = tphase + r * pitch + ky * (KS * C);
#pragma unroll
                for (int b = 0; b < KS; ++b)
#pragma unroll
                    for (int k = 0; k < C; ++k) v[r][b][k] = trow[b * (KC - C) + k];
            }
            bool store = false;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int ky = d - r, oy = oy0 + r;
                const bool valid = mine && ky >= 0 && ky < KS && oy < pl.oh;
                const bool first = ky == KS - 1 || oy == 0;       // the row's first col row starts from the old value
#pragma unroll
                for (int k = 0; k < C; ++k) {
                    float sum = first ? old_value[k] : acc[k];
#pragma unroll
                    for (int b = 0; b < KS; ++b) sum = xok[b] ? sum + v[r][b][k] : sum;
                    acc[k] = valid ? sum : acc[k];
                }
                store = store || (valid && (ky == 0 || oy == pl.oh - 1));       // its last one
            }
            if (store) {
                float* q = img + static_cast<int64_t>(y) * wc + eoff;
#pragma unroll
                for (int k = 0; k < C; ++k) q[k] = acc[k];
            }
        }
        slot = slot == DEPTH ? 0 : slot + 1;
        mm += R % M;
        if (mm >= M) mm -= M;
        old_pos += R;
        if (old_pos >= pl.old_ring) old_pos -= pl.old_ring;
        if (++phase == pl.phases) {
            phase = 0;
            img += old_step;
            mm = m_start;
            old_pos += pl.old_image_step;
            if (old_pos >= pl.old_ring) old_pos -= pl.old_ring;
        }
    }
}

// _cpuop 57-80: strict '>' from -FLT_MAX, so the first maximum in (y, x) scan
// order wins and NaN never does; empty windows give output 0 and argmax -1.
// One lane per W channels of one output position; lanes_per_image = oh*ow*cv.
// K > 0: the window is K x K, known at compile time; all K*K loads are issued first
// (positions outside the image read a clamped address and are skipped in the scan).
template <int W, bool AL, int K>
__device__ __forceinline__ void maxpool_fwd_body(const float* __restrict__ in, float* __restrict__ out,
                                                 float* __restrict__ argmax, int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t opix, chv, oy, ox;
    pl.d_cv.divmod(p, opix, chv);
    pl.d_ow.divmod(opix, oy, ox);
    const int y = static_cast<int>(oy) * g.sh - g.pad, x = static_cast<int>(ox) * g.sw - g.pad;
    const int y0 = imax(y, 0), y1 = imin(y + g.kh, g.h);
    const int x0 = imax(x, 0), x1 = imin(x + g.kw, g.w);
    const int64_t in_img = pl.in_pitch;
    const int64_t out_img = pl.out_pitch;
    const int ch0 = static_cast<int>(chv) * W;
    typedef typename VecT<W>::type R;
    for (int64_t img = group; img < n; img += pl.groups) {
        const float* base = in + img * in_img + ch0;
        R best = vsplat<W>(-FLT_MAX), where = vsplat<W>(-1.0f);
        auto take = [&](R v, int k) {
#pragma unroll
            for (int j = 0; j < W; ++j)
                if (comp<W>(v, j) > comp<W>(best, j)) {
                    comp<W>(best, j) = comp<W>(v, j);
                    comp<W>(where, j) = static_cast<float>(k + ch0 + j);
                }
        };
        if constexpr (K > 0) {
            R v[K * K];
#pragma unroll
            for (int a = 0; a < K; ++a)
#pragma unroll
                for (int b = 0; b < K; ++b) {
                    const int iy = imin(imax(y + a, 0), g.h - 1), ix = imin(imax(x + b, 0), g.w - 1);
                    v[a * K + b] = img_load<W, AL>(base + (iy * g.w + ix) * g.c);
                }
#pragma unroll
            for (int a = 0; a < K; ++a)
#pragma unroll
                for (int b = 0; b < K; ++b)
                    if (y + a >= y0 && y + a < y1 && x + b >= x0 && x + b < x1)
                        take(v[a * K + b], ((y + a) * g.w + (x + b)) * g.c);
        } else {
            for (int iy = y0; iy < y1; ++iy)
                for (int ix = x0; ix < x1; ++ix) {
                    const int k = (iy * g.w + ix) * g.c;
                    take(img_load<W, AL>(base + k), k);
                }
        }
#pragma unroll
        for (int j = 0; j < W; ++j)
            if (comp<W>(where, j) < 0.0f) comp<W>(best, j) = 0.0f;
        vstore<W, AL>(out + img * out_img + static_cast<int64_t>(p) * W, best);
        vstore<W, AL>(argmax + img * pl.aux_pitch + static_cast<int64_t>(p) * W, where);
    }
}
#define BSHIP_POOL_FWD_KERNEL(name, K)                                                                   \
    template <int W, bool AL>                                                                            \
    __global__ __launch_bounds__(kBlock) void name(const float* __restrict__ in, float* __restrict__ out, \
                                                   float* __restrict__ argmax, int64_t n, ImgPlan pl) {  \
        maxpool_fwd_body<W, AL, K>(in, out, argmax, n, pl);                                              \
    }
BSHIP_POOL_FWD_KERNEL(maxpool_fwd_kernel, 0)
BSHIP_POOL_FWD_KERNEL(maxpool_fwd_kernel_2x2, 2)
BSHIP_POOL_FWD_KERNEL(maxpool_fwd_kernel_3x3, 3)

// _cpuop 103-115 in gather form. One lane per W channels of one input pixel.
// C > 0: at most C x C output positions cover a pixel (C = ceil(window / stride), known at
// compile time); their loads are issued first, positions beyond the cover read a clamped address.
template <int W, bool AL, int C>
__device__ __forceinline__ void maxpool_bwd_body(const float* __restrict__ argmax,
                                                 const float* __restrict__ out_deltas,
                                                 float* __restrict__ in_deltas, int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t pix, chv, yy, xx;
    pl.d_cv.divmod(p, pix, chv);
    pl.d_w.divmod(pix, yy, xx);
    const int y = static_cast<int>(yy), x = static_cast<int>(xx);
    const int ch0 = static_cast<int>(chv) * W;
    const int self = (y * g.w + x) * g.c + ch0;        // what argmax holds for this pixel's first channel
    int oy0, oy1, ox0, ox1;
    cover_range(y, g.pad, pl.d_sh, g.kh, g.oh, oy0, oy1);
    cover_range(x, g.pad, pl.d_sw, g.kw, g.ow, ox0, ox1);
    const int64_t in_img = pl.in_pitch;
    const int64_t out_img = pl.out_pitch;
    typedef typename VecT<W>::type R;
    for (int64_t img = group; img < n; img += pl.groups) {
        float* q = in_deltas + img * in_img + static_cast<int64_t>(p) * W;
        R acc = vload<W, AL>(q);
        auto take = [&](R am, R d) {
#pragma unroll
            for (int j = 0; j < W; ++j)
                if (static_cast<int>(comp<W>(am, j)) == self + j) comp<W>(acc, j) += comp<W>(d, j);
        };
        if constexpr (C > 0) {
            R am[C * C], d[C * C];
#pragma unroll
            for (int a = 0; a < C; ++a)
#pragma unroll
                for (int b = 0; b < C; ++b) {
                    const int oy = imin(oy0 + a, g.oh - 1), ox = imin(ox0 + b, g.ow - 1);
                    const int64_t o = (static_cast<int64_t>(oy) * g.ow + ox) * g.c + ch0;
                    am[a * C + b] = img_load<W, AL>(argmax + img * pl.aux_pitch + o);
                    d[a * C + b] = img_load<W, AL>(out_deltas + img * out_img + o);
                }
#pragma unroll
            for (int a = 0; a < C; ++a)
#pragma unroll
                for (int b = 0; b < C; ++b)
                    if (oy0 + a < oy1 && ox0 + b < ox1) take(am[a * C + b], d[a * C + b]);
        } else {
            for (int oy = oy0; oy < oy1; ++oy)
                for (int ox = ox0; ox < ox1; ++ox) {
                    const int64_t o = (static_cast<int64_t>(oy) * g.ow + ox) * g.c + ch0;
                    take(img_load<W, AL>(argmax + img * pl.aux_pitch + o), img_load<W, AL>(out_deltas + img * out_img + o));
                }
        }
        vstore<W, AL>(q, acc, pl.through);
    }
}
#define BSHIP_POOL_BWD_KERNEL(name, C)                                                                   \
    template <int W, bool AL>                                                                            \
    __global__ __launch_bounds__(kBlock) void name(const float* __restrict__ argmax,                     \
                                                   const float* __restrict__ out_deltas,                 \
                                                   float* __restrict__ in_deltas, int64_t n, ImgPlan pl) { \
        maxpool_bwd_body<W, AL, C>(argmax, out_deltas, in_deltas, n, pl);                                \
    }
BSHIP_POOL_BWD_KERNEL(maxpool_bwd_kernel, 0)
BSHIP_POOL_BWD_KERNEL(maxpool_bwd_kernel_c1, 1)
BSHIP_POOL_BWD_KERNEL(maxpool_bwd_kernel_c2, 2)

// _cpuop 143-162: mean over the non-padding pixels of the window. K as for max pooling.
template <int W, bool AL, int K>
__device__ __forceinline__ void avgpool_fwd_body(const float* __restrict__ in, float* __restrict__ out,
                                                 int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t opix, chv, oy, ox;
    pl.d_cv.divmod(p, opix, chv);
    pl.d_ow.divmod(opix, oy, ox);
    const int y = static_cast<int>(oy) * g.sh - g.pad, x = static_cast<int>(ox) * g.sw - g.pad;
    const int y0 = imax(y, 0), y1 = imin(y + g.kh, g.h);
    const int x0 = imax(x, 0), x1 = imin(x + g.kw, g.w);
    const float size = static_cast<float>(imax((y1 - y0) * (x1 - x0), 1));
    const int64_t in_img = pl.in_pitch;
    const int64_t out_img = pl.out_pitch;
    typedef typename VecT<W>::type R;
    for (int64_t img = group; img < n; img += pl.groups) {
        const float* base = in + img * in_img + chv * W;
        R sum = vsplat<W>(0.0f);
        if constexpr (K > 0) {
            R v[K * K];
#pragma unroll
            for (int a = 0; a < K; ++a)
#pragma unroll
                for (int b = 0; b < K; ++b) {
                    const int iy = imin(imax(y + a, 0), g.h - 1), ix = imin(imax(x + b, 0), g.w - 1);
                    v[a * K + b] = img_load<W, AL>(base + (iy * g.w + ix) * g.c);
                }
#pragma unroll
            for (int a = 0; a < K; ++a)
#pragma unroll
                for (int b = 0; b < K; ++b)
                    if (y + a >= y0 && y + a < y1 && x + b >= x0 && x + b < x1) sum += v[a * K + b];
        } else {
            for (int iy = y0; iy < y1; ++iy)
                for (int ix = x0; ix < x1; ++ix) sum += img_load<W, AL>(base + (iy * g.w + ix) * g.c);
        }
#pragma unroll
        for (int j = 0; j < W; ++j) comp<W>(sum, j) = comp<W>(sum, j) / size;
        vstore<W, AL>(out + img * out_img + static_cast<int64_t>(p) * W, sum);
    }
}
#define BSHIP_AVG_FWD_KERNEL(name, K)                                                                    \
    template <int W, bool AL>                                                                            \
    __global__ __launch_bounds__(kBlock) void name(const float* __restrict__ in, float* __restrict__ out, \
                                                   int64_t n, ImgPlan pl) {                              \
        avgpool_fwd_body<W, AL, K>(in, out, n, pl);                                                      \
    }
BSHIP_AVG_FWD_KERNEL(avgpool_fwd_kernel, 0)
BSHIP_AVG_FWD_KERNEL(avgpool_fwd_kernel_2x2, 2)
BSHIP_AVG_FWD_KERNEL(avgpool_fwd_kernel_3x3, 3)

// _cpuop 187-202 in gather form. C as for max pooling.
template <int W, bool AL, int C>
__device__ __forceinline__ void avgpool_bwd_body(const float* __restrict__ out_deltas,
                                                 float* __restrict__ in_deltas, int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t pix, chv, yy, xx;
    pl.d_cv.divmod(p, pix, chv);
    pl.d_w.divmod(pix, yy, xx);
    const int y = static_cast<int>(yy), x = static_cast<int>(xx);
    int oy0, oy1, ox0, ox1;
    cover_range(y, g.pad, pl.d_sh, g.kh, g.oh, oy0, oy1);
    cover_range(x, g.pad, pl.d_sw, g.kw, g.ow, ox0, ox1);
    const int64_t in_img = pl.in_pitch;
    const int64_t out_img = pl.out_pitch;
    typedef typename VecT<W>::type R;
    // number of image pixels under the window at output position (oy, ox)
    auto window_size = [&](int oy, int ox) {
        const int wy = oy * g.sh - g.pad, wx = ox * g.sw - g.pad;
        const int ny = imin(wy + g.kh, g.h) - imax(wy, 0);
        const int nx = imin(wx + g.kw, g.w) - imax(wx, 0);
        return static_cast<float>(ny * nx);
    };
    for (int64_t img = group; img < n; img += pl.groups) {
        float* q = in_deltas + img * in_img + static_cast<int64_t>(p) * W;
        R acc = vload<W, AL>(q);
        const float* dimg = out_deltas + img * out_img + chv * W;
        if constexpr (C > 0) {
            R d[C * C];
#pragma unroll
            for (int a = 0; a < C; ++a)
#pragma unroll
                for (int b = 0; b < C; ++b) {
                    const int oy = imin(oy0 + a, g.oh - 1), ox = imin(ox0 + b, g.ow - 1);
                    d[a * C + b] = img_load<W, AL>(dimg + (static_cast<int64_t>(oy) * g.ow + ox) * g.c);
                }
#pragma unroll
            for (int a = 0; a < C; ++a)
#pragma unroll
                for (int b = 0; b < C; ++b)
                    if (oy0 + a < oy1 && ox0 + b < ox1) {
                        const float size = window_size(oy0 + a, ox0 + b);
#pragma unroll
                        for (int j = 0; j < W; ++j) comp<W>(acc, j) += comp<W>(d[a * C + b], j) / size;
                    }
        } else {
            for (int oy = oy0; oy < oy1; ++oy)
                for (int ox = ox0; ox < ox1; ++ox) {
                    const float size = window_size(oy, ox);
                    R d = img_load<W, AL>(dimg + (static_cast<int64_t>(oy) * g.ow + ox) * g.c);
#pragma unroll
                    for (int j = 0; j < W; ++j) comp<W>(acc, j) += comp<W>(d, j) / size;
                }
        }
        vstore<W, AL>(q, acc, pl.through);
    }
}
#define BSHIP_AVG_BWD_KERNEL(name, C)                                                                    \
    template <int W, bool AL>                                                                            \
    __global__ __launch_bounds__(kBlock) void name(const float* __restrict__ out_deltas,                 \
                                                   float* __restrict__ in_deltas, int64_t n, ImgPlan pl) { \
        avgpool_bwd_body<W, AL, C>(out_deltas, in_deltas, n, pl);                                        \
    }
BSHIP_AVG_BWD_KERNEL(avgpool_bwd_kernel, 0)
BSHIP_AVG_BWD_KERNEL(avgpool_bwd_kernel_c1, 1)
BSHIP_AVG_BWD_KERNEL(avgpool_bwd_kernel_c2, 2)

// Pooling backward for strides above 1 (_cpuop 103-115 and 187-202, gather form): one lane owns W
// channels of a stride-aligned S x S patch of input pixels, (y + pad) / S = pi and (x + pad) / S = pj.
// The windows that cover any pixel of the patch are the C x C output positions
// (pi - C + 1 .. pi) x (pj - C + 1 .. pj) with C = (k - 1) / S + 1, so a lane reads C*C window
// entries for S*S pixels (3x3 windows, stride 2: 2 per pixel) where a lane per pixel reads up to
// C*C for each (8 of its 10 accesses, which kept the vector memory path busier than HBM). Every
// pixel still adds its terms in (oy, ox) scan order. lanes_per_image = patch rows x patch columns x cv.
// MAX: max pooling (argmax holds the winner's index), otherwise average pooling.
template <int W, bool AL, int S, int C, bool MAX>
__device__ __forceinline__ void pool_bwd_patch_body(const float* __restrict__ argmax,
                                                    const float* __restrict__ out_deltas,
                                                    float* __restrict__ in_deltas, int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    uint32_t tile, group;
    if (!img_block(pl, tile, group)) return;
    const uint32_t p = tile * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t patch, chv, pi, pj;
    pl.d_cv.divmod(p, patch, chv);
    pl.d_pw.divmod(patch, pi, pj);
    const int ch0 = static_cast<int>(chv) * W;
    const int y0 = static_cast<int>(pi) * S - g.pad, x0 = static_cast<int>(pj) * S - g.pad;
    const int oyb = static_cast<int>(pi) - (C - 1), oxb = static_cast<int>(pj) - (C - 1);
    const int64_t in_img = pl.in_pitch;
    const int64_t out_img = pl.out_pitch;
    typedef typename VecT<W>::type R;
    bool valid[S * S];
    int pix_off[S * S];
#pragma unroll
    for (int r = 0; r < S; ++r)
#pragma unroll
        for (int t = 0; t < S; ++t) {
            const int y = y0 + r, x = x0 + t;
            valid[r * S + t] = y >= 0 && y < g.h && x >= 0 && x < g.w;
            pix_off[r * S + t] = (imin(imax(y, 0), g.h - 1) * g.w + imin(imax(x, 0), g.w - 1)) * g.c + ch0;
        }
    // window (a, b) of the cover: whether it exists, and for average pooling its pixel count
    bool exists[C * C];
    int win_off[C * C];
    float win_size[C * C];
#pragma unroll
    for (int a = 0; a < C; ++a)
#pragma unroll
        for (int b = 0; b < C; ++b) {
            const int oy = oyb + a, ox = oxb + b;
            exists[a * C + b] = oy >= 0 && oy < g.oh && ox >= 0 && ox < g.ow;
            win_off[a * C + b] = (imin(imax(oy, 0), g.oh - 1) * g.ow + imin(imax(ox, 0), g.ow - 1)) * g.c + ch0;
            const int wy = oy * S - g.pad, wx = ox * S - g.pad;
            win_size[a * C + b] = static_cast<float>((imin(wy + g.kh, g.h) - imax(wy, 0)) *
                                                     (imin(wx + g.kw, g.w) - imax(wx, 0)));
        }
    for (int64_t img = group; img < n; img += pl.groups) {
        float* q = in_deltas + img * in_img;
        R acc[S * S], am[C * C], d[C * C];
#pragma unroll
        for (int k = 0; k < S * S; ++k)
            if (valid[k]) acc[k] = vload<W, AL>(q + pix_off[k]);
#pragma unroll
        for (int k = 0; k < C * C; ++k) {
            if constexpr (MAX) am[k] = img_load<W, AL>(argmax + img * pl.aux_pitch + win_off[k]);
            d[k] = img_load<W, AL>(out_deltas + img * out_img + win_off[k]);
        }
        if constexpr (!MAX) {
            // a window's share delta / size is the same quotient for every pixel under it
#pragma unroll
            for (int k = 0; k < C * C; ++k)
#pragma unroll
                for (int j = 0; j < W; ++j) comp<W>(d[k], j) = comp<W>(d[k], j) / win_size[k];
        }
#pragma unroll
        for (int r = 0; r < S; ++r)
#pragma unroll
            for (int t = 0; t < S; ++t) {
                if (!valid[r * S + t]) continue;
#pragma unroll
                for (int a = 0; a < C; ++a)
#pragma unroll
                    for (int b = 0; b < C; ++b) {
                        // the pixel's offset inside window (a, b): S * (C - 1 - a) + r rows down
                        const bool covers = exists[a * C + b] && S * (C - 1 - a) + r < g.kh &&
                                            S * (C - 1 - b) + t < g.kw;
                        if (!covers) continue;
#pragma unroll
                        for (int j = 0; j < W; ++j) {
                            if constexpr (MAX) {
                                if (static_cast<int>(comp<W>(am[a * C + b], j)) == pix_off[r * S + t] + j)
                                    comp<W>(acc[r * S + t], j) += comp<W>(d[a * C + b], j);
                            } else {
                                comp<W>(acc[r * S + t], j) += comp<W>(d[a * C + b], j);
                            }
                        }
                    }
            }
#pragma unroll
        for (int k = 0; k < S * S; ++k)
            if (valid[k]) vstore<W, AL>(q + pix_off[k], acc[k], pl.through);
    }
}
#define BSHIP_POOL_BWD_PATCH_KERNELS(suffix, S, C)                                                       \
    template <int W, bool AL>                                                                            \
    __global__ __launch_bounds__(kBlock) void maxpool_bwd_patch_##suffix(                                \
        const float* __restrict__ argmax, const float* __restrict__ out_deltas,                          \
        float* __restrict__ in_deltas, int64_t n, ImgPlan pl) {                                          \
        pool_bwd_patch_body<W, AL, S, C, true>(argmax, out_deltas, in_deltas, n, pl);                    \
    }                                                                                                    \
    template <int W, bool AL>                                                                            \
    __global__ __launch_bounds__(kBlock) void avgpool_bwd_patch_##suffix(                                \
        const float* __restrict__ out_deltas, float* __restrict__ in_deltas, int64_t n, ImgPlan pl) {    \
        pool_bwd_patch_body<W, AL, S, C, false>(nullptr, out_deltas, in_deltas, n, pl);                  \
    }
BSHIP_POOL_BWD_PATCH_KERNELS(s2c1, 2, 1)
BSHIP_POOL_BWD_PATCH_KERNELS(s2c2, 2, 2)
BSHIP_POOL_BWD_PATCH_KERNELS(s3c1, 3, 1)

static int check_geom(const char* fn, int64_t n, const ImgGeom& g) {
    if (n < 0 || g.h < 0 || g.w < 0 || g.c < 0 || g.oh < 0 || g.ow < 0 || g.kh < 1 || g.kw < 1 ||
        g.pad < 0 || g.sh < 1 || g.sw < 1)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: bad geometry (n=%lld h=%d w=%d c=%d oh=%d ow=%d "
                         "k=%dx%d pad=%d stride=%dx%d)", fn, (long long)n, g.h, g.w, g.c, g.oh, g.ow,
                         g.kh, g.kw, g.pad, g.sh, g.sw);
    // per-image indices are held in int (and in float32 by argmax)
    if (static_cast<int64_t>(g.h) * g.w * g.c > 0x7fffffff ||
        static_cast<int64_t>(g.oh) * g.ow * g.c > 0x7fffffff)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: one image exceeds 2^31 elements", fn);
    return 0;
}

static inline int conv_out(int in, int k, int pad, int stride) { return (in + 2 * pad - k) / stride + 1; }

// Band size of im2col_band: about kBandFloats col floats, whole output rows when a row is a
// multiple of 4 floats, fewer when the batch is small (to keep every compute unit busy), and such
// that the two LDS tiles fit. Returns false when the geometry does not suit the banded kernel
// (col rows of an image not a multiple of 4 floats in total, or image rows too wide for LDS).
constexpr int64_t kBandFloats = 8192;
constexpr int64_t kBandMinWorkgroups = 1024;
constexpr size_t kBandLdsBytes = 64 * 1024;

static bool plan_im2col_band(const ImgGeom& g, int64_t n, int64_t per_image, BandPlan* out) {
    if (per_image % 4 != 0 || per_image > 0x7fffffff || per_image == 0) return false;
    const int64_t owk = static_cast<int64_t>(g.ow) * g.kh * g.kw * g.c;
    const int64_t wpc = (static_cast<int64_t>(g.w) + 2 * g.pad) * g.c;
    auto tile_rows_of = [&](int64_t band) {
        // output rows that `band` consecutive floats can touch, wherever they start
        const int64_t span = owk % 4 == 0 ? band / owk : (band >= 2 ? (band - 2) / owk + 2 : 1);
        return (span - 1) * g.sh + g.kh;
    };
    auto fits = [&](int64_t band) {
        return 2 * static_cast<size_t>(tile_rows_of(band) * wpc) * sizeof(float) <= kBandLdsBytes;
    };
    int64_t band;
    if (owk % 4 == 0) {
        int64_t rows = ceil_div(kBandFloats, owk);
        if (rows > g.oh) rows = g.oh;
        while (rows > 1 && (ceil_div(g.oh, rows) * n < kBandMinWorkgroups || !fits(rows * owk))) rows = (rows + 1) / 2;
        band = rows * owk;
    } else {
        band = kBandFloats;
        while (band > 1024 && (ceil_div(per_image, band) * n < kBandMinWorkgroups || !fits(band))) band /= 2;
    }
    if (!fits(band)) return false;
    out->g = g;
    out->band = static_cast<uint32_t>(band);
    out->per_image = static_cast<uint32_t>(per_image);
    out->tile_rows = static_cast<int>(tile_rows_of(band));
    out->wpc = static_cast<int>(wpc);
    out->d_k = FastDiv(static_cast<uint32_t>(g.kh * g.kw * g.c));
    out->d_ow = FastDiv(static_cast<uint32_t>(g.ow));
    out->d_kwc = FastDiv(static_cast<uint32_t>(g.kw * g.c));
    out->d_wpc = FastDiv(static_cast<uint32_t>(wpc));
    out->d_owk = FastDiv(static_cast<uint32_t>(owk));
    return true;
}

// Host mirror of cover_range().
static void cover_range_host(int p, int pad, int stride, int k, int n_out, int* lo, int* hi) {
    const int q = p + pad;
    *hi = imin(q / stride + 1, n_out);
    const int t = q - k + 1;
    *lo = t <= 0 ? 0 : (t + stride - 1) / stride;
}

// Phases of `rows` image rows: the most col rows one phase needs (`ring`) and the most col rows
// a phase adds to those of the phase before (`fresh`).
static void col2im_phase_extent(const ImgGeom& g, int rows, int* ring, int* fresh) {
    *ring = 0;
    *fresh = 0;
    int have_hi = 0;
    for (int y0 = 0; y0 < g.h; y0 += rows) {
        int lo, hi, unused;
        cover_range_host(y0, g.pad, g.sh, g.kh, g.oh, &lo, &unused);
        cover_range_host(imin(y0 + rows, g.h) - 1, g.pad, g.sh, g.kh, g.oh, &unused, &hi);
        *ring = imax(*ring, hi - lo);
        if (y0 > 0) *fresh = imax(*fresh, hi - imax(have_hi, lo));
        have_hi = imax(have_hi, imax(hi, lo));
    }
}

// col2im_band is used for fewer than 16 channels when the col rows are multiples of 4 floats and
// a ring for at least one image row per phase fits half of a compute unit's LDS. A workgroup gets
// as many phases as leave about kCol2imMinWorkgroups workgroups in the launch.
constexpr size_t kCol2imLdsBytes = 80 * 1024;
constexpr int64_t kCol2imMinWorkgroups = 1024;

static bool plan_col2im_band(const ImgGeom& g, int64_t n, Col2imBandPlan* out, size_t* lds_bytes) {
    if (g.c >= 16 || g.h == 0 || g.w == 0 || g.c == 0 || g.oh == 0 || g.ow == 0 || n == 0) return false;
    const int64_t owk = static_cast<int64_t>(g.ow) * g.kh * g.kw * g.c;
    if (owk % 4 != 0 || owk * g.oh > 0x7fffffff) return false;
    int rows = 0, ring = 0;
    for (int r = 1; r <= g.h; ++r) {
        int rg, fresh;
        col2im_phase_extent(g, r, &rg, &fresh);
        if (static_cast<size_t>(rg) * owk * sizeof(float) > kCol2imLdsBytes ||
            static_cast<int64_t>(fresh) * (owk / 4) > static_cast<int64_t>(kCol2imPrefetch) * kCol2imThreads ||
            static_cast<int64_t>(r) * g.w * g.c > static_cast<int64_t>(kCol2imOutsPerLane) * kCol2imThreads)
            break;
        rows = r;
        ring = rg;
    }
    if (rows == 0 || ring == 0) return false;
    const int64_t all_phases = ceil_div(g.h, rows);
    int64_t phases = n * all_phases / kCol2imMinWorkgroups;
    if (phases < 1) phases = 1;
    if (phases > all_phases) phases = all_phases;
    out->g = g;
    out->rows = rows;
    out->phases = static_cast<int>(phases);
    out->bands = static_cast<int>(ceil_div(all_phases, phases));
    out->ring = ring;
    out->owk = static_cast<uint32_t>(owk);
    out->d_bands = FastDiv(static_cast<uint32_t>(out->bands));
    out->d_wc = FastDiv(static_cast<uint32_t>(g.w * g.c));
    out->d_w = FastDiv(static_cast<uint32_t>(g.w));
    out->d_sh = FastDiv(static_cast<uint32_t>(g.sh));
    out->d_sw = FastDiv(static_cast<uint32_t>(g.sw));
    out->d_ring = FastDiv(static_cast<uint32_t>(ring));
    out->d_owk4 = FastDiv(static_cast<uint32_t>(owk / 4));
    *lds_bytes = static_cast<size_t>(ring) * owk * sizeof(float);
    return true;
}

// col2im_stream with `rows` col rows per phase, requests `depth` phases ahead and `per` loads per phase
// and requesting wavefront.
static bool plan_col2im_stream(const ImgGeom& g, int rows, int depth, int threads, int per, Col2imStreamPlan* out,
                               size_t* lds_bytes) {
    if (g.kh != g.kw || g.sh != 1 || g.sw != 1 || g.pad > g.kh - 1 || g.c >= 16) return false;
    if (g.h == 0 || g.w == 0 || g.c == 0 || g.oh == 0 || g.ow == 0 || rows < 1 || depth < 1) return false;
    const int kc = g.kh * g.kw * g.c;
    const int64_t owk = static_cast<int64_t>(g.ow) * kc;
    const int64_t wc = static_cast<int64_t>(g.w) * g.c;
    if (owk % 4 != 0 || wc % 4 != 0 || owk * g.oh > 0x7fffffff) return false;
    const int m = g.kh + rows - 1;                      // image rows a phase adds to
    // wavefronts left to request a phase's data with `per` loads each
    const int64_t add_waves = (static_cast<int64_t>(m) * g.w + kWave - 1) / kWave;   // one lane per pixel of those rows
    const int64_t req_waves = threads / kWave - add_waves;
    const int64_t pieces = (rows * owk + kPieceFloats - 1) / kPieceFloats +
                           imin(m - g.pad, g.h) * ((wc + kPieceFloats - 1) / kPieceFloats);
    if (req_waves < 1 || per * req_waves < pieces || (depth - 1) * per > 63) return false;
    const int old_ring = (depth + 1) * rows + g.kh;
    if (g.pad >= old_ring) return false;
    // reads of terms beyond the left and right image borders fall this far outside a col row
    const int guard = ((g.kh - 1) * (kc - g.c) + 3) / 4 * 4;
    const int back = imax((g.kh - 1) * kc, 4);
    const size_t bytes = (static_cast<size_t>(guard) + static_cast<size_t>(depth + 1) * rows * owk +
                          static_cast<size_t>(old_ring) * wc + back) * sizeof(float);
    if (bytes > 160 * 1024) return false;
    out->h = g.h; out->w = g.w; out->oh = g.oh; out->ow = g.ow; out->pad = g.pad;
    out->phases = (g.oh + rows - 1) / rows;
    out->add_waves = static_cast<int>(add_waves);
    out->old_ring = old_ring;
    // image row "oy0 - pad" of an image's last phase is row (phases-1)*rows - pad; of the next image's first
    // phase it is row -pad, h rows further on in the sequence of all image rows; every phase steps by `rows`
    out->old_image_step = ((g.h - out->phases * rows) % old_ring + old_ring) % old_ring;
    out->guard = guard;
    out->owk = static_cast<int>(owk);
    out->d_w = FastDiv(static_cast<uint32_t>(g.w));
    *lds_bytes = bytes;
    return true;
}

// Lets `kernel` use `bytes` of dynamic LDS (more than the default limit has to be asked for);
// remembers what each kernel was granted.
static bool allow_dynamic_lds_impl(const void* kernel, size_t bytes) {
    static std::mutex mutex;
    static std::map<const void*, size_t> granted;
    std::lock_guard<std::mutex> lock(mutex);
    auto it = granted.find(kernel);
    if (it != granted.end() && it->second >= bytes) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)) != hipSuccess)
        return false;
    granted[kernel] = bytes;
    return true;
}
template <typename K>
static bool allow_dynamic_lds(K kernel, size_t bytes) {
    return allow_dynamic_lds_impl(reinterpret_cast<const void*>(kernel), bytes);
}

// col2im_stream for 5x5 windows on 1 or 3 channels and 3x3 windows on 3, stride 1. A phase costs about 0.4 us whatever
// it carries, so the kernel is used where a phase of four (or two) col rows holds at least kStreamMinPhaseBytes.
// Measured at batch 2048 against the banded kernel: 32x32x3 under 5x5 (col rows of 9.6 KB) 118 us against 138,
// and 16 against 24 at batch 256; 24x24x3 (7.2 KB) 66 against 79; 64x64x1 at batch 1024 (6.4 KB) 76 against 88;
// 64x64x3 under 3x3 (6.9 KB) 195 against 213, 96x96x3 at batch 1024 221 against 256; 16x16x3 and 48x48x1
// (4.8 KB) 7 % ahead; col rows of 4.0 KB 6 % behind, 28x28x1 (2.8 KB, eight rows per phase) 20 % behind.
// Needs at least one image per workgroup. *launched says whether it ran.
constexpr size_t kStreamMinPhaseBytes = 18 * 1024;
constexpr int kStreamThreads = 1024, kStreamMinRequesters = 6;
static int try_col2im_stream(const ImgGeom& g, const float* col, float* in_deltas, int64_t in_pitch, int64_t n,
                             int* launched) {
    *launched = 0;
    const Context& c = ctx();
    const int64_t min_per_cu = c.col2im_stream_min_images_per_cu;
    if (min_per_cu <= 0 || n < min_per_cu * c.num_cus || !aligned16(col) || !aligned16(in_deltas) || in_pitch % 4 != 0)
        return 0;
    // (3x3 windows on one channel: col rows long enough would need more adding wavefronts than the rules below allow)
    if (!((g.kh == 5 && (g.c == 1 || g.c == 3)) || (g.kh == 3 && g.c == 3))) return 0;
    const size_t col_row_bytes = static_cast<size_t>(g.ow) * g.kh * g.kw * g.c * sizeof(float);
    if ((n / c.num_cus + 1) * g.oh > 0x7fffffff) return 0;
    // four col rows per phase and two phases in flight where the lanes and the LDS allow it (32x32x3 at batch
    // 2048: 117.5-118 us against 119-119.5 for two rows and four phases), else two rows and four phases
    Col2imStreamPlan sp;
    size_t lds = 0;
    int rows = 0, per = 0;
    for (int r : {4, 2}) {
        if (r * col_row_bytes < kStreamMinPhaseBytes) continue;
        for (int p : {2, 4, 8, 12}) {
            Col2imStreamPlan candidate;
            if (per != 0 || !plan_col2im_stream(g, r, r == 2 ? 4 : 2, kStreamThreads, p, &candidate, &lds)) continue;
            // with fewer requesting wavefronts the kernel falls behind the banded one (128x128x1 under 3x3:
            // 12 adding and 4 requesting wavefronts, 166 us against 140)
            if (kStreamThreads / kWave - candidate.add_waves < kStreamMinRequesters) continue;
            sp = candidate; rows = r; per = p;
        }
    }
    if (per == 0) return 0;
    sp.in_pitch = in_pitch;
    const dim3 grid(static_cast<unsigned>(c.num_cus));      // one workgroup per compute unit: it takes most of the LDS
#define BSHIP_COL2IM_STREAM(KS_, C_, R_, D_, P_)                                                                  \
    if (g.kh == KS_ && g.c == C_ && rows == R_ && per == P_) {                                                    \
        auto kernel = col2im_stream<KS_, C_, R_, kStreamThreads, D_, P_>;                                         \
        if (!allow_dynamic_lds(kernel, lds)) { (void)hipGetLastError(); return 0; }                               \
        hipLaunchKernelGGL(kernel, grid, dim3(kStreamThreads), lds, c.stream, col, in_deltas, n, sp);             \
        *launched = 1;                                                                                            \
        return check_launch("col2im");                                                                            \
    }
#define BSHIP_COL2IM_STREAM_PER(KS_, C_, R_, D_)                                                 \
    BSHIP_COL2IM_STREAM(KS_, C_, R_, D_, 2) BSHIP_COL2IM_STREAM(KS_, C_, R_, D_, 4)             \
    BSHIP_COL2IM_STREAM(KS_, C_, R_, D_, 8) BSHIP_COL2IM_STREAM(KS_, C_, R_, D_, 12)
    BSHIP_COL2IM_STREAM_PER(5, 3, 4, 2)
    BSHIP_COL2IM_STREAM_PER(5, 3, 2, 4)
    BSHIP_COL2IM_STREAM_PER(5, 1, 4, 2)
    BSHIP_COL2IM_STREAM_PER(5, 1, 2, 4)
    BSHIP_COL2IM_STREAM_PER(3, 3, 4, 2)
    BSHIP_COL2IM_STREAM_PER(3, 3, 2, 4)
#undef BSHIP_COL2IM_STREAM_PER
#undef BSHIP_COL2IM_STREAM
    return 0;
}

}  // namespace bship

using namespace bship;

// Launches kernel<W, AL> over lanes_per_image x n: W = 4 when the channels come in fours,
// AL when additionally every pointer is 16-byte aligned. The image pitches of the plan are the
// caller's local variables in_pitch, out_pitch and aux_pitch; through_out, another local, says whether
// the kernel stores its result write-through (ImgPlan::through).
#define BSHIP_LAUNCH_IMG(kernel, name, positions, aligned, ...) \
    BSHIP_LAUNCH_IMG_FULL(kernel, name, positions, aligned, kImagesPerWorkgroup, false, true, __VA_ARGS__)
// in_order: tiles in dispatch order instead of one run per XCD (img_block)
#define BSHIP_LAUNCH_IMG_ORDER(kernel, name, positions, aligned, order_, ...) \
    BSHIP_LAUNCH_IMG_FULL(kernel, name, positions, aligned, kImagesPerWorkgroup, order_, true, __VA_ARGS__)
#define BSHIP_LAUNCH_IMG_N(kernel, name, positions, aligned, images_per_wg, ...) \
    BSHIP_LAUNCH_IMG_FULL(kernel, name, positions, aligned, images_per_wg, false, true, __VA_ARGS__)
// for kernels that take exactly kImagesPerWorkgroup images at a time (im2col_body)
#define BSHIP_LAUNCH_IMG_EXACT(kernel, name, positions, aligned, ...) \
    BSHIP_LAUNCH_IMG_FULL(kernel, name, positions, aligned, kImagesPerWorkgroup, false, false, __VA_ARGS__)
// images_per_wg: how many images a workgroup walks through, one after the other (kernels whose image
// loop is `img = group; img += groups`; im2col_body needs kImagesPerWorkgroup). Measured at batch 2048:
// the pooling backward kernels (read-modify-write of in_deltas) want 1 (max 32x32x32: 0.75 -> 0.89 of
// peak, avg 0.71 -> 0.80), max pooling forward 4 (0.90 against 0.82 with 1).
#define BSHIP_LAUNCH_IMG_FULL(kernel, name, positions, aligned, images_per_wg, order_, few_ok_, ...)    \
    do {                                                                                                \
        const bool vec4_ = (g.c % 4 == 0);                                                              \
        const int cv_ = vec4_ ? g.c / 4 : g.c;                                                          \
        const int64_t lanes_ = static_cast<int64_t>(positions) * cv_;                                   \
        if (lanes_ > 0x7fffffff)                                                                        \
            return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: one image exceeds 2^31 elements", name);     \
        ImgPlan pl_;                                                                                    \
        pl_.g = g;                                                                                      \
        pl_.lanes_per_image = static_cast<uint32_t>(lanes_);                                            \
        pl_.d_cv = FastDiv(static_cast<uint32_t>(imax(cv_, 1)));                                        \
        pl_.d_w = FastDiv(static_cast<uint32_t>(imax(g.w, 1)));                                         \
        pl_.d_ow = FastDiv(static_cast<uint32_t>(imax(g.ow, 1)));                                       \
        pl_.d_kcv = FastDiv(static_cast<uint32_t>(imax(g.kh * g.kw * cv_, 1)));                         \
        pl_.d_kwcv = FastDiv(static_cast<uint32_t>(imax(g.kw * cv_, 1)));                               \
        pl_.d_sh = FastDiv(static_cast<uint32_t>(g.sh));                                                \
        pl_.d_sw = FastDiv(static_cast<uint32_t>(g.sw));                                                \
        pl_.d_pw = FastDiv(static_cast<uint32_t>(imax((g.w - 1 + g.pad) / g.sw + 1, 1)));               \
        pl_.in_pitch = in_pitch;                                                                        \
        pl_.out_pitch = out_pitch;                                                                      \
        pl_.aux_pitch = aux_pitch;                                                                      \
        pl_.tiles = static_cast<uint32_t>(ceil_div(lanes_, kBlock));                                    \
        /* a small batch: one image per workgroup when several would leave compute units without work */ \
        const int64_t ipw_ = ((few_ok_) && static_cast<int64_t>(pl_.tiles) * ceil_div(n, images_per_wg) <  \
                                               4 * static_cast<int64_t>(ctx().num_cus)) ? 1 : (images_per_wg); \
        const int64_t gy_ = ceil_div(n, ipw_);                                                          \
        pl_.groups = static_cast<uint32_t>(gy_ < 65535 ? gy_ : 65535);                                  \
        if (static_cast<int64_t>(pl_.tiles) * pl_.groups > 0x7ffffff0)                                  \
            pl_.groups = static_cast<uint32_t>(imax(1, static_cast<int>(0x7ffffff0 / pl_.tiles)));      \
        pl_.d_tiles = FastDiv(pl_.tiles);                                                               \
        pl_.per_xcd = static_cast<uint32_t>(ceil_div(static_cast<int64_t>(pl_.tiles) * pl_.groups, kXcdCount)); \
        pl_.in_order = (order_);                                                                        \
        pl_.through = through_out;                                                                      \
        const dim3 grid_(pl_.per_xcd * kXcdCount);                                                      \
        if (vec4_ && (aligned))                                                                         \
            hipLaunchKernelGGL((kernel<4, true>), grid_, dim3(kBlock), 0, ctx().stream, __VA_ARGS__, n, pl_); \
        else if (vec4_)                                                                                 \
            hipLaunchKernelGGL((kernel<4, false>), grid_, dim3(kBlock), 0, ctx().stream, __VA_ARGS__, n, pl_); \
        else                                                                                            \
            hipLaunchKernelGGL((kernel<1, false>), grid_, dim3(kBlock), 0, ctx().stream, __VA_ARGS__, n, pl_); \
        return check_launch(name);                                                                      \
    } while (0)
extern "C" {

int bship_im2col_nhwc_f32(const float* in, float* col, int64_t n, int h, int w, int c, int kh,
                          int kw, int pad, int stride_h, int stride_w) {
    return bship_im2col_nhwc_pitched_f32(in, static_cast<int64_t>(h) * w * c, col, n, h, w, c, kh, kw, pad,
                                         stride_h, stride_w);
}

int bship_im2col_nhwc_pitched_f32(const float* in, int64_t in_pitch, float* col, int64_t n, int h, int w,
                                  int c, int kh, int kw, int pad, int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    const bool through_out = false;   // these kernels keep their stores (pooling forward loses with write-through)
    BSHIP_REQUIRE_DIM(kh >= 1 && kw >= 1 && stride_h >= 1 && stride_w >= 1 && pad >= 0);
    BSHIP_REQUIRE_DIM(h + 2 * pad >= kh && w + 2 * pad >= kw);
    ImgGeom g{h, w, c, conv_out(h, kh, pad, stride_h), conv_out(w, kw, pad, stride_w), kh, kw, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c);
    const int64_t total = n * g.oh * g.ow * kh * kw * c;
    if (total == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(col);
    BSHIP_REQUIRE_F32_ALIGNED(in);
    BSHIP_REQUIRE_F32_ALIGNED(col);
    // write-through stores from 1 MB on: a col matrix beyond the last-level cache's 256 MB is written fastest
    // that way (a pure write stream), a smaller one is left in that cache for the product that reads it next
    // (CNN step at batch 100, col matrices of 31 and 72 MB: 0.460 -> 0.456 ms)
    const bool write_through = static_cast<size_t>(total) >= ctx().store_through_min;
    const int64_t per_image = static_cast<int64_t>(g.oh) * g.ow * kh * kw * c;
    const int64_t out_pitch = per_image, aux_pitch = 0;
    BandPlan bp;
    if (plan_im2col_band(g, n, per_image, &bp)) {
        bp.in_pitch = in_pitch;
        const size_t lds = 2 * static_cast<size_t>(bp.tile_rows) * bp.wpc * sizeof(float);
        const dim3 grid(static_cast<unsigned>(ceil_div(per_image, bp.band)), static_cast<unsigned>(n < 65535 ? n : 65535));
        const int64_t K = static_cast<int64_t>(kh) * kw * c;
        const int64_t owk = g.ow * K;
        if (c % 4 == 0) {
            if (write_through) hipLaunchKernelGGL((im2col_band<4, true>), grid, dim3(kBlock), lds, ctx().stream, in, col, n, bp);
            else               hipLaunchKernelGGL((im2col_band<4, false>), grid, dim3(kBlock), lds, ctx().stream, in, col, n, bp);
        } else if (g.ow % 4 == 0 && bp.band % owk == 0 && (bp.tile_rows * bp.wpc) % 4 == 0 &&
                   lds + static_cast<size_t>(K) * 16 <= kBandLdsBytes) {
            // bands of whole output rows, 4 pixels = K stores: the stores' sources come from a table
            const size_t lds_t = lds + static_cast<size_t>(K) * 16;
            const FastDiv d_K(static_cast<uint32_t>(K)), d_gpr(static_cast<uint32_t>(g.ow / 4));
            if (write_through) hipLaunchKernelGGL(im2col_band_groups<true>, grid, dim3(kBlock), lds_t, ctx().stream, in, col, n, bp, d_K, d_gpr);
            else               hipLaunchKernelGGL(im2col_band_groups<false>, grid, dim3(kBlock), lds_t, ctx().stream, in, col, n, bp, d_K, d_gpr);
        } else {
            if (write_through) hipLaunchKernelGGL((im2col_band<1, true>), grid, dim3(kBlock), lds, ctx().stream, in, col, n, bp);
            else               hipLaunchKernelGGL((im2col_band<1, false>), grid, dim3(kBlock), lds, ctx().stream, in, col, n, bp);
        }
        return check_launch("im2col");
    }
    if (c % 4 != 0 && per_image % 4 == 0 && per_image <= 0x7fffffff) {
        ImgPlan pl;
        pl.g = g;
        pl.lanes_per_image = static_cast<uint32_t>(per_image / 4);
        pl.d_cv = FastDiv(static_cast<uint32_t>(c));
        pl.d_ow = FastDiv(static_cast<uint32_t>(g.ow));
        pl.d_kcv = FastDiv(static_cast<uint32_t>(kh * kw * c));
        pl.d_kwcv = FastDiv(static_cast<uint32_t>(kw * c));
        pl.in_pitch = in_pitch;
        pl.out_pitch = out_pitch;
        pl.aux_pitch = 0;
        const int64_t gy = ceil_div(n, kImagesPerWorkgroup);
        pl.tiles = static_cast<uint32_t>(ceil_div(per_image / 4, kBlock));
        pl.groups = static_cast<uint32_t>(gy < 65535 ? gy : 65535);
        if (static_cast<int64_t>(pl.tiles) * pl.groups > 0x7ffffff0)
            pl.groups = static_cast<uint32_t>(imax(1, static_cast<int>(0x7ffffff0 / pl.tiles)));
        pl.d_tiles = FastDiv(pl.tiles);
        pl.per_xcd = static_cast<uint32_t>(ceil_div(static_cast<int64_t>(pl.tiles) * pl.groups, kXcdCount));
        const dim3 grid(pl.per_xcd * kXcdCount);
        if (write_through) hipLaunchKernelGGL(im2col_gather4<true>, grid, dim3(kBlock), 0, ctx().stream, in, col, n, pl);
        else               hipLaunchKernelGGL(im2col_gather4<false>, grid, dim3(kBlock), 0, ctx().stream, in, col, n, pl);
        return check_launch("im2col");
    }
    const bool al = aligned16(in) && aligned16(col) && in_pitch % 4 == 0;
    if (write_through)
        BSHIP_LAUNCH_IMG_EXACT(im2col_wt, "im2col", static_cast<int64_t>(g.oh) * g.ow * kh * kw, al, in, col);
    BSHIP_LAUNCH_IMG_EXACT(im2col_cached, "im2col", static_cast<int64_t>(g.oh) * g.ow * kh * kw, al, in, col);
}

int bship_col2im_nhwc_f32(const float* col, float* in_deltas, int64_t n, int h, int w, int c,
                          int kh, int kw, int pad, int stride_h, int stride_w) {
    return bship_col2im_nhwc_pitched_f32(col, in_deltas, static_cast<int64_t>(h) * w * c, n, h, w, c, kh, kw,
                                         pad, stride_h, stride_w);
}

int bship_col2im_nhwc_pitched_f32(const float* col, float* in_deltas, int64_t in_pitch, int64_t n, int h,
                                  int w, int c, int kh, int kw, int pad, int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    const bool through_out = false;   // these kernels keep their stores (pooling forward loses with write-through)
    BSHIP_REQUIRE_DIM(kh >= 1 && kw >= 1 && stride_h >= 1 && stride_w >= 1 && pad >= 0);
    BSHIP_REQUIRE_DIM(h + 2 * pad >= kh && w + 2 * pad >= kw);
    ImgGeom g{h, w, c, conv_out(h, kh, pad, stride_h), conv_out(w, kw, pad, stride_w), kh, kw, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c);
    const int64_t total = n * h * w * c;
    if (total == 0) return 0;
    BSHIP_REQUIRE_PTR(col);
    BSHIP_REQUIRE_PTR(in_deltas);
    BSHIP_REQUIRE_F32_ALIGNED(col);
    BSHIP_REQUIRE_F32_ALIGNED(in_deltas);
    const int64_t out_pitch = 0, aux_pitch = 0;
    {
        int launched = 0;
        st = try_col2im_stream(g, col, in_deltas, in_pitch, n, &launched);
        if (launched) return st;
    }
    Col2imBandPlan bp;
    size_t lds = 0;
    if (plan_col2im_band(g, n, &bp, &lds)) {
        bp.in_pitch = in_pitch;
        const int ks = (kh == kw && stride_h == 1 && stride_w == 1 && (kh == 3 || kh == 5)) ? kh : 0;
        const int64_t groups = ceil_div(n, kXcds) * bp.bands;
        if (groups * kXcds <= 0x7fffffff) {
            const dim3 grid(static_cast<unsigned>(groups * kXcds));
#define BSHIP_COL2IM_BAND(KS_)                                                                          \
            if (ks == KS_ && allow_dynamic_lds(col2im_band<KS_>, lds)) {                                \
                hipLaunchKernelGGL(col2im_band<KS_>, grid, dim3(kCol2imThreads), lds, ctx().stream, col,        \
                                   in_deltas, n, bp);                                                   \
                return check_launch("col2im");                                                          \
            }
            BSHIP_COL2IM_BAND(5)
            BSHIP_COL2IM_BAND(3)
            BSHIP_COL2IM_BAND(0)
#undef BSHIP_COL2IM_BAND
        }
        (void)hipGetLastError();   // the attribute was refused: use the kernel without LDS
    }
    const bool al = aligned16(col) && aligned16(in_deltas) && in_pitch % 4 == 0;
    // one image's col matrix must be addressable with 32-bit offsets for the compile-time windows
    const bool small_image = static_cast<int64_t>(g.oh) * g.ow * kh * kw * c <= 0x7fffffff;
    // for launches of up to 8 workgroups per compute unit: with more, enough wavefronts wait side by side and the
    // plain loops are as fast (15x15x32, 5x5: batch 100 35.7 -> 18 us, CNN step 0.457 -> 0.437 ms; batch 2048
    // 0.756 against 0.751 of peak)
    const int64_t workgroups = ceil_div(static_cast<int64_t>(h) * w * (c % 4 == 0 ? c / 4 : c), kBlock) *
                               ceil_div(n, kImagesPerWorkgroup);
    const int ks_gather = (kh == kw && stride_h == 1 && stride_w == 1 && small_image &&
                           workgroups <= 8 * static_cast<int64_t>(ctx().num_cus)) ? kh : 0;
    if (ks_gather == 5)
        BSHIP_LAUNCH_IMG_ORDER(col2im_kernel_k5, "col2im", static_cast<int64_t>(h) * w, al, true, col, in_deltas);
    if (ks_gather == 3)
        BSHIP_LAUNCH_IMG_ORDER(col2im_kernel_k3, "col2im", static_cast<int64_t>(h) * w, al, true, col, in_deltas);
    BSHIP_LAUNCH_IMG_ORDER(col2im_kernel, "col2im", static_cast<int64_t>(h) * w, al, true, col, in_deltas);
}

int bship_maxpool_fwd_nhwc_f32(const float* in, float* out, float* argmax, int64_t n, int h, int w,
                               int c, int out_h, int out_w, int pool_h, int pool_w, int pad,
                               int stride_h, int stride_w) {
    const int64_t o = static_cast<int64_t>(out_h) * out_w * c;
    return bship_maxpool_fwd_nhwc_pitched_f32(in, static_cast<int64_t>(h) * w * c, out, o, argmax, o, n, h, w, c,
                                              out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w);
}

int bship_maxpool_fwd_nhwc_pitched_f32(const float* in, int64_t in_pitch, float* out, int64_t out_pitch,
                                       float* argmax, int64_t aux_pitch, int64_t n, int h, int w, int c,
                                       int out_h, int out_w, int pool_h, int pool_w, int pad, int stride_h,
                                       int stride_w) {
    BSHIP_REQUIRE_INIT();
    const bool through_out = false;   // these kernels keep their stores (pooling forward loses with write-through)
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t out_image = static_cast<int64_t>(out_h) * out_w * c;
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c && out_pitch >= out_image && aux_pitch >= out_image);
    if (n * out_image == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_PTR(argmax);
    BSHIP_REQUIRE_F32_ALIGNED(in);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    BSHIP_REQUIRE_F32_ALIGNED(argmax);
    const bool al = aligned16(in) && aligned16(out) && aligned16(argmax) && (in_pitch | out_pitch | aux_pitch) % 4 == 0;
    if (pool_h == 3 && pool_w == 3 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG(maxpool_fwd_kernel_3x3, "maxpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out, argmax);
    if (pool_h == 2 && pool_w == 2 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG(maxpool_fwd_kernel_2x2, "maxpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out, argmax);
    BSHIP_LAUNCH_IMG(maxpool_fwd_kernel, "maxpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out, argmax);
}

int bship_maxpool_bwd_nhwc_f32(const float* argmax, const float* out_deltas, float* in_deltas,
                               int64_t n, int h, int w, int c, int out_h, int out_w, int pool_h,
                               int pool_w, int pad, int stride_h, int stride_w) {
    const int64_t o = static_cast<int64_t>(out_h) * out_w * c;
    return bship_maxpool_bwd_nhwc_pitched_f32(argmax, o, out_deltas, o, in_deltas, static_cast<int64_t>(h) * w * c, n,
                                              h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w);
}

int bship_maxpool_bwd_nhwc_pitched_f32(const float* argmax, int64_t aux_pitch, const float* out_deltas,
                                       int64_t out_pitch, float* in_deltas, int64_t in_pitch, int64_t n, int h,
                                       int w, int c, int out_h, int out_w, int pool_h, int pool_w, int pad,
                                       int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t out_image = static_cast<int64_t>(out_h) * out_w * c;
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c && out_pitch >= out_image && aux_pitch >= out_image);
    const int64_t total = n * h * w * c;
    if (total == 0 || out_h == 0 || out_w == 0) return 0;
    // in_deltas of up to half the last-level cache's size (they are read as well as written): write-through.
    // 15x15x64 at batch 2048, 118 MB: max pooling backward 0.79 -> 0.89 of peak, average 0.75 -> 0.86;
    // 32x32x32, 256 MB, loses with it: 0.86 -> 0.72 and 0.81 -> 0.73.
    const bool through_out = store_through(2 * static_cast<size_t>(total));
    BSHIP_REQUIRE_PTR(argmax);
    BSHIP_REQUIRE_PTR(out_deltas);
    BSHIP_REQUIRE_PTR(in_deltas);
    BSHIP_REQUIRE_F32_ALIGNED(argmax);
    BSHIP_REQUIRE_F32_ALIGNED(out_deltas);
    BSHIP_REQUIRE_F32_ALIGNED(in_deltas);
    const bool al = aligned16(argmax) && aligned16(out_deltas) && aligned16(in_deltas) &&
                    (in_pitch | out_pitch | aux_pitch) % 4 == 0;
    // square windows and strides above 1: a lane per stride-aligned patch of pixels
    if (pool_h == pool_w && stride_h == stride_w && (stride_h == 2 || stride_h == 3)) {
        const int64_t patches = static_cast<int64_t>((h - 1 + pad) / stride_h + 1) * ((w - 1 + pad) / stride_w + 1);
        const int cover_patch = (pool_h - 1) / stride_h + 1;
        if (stride_h == 2 && cover_patch == 1)
            BSHIP_LAUNCH_IMG_N(maxpool_bwd_patch_s2c1, "maxpool2d_backward_batch", patches, al, 1, argmax, out_deltas, in_deltas);
        if (stride_h == 2 && cover_patch == 2)
            BSHIP_LAUNCH_IMG_N(maxpool_bwd_patch_s2c2, "maxpool2d_backward_batch", patches, al, 1, argmax, out_deltas, in_deltas);
        if (stride_h == 3 && cover_patch == 1)
            BSHIP_LAUNCH_IMG_N(maxpool_bwd_patch_s3c1, "maxpool2d_backward_batch", patches, al, 1, argmax, out_deltas, in_deltas);
    }
    // how many output positions can cover one pixel along each axis
    const int cover = imax((pool_h + stride_h - 1) / stride_h, (pool_w + stride_w - 1) / stride_w);
    if (cover == 1)
        BSHIP_LAUNCH_IMG(maxpool_bwd_kernel_c1, "maxpool2d_backward_batch", static_cast<int64_t>(h) * w, al, argmax, out_deltas, in_deltas);
    if (cover == 2)
        BSHIP_LAUNCH_IMG(maxpool_bwd_kernel_c2, "maxpool2d_backward_batch", static_cast<int64_t>(h) * w, al, argmax, out_deltas, in_deltas);
    BSHIP_LAUNCH_IMG(maxpool_bwd_kernel, "maxpool2d_backward_batch", static_cast<int64_t>(h) * w, al, argmax, out_deltas, in_deltas);
}

int bship_avgpool_fwd_nhwc_f32(const float* in, float* out, int64_t n, int h, int w, int c,
                               int out_h, int out_w, int pool_h, int pool_w, int pad, int stride_h,
                               int stride_w) {
    return bship_avgpool_fwd_nhwc_pitched_f32(in, static_cast<int64_t>(h) * w * c, out,
                                              static_cast<int64_t>(out_h) * out_w * c, n, h, w, c, out_h, out_w,
                                              pool_h, pool_w, pad, stride_h, stride_w);
}

int bship_avgpool_fwd_nhwc_pitched_f32(const float* in, int64_t in_pitch, float* out, int64_t out_pitch, int64_t n,
                                       int h, int w, int c, int out_h, int out_w, int pool_h, int pool_w, int pad,
                                       int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    const bool through_out = false;   // these kernels keep their stores (pooling forward loses with write-through)
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t out_image = static_cast<int64_t>(out_h) * out_w * c;
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c && out_pitch >= out_image);
    if (n * out_image == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(in);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    const int64_t aux_pitch = 0;
    const bool al = aligned16(in) && aligned16(out) && (in_pitch | out_pitch) % 4 == 0;
    if (pool_h == 3 && pool_w == 3 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG_N(avgpool_fwd_kernel_3x3, "avgpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, 1, in, out);
    if (pool_h == 2 && pool_w == 2 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG_N(avgpool_fwd_kernel_2x2, "avgpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, 1, in, out);
    BSHIP_LAUNCH_IMG(avgpool_fwd_kernel, "avgpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out);
}

int bship_avgpool_bwd_nhwc_f32(const float* out_deltas, float* in_deltas, int64_t n, int h, int w,
                               int c, int out_h, int out_w, int pool_h, int pool_w, int pad,
                               int stride_h, int stride_w) {
    return bship_avgpool_bwd_nhwc_pitched_f32(out_deltas, static_cast<int64_t>(out_h) * out_w * c, in_deltas,
                                              static_cast<int64_t>(h) * w * c, n, h, w, c, out_h, out_w, pool_h,
                                              pool_w, pad, stride_h, stride_w);
}

int bship_avgpool_bwd_nhwc_pitched_f32(const float* out_deltas, int64_t out_pitch, float* in_deltas, int64_t in_pitch,
                                       int64_t n, int h, int w, int c, int out_h, int out_w, int pool_h, int pool_w,
                                       int pad, int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    BSHIP_REQUIRE_DIM(in_pitch >= static_cast<int64_t>(h) * w * c &&
                      out_pitch >= static_cast<int64_t>(out_h) * out_w * c);
    const int64_t total = n * h * w * c;
    if (total == 0 || out_h == 0 || out_w == 0) return 0;
    // in_deltas of up to half the last-level cache's size (they are read as well as written): write-through.
    // 15x15x64 at batch 2048, 118 MB: max pooling backward 0.79 -> 0.89 of peak, average 0.75 -> 0.86;
    // 32x32x32, 256 MB, loses with it: 0.86 -> 0.72 and 0.81 -> 0.73.
    const bool through_out = store_through(2 * static_cast<size_t>(total));
    BSHIP_REQUIRE_PTR(out_deltas);
    BSHIP_REQUIRE_PTR(in_deltas);
    BSHIP_REQUIRE_F32_ALIGNED(out_deltas);
    BSHIP_REQUIRE_F32_ALIGNED(in_deltas);
    const int64_t aux_pitch = 0;
    const bool al = aligned16(out_deltas) && aligned16(in_deltas) && (in_pitch | out_pitch) % 4 == 0;
    if (pool_h == pool_w && stride_h == stride_w && (stride_h == 2 || stride_h == 3)) {
        const int64_t patches = static_cast<int64_t>((h - 1 + pad) / stride_h + 1) * ((w - 1 + pad) / stride_w + 1);
        const int cover_patch = (pool_h - 1) / stride_h + 1;
        if (stride_h == 2 && cover_patch == 1)
            BSHIP_LAUNCH_IMG_N(avgpool_bwd_patch_s2c1, "avgpool2d_backward_batch", patches, al, 1, out_deltas, in_deltas);
        if (stride_h == 2 && cover_patch == 2)
            BSHIP_LAUNCH_IMG_N(avgpool_bwd_patch_s2c2, "avgpool2d_backward_batch", patches, al, 1, out_deltas, in_deltas);
        if (stride_h == 3 && cover_patch == 1)
            BSHIP_LAUNCH_IMG_N(avgpool_bwd_patch_s3c1, "avgpool2d_backward_batch", patches, al, 1, out_deltas, in_deltas);
    }
    const int cover = imax((pool_h + stride_h - 1) / stride_h, (pool_w + stride_w - 1) / stride_w);
    if (cover == 1)
        BSHIP_LAUNCH_IMG(avgpool_bwd_kernel_c1, "avgpool2d_backward_batch", static_cast<int64_t>(h) * w, al, out_deltas, in_deltas);
    if (cover == 2)
        BSHIP_LAUNCH_IMG(avgpool_bwd_kernel_c2, "avgpool2d_backward_batch", static_cast<int64_t>(h) * w, al, out_deltas, in_deltas);
    BSHIP_LAUNCH_IMG(avgpool_bwd_kernel, "avgpool2d_backward_batch", static_cast<int64_t>(h) * w, al, out_deltas, in_deltas);
}

}  // extern "C"
