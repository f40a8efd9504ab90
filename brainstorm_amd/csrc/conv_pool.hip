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

// Range [lo, hi) of output positions o with  o*stride - pad <= p < o*stride - pad + k.
__device__ __forceinline__ void cover_range(int p, int pad, const FastDiv& stride, int k, int n_out,
                                            int& lo, int& hi) {
    const int q = p + pad;                       // o*stride <= q < o*stride + k
    hi = imin(static_cast<int>(stride.div(static_cast<uint32_t>(q))) + 1, n_out);
    const int t = q - k + 1;                     // o*stride >= t
    lo = t <= 0 ? 0 : static_cast<int>(stride.div(static_cast<uint32_t>(t) + stride.d - 1));
}

// Cached (not streaming) accesses: the images are re-read by overlapping windows.
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
};

// col[(img, oy, ox), (ky, kx, ch)] = in[img, oy*sh-pad+ky, ox*sw-pad+kx, ch] or 0   (_cpuop 264-277)
// One lane per W channels of one (oy, ox, ky, kx); lanes_per_image = oh*ow*kh*kw*cv.
// WT: write-through stores for a col matrix too large to stay in the caches.
template <int W, bool AL, bool WT>
__device__ __forceinline__ void im2col_body(const float* __restrict__ in, float* __restrict__ col,
                                            int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
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
    const int64_t in_img = static_cast<int64_t>(g.h) * g.w * g.c;
    const int64_t col_img = static_cast<int64_t>(pl.lanes_per_image) * W;
    // kImagesPerWorkgroup images at a time: all loads first, then all stores
    for (int64_t img0 = static_cast<int64_t>(blockIdx.y) * kImagesPerWorkgroup; img0 < n;
         img0 += static_cast<int64_t>(gridDim.y) * kImagesPerWorkgroup) {
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
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
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
    const int64_t in_img = static_cast<int64_t>(g.h) * g.w * g.c;
    const int64_t col_img = static_cast<int64_t>(pl.lanes_per_image) * 4;
    for (int64_t img0 = static_cast<int64_t>(blockIdx.y) * kImagesPerWorkgroup; img0 < n;
         img0 += static_cast<int64_t>(gridDim.y) * kImagesPerWorkgroup) {
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

// in_deltas[img, y, x, ch] += sum over covering (oy, ox), in scan order, of
// col[(img, oy, ox), (y - (oy*sh-pad), x - (ox*sw-pad), ch)]               (_cpuop 295-309)
// One lane per W channels of one input pixel; lanes_per_image = h*w*cv.
template <int W, bool AL>
__global__ __launch_bounds__(kBlock) void col2im_kernel(const float* __restrict__ col,
                                                        float* __restrict__ in_deltas, int64_t n,
                                                        ImgPlan pl) {
    const ImgGeom& g = pl.g;
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t pix, chv, yy, xx;
    pl.d_cv.divmod(p, pix, chv);
    pl.d_w.divmod(pix, yy, xx);
    const int y = static_cast<int>(yy), x = static_cast<int>(xx);
    int oy0, oy1, ox0, ox1;
    cover_range(y, g.pad, pl.d_sh, g.kh, g.oh, oy0, oy1);
    cover_range(x, g.pad, pl.d_sw, g.kw, g.ow, ox0, ox1);
    const int64_t kc = static_cast<int64_t>(g.kh) * g.kw * g.c;
    const int64_t in_img = static_cast<int64_t>(g.h) * g.w * g.c;
    const int64_t col_img = static_cast<int64_t>(g.oh) * g.ow * kc;
    for (int64_t img = blockIdx.y; img < n; img += gridDim.y) {
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

// _cpuop 57-80: strict '>' from -FLT_MAX, so the first maximum in (y, x) scan
// order wins and NaN never does; empty windows give output 0 and argmax -1.
// One lane per W channels of one output position; lanes_per_image = oh*ow*cv.
// K > 0: the window is K x K, known at compile time; all K*K loads are issued first
// (positions outside the image read a clamped address and are skipped in the scan).
template <int W, bool AL, int K>
__device__ __forceinline__ void maxpool_fwd_body(const float* __restrict__ in, float* __restrict__ out,
                                                 float* __restrict__ argmax, int64_t n, const ImgPlan& pl) {
    const ImgGeom& g = pl.g;
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t opix, chv, oy, ox;
    pl.d_cv.divmod(p, opix, chv);
    pl.d_ow.divmod(opix, oy, ox);
    const int y = static_cast<int>(oy) * g.sh - g.pad, x = static_cast<int>(ox) * g.sw - g.pad;
    const int y0 = imax(y, 0), y1 = imin(y + g.kh, g.h);
    const int x0 = imax(x, 0), x1 = imin(x + g.kw, g.w);
    const int64_t in_img = static_cast<int64_t>(g.h) * g.w * g.c;
    const int64_t out_img = static_cast<int64_t>(pl.lanes_per_image) * W;
    const int ch0 = static_cast<int>(chv) * W;
    typedef typename VecT<W>::type R;
    for (int64_t img = blockIdx.y; img < n; img += gridDim.y) {
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
        img_store<W, AL>(out + img * out_img + static_cast<int64_t>(p) * W, best);
        img_store<W, AL>(argmax + img * out_img + static_cast<int64_t>(p) * W, where);
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
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
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
    const int64_t in_img = static_cast<int64_t>(g.h) * g.w * g.c;
    const int64_t out_img = static_cast<int64_t>(g.oh) * g.ow * g.c;
    typedef typename VecT<W>::type R;
    for (int64_t img = blockIdx.y; img < n; img += gridDim.y) {
        float* q = in_deltas + img * in_img + static_cast<int64_t>(p) * W;
        R acc = img_load<W, AL>(q);
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
                    const int64_t o = img * out_img + (static_cast<int64_t>(oy) * g.ow + ox) * g.c + ch0;
                    am[a * C + b] = img_load<W, AL>(argmax + o);
                    d[a * C + b] = img_load<W, AL>(out_deltas + o);
                }
#pragma unroll
            for (int a = 0; a < C; ++a)
#pragma unroll
                for (int b = 0; b < C; ++b)
                    if (oy0 + a < oy1 && ox0 + b < ox1) take(am[a * C + b], d[a * C + b]);
        } else {
            for (int oy = oy0; oy < oy1; ++oy)
                for (int ox = ox0; ox < ox1; ++ox) {
                    const int64_t o = img * out_img + (static_cast<int64_t>(oy) * g.ow + ox) * g.c + ch0;
                    take(img_load<W, AL>(argmax + o), img_load<W, AL>(out_deltas + o));
                }
        }
        img_store<W, AL>(q, acc);
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
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t opix, chv, oy, ox;
    pl.d_cv.divmod(p, opix, chv);
    pl.d_ow.divmod(opix, oy, ox);
    const int y = static_cast<int>(oy) * g.sh - g.pad, x = static_cast<int>(ox) * g.sw - g.pad;
    const int y0 = imax(y, 0), y1 = imin(y + g.kh, g.h);
    const int x0 = imax(x, 0), x1 = imin(x + g.kw, g.w);
    const float size = static_cast<float>(imax((y1 - y0) * (x1 - x0), 1));
    const int64_t in_img = static_cast<int64_t>(g.h) * g.w * g.c;
    const int64_t out_img = static_cast<int64_t>(pl.lanes_per_image) * W;
    typedef typename VecT<W>::type R;
    for (int64_t img = blockIdx.y; img < n; img += gridDim.y) {
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
        img_store<W, AL>(out + img * out_img + static_cast<int64_t>(p) * W, sum);
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
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= pl.lanes_per_image) return;
    uint32_t pix, chv, yy, xx;
    pl.d_cv.divmod(p, pix, chv);
    pl.d_w.divmod(pix, yy, xx);
    const int y = static_cast<int>(yy), x = static_cast<int>(xx);
    int oy0, oy1, ox0, ox1;
    cover_range(y, g.pad, pl.d_sh, g.kh, g.oh, oy0, oy1);
    cover_range(x, g.pad, pl.d_sw, g.kw, g.ow, ox0, ox1);
    const int64_t in_img = static_cast<int64_t>(g.h) * g.w * g.c;
    const int64_t out_img = static_cast<int64_t>(g.oh) * g.ow * g.c;
    typedef typename VecT<W>::type R;
    // number of image pixels under the window at output position (oy, ox)
    auto window_size = [&](int oy, int ox) {
        const int wy = oy * g.sh - g.pad, wx = ox * g.sw - g.pad;
        const int ny = imin(wy + g.kh, g.h) - imax(wy, 0);
        const int nx = imin(wx + g.kw, g.w) - imax(wx, 0);
        return static_cast<float>(ny * nx);
    };
    for (int64_t img = blockIdx.y; img < n; img += gridDim.y) {
        float* q = in_deltas + img * in_img + static_cast<int64_t>(p) * W;
        R acc = img_load<W, AL>(q);
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
        img_store<W, AL>(q, acc);
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

}  // namespace bship

using namespace bship;

// Launches kernel<W, AL> over lanes_per_image x n: W = 4 when the channels come in fours,
// AL when additionally every pointer is 16-byte aligned.
#define BSHIP_LAUNCH_IMG(kernel, name, positions, aligned, ...)                                         \
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
        const int64_t gy_ = ceil_div(n, kImagesPerWorkgroup);                                           \
        const dim3 grid_(static_cast<unsigned>(ceil_div(lanes_, kBlock)),                               \
                         static_cast<unsigned>(gy_ < 65535 ? gy_ : 65535));                             \
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
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(kh >= 1 && kw >= 1 && stride_h >= 1 && stride_w >= 1 && pad >= 0);
    BSHIP_REQUIRE_DIM(h + 2 * pad >= kh && w + 2 * pad >= kw);
    ImgGeom g{h, w, c, conv_out(h, kh, pad, stride_h), conv_out(w, kw, pad, stride_w), kh, kw, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t total = n * g.oh * g.ow * kh * kw * c;
    if (total == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(col);
    const bool write_through = static_cast<size_t>(total) >= (size_t(1) << 26);   // 256 MiB: beyond the last-level cache
    const int64_t per_image = static_cast<int64_t>(g.oh) * g.ow * kh * kw * c;
    if (c % 4 != 0 && per_image % 4 == 0 && per_image <= 0x7fffffff) {
        ImgPlan pl;
        pl.g = g;
        pl.lanes_per_image = static_cast<uint32_t>(per_image / 4);
        pl.d_cv = FastDiv(static_cast<uint32_t>(c));
        pl.d_ow = FastDiv(static_cast<uint32_t>(g.ow));
        pl.d_kcv = FastDiv(static_cast<uint32_t>(kh * kw * c));
        pl.d_kwcv = FastDiv(static_cast<uint32_t>(kw * c));
        const int64_t gy = ceil_div(n, kImagesPerWorkgroup);
        const dim3 grid(static_cast<unsigned>(ceil_div(per_image / 4, kBlock)), static_cast<unsigned>(gy < 65535 ? gy : 65535));
        if (write_through) hipLaunchKernelGGL(im2col_gather4<true>, grid, dim3(kBlock), 0, ctx().stream, in, col, n, pl);
        else               hipLaunchKernelGGL(im2col_gather4<false>, grid, dim3(kBlock), 0, ctx().stream, in, col, n, pl);
        return check_launch("im2col");
    }
    if (write_through)
        BSHIP_LAUNCH_IMG(im2col_wt, "im2col", static_cast<int64_t>(g.oh) * g.ow * kh * kw,
                         aligned16(in) && aligned16(col), in, col);
    BSHIP_LAUNCH_IMG(im2col_cached, "im2col", static_cast<int64_t>(g.oh) * g.ow * kh * kw,
                     aligned16(in) && aligned16(col), in, col);
}

int bship_col2im_nhwc_f32(const float* col, float* in_deltas, int64_t n, int h, int w, int c,
                          int kh, int kw, int pad, int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(kh >= 1 && kw >= 1 && stride_h >= 1 && stride_w >= 1 && pad >= 0);
    BSHIP_REQUIRE_DIM(h + 2 * pad >= kh && w + 2 * pad >= kw);
    ImgGeom g{h, w, c, conv_out(h, kh, pad, stride_h), conv_out(w, kw, pad, stride_w), kh, kw, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t total = n * h * w * c;
    if (total == 0) return 0;
    BSHIP_REQUIRE_PTR(col);
    BSHIP_REQUIRE_PTR(in_deltas);
    BSHIP_LAUNCH_IMG(col2im_kernel, "col2im", static_cast<int64_t>(h) * w,
                     aligned16(col) && aligned16(in_deltas), col, in_deltas);
}

int bship_maxpool_fwd_nhwc_f32(const float* in, float* out, float* argmax, int64_t n, int h, int w,
                               int c, int out_h, int out_w, int pool_h, int pool_w, int pad,
                               int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t total = n * out_h * out_w * c;
    if (total == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_PTR(argmax);
    const bool al = aligned16(in) && aligned16(out) && aligned16(argmax);
    if (pool_h == 3 && pool_w == 3 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG(maxpool_fwd_kernel_3x3, "maxpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out, argmax);
    if (pool_h == 2 && pool_w == 2 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG(maxpool_fwd_kernel_2x2, "maxpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out, argmax);
    BSHIP_LAUNCH_IMG(maxpool_fwd_kernel, "maxpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out, argmax);
}

int bship_maxpool_bwd_nhwc_f32(const float* argmax, const float* out_deltas, float* in_deltas,
                               int64_t n, int h, int w, int c, int out_h, int out_w, int pool_h,
                               int pool_w, int pad, int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t total = n * h * w * c;
    if (total == 0 || out_h == 0 || out_w == 0) return 0;
    BSHIP_REQUIRE_PTR(argmax);
    BSHIP_REQUIRE_PTR(out_deltas);
    BSHIP_REQUIRE_PTR(in_deltas);
    const bool al = aligned16(argmax) && aligned16(out_deltas) && aligned16(in_deltas);
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
    BSHIP_REQUIRE_INIT();
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t total = n * out_h * out_w * c;
    if (total == 0) return 0;
    BSHIP_REQUIRE_PTR(in);
    BSHIP_REQUIRE_PTR(out);
    const bool al = aligned16(in) && aligned16(out);
    if (pool_h == 3 && pool_w == 3 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG(avgpool_fwd_kernel_3x3, "avgpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out);
    if (pool_h == 2 && pool_w == 2 && h >= 1 && w >= 1)
        BSHIP_LAUNCH_IMG(avgpool_fwd_kernel_2x2, "avgpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out);
    BSHIP_LAUNCH_IMG(avgpool_fwd_kernel, "avgpool2d_forward_batch", static_cast<int64_t>(out_h) * out_w, al, in, out);
}

int bship_avgpool_bwd_nhwc_f32(const float* out_deltas, float* in_deltas, int64_t n, int h, int w,
                               int c, int out_h, int out_w, int pool_h, int pool_w, int pad,
                               int stride_h, int stride_w) {
    BSHIP_REQUIRE_INIT();
    ImgGeom g{h, w, c, out_h, out_w, pool_h, pool_w, pad, stride_h, stride_w};
    int st = check_geom(__func__, n, g);
    if (st != 0) return st;
    const int64_t total = n * h * w * c;
    if (total == 0 || out_h == 0 || out_w == 0) return 0;
    BSHIP_REQUIRE_PTR(out_deltas);
    BSHIP_REQUIRE_PTR(in_deltas);
    const bool al = aligned16(out_deltas) && aligned16(in_deltas);
    const int cover = imax((pool_h + stride_h - 1) / stride_h, (pool_w + stride_w - 1) / stride_w);
    if (cover == 1)
        BSHIP_LAUNCH_IMG(avgpool_bwd_kernel_c1, "avgpool2d_backward_batch", static_cast<int64_t>(h) * w, al, out_deltas, in_deltas);
    if (cover == 2)
        BSHIP_LAUNCH_IMG(avgpool_bwd_kernel_c2, "avgpool2d_backward_batch", static_cast<int64_t>(h) * w, al, out_deltas, in_deltas);
    BSHIP_LAUNCH_IMG(avgpool_bwd_kernel, "avgpool2d_backward_batch", static_cast<int64_t>(h) * w, al, out_deltas, in_deltas);
}

}  // extern "C"
