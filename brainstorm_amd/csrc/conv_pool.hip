// NHWC image kernels: im2col / col2im for the convolution GEMMs and max /
// average pooling, forward and backward. One thread per output element with the
// channel index fastest, so neighbouring lanes touch neighbouring addresses.
//
// The backward kernels are written in gather form (one thread per input
// element, visiting the output positions that cover it in row-major order):
// that is the order in which the reference's serial loops add their terms, so
// results are deterministic and match the reference bit for bit.
#pragma clang fp contract(off)

#include <cfloat>

#include "common.h"

namespace bship {

struct ImgGeom {
    int h, w, c;          // input image
    int oh, ow;           // output positions
    int kh, kw;           // window / kernel
    int pad, sh, sw;
};

__host__ __device__ inline int imax(int a, int b) { return a > b ? a : b; }
__host__ __device__ inline int imin(int a, int b) { return a < b ? a : b; }

// Range [lo, hi) of output positions o with  o*stride - pad <= p < o*stride - pad + k.
__device__ __forceinline__ void cover_range(int p, int pad, int stride, int k, int n_out, int& lo,
                                            int& hi) {
    const int q = p + pad;                       // o*stride <= q < o*stride + k
    hi = imin(q / stride + 1, n_out);
    const int t = q - k + 1;                     // o*stride >= t
    lo = t <= 0 ? 0 : (t + stride - 1) / stride;
}

// col[(img, oy, ox), (ky, kx, ch)] = in[img, oy*sh-pad+ky, ox*sw-pad+kx, ch] or 0   (_cpuop 264-277)
__global__ __launch_bounds__(kBlock) void im2col_kernel(const float* __restrict__ in,
                                                        float* __restrict__ col, int64_t total,
                                                        ImgGeom g) {
    const int64_t kc = static_cast<int64_t>(g.kh) * g.kw * g.c;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < total;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int64_t row = e / kc;              // (img*oh + oy)*ow + ox
        int r = static_cast<int>(e - row * kc);
        const int ch = r % g.c; r /= g.c;
        const int kx = r % g.kw;
        const int ky = r / g.kw;
        const int ox = static_cast<int>(row % g.ow);
        const int64_t t = row / g.ow;
        const int oy = static_cast<int>(t % g.oh);
        const int64_t img = t / g.oh;
        const int iy = oy * g.sh - g.pad + ky;
        const int ix = ox * g.sw - g.pad + kx;
        float v = 0.0f;
        if (iy >= 0 && iy < g.h && ix >= 0 && ix < g.w)
            v = in[((img * g.h + iy) * g.w + ix) * g.c + ch];
        col[e] = v;
    }
}

// in_deltas[img, y, x, ch] += sum over covering (oy, ox), in scan order, of
// col[(img, oy, ox), (y - (oy*sh-pad), x - (ox*sw-pad), ch)]               (_cpuop 295-309)
__global__ __launch_bounds__(kBlock) void col2im_kernel(const float* __restrict__ col,
                                                        float* __restrict__ in_deltas,
                                                        int64_t total, ImgGeom g) {
    const int64_t kc = static_cast<int64_t>(g.kh) * g.kw * g.c;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < total;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int ch = static_cast<int>(e % g.c);
        int64_t t = e / g.c;
        const int x = static_cast<int>(t % g.w); t /= g.w;
        const int y = static_cast<int>(t % g.h);
        const int64_t img = t / g.h;
        int oy0, oy1, ox0, ox1;
        cover_range(y, g.pad, g.sh, g.kh, g.oh, oy0, oy1);
        cover_range(x, g.pad, g.sw, g.kw, g.ow, ox0, ox1);
        float acc = in_deltas[e];
        for (int oy = oy0; oy < oy1; ++oy) {
            const int ky = y - (oy * g.sh - g.pad);
            for (int ox = ox0; ox < ox1; ++ox) {
                const int kx = x - (ox * g.sw - g.pad);
                const int64_t row = (img * g.oh + oy) * g.ow + ox;
                acc += col[row * kc + (static_cast<int64_t>(ky) * g.kw + kx) * g.c + ch];
            }
        }
        in_deltas[e] = acc;
    }
}

// _cpuop 57-80: strict '>' from -FLT_MAX, so the first maximum in (y, x) scan
// order wins and NaN never does; empty windows give output 0 and argmax -1.
__global__ __launch_bounds__(kBlock) void maxpool_fwd_kernel(const float* __restrict__ in,
                                                             float* __restrict__ out,
                                                             float* __restrict__ argmax,
                                                             int64_t total, ImgGeom g) {
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < total;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int ch = static_cast<int>(e % g.c);
        int64_t t = e / g.c;
        const int ox = static_cast<int>(t % g.ow); t /= g.ow;
        const int oy = static_cast<int>(t % g.oh);
        const int64_t img = t / g.oh;
        const int y = oy * g.sh - g.pad, x = ox * g.sw - g.pad;
        const int y0 = imax(y, 0), y1 = imin(y + g.kh, g.h);
        const int x0 = imax(x, 0), x1 = imin(x + g.kw, g.w);
        const float* base = in + img * g.h * g.w * g.c;
        float best = -FLT_MAX;
        int idx = -1;
        for (int iy = y0; iy < y1; ++iy)
            for (int ix = x0; ix < x1; ++ix) {
                const int k = (iy * g.w + ix) * g.c + ch;
                const float v = base[k];
                if (v > best) { best = v; idx = k; }
            }
        out[e] = idx == -1 ? 0.0f : best;
        argmax[e] = static_cast<float>(idx);
    }
}

// _cpuop 103-115 in gather form.
__global__ __launch_bounds__(kBlock) void maxpool_bwd_kernel(const float* __restrict__ argmax,
                                                             const float* __restrict__ out_deltas,
                                                             float* __restrict__ in_deltas,
                                                             int64_t total, ImgGeom g) {
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < total;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int ch = static_cast<int>(e % g.c);
        int64_t t = e / g.c;
        const int x = static_cast<int>(t % g.w); t /= g.w;
        const int y = static_cast<int>(t % g.h);
        const int64_t img = t / g.h;
        const int self = (y * g.w + x) * g.c + ch;        // what argmax holds for this pixel
        int oy0, oy1, ox0, ox1;
        cover_range(y, g.pad, g.sh, g.kh, g.oh, oy0, oy1);
        cover_range(x, g.pad, g.sw, g.kw, g.ow, ox0, ox1);
        float acc = in_deltas[e];
        for (int oy = oy0; oy < oy1; ++oy)
            for (int ox = ox0; ox < ox1; ++ox) {
                const int64_t o = ((img * g.oh + oy) * g.ow + ox) * g.c + ch;
                if (static_cast<int>(argmax[o]) == self) acc += out_deltas[o];
            }
        in_deltas[e] = acc;
    }
}

// _cpuop 143-162: mean over the non-padding pixels of the window.
__global__ __launch_bounds__(kBlock) void avgpool_fwd_kernel(const float* __restrict__ in,
                                                             float* __restrict__ out, int64_t total,
                                                             ImgGeom g) {
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < total;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int ch = static_cast<int>(e % g.c);
        int64_t t = e / g.c;
        const int ox = static_cast<int>(t % g.ow); t /= g.ow;
        const int oy = static_cast<int>(t % g.oh);
        const int64_t img = t / g.oh;
        const int y = oy * g.sh - g.pad, x = ox * g.sw - g.pad;
        const int y0 = imax(y, 0), y1 = imin(y + g.kh, g.h);
        const int x0 = imax(x, 0), x1 = imin(x + g.kw, g.w);
        const float* base = in + img * g.h * g.w * g.c;
        float sum = 0.0f;
        for (int iy = y0; iy < y1; ++iy)
            for (int ix = x0; ix < x1; ++ix) sum += base[(iy * g.w + ix) * g.c + ch];
        const int size = imax((y1 - y0) * (x1 - x0), 1);
        out[e] = sum / static_cast<float>(size);
    }
}

// _cpuop 187-202 in gather form.
__global__ __launch_bounds__(kBlock) void avgpool_bwd_kernel(const float* __restrict__ out_deltas,
                                                             float* __restrict__ in_deltas,
                                                             int64_t total, ImgGeom g) {
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < total;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int ch = static_cast<int>(e % g.c);
        int64_t t = e / g.c;
        const int x = static_cast<int>(t % g.w); t /= g.w;
        const int y = static_cast<int>(t % g.h);
        const int64_t img = t / g.h;
        int oy0, oy1, ox0, ox1;
        cover_range(y, g.pad, g.sh, g.kh, g.oh, oy0, oy1);
        cover_range(x, g.pad, g.sw, g.kw, g.ow, ox0, ox1);
        float acc = in_deltas[e];
        for (int oy = oy0; oy < oy1; ++oy) {
            const int wy = oy * g.sh - g.pad;
            const int ny = imin(wy + g.kh, g.h) - imax(wy, 0);
            for (int ox = ox0; ox < ox1; ++ox) {
                const int wx = ox * g.sw - g.pad;
                const int nx = imin(wx + g.kw, g.w) - imax(wx, 0);
                const int64_t o = ((img * g.oh + oy) * g.ow + ox) * g.c + ch;
                acc += out_deltas[o] / static_cast<float>(ny * nx);
            }
        }
        in_deltas[e] = acc;
    }
}

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

#define BSHIP_LAUNCH_IMG(kernel, total, ...)                                                  \
    hipLaunchKernelGGL(kernel, dim3(stream_grid(ceil_div((total), kBlock))), dim3(kBlock), 0, \
                       ctx().stream, __VA_ARGS__)

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
    BSHIP_LAUNCH_IMG(im2col_kernel, total, in, col, total, g);
    return check_launch("im2col");
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
    BSHIP_LAUNCH_IMG(col2im_kernel, total, col, in_deltas, total, g);
    return check_launch("col2im");
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
    BSHIP_LAUNCH_IMG(maxpool_fwd_kernel, total, in, out, argmax, total, g);
    return check_launch("maxpool2d_forward_batch");
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
    BSHIP_LAUNCH_IMG(maxpool_bwd_kernel, total, argmax, out_deltas, in_deltas, total, g);
    return check_launch("maxpool2d_backward_batch");
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
    BSHIP_LAUNCH_IMG(avgpool_fwd_kernel, total, in, out, total, g);
    return check_launch("avgpool2d_forward_batch");
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
    BSHIP_LAUNCH_IMG(avgpool_bwd_kernel, total, out_deltas, in_deltas, total, g);
    return check_launch("avgpool2d_backward_batch");
}

}  // extern "C"
