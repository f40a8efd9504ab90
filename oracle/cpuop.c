/*
 * TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
 *
 * Plain-C restatement of brainstorm's one compiled module,
 * brainstorm/handlers/_cpuop.pyx (NHWC pooling, im2col, col2im), used as the
 * CPU oracle for the HIP kernels of the same names. Only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline may load it.
 *
 * Each function cites the lines of _cpuop.pyx it follows. The order in which
 * floating-point terms are added into one memory cell is kept identical to the
 * reference (that is what the bit-exact backward tests rely on); loops over
 * independent cells (images, channels) are ordered for cache friendliness.
 * Compile without fast-math and without FMA contraction (see the Makefile).
 *
 * Every routine exists for float (suffix _f32) and double (suffix _f64), like
 * the fused DTYPE_t of the reference (_cpuop.pyx 12-14).
 */
#include <float.h>
#include <stddef.h>

static int imax(int a, int b) { return a > b ? a : b; }
static int imin(int a, int b) { return a < b ? a : b; }

#define IDX4(i, y, x, ch, H, W, C) ((((size_t)(i) * (H) + (y)) * (W) + (x)) * (C) + (ch))

#define DEFINE_CPUOP(T, SUF, TMAX)                                                          \
                                                                                             \
/* _cpuop.pyx 57-80: start from -TMAX, strict '>' (first maximum in (y,x) scan order wins,  \
 * NaN never wins); argmax = (y*W + x)*C + c as a float, -1 and output 0 for no hit. */     \
void bs_maxpool_fwd_##SUF(const T* in, T* out, T* argmax, long n, int h, int w, int c,      \
                          int oh, int ow, int ph, int pw, int pad, int sh, int sw) {        \
    for (long i = 0; i < n; ++i)                                                             \
        for (int yo = 0; yo < oh; ++yo) {                                                    \
            const int y = yo * sh - pad;                                                     \
            const int y0 = imax(y, 0), y1 = imin(y + ph, h);                                 \
            for (int xo = 0; xo < ow; ++xo) {                                                \
                const int x = xo * sw - pad;                                                 \
                const int x0 = imax(x, 0), x1 = imin(x + pw, w);                             \
                for (int ch = 0; ch < c; ++ch) {                                             \
                    T best = -TMAX;                                                          \
                    int best_idx = -1;                                                       \
                    for (int iy = y0; iy < y1; ++iy)                                         \
                        for (int ix = x0; ix < x1; ++ix) {                                   \
                            const T v = in[IDX4(i, iy, ix, ch, h, w, c)];                    \
                            if (v > best) {                                                  \
                                best = v;                                                    \
                                best_idx = (iy * w + ix) * c + ch;                           \
                            }                                                                \
                        }                                                                    \
                    const size_t o = IDX4(i, yo, xo, ch, oh, ow, c);                         \
                    out[o] = best_idx == -1 ? (T)0 : best;                                   \
                    argmax[o] = (T)best_idx;                                                 \
                }                                                                            \
            }                                                                                \
        }                                                                                    \
}                                                                                            \
                                                                                             \
/* _cpuop.pyx 103-115: for every output position in (y,x) scan order add its delta to the  \
 * input cell its argmax names. */                                                           \
void bs_maxpool_bwd_##SUF(const T* argmax, const T* out_deltas, T* in_deltas, long n, int h, \
                          int w, int c, int oh, int ow) {                                    \
    for (long i = 0; i < n; ++i)                                                             \
        for (int yo = 0; yo < oh; ++yo)                                                      \
            for (int xo = 0; xo < ow; ++xo)                                                  \
                for (int ch = 0; ch < c; ++ch) {                                             \
                    const size_t o = IDX4(i, yo, xo, ch, oh, ow, c);                         \
                    const int idx = (int)argmax[o];                                          \
                    if (idx == -1) continue;                                                 \
                    const int loc = idx / c;                                                 \
                    const int iy = loc / w, ix = loc % w;                                    \
                    if (iy >= 0 && ix >= 0) in_deltas[IDX4(i, iy, ix, ch, h, w, c)] += out_deltas[o]; \
                }                                                                            \
}                                                                                            \
                                                                                             \
/* _cpuop.pyx 143-162: sum in (y,x) scan order, divide by the number of non-padding         \
 * pixels (at least 1). */                                                                   \
void bs_avgpool_fwd_##SUF(const T* in, T* out, long n, int h, int w, int c, int oh, int ow, \
                          int ph, int pw, int pad, int sh, int sw) {                         \
    for (long i = 0; i < n; ++i)                                                             \
        for (int yo = 0; yo < oh; ++yo) {                                                    \
            const int y = yo * sh - pad;                                                     \
            const int y0 = imax(y, 0), y1 = imin(y + ph, h);                                 \
            for (int xo = 0; xo < ow; ++xo) {                                                \
                const int x = xo * sw - pad;                                                 \
                const int x0 = imax(x, 0), x1 = imin(x + pw, w);                             \
                const int size = imax((y1 - y0) * (x1 - x0), 1);                             \
                for (int ch = 0; ch < c; ++ch) {                                             \
                    T sum = 0;                                                               \
                    for (int iy = y0; iy < y1; ++iy)                                         \
                        for (int ix = x0; ix < x1; ++ix) sum += in[IDX4(i, iy, ix, ch, h, w, c)]; \
                    out[IDX4(i, yo, xo, ch, oh, ow, c)] = sum / size;                        \
                }                                                                            \
            }                                                                                \
        }                                                                                    \
}                                                                                            \
                                                                                             \
/* _cpuop.pyx 187-202: every output position, in (y,x) scan order, spreads delta/size over  \
 * the input pixels of its window. */                                                        \
void bs_avgpool_bwd_##SUF(const T* out_deltas, T* in_deltas, long n, int h, int w, int c,   \
                          int oh, int ow, int ph, int pw, int pad, int sh, int sw) {         \
    for (long i = 0; i < n; ++i)                                                             \
        for (int yo = 0; yo < oh; ++yo) {                                                    \
            const int y = yo * sh - pad;                                                     \
            const int y0 = imax(y, 0), y1 = imin(y + ph, h);                                 \
            for (int xo = 0; xo < ow; ++xo) {                                                \
                const int x = xo * sw - pad;                                                 \
                const int x0 = imax(x, 0), x1 = imin(x + pw, w);                             \
                const int size = (y1 - y0) * (x1 - x0);                                      \
                for (int iy = y0; iy < y1; ++iy)                                             \
                    for (int ix = x0; ix < x1; ++ix)                                         \
                        for (int ch = 0; ch < c; ++ch)                                       \
                            in_deltas[IDX4(i, iy, ix, ch, h, w, c)] +=                       \
                                out_deltas[IDX4(i, yo, xo, ch, oh, ow, c)] / size;           \
            }                                                                                \
        }                                                                                    \
}                                                                                            \
                                                                                             \
/* _cpuop.pyx 258-277 for ONE image: col[(yo, xo), (ky, kx, ch)], zero outside the image. */ \
void bs_im2col_##SUF(const T* in, T* col, int h, int w, int c, int kh, int kw, int pad_t,    \
                     int pad_l, int pad_b, int pad_r, int sh, int sw) {                      \
    const int oh = (h + pad_t + pad_b - kh) / sh + 1;                                        \
    const int ow = (w + pad_l + pad_r - kw) / sw + 1;                                        \
    size_t k = 0;                                                                            \
    for (int yo = 0; yo < oh; ++yo)                                                          \
        for (int xo = 0; xo < ow; ++xo)                                                      \
            for (int ky = 0; ky < kh; ++ky)                                                  \
                for (int kx = 0; kx < kw; ++kx) {                                            \
                    const int iy = yo * sh - pad_t + ky, ix = xo * sw - pad_l + kx;          \
                    const int inside = iy >= 0 && iy < h && ix >= 0 && ix < w;               \
                    for (int ch = 0; ch < c; ++ch)                                           \
                        col[k++] = inside ? in[((size_t)iy * w + ix) * c + ch] : (T)0;       \
                }                                                                            \
}                                                                                            \
                                                                                             \
/* _cpuop.pyx 288-309 for ONE image: in_deltas += col, patches visited in (yo, xo) order. */ \
void bs_col2im_##SUF(const T* col, T* in_deltas, int h, int w, int c, int kh, int kw,        \
                     int pad_t, int pad_l, int pad_b, int pad_r, int sh, int sw) {           \
    const int oh = (h + pad_t + pad_b - kh) / sh + 1;                                        \
    const int ow = (w + pad_l + pad_r - kw) / sw + 1;                                        \
    size_t k = 0;                                                                            \
    for (int yo = 0; yo < oh; ++yo)                                                          \
        for (int xo = 0; xo < ow; ++xo)                                                      \
            for (int ky = 0; ky < kh; ++ky)                                                  \
                for (int kx = 0; kx < kw; ++kx) {                                            \
                    const int iy = yo * sh - pad_t + ky, ix = xo * sw - pad_l + kx;          \
                    if (iy >= 0 && iy < h && ix >= 0 && ix < w)                              \
                        for (int ch = 0; ch < c; ++ch)                                       \
                            in_deltas[((size_t)iy * w + ix) * c + ch] += col[k + ch];        \
                    k += c;                                                                  \
                }                                                                            \
}

DEFINE_CPUOP(float, f32, FLT_MAX)
DEFINE_CPUOP(double, f64, DBL_MAX)
