// Broadcast operations: matrix (op) vector with a row vector (1,N) or a column
// vector (M,1), broadcast_t along a size-1 axis, and merge/split on the last
// axis. All are HBM-bound; the matrix is streamed once, the vector operand is
// small and comes out of the caches.
#pragma clang fp contract(off)

#include "common.h"
#include "window.h"

namespace bship {

// ---- small helpers so one kernel body serves float and 4-wide vectors ----
template <typename F> __device__ __forceinline__ float vmap(F f, float a, float b, float c) {
    return f.apply(a, b, c);
}
template <typename F> __device__ __forceinline__ f4 vmap(F f, f4 a, f4 b, f4 c) {
    f4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = f.apply(a[k], b[k], c[k]);
    return o;
}
__device__ __forceinline__ f4 splat(f4, float s) { f4 r = {s, s, s, s}; return r; }
__device__ __forceinline__ float splat(float, float s) { return s; }

// functors: apply(m, v, old_out)
template <bool ACC> struct MvAdd { __device__ float apply(float m, float v, float o) const { float r = m + v; return ACC ? o + r : r; } };
template <bool ACC> struct MvSub { __device__ float apply(float m, float v, float o) const { float r = m - v; return ACC ? o + r : r; } };
template <bool ACC> struct MvMul { __device__ float apply(float m, float v, float o) const { float r = m * v; return ACC ? o + r : r; } };
template <bool ACC> struct MvDiv { __device__ float apply(float m, float v, float o) const { float r = m / v; return ACC ? o + r : r; } };

// Row vector: a workgroup handles R (= kMvRows) consecutive rows of one tile of kBlock*W
// columns; each lane loads its slice of v once and applies it to R rows.
// One workgroup per tile (see elementwise.hip for why). NW = N / W.
template <int W, bool AL, bool ACC, int R, typename F>
__global__ __launch_bounds__(kBlock) void mv_rowvec_kernel(F f, const float* m, const float* v,
                                                           float* out, int64_t M, int64_t NW,
                                                           unsigned col_tiles, bool through) {
    typedef typename VecT<W>::type T;
    const unsigned ct = blockIdx.x % col_tiles;
    const int64_t r0 = static_cast<int64_t>(blockIdx.x / col_tiles) * R;
    const int64_t c = static_cast<int64_t>(ct) * kBlock + threadIdx.x;
    if (c >= NW) return;
    const T vv = vload<W, AL>(v + c * W);
    T a[R], o[R];
#pragma unroll
    for (int u = 0; u < R; ++u) {
        if (r0 + u < M) {
            const int64_t e = ((r0 + u) * NW + c) * W;
            a[u] = vload<W, AL>(m + e);
            if (ACC) o[u] = vload<W, AL>(out + e);
        }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        if (r0 + u < M) {
            const int64_t e = ((r0 + u) * NW + c) * W;
            vstore<W, AL>(out + e, vmap(f, a[u], vv, ACC ? o[u] : a[u]), through);
        }
    }
}

// Column vector: one workgroup per tile of kBlock*W columns of one row; v[row]
// is one broadcast load per tile.
template <int W, bool AL, bool ACC, typename F>
__global__ __launch_bounds__(kBlock) void mv_colvec_kernel(F f, const float* m, const float* v,
                                                           float* out, int64_t M, int64_t NW,
                                                           unsigned tiles_per_row, bool through) {
    typedef typename VecT<W>::type T;
    const int64_t row = blockIdx.x / tiles_per_row;
    const int64_t c = static_cast<int64_t>(blockIdx.x % tiles_per_row) * kBlock + threadIdx.x;
    if (c >= NW) return;
    const int64_t e = (row * NW + c) * W;
    const float s = v[row];
    const T a = vload<W, AL>(m + e);
    T o = a;
    if (ACC) o = vload<W, AL>(out + e);
    vstore<W, AL>(out + e, vmap(f, a, splat(a, s), o), through);
}

// rows per workgroup; measured at 8192^2 / 16384^2: add_mv 0.79/0.76 of peak with 1 row,
// 0.81/0.80 with 2, 0.75/0.79 with 4, 0.71/0.71 with 8
constexpr int kMvRows = 2;

template <bool ACC, typename F>
int launch_mv(const char* name, F f, const float* m, const float* v, float* out, int64_t M,
              int64_t N, int v_is_col) {
    const Context& c = ctx();
    const bool vec = (N % 4 == 0);
    const int64_t NW = vec ? N / 4 : N;
    const dim3 blk(kBlock);
    const int64_t col_tiles = ceil_div(NW, kBlock);
    const bool through = store_through(static_cast<size_t>(M) * static_cast<size_t>(N));
    if (!v_is_col) {
        const bool al = aligned16(m) && aligned16(out) && aligned16(v);
        const int64_t blocks = col_tiles * ceil_div(M, kMvRows);
        if (blocks > 0x7fffffff || col_tiles > 0x7fffffff)
            return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: matrix too large for one launch", name);
        const dim3 grid(static_cast<unsigned>(blocks));
        const unsigned ctl = static_cast<unsigned>(col_tiles);
        if (vec && al)
            hipLaunchKernelGGL((mv_rowvec_kernel<4, true, ACC, kMvRows, F>), grid, blk, 0, c.stream, f, m, v, out, M, NW, ctl, through);
        else if (vec)
            hipLaunchKernelGGL((mv_rowvec_kernel<4, false, ACC, kMvRows, F>), grid, blk, 0, c.stream, f, m, v, out, M, NW, ctl, through);
        else
            hipLaunchKernelGGL((mv_rowvec_kernel<1, false, ACC, kMvRows, F>), grid, blk, 0, c.stream, f, m, v, out, M, NW, ctl, through);
    } else {
        const bool al = aligned16(m) && aligned16(out);
        const int64_t blocks = col_tiles * M;
        if (blocks > 0x7fffffff)
            return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: matrix too large for one launch", name);
        const dim3 grid(static_cast<unsigned>(blocks));
        const unsigned tpr = static_cast<unsigned>(col_tiles);
        if (vec && al)
            hipLaunchKernelGGL((mv_colvec_kernel<4, true, ACC, F>), grid, blk, 0, c.stream, f, m, v, out, M, NW, tpr, through);
        else if (vec)
            hipLaunchKernelGGL((mv_colvec_kernel<4, false, ACC, F>), grid, blk, 0, c.stream, f, m, v, out, M, NW, tpr, through);
        else
            hipLaunchKernelGGL((mv_colvec_kernel<1, false, ACC, F>), grid, blk, 0, c.stream, f, m, v, out, M, NW, tpr, through);
    }
    return check_launch(name);
}

// out(outer, bdim, inner) = a(outer, 1, inner)
__global__ __launch_bounds__(kBlock) void broadcast_kernel(const float* __restrict__ a,
                                                           float* __restrict__ out, int64_t outer,
                                                           int64_t bdim, int64_t inner) {
    const int64_t n = outer * bdim * inner;
    const int64_t slab = bdim * inner;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < n;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int64_t o = e / slab;
        const int64_t i = (e - o * slab) % inner;
        out[e] = a[o * inner + i];
    }
}

// out(rows, na+nb): [:, :na] = a, [:, na:] = b
__global__ __launch_bounds__(kBlock) void merge_kernel(const float* __restrict__ a,
                                                       const float* __restrict__ b,
                                                       float* __restrict__ out, int64_t rows,
                                                       int64_t na, int64_t nb) {
    const int64_t w = na + nb;
    const int64_t n = rows * w;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < n;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int64_t r = e / w;
        const int64_t c = e - r * w;
        out[e] = c < na ? a[r * na + c] : b[r * nb + (c - na)];
    }
}

// oa += x[:, :na]; ob += x[:, na:]
__global__ __launch_bounds__(kBlock) void split_add_kernel(const float* __restrict__ x, float* oa,
                                                           float* ob, int64_t rows, int64_t na,
                                                           int64_t nb) {
    const int64_t w = na + nb;
    const int64_t n = rows * w;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; e < n;
         e += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int64_t r = e / w;
        const int64_t c = e - r * w;
        if (c < na) oa[r * na + c] += x[e];
        else ob[r * nb + (c - na)] += x[e];
    }
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_mv_f32(int op, const float* m, const float* v, float* out, int64_t M, int64_t N,
                 int v_is_col, int accumulate) {
    BSHIP_REQUIRE_INIT_NO_FLUSH();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0);
    if (M == 0 || N == 0) return 0;
    BSHIP_REQUIRE_PTR(m);
    BSHIP_REQUIRE_PTR(v);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(m);
    BSHIP_REQUIRE_F32_ALIGNED(v);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    if (op < BSHIP_ADD || op > BSHIP_DIV) return set_error(BSHIP_ERR_BAD_OP, "bship_mv_f32: unknown op %d", op);
    // matrix-vector operations open and fill most of the layers' sequences: through the fusing window
    if (window_takes()) return window_push(window::rec_mv(op, m, v, out, M, N, v_is_col != 0, accumulate != 0));
    BSHIP_FLUSH_PENDING();
    if (accumulate) {
        switch (op) {
            case BSHIP_ADD: return launch_mv<true>("add_mv(acc)", MvAdd<true>{}, m, v, out, M, N, v_is_col);
            case BSHIP_SUB: return launch_mv<true>("subtract_mv(acc)", MvSub<true>{}, m, v, out, M, N, v_is_col);
            case BSHIP_MUL: return launch_mv<true>("mult_add_mv", MvMul<true>{}, m, v, out, M, N, v_is_col);
            case BSHIP_DIV: return launch_mv<true>("divide_mv(acc)", MvDiv<true>{}, m, v, out, M, N, v_is_col);
        }
    } else {
        switch (op) {
            case BSHIP_ADD: return launch_mv<false>("add_mv", MvAdd<false>{}, m, v, out, M, N, v_is_col);
            case BSHIP_SUB: return launch_mv<false>("subtract_mv", MvSub<false>{}, m, v, out, M, N, v_is_col);
            case BSHIP_MUL: return launch_mv<false>("mult_mv", MvMul<false>{}, m, v, out, M, N, v_is_col);
            case BSHIP_DIV: return launch_mv<false>("divide_mv", MvDiv<false>{}, m, v, out, M, N, v_is_col);
        }
    }
    return set_error(BSHIP_ERR_BAD_OP, "bship_mv_f32: unknown op %d", op);
}

int bship_broadcast_f32(const float* a, float* out, int64_t outer, int64_t bdim, int64_t inner) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(outer >= 0 && bdim >= 0 && inner >= 0);
    const int64_t n = outer * bdim * inner;
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(a);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_DIM(a != out);
    // up to 2^32 - 1 elements: the vectorised kernel of the run-pitched form, with one run each
    if (n <= 0xffffffffll)
        return bship_broadcast_pitched_f32(a, outer * inner, outer * inner, out, n, n, outer, bdim, inner);
    hipLaunchKernelGGL(broadcast_kernel, dim3(stream_grid(ceil_div(n, kBlock))), dim3(kBlock), 0,
                       ctx().stream, a, out, outer, bdim, inner);
    return check_launch("broadcast_t");
}

int bship_merge_f32(const float* a, const float* b, float* out, int64_t rows, int64_t na,
                    int64_t nb) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(rows >= 0 && na >= 0 && nb >= 0);
    const int64_t n = rows * (na + nb);
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(out);
    if (na > 0) BSHIP_REQUIRE_PTR(a);
    if (nb > 0) BSHIP_REQUIRE_PTR(b);
    hipLaunchKernelGGL(merge_kernel, dim3(stream_grid(ceil_div(n, kBlock))), dim3(kBlock), 0,
                       ctx().stream, a, b, out, rows, na, nb);
    return check_launch("merge_tt");
}

int bship_split_add_f32(const float* x, float* oa, float* ob, int64_t rows, int64_t na,
                        int64_t nb) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(rows >= 0 && na >= 0 && nb >= 0);
    const int64_t n = rows * (na + nb);
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(x);
    if (na > 0) BSHIP_REQUIRE_PTR(oa);
    if (nb > 0) BSHIP_REQUIRE_PTR(ob);
    hipLaunchKernelGGL(split_add_kernel, dim3(stream_grid(ceil_div(n, kBlock))), dim3(kBlock), 0,
                       ctx().stream, x, oa, ob, rows, na, nb);
    return check_launch("split_add_tt");
}

}  // extern "C"
