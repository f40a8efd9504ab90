// Column sums (sum over axis 0) of a row-major (M,N) matrix whose elements come
// from a source functor: the plain matrix for sum_t, or a per-element expression
// of one or two matrices for the fused layer kernels, which then add up exactly
// the values, in exactly the order, that the single operations would.
#pragma once
#pragma clang fp contract(off)

#include "common.h"

namespace bship {

__device__ __forceinline__ float hsum(float v) { return v; }
__device__ __forceinline__ float hsum(f4 v) { return (v[0] + v[1]) + (v[2] + v[3]); }
__device__ __forceinline__ float hmax(float v) { return v; }
__device__ __forceinline__ float hmax(f4 v) { return fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])); }
template <typename R> __device__ __forceinline__ R vzero();
template <> __device__ __forceinline__ float vzero<float>() { return 0.0f; }
template <> __device__ __forceinline__ f4 vzero<f4>() { f4 z = {0.0f, 0.0f, 0.0f, 0.0f}; return z; }

// A workgroup is (for wide matrices) 64 column-lanes x 4 row-lanes, one wavefront per row-lane: each
// wavefront reads 64*W consecutive columns of one row per access, walks down the
// rows of its band with 4 independent accumulators, and the 4 wavefronts are
// combined through LDS. grid.x tiles the columns, grid.y splits the rows into bands;
// with more than one band the bands write partial sums that a second launch adds up.
// NW = N / W.
//
// Source functors provide
//   bool aligned() const                         all pointers 16-byte aligned (host)
//   R prep<W, AL>(col_offset) const              per-lane column context, loaded once
//   R load<W, AL>(element_offset, ctx) const     the value to add (may store side results)
struct PlainSrc {
    const float* a;
    bool aligned() const { return aligned16(a); }
    template <int W, bool AL> __device__ typename VecT<W>::type prep(int64_t) const {
        return vzero<typename VecT<W>::type>();
    }
    template <int W, bool AL>
    __device__ typename VecT<W>::type load(int64_t off, typename VecT<W>::type) const {
        return vload<W, AL>(a + off);
    }
};

// CL column-lanes x (kBlock / CL) row-lanes. CL = 64 for matrices at least 64 accesses wide;
// narrower matrices (bias gradients of small layers, image channels) take CL = 8, 16 or 32 so
// that the lanes that would have no column walk down more rows instead.
template <int W, bool AL, int CL, typename Src>
__global__ __launch_bounds__(kBlock) void colsum_kernel(Src src, float* out, int64_t M, int64_t NW, int64_t ld) {
    typedef typename VecT<W>::type R;
    constexpr int RL = kBlock / CL;                          // row-lanes
    constexpr int GROUP = 4 * RL;                            // rows per group: 4 per row-lane
    __shared__ R lds[kBlock];
    const int lane = threadIdx.x & (CL - 1);
    const int rl = threadIdx.x / CL;
    const int64_t c = static_cast<int64_t>(blockIdx.x) * CL + lane;
    R acc0 = vzero<R>(), acc1 = vzero<R>(), acc2 = vzero<R>(), acc3 = vzero<R>();
    if (c < NW) {
        const int64_t col = c * W;
        const int64_t pitch = ld;                 // elements from one row of the source to the next
        const R cx = src.template prep<W, AL>(col);
        // Groups of rows are dealt round-robin to the row bands (blockIdx.y), so all bands
        // together read one contiguous region that moves down the matrix. (Bands of
        // consecutive rows start a power-of-two number of bytes apart for the usual matrix
        // sizes and were measured 5-10 % slower.)
        for (int64_t g = blockIdx.y; g * GROUP < M; g += gridDim.y) {
            int64_t r = g * GROUP + rl;
            if (r + 3 * RL < M) {
                R x0 = src.template load<W, AL>(col + r * pitch, cx);
                R x1 = src.template load<W, AL>(col + (r + RL) * pitch, cx);
                R x2 = src.template load<W, AL>(col + (r + 2 * RL) * pitch, cx);
                R x3 = src.template load<W, AL>(col + (r + 3 * RL) * pitch, cx);
                acc0 += x0; acc1 += x1; acc2 += x2; acc3 += x3;
            } else {
                for (; r < M; r += RL) acc0 += src.template load<W, AL>(col + r * pitch, cx);
            }
        }
    }
    lds[threadIdx.x] = (acc0 + acc1) + (acc2 + acc3);
    __syncthreads();
    if (rl == 0 && c < NW) {
        R t;
        if constexpr (RL == 4) {
            t = (lds[lane] + lds[lane + CL]) + (lds[lane + 2 * CL] + lds[lane + 3 * CL]);
        } else {
            t = lds[lane];
#pragma unroll
            for (int k = 1; k < RL; ++k) t += lds[lane + k * CL];
        }
        vstore<W, AL>(out + (static_cast<int64_t>(blockIdx.y) * NW + c) * W, t);
    }
}

// Matrices of up to this many rows are summed by one band of workgroups (one launch).
constexpr int64_t kColsumSingleBandRows = 256;

// Column-lanes for a matrix of NW accesses per row.
static inline int colsum_lanes(int64_t NW) { return NW > 32 ? 64 : NW > 16 ? 32 : NW > 8 ? 16 : 8; }

template <int W, bool AL, typename Src>
static void launch_colsum_lanes(int cl, dim3 grid, Src src, float* dst, int64_t M, int64_t NW, int64_t ld) {
    hipStream_t s = ctx().stream;
    switch (cl) {
        case 8:  hipLaunchKernelGGL((colsum_kernel<W, AL, 8, Src>), grid, dim3(kBlock), 0, s, src, dst, M, NW, ld); break;
        case 16: hipLaunchKernelGGL((colsum_kernel<W, AL, 16, Src>), grid, dim3(kBlock), 0, s, src, dst, M, NW, ld); break;
        case 32: hipLaunchKernelGGL((colsum_kernel<W, AL, 32, Src>), grid, dim3(kBlock), 0, s, src, dst, M, NW, ld); break;
        default: hipLaunchKernelGGL((colsum_kernel<W, AL, 64, Src>), grid, dim3(kBlock), 0, s, src, dst, M, NW, ld); break;
    }
}

template <typename Src>
static void launch_colsum_kernel(bool vec, bool al, int cl, dim3 grid, Src src, float* dst, int64_t M,
                                 int64_t NW, int64_t ld) {
    if (vec && al) launch_colsum_lanes<4, true, Src>(cl, grid, src, dst, M, NW, ld);
    else if (vec)  launch_colsum_lanes<4, false, Src>(cl, grid, src, dst, M, NW, ld);
    else           launch_colsum_lanes<1, false, Src>(cl, grid, src, dst, M, NW, ld);
}

// Where the partial sums of a multi-band launch go: a block of the pool (ptr == nullptr), or a
// buffer the caller owns that holds `floats` floats (callers that must not allocate).
struct PartialsBuffer {
    float* ptr = nullptr;
    size_t floats = 0;
};

// ld: elements from one row of the source matrices to the next (0: dense, ld = N).
template <typename Src>
static int launch_colsum(Src src, float* out, int64_t M, int64_t N, int64_t ld = 0,
                         PartialsBuffer ws = PartialsBuffer()) {
    const Context& c = ctx();
    if (ld == 0) ld = N;
    const bool vec = (N % 4 == 0);
    const int64_t NW = vec ? N / 4 : N;
    const int cl = colsum_lanes(NW);
    const int64_t gx = ceil_div(NW, cl);
    const int64_t target = static_cast<int64_t>(c.num_cus) * c.colsum_blocks_per_cu;
    int64_t bands = target / gx;
    if (bands < 1) bands = 1;
    const int64_t min_rows = 4 * (4 * kBlock / cl);      // at least 4 unrolled steps per lane
    if (bands > ceil_div(M, min_rows)) bands = ceil_div(M, min_rows);
    if (bands > 1024) bands = 1024;
    // few rows (bias gradients at small batch): a second launch costs more than one band loses
    // (100 x 1200: 3.6 us against 7; 1000 x 200 would take 20 against 7)
    if (M <= kColsumSingleBandRows) bands = 1;
    float* dst = out;
    float* partial = nullptr;
    if (bands > 1 && ws.ptr) {
        if (static_cast<size_t>(bands) * N > ws.floats)
            return set_error(BSHIP_ERR_BAD_DIMENSION,
                             "sum over axis 0 of a (%lld, %lld) matrix needs %lld floats of partial sums, "
                             "the buffer given holds %zu", static_cast<long long>(M), static_cast<long long>(N),
                             static_cast<long long>(bands * N), ws.floats);
        dst = ws.ptr;
    } else if (bands > 1) {
        void* p = nullptr;
        int st = pool_alloc_raw(static_cast<size_t>(bands) * N * sizeof(float), &p);
        if (st != 0) return st;
        partial = static_cast<float*>(p);
        dst = partial;
    }
    // 16-byte accesses need every row start aligned: the base, and a pitch of whole vectors
    launch_colsum_kernel(vec, src.aligned() && aligned16(dst) && ld % 4 == 0, cl,
                         dim3(static_cast<unsigned>(gx), static_cast<unsigned>(bands)), src, dst, M, NW, ld);
    int st = check_launch("sum over axis 0");
    if (dst != out) {
        if (st == 0) {
            // second stage: column sums of the (bands, N) partials in one band
            launch_colsum_kernel(vec, aligned16(dst) && aligned16(out), cl,
                                 dim3(static_cast<unsigned>(gx), 1), PlainSrc{dst}, out, bands, NW, N);
            st = check_launch("sum over axis 0, stage 2");
        }
        if (partial) pool_free_raw(partial);   // a later owner of the block runs after this launch
    }
    return st;
}

}  // namespace bship
