// Integer-label operations: one-hot rows (binarize_v) and the per-row gather
// (index_m_by_v). Labels are float32-valued integers, truncated toward zero
// like NumPy's astype(int32); negative labels count from the last column, as
// NumPy's indexing does (label_column in common.h).
#include "common.h"
#include "window.h"

namespace bship {

// out[i, j] = (j == label_column(v[i])). Write-only: one workgroup per tile of kBlock*W
// columns of one row, one store per lane (the shape of the fill kernel).
// WT selects write-through stores (large outputs). KW = K / W.
template <int W, bool AL, bool WT>
__global__ __launch_bounds__(kBlock) void binarize_kernel(const float* __restrict__ v, int64_t ldv,
                                                          float* __restrict__ out, int64_t ldo, int64_t KW,
                                                          int64_t K, unsigned tiles_per_row) {
    const int64_t row = blockIdx.x / tiles_per_row;
    const int64_t c = static_cast<int64_t>(blockIdx.x % tiles_per_row) * kBlock + threadIdx.x;
    if (c >= KW) return;
    const int64_t hot = label_column(v[row * ldv], K);
    float* q = out + row * ldo + c * W;         // ldv, ldo: elements from one row to the next
    typename VecT<W>::type r;
    if constexpr (W == 4) {
        const int64_t j = c * 4;
        r = f4{j == hot ? 1.0f : 0.0f, j + 1 == hot ? 1.0f : 0.0f, j + 2 == hot ? 1.0f : 0.0f,
               j + 3 == hot ? 1.0f : 0.0f};
    } else {
        r = (c == hot) ? 1.0f : 0.0f;
    }
    if constexpr (WT) vstore_writeonly<W>(q, r);
    else vstore<W, AL>(q, r);
}

// The ones of a large one-hot matrix whose zeros a fill has written: one lane per row.
__global__ __launch_bounds__(kBlock) void one_hot_ones_kernel(const float* __restrict__ v, int64_t ldv,
                                                              float* __restrict__ out, int64_t ldo, int64_t M,
                                                              int64_t K) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (row >= M) return;
    const int64_t hot = label_column(v[row * ldv], K);
    if (hot >= 0) out[row * ldo + hot] = 1.0f;
}

// out[i] = m[i, label_column(v[i])]; labels outside [-K,K) read as 0.
__global__ __launch_bounds__(kBlock) void index_m_by_v_kernel(const float* __restrict__ m, int64_t ldm,
                                                              const float* __restrict__ v, int64_t ldv,
                                                              float* __restrict__ out, int64_t ldo, int64_t M,
                                                              int64_t K) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (row >= M) return;
    const int64_t j = label_column(v[row * ldv], K);
    out[row * ldo] = j >= 0 ? m[row * ldm + j] : 0.0f;
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_binarize_f32(const float* v, float* out, int64_t M, int64_t K) {
    // the first call of the softmax cross-entropy layer's backward sequence: through the fusing window
    if (window_takes() && M >= 1 && K >= 1 && v && out &&
        ((reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out)) & 3u) == 0) {
        BSHIP_REQUIRE_INIT_NO_FLUSH();
        return window_push(window::rec_binarize(v, out, M, K));
    }
    return bship_binarize_pitched_f32(v, 1, out, K, M, K);
}

int bship_binarize_pitched_f32(const float* v, int64_t ld_v, float* out, int64_t ld_out, int64_t M, int64_t K) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && K >= 0);
    BSHIP_REQUIRE_DIM(ld_v >= 1 && ld_out >= K);
    if (M == 0 || K == 0) return 0;
    BSHIP_REQUIRE_PTR(v);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(v);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    const bool vec = (K % 4 == 0);
    const int64_t KW = vec ? K / 4 : K;
    const bool al = aligned16(out) && ld_out % 4 == 0;
    const int64_t tiles_per_row = ceil_div(KW, kBlock);
    BSHIP_REQUIRE_DIM(tiles_per_row * M <= 0x7fffffff);
    const dim3 grid(static_cast<unsigned>(tiles_per_row * M)), blk(kBlock);
    const unsigned tpr = static_cast<unsigned>(tiles_per_row);
    const bool wt = static_cast<size_t>(M) * static_cast<size_t>(K) >= ctx().write_through_min;
    hipStream_t s = ctx().stream;
    if (wt && ld_out == K && store_through(static_cast<size_t>(M) * static_cast<size_t>(K))) {
        // A large dense one-hot matrix of a size at which the kernels around it store write-through: zeros
        // from the fill kernel, then the ones. binarize_kernel's workgroups wait for their row's label before
        // they store, and a write stream is only fast when its stores are issued at once: 0.91-0.95 of peak
        // while the labels stay in the L2 from one call to the next, 0.61 after write-through kernels have
        // swept the L2 (measured at 8192 x 8192); fill + ones: 0.89 there.
        int st = launch_fill(out, 0.0f, static_cast<size_t>(M) * static_cast<size_t>(K));
        if (st != 0) return st;
        hipLaunchKernelGGL(one_hot_ones_kernel, dim3(static_cast<unsigned>(ceil_div(M, kBlock))), blk, 0, s, v, ld_v,
                           out, ld_out, M, K);
        return check_launch("binarize_v");
    }
    if (vec && wt)                   hipLaunchKernelGGL((binarize_kernel<4, false, true>), grid, blk, 0, s, v, ld_v, out, ld_out, KW, K, tpr);
    else if (vec && al)              hipLaunchKernelGGL((binarize_kernel<4, true, false>), grid, blk, 0, s, v, ld_v, out, ld_out, KW, K, tpr);
    else if (vec)                    hipLaunchKernelGGL((binarize_kernel<4, false, false>), grid, blk, 0, s, v, ld_v, out, ld_out, KW, K, tpr);
    else if (wt)                     hipLaunchKernelGGL((binarize_kernel<1, false, true>), grid, blk, 0, s, v, ld_v, out, ld_out, KW, K, tpr);
    else                             hipLaunchKernelGGL((binarize_kernel<1, false, false>), grid, blk, 0, s, v, ld_v, out, ld_out, KW, K, tpr);
    return check_launch("binarize_v");
}

int bship_index_m_by_v_f32(const float* m, const float* v, float* out, int64_t M, int64_t K) {
    if (window_takes() && M >= 1 && K >= 0 && m && v && out) {      // part of the softmax cross-entropy forward sequence
        BSHIP_REQUIRE_INIT_NO_FLUSH();
        return window_push(window::rec_index(m, v, out, M, K));
    }
    return bship_index_m_by_v_pitched_f32(m, K, v, 1, out, 1, M, K);
}

int bship_index_m_by_v_pitched_f32(const float* m, int64_t ld_m, const float* v, int64_t ld_v, float* out,
                                   int64_t ld_out, int64_t M, int64_t K) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && K >= 0);
    BSHIP_REQUIRE_DIM(ld_m >= K && ld_v >= 1 && ld_out >= 1);
    if (M == 0) return 0;
    BSHIP_REQUIRE_PTR(m);
    BSHIP_REQUIRE_PTR(v);
    BSHIP_REQUIRE_PTR(out);
    hipLaunchKernelGGL(index_m_by_v_kernel, dim3(static_cast<unsigned>(ceil_div(M, kBlock))),
                       dim3(kBlock), 0, ctx().stream, m, ld_m, v, ld_v, out, ld_out, M, K);
    return check_launch("index_m_by_v");
}

}  // extern "C"
