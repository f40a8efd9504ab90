// Integer-label operations: one-hot rows (binarize_v) and the per-row gather
// (index_m_by_v). Labels are float32-valued integers, truncated toward zero
// like NumPy's astype(int32).
#include "common.h"

namespace bship {

// out[i, j] = (j == (int)v[i]); a wavefront writes one row, 4 rows per workgroup.
template <int W, bool AL>
__global__ __launch_bounds__(kBlock) void binarize_kernel(const float* __restrict__ v,
                                                          float* __restrict__ out, int64_t M,
                                                          int64_t K) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave;
    if (row >= M) return;
    const int64_t hot = static_cast<int64_t>(static_cast<int>(v[row]));
    float* q = out + row * K;
    const int64_t KW = K / W;
    for (int64_t i = lane; i < KW; i += kWave) {
        if constexpr (W == 4) {
            const int64_t j = i * 4;
            f4 r = {j == hot ? 1.0f : 0.0f, j + 1 == hot ? 1.0f : 0.0f,
                    j + 2 == hot ? 1.0f : 0.0f, j + 3 == hot ? 1.0f : 0.0f};
            vstore<4, AL>(q + j, r);
        } else {
            q[i] = (i == hot) ? 1.0f : 0.0f;
        }
    }
}

// out[i] = m[i, (int)v[i]]; labels outside [0,K) read as 0.
__global__ __launch_bounds__(kBlock) void index_m_by_v_kernel(const float* __restrict__ m,
                                                              const float* __restrict__ v,
                                                              float* __restrict__ out, int64_t M,
                                                              int64_t K) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (row >= M) return;
    const int64_t j = static_cast<int64_t>(static_cast<int>(v[row]));
    out[row] = (j >= 0 && j < K) ? m[row * K + j] : 0.0f;
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_binarize_f32(const float* v, float* out, int64_t M, int64_t K) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && K >= 0);
    if (M == 0 || K == 0) return 0;
    BSHIP_REQUIRE_PTR(v);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(v);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    BSHIP_REQUIRE_DIM(M <= 0x7fffffff);
    dim3 grid(static_cast<unsigned>(ceil_div(M, kBlock / kWave)));
    if (K % 4 == 0 && aligned16(out))
        hipLaunchKernelGGL((binarize_kernel<4, true>), grid, dim3(kBlock), 0, ctx().stream, v, out, M, K);
    else if (K % 4 == 0)
        hipLaunchKernelGGL((binarize_kernel<4, false>), grid, dim3(kBlock), 0, ctx().stream, v, out, M, K);
    else
        hipLaunchKernelGGL((binarize_kernel<1, false>), grid, dim3(kBlock), 0, ctx().stream, v, out, M, K);
    return check_launch("binarize_v");
}

int bship_index_m_by_v_f32(const float* m, const float* v, float* out, int64_t M, int64_t K) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && K >= 0);
    if (M == 0) return 0;
    BSHIP_REQUIRE_PTR(m);
    BSHIP_REQUIRE_PTR(v);
    BSHIP_REQUIRE_PTR(out);
    hipLaunchKernelGGL(index_m_by_v_kernel, dim3(static_cast<unsigned>(ceil_div(M, kBlock))),
                       dim3(kBlock), 0, ctx().stream, m, v, out, M, K);
    return check_launch("index_m_by_v");
}

}  // extern "C"
