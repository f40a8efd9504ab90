// Matrix products with a THIN left operand, for the recurrent steps of lstm_layer.py:115-145 and 180-205
// (dot_mm / dot_add_mm of a (batch, n) slab with a square-ish weight matrix, batch <= 128):
//
//     C (M x N)  =  A (M x K) . B (K x N),   M <= 128,   A given TRANSPOSED: aT is K rows of 128 floats
//
// Why transposed: v_mfma_f32_16x16x4f32 takes A[l % 16][l / 16] and B[l / 16][l % 16] from lane l, i.e. the
// 16 lanes of a group hold 16 different rows of A (or columns of B) at the same k. Read from a row-major
// A those are 16 separate cache lines per load; read from the transposed copy and from a row-major B they
// are neighbours in memory. Lane (m = l % 16, g = l / 16) loads, for k = kb + 4g + j, the NT consecutive rows
// base + NT*m .. of A (one load of NT floats from aT) and the 2 consecutive columns n0 + 2m, n0 + 2m + 1 of B;
// component r of the first and c of the second are its operands for the tile pair (r, c), whose rows are
// base + NT*m' + r and whose columns are n0 + 2m' + c (a tile need not be contiguous).
//
// A workgroup (256 lanes) computes up to 64 rows x 32 columns over one K-range; wavefront w takes the
// quarter w of that range and the four partial sums meet in LDS in a fixed order. More than 64 rows are
// two row groups (two workgroups per column group, placed on the same XCD so that they share the columns
// of B in its L2); `splits` > 1 cuts K into that many ranges whose results go to separate output slabs
// (c + s * c_split_stride) for the caller to add in a fixed order - nothing here depends on the order in
// which workgroups finish. Loads run 5-7 k blocks ahead of the matrix-core instructions through
// bounds-checked buffer loads: a load beyond the end of an operand returns zeros without touching memory,
// so ragged K needs no branch around a load.
#pragma clang fp contract(off)

#include "buffer_loads.h"
#include "common.h"

namespace bship {

constexpr int kDsThreads = 256;
constexpr int kDsRows = 64;                       // rows per workgroup: up to 4 row tiles of 16
constexpr int kDsCols = 32;                       // columns per workgroup: 2 column tiles of 16
constexpr int kDsPitchT = 128;                    // floats per row of the transposed operand

typedef float v4f __attribute__((ext_vector_type(4)));

struct DotSmallArgs {
    const float* aT;       // (K, 128): column i is row i of A; columns >= M are zero
    const float* b;        // (K, N), row pitch ldb
    float* c;              // (splits, M, N) with row pitch ldc and slab pitch c_split_stride
    int M, N, K, ldb, ldc;
    int64_t c_split_stride;
    int col_groups;        // ceil(N / 32)
    int slices;            // col_groups * splits
    int halves;            // 1 or 2 row groups
    int base1, nt0, nt1;   // first row and tiles of group 1; tiles of group 0
    int split_blocks;      // k blocks (of 16) per split
    int wave_blocks;       // k blocks per wavefront
};

template <int NT>
__device__ __forceinline__ void dot_small_body(const DotSmallArgs& a, float* P, int colgroup, int split, int base,
                                               int rows) {
    const int tid = static_cast<int>(threadIdx.x);
    const int lane = tid & 63, kq = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    const int n0 = colgroup * kDsCols;
    const __amdgpu_buffer_rsrc_t ra = uniform_rsrc(a.aT, a.K * kDsPitchT * 4);
    const __amdgpu_buffer_rsrc_t rb = uniform_rsrc(a.b, ((a.K - 1) * a.ldb + a.N) * 4);
    const int total_blocks = (a.K + 15) / 16;
    const int first = split * a.split_blocks + kq * a.wave_blocks;
    int last = first + a.wave_blocks;
    if (last > (split + 1) * a.split_blocks) last = (split + 1) * a.split_blocks;
    if (last > total_blocks) last = total_blocks;
    const int nblocks = last > first ? last - first : 0;
    const int col_off = n0 + 2 * m < a.N ? (n0 + 2 * m) * 4 : kBufferOob;      // columns beyond N read zeros

    v4f acc[NT][2];
#pragma unroll
    for (int r = 0; r < NT; ++r) { acc[r][0] = v4f{0.0f, 0.0f, 0.0f, 0.0f}; acc[r][1] = v4f{0.0f, 0.0f, 0.0f, 0.0f}; }
    struct Block { Piece<NT> pa[4]; Piece<2> pb[4]; };
    auto load_block = [&](int ib, Block& blk) {
        const int k = (first + ib) * 16 + 4 * g;
        const int va = ib < nblocks ? (k * kDsPitchT + base + NT * m) * 4 : kBufferOob;
        const int vb = ib < nblocks ? k * a.ldb * 4 + col_off : kBufferOob;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            blk.pa[j] = load_piece<NT>(ra, va + j * kDsPitchT * 4);
            blk.pb[j] = load_piece<2>(rb, vb + j * a.ldb * 4);
        }
    };
    auto multiply = [&](const Block& blk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int r = 0; r < NT; ++r) {
                acc[r][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(blk.pa[j].v[r], blk.pb[j].v[0], acc[r][0], 0, 0, 0);
                acc[r][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(blk.pa[j].v[r], blk.pb[j].v[1], acc[r][1], 0, 0, 0);
            }
        }
    };
    {
        constexpr int kSets = NT >= 3 ? 6 : 8;                     // what 256 registers per lane hold
        Block blk[kSets];
#pragma unroll
        for (int s = 0; s < kSets - 1; ++s) load_block(s, blk[s]);
        for (int ib = 0; ib < nblocks; ib += kSets) {
#pragma unroll
            for (int s = 0; s < kSets; ++s) {
                load_block(ib + s + kSets - 1, blk[(s + kSets - 1) % kSets]);
                if (ib + s < nblocks) multiply(blk[s]);
            }
        }
    }
    // lane (m, g) holds, of tile pair (r, c), the rows m' = 4g + q (q = 0..3) of column m:
    // group row NT * m' + r, group column 2 * m + c
#pragma unroll
    for (int r = 0; r < NT; ++r) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float* p = P + (kq * kDsRows + NT * (4 * g + q) + r) * kDsCols + 2 * m;
            p[0] = acc[r][0][q];
            p[1] = acc[r][1][q];
        }
    }
    __syncthreads();
    float* out = a.c + static_cast<int64_t>(split) * a.c_split_stride;
    const int col = tid & 31;
    if (n0 + col < a.N) {
        for (int lr = tid >> 5; lr < rows; lr += kDsThreads / 32) {
            const float p0 = P[(0 * kDsRows + lr) * kDsCols + col], p1 = P[(1 * kDsRows + lr) * kDsCols + col];
            const float p2 = P[(2 * kDsRows + lr) * kDsCols + col], p3 = P[(3 * kDsRows + lr) * kDsCols + col];
            out[static_cast<int64_t>(base + lr) * a.ldc + n0 + col] = (p0 + p1) + (p2 + p3);
        }
    }
}

// two wavefronts per SIMD
__global__ __launch_bounds__(kDsThreads, 2) void dot_small_kernel(DotSmallArgs a) {
    __shared__ float P[4 * kDsRows * kDsCols];
    // Workgroups are dealt to the 8 XCDs by number. With two row groups, the two workgroups of a slice
    // (column group x split) are numbers i and i + 8: the same XCD, whose L2 then holds that slice of B once.
    int slice, half;
    if (a.halves == 2) {
        const int xcd = static_cast<int>(blockIdx.x) & 7, slot = static_cast<int>(blockIdx.x) >> 3;
        half = slot & 1;
        slice = (slot >> 1) * 8 + xcd;
    } else {
        half = 0;
        slice = static_cast<int>(blockIdx.x);
    }
    if (slice >= a.slices) return;
    const int colgroup = slice % a.col_groups, split = slice / a.col_groups;
    const int base = half == 0 ? 0 : a.base1;
    const int nt = half == 0 ? a.nt0 : a.nt1;
    const int rows = (half == 0 && a.nt1 > 0 ? a.base1 : a.M) - base;
    switch (nt) {
        case 1: dot_small_body<1>(a, P, colgroup, split, base, rows); break;
        case 2: dot_small_body<2>(a, P, colgroup, split, base, rows); break;
        case 3: dot_small_body<3>(a, P, colgroup, split, base, rows); break;
        default: dot_small_body<4>(a, P, colgroup, split, base, rows); break;
    }
}

// dst (cols x ld_dst) = src (rows x cols, pitch ld_src) transposed; columns >= rows of dst are left alone
__global__ __launch_bounds__(256) void transpose_kernel(const float* __restrict__ src, float* __restrict__ dst, int rows,
                                                        int cols, int64_t ld_src, int64_t ld_dst, unsigned col_tiles) {
    __shared__ float tile[32][33];
    const int tx = static_cast<int>(threadIdx.x) & 31, ty = static_cast<int>(threadIdx.x) >> 5;
    const int r0 = static_cast<int>(blockIdx.x / col_tiles) * 32, c0 = static_cast<int>(blockIdx.x % col_tiles) * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = r0 + ty + 8 * i, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + 8 * i][tx] = src[r * ld_src + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = c0 + ty + 8 * i, r = r0 + tx;
        if (r < rows && c < cols) dst[c * ld_dst + r] = tile[tx][ty + 8 * i];
    }
}

}  // namespace bship

using namespace bship;

extern "C" int bship_dot_small_tn_f32(const float* aT, const float* b, float* c, int64_t M, int64_t N, int64_t K,
                                      int64_t ldb, int64_t ldc, int splits, int64_t c_split_stride) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0 && K >= 0 && ldb >= N && ldc >= N && splits >= 1 && splits <= 64);
    BSHIP_REQUIRE_DIM(splits == 1 || c_split_stride >= M * ldc);
    if (M > 2 * kDsRows)
        return set_error(BSHIP_ERR_UNSUPPORTED, "%s: at most %d rows, got %lld", __func__, 2 * kDsRows, static_cast<long long>(M));
    if (K * kDsPitchT * 4 >= kBufferOob || ((K - 1) * ldb + N) * 4 >= kBufferOob)
        return set_error(BSHIP_ERR_UNSUPPORTED, "%s: operands of 1 GiB and more are not addressed", __func__);
    if (M == 0 || N == 0) return 0;
    BSHIP_REQUIRE_PTR(c); BSHIP_REQUIRE_F32_ALIGNED(c);
    if (K == 0) {
        // an empty sum: zeros, without a launch that would build descriptors over nothing
        for (int sp = 0; sp < splits; ++sp)
            for (int64_t r = 0; r < M; ++r) {
                const int st = launch_fill(c + sp * c_split_stride + r * ldc, 0.0f, static_cast<size_t>(N));
                if (st != 0) return st;
            }
        return 0;
    }
    BSHIP_REQUIRE_PTR(aT); BSHIP_REQUIRE_PTR(b); BSHIP_REQUIRE_F32_ALIGNED(aT); BSHIP_REQUIRE_F32_ALIGNED(b);
    if ((reinterpret_cast<uintptr_t>(aT) & 15) != 0)
        return set_error(BSHIP_ERR_BAD_POINTER, "%s: the transposed operand must be aligned to 16 bytes", __func__);
    DotSmallArgs a;
    a.aT = aT; a.b = b; a.c = c;
    a.M = static_cast<int>(M); a.N = static_cast<int>(N); a.K = static_cast<int>(K);
    a.ldb = static_cast<int>(ldb); a.ldc = static_cast<int>(ldc);
    a.c_split_stride = c_split_stride;
    // row tiles: one group of up to 4, or two groups that share them as evenly as they divide
    const int tiles = static_cast<int>(ceil_div(M, 16));
    a.nt0 = tiles <= 4 ? tiles : (tiles + 1) / 2;
    a.nt1 = tiles - a.nt0;
    a.base1 = 16 * a.nt0;
    a.halves = a.nt1 > 0 ? 2 : 1;
    a.col_groups = static_cast<int>(ceil_div(N, kDsCols));
    a.slices = a.col_groups * splits;
    const int total_blocks = static_cast<int>(ceil_div(K, 16));
    a.split_blocks = static_cast<int>(ceil_div(total_blocks, splits));
    a.wave_blocks = (a.split_blocks + 3) / 4;
    const int64_t grid = a.halves == 2 ? ceil_div(a.slices, 8) * 16 : a.slices;
    hipLaunchKernelGGL(dot_small_kernel, dim3(static_cast<unsigned>(grid)), dim3(kDsThreads), 0, ctx().stream, a);
    return check_launch("dot_small_tn");
}

extern "C" int bship_transpose_f32(const float* src, int64_t rows, int64_t cols, int64_t ld_src, float* dst,
                                   int64_t ld_dst) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(rows >= 0 && cols >= 0 && ld_src >= cols && ld_dst >= rows);
    BSHIP_REQUIRE_DIM(rows < (1 << 30) && cols < (1 << 30));
    if (rows == 0 || cols == 0) return 0;
    BSHIP_REQUIRE_PTR(src); BSHIP_REQUIRE_PTR(dst); BSHIP_REQUIRE_F32_ALIGNED(src); BSHIP_REQUIRE_F32_ALIGNED(dst);
    const int64_t row_tiles = ceil_div(rows, 32), col_tiles = ceil_div(cols, 32);
    BSHIP_REQUIRE_DIM(row_tiles * col_tiles < (1ll << 31));
    hipLaunchKernelGGL(transpose_kernel, dim3(static_cast<unsigned>(row_tiles * col_tiles)), dim3(256), 0, ctx().stream,
                       src, dst, static_cast<int>(rows), static_cast<int>(cols), ld_src, ld_dst,
                       static_cast<unsigned>(col_tiles));
    return check_launch("transpose");
}
