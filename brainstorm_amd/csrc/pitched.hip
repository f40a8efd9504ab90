// Elementwise and matrix-vector operations on row-pitched matrices.
//
// brainstorm lets several layers write side by side into one hub and hands each
// of them the feature slice hub[:, :, a:b] (buffer_structure.py:232-245): a
// (rows, cols) matrix whose rows lie `pitch` elements apart. NumPy addresses it
// with strides; here one kernel template serves every elementwise operation and
// every matrix (op) vector operation on such operands. Each input is described
// by a row stride and a column stride of 0 or 1:
//     matrix         row stride = its pitch   column stride 1
//     row vector     row stride = 0           column stride 1
//     column vector  row stride = 1           column stride 0
// so add_mv is AddOp with a vector for its second input, and mult_add_mv is
// MultAddOp. The arithmetic is that of functors.h: the results equal those of
// the dense kernels bit for bit.
//
// Shape of the kernel: as for the dense streams, one workgroup per tile of
// kBlock*4 columns of one row (or several rows, when they are narrower than a
// tile), one 128-bit access per lane and operand. Rows of
// a pitched view start wherever the slice starts, so the wide accesses promise
// only 4-byte alignment (the memory system takes dword-aligned wide accesses).
#pragma clang fp contract(off)

#include "common.h"
#include "functors.h"

namespace bship {

struct Operand2d {
    const float* p;
    int64_t row_stride;   // elements between rows (0: the same row for every row)
    int col_stride;       // 1, or 0 for one value per row
};

__device__ __forceinline__ f4 load4(const Operand2d& o, int64_t row, int64_t c) {
    const float* q = o.p + row * o.row_stride;
    if (o.col_stride == 0) { const float s = *q; return f4{s, s, s, s}; }
    return vload<4, false>(q + c);
}
__device__ __forceinline__ float load1(const Operand2d& o, int64_t row, int64_t c) {
    return o.p[row * o.row_stride + c * o.col_stride];
}

// Lanes that share a row: the power of two that covers the row's 128-bit accesses, 256 at most.
// Narrow slices then put several rows into one workgroup instead of leaving its lanes idle.
static inline int row_lanes_log2(int64_t cols) {
    int l = 0;
    while (l < 8 && (int64_t(4) << l) < cols) ++l;
    return l;
}

// out[row, c] = f(in0, in1, in2)[row, c]; an input may be `out` itself (a lane reads all of
// its operands before it writes). A workgroup covers 2^(8-L) rows x one tile of VPL * 2^L accesses
// (VPL = 2 for the float64 transcendentals, as in the dense kernels: more loads in flight per
// wavefront to cover the long arithmetic phase).
template <int NIN, int VPL, typename F>
__global__ __launch_bounds__(kBlock) void map2d_kernel(F f, Operand2d in0, Operand2d in1, Operand2d in2,
                                                       float* out, int64_t ldo, int64_t rows, int64_t cols,
                                                       unsigned tiles_per_row, int L, bool through) {
    const int64_t row = (static_cast<int64_t>(blockIdx.x / tiles_per_row) << (8 - L)) + (threadIdx.x >> L);
    const int64_t c0 = ((static_cast<int64_t>(blockIdx.x % tiles_per_row) * VPL << L) + (threadIdx.x & ((1u << L) - 1))) * 4;
    if (row >= rows) return;
    const f4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    f4 v0[VPL], v1[VPL], v2[VPL];
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const int64_t c = c0 + (static_cast<int64_t>(u) << (L + 2));
        if (c + 4 <= cols) {
            v0[u] = NIN > 0 ? load4(in0, row, c) : zero;
            v1[u] = NIN > 1 ? load4(in1, row, c) : zero;
            v2[u] = NIN > 2 ? load4(in2, row, c) : zero;
        }
    }
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const int64_t c = c0 + (static_cast<int64_t>(u) << (L + 2));
        if (c >= cols) continue;
        float* q = out + row * ldo + c;
        if (c + 4 <= cols) {
            f4 o;
#pragma unroll
            for (int k = 0; k < 4; ++k) o[k] = f.apply(v0[u][k], v1[u][k], v2[u][k]);
            vstore<4, false>(q, o, through);
        } else {
            for (int64_t j = 0; c + j < cols; ++j)
                q[j] = f.apply(NIN > 0 ? load1(in0, row, c + j) : 0.0f, NIN > 1 ? load1(in1, row, c + j) : 0.0f,
                               NIN > 2 ? load1(in2, row, c + j) : 0.0f);
        }
    }
}

struct FillOp { float val; __device__ float apply(float, float, float) const { return val; } };

template <typename F, typename = void> struct VectorsPerLane2d { static constexpr int value = 1; };
template <typename F> struct VectorsPerLane2d<F, std::void_t<decltype(F::kVectorsPerLane)>> {
    static constexpr int value = F::kVectorsPerLane;
};

template <int NIN, typename F>
static int launch_map2d(const char* name, F f, Operand2d in0, Operand2d in1, Operand2d in2, float* out,
                        int64_t ldo, int64_t rows, int64_t cols) {
    constexpr int VPL = VectorsPerLane2d<F>::value;
    const int L = row_lanes_log2(cols);
    const bool wide = VPL > 1 && L == 8 && cols > (int64_t(4) << 8);      // rows longer than one tile
    const int vpl = wide ? VPL : 1;
    const int64_t tiles_per_row = ceil_div(cols, (int64_t(4) << L) * vpl);
    const int64_t row_groups = ceil_div(rows, int64_t(1) << (8 - L));
    if (tiles_per_row * row_groups > 0x7fffffff)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: %lld x %lld elements exceed one launch", name,
                         static_cast<long long>(rows), static_cast<long long>(cols));
    const dim3 grid(static_cast<unsigned>(tiles_per_row * row_groups));
    const bool through = store_through(static_cast<size_t>(rows) * static_cast<size_t>(cols));
    if (wide)
        hipLaunchKernelGGL((map2d_kernel<NIN, VPL, F>), grid, dim3(kBlock), 0, ctx().stream, f, in0, in1, in2, out, ldo,
                           rows, cols, static_cast<unsigned>(tiles_per_row), L, through);
    else
        hipLaunchKernelGGL((map2d_kernel<NIN, 1, F>), grid, dim3(kBlock), 0, ctx().stream, f, in0, in1, in2, out, ldo,
                           rows, cols, static_cast<unsigned>(tiles_per_row), L, through);
    return check_launch(name);
}

// broadcast_t (numpy 103-105) between arrays made of contiguous runs: element e of the dense
// order of `out`, e = (o * bdim + b) * inner + i, is element o * inner + i of the dense order of
// `a`; dense element k of an array lies at (k / run) * pitch + k % run. W = 4 when inner and both
// runs are multiples of 4: four consecutive elements then share their rows on both sides.
struct BroadcastPlan {
    uint32_t groups;             // lanes: n / W
    uint32_t inner;
    int64_t ld_a, ld_out;
    FastDiv d_inner, d_bdim, d_arun, d_orun;
};
// WT: write-through stores (outputs too large to be read again from the caches soon).
template <int W, bool WT>
__global__ __launch_bounds__(kBlock) void broadcast_pitched_kernel(const float* __restrict__ a,
                                                                   float* __restrict__ out, BroadcastPlan pl) {
    const uint32_t g = blockIdx.x * kBlock + threadIdx.x;
    if (g >= pl.groups) return;
    const uint32_t e = g * W;
    uint32_t ob, i, o, b, ar, ac, orow, oc;
    pl.d_inner.divmod(e, ob, i);
    pl.d_bdim.divmod(ob, o, b);
    pl.d_arun.divmod(o * pl.inner + i, ar, ac);
    pl.d_orun.divmod(e, orow, oc);
    const float* src = a + static_cast<int64_t>(ar) * pl.ld_a + ac;
    float* dst = out + static_cast<int64_t>(orow) * pl.ld_out + oc;
    if constexpr (W == 4) {
        const f4 v = *reinterpret_cast<const f4u*>(src);        // the source is read bdim times: cached
        if constexpr (WT) vstore_writeonly<4>(dst, v);
        else vstore<4, false>(dst, v);
    } else {
        *dst = *src;
    }
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_broadcast_pitched_f32(const float* a, int64_t a_run, int64_t ld_a, float* out, int64_t out_run,
                                int64_t ld_out, int64_t outer, int64_t bdim, int64_t inner) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(outer >= 0 && bdim >= 0 && inner >= 0);
    const int64_t n = outer * bdim * inner;
    if (n == 0) return 0;
    BSHIP_REQUIRE_DIM(a_run >= 1 && out_run >= 1 && ld_a >= a_run && ld_out >= out_run);
    BSHIP_REQUIRE_DIM((outer * inner) % a_run == 0 && n % out_run == 0);
    BSHIP_REQUIRE_DIM(n <= 0xffffffffll);
    BSHIP_REQUIRE_PTR(a);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(a);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    BSHIP_REQUIRE_DIM(a != out);
    const bool vec = inner % 4 == 0 && a_run % 4 == 0 && out_run % 4 == 0;
    BroadcastPlan pl;
    pl.groups = static_cast<uint32_t>(vec ? n / 4 : n);
    pl.inner = static_cast<uint32_t>(inner);
    pl.ld_a = ld_a;
    pl.ld_out = ld_out;
    pl.d_inner = FastDiv(static_cast<uint32_t>(inner));
    pl.d_bdim = FastDiv(static_cast<uint32_t>(bdim));
    pl.d_arun = FastDiv(static_cast<uint32_t>(a_run));
    pl.d_orun = FastDiv(static_cast<uint32_t>(out_run));
    const dim3 grid(static_cast<unsigned>(ceil_div(pl.groups, kBlock)));
    const bool wt = static_cast<size_t>(n) >= ctx().write_through_min;
    if (vec && wt) hipLaunchKernelGGL((broadcast_pitched_kernel<4, true>), grid, dim3(kBlock), 0, ctx().stream, a, out, pl);
    else if (vec)  hipLaunchKernelGGL((broadcast_pitched_kernel<4, false>), grid, dim3(kBlock), 0, ctx().stream, a, out, pl);
    else           hipLaunchKernelGGL((broadcast_pitched_kernel<1, false>), grid, dim3(kBlock), 0, ctx().stream, a, out, pl);
    return check_launch("broadcast_t");
}

int bship_elementwise_pitched_f32(int family, int op, float s0, float s1,
                                  const float* a, int64_t a_row_stride, int a_col_stride,
                                  const float* b, int64_t b_row_stride, int b_col_stride,
                                  float* out, int64_t ld_out, int64_t rows, int64_t cols) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(rows >= 0 && cols >= 0);
    if (rows == 0 || cols == 0) return 0;
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    BSHIP_REQUIRE_F32_ALIGNED(a);
    BSHIP_REQUIRE_F32_ALIGNED(b);
    BSHIP_REQUIRE_DIM(ld_out >= cols);
    BSHIP_REQUIRE_DIM((a_col_stride == 0 || a_col_stride == 1) && (b_col_stride == 0 || b_col_stride == 1));
    BSHIP_REQUIRE_DIM(a_row_stride >= 0 && b_row_stride >= 0);
    const Operand2d A = {a, a_row_stride, a_col_stride};
    const Operand2d B = {b, b_row_stride, b_col_stride};
    const Operand2d O = {out, ld_out, 1};
    const Operand2d none = {nullptr, 0, 0};
#define BSHIP_MAP(NIN, name, f, i0, i1, i2) return launch_map2d<NIN>(name, f, i0, i1, i2, out, ld_out, rows, cols)
    switch (family) {
        case BSHIP_PITCHED_BINARY:
            BSHIP_REQUIRE_PTR(a);
            BSHIP_REQUIRE_PTR(b);
            switch (op) {
                case BSHIP_ADD:  BSHIP_MAP(2, "add (pitched)", AddOp{}, A, B, none);
                case BSHIP_SUB:  BSHIP_MAP(2, "subtract (pitched)", SubOp{}, A, B, none);
                case BSHIP_MUL:  BSHIP_MAP(2, "mult (pitched)", MulOp{}, A, B, none);
                case BSHIP_DIV:  BSHIP_MAP(2, "divide (pitched)", DivOp{}, A, B, none);
                case BSHIP_FMOD: BSHIP_MAP(2, "modulo (pitched)", FmodOp{}, A, B, none);
            }
            break;
        case BSHIP_PITCHED_MULT_ADD:
            BSHIP_REQUIRE_PTR(a);
            BSHIP_REQUIRE_PTR(b);
            BSHIP_MAP(3, "mult_add (pitched)", MultAddOp{}, A, B, O);
        case BSHIP_PITCHED_SCALAR:
            BSHIP_REQUIRE_PTR(a);
            switch (op) {
                case BSHIP_ADD_ST:      BSHIP_MAP(1, "add_st (pitched)", AddStOp{s0}, A, none, none);
                case BSHIP_MULT_ST:     BSHIP_MAP(1, "mult_st (pitched)", MultStOp{s0}, A, none, none);
                case BSHIP_MULT_ADD_ST: BSHIP_MAP(2, "mult_add_st (pitched)", MultAddStOp{s0}, A, O, none);
            }
            break;
        case BSHIP_PITCHED_UNARY:
            BSHIP_REQUIRE_PTR(a);
            switch (op) {
                case BSHIP_ABS:     BSHIP_MAP(1, "abs_t (pitched)", AbsOp{}, A, none, none);
                case BSHIP_SIGN:    BSHIP_MAP(1, "sign_t (pitched)", SignOp{}, A, none, none);
                case BSHIP_SQRT:    BSHIP_MAP(1, "sqrt_t (pitched)", SqrtOp{}, A, none, none);
                case BSHIP_LOG:     BSHIP_MAP(1, "log_t (pitched)", LogOp{}, A, none, none);
                case BSHIP_SIGMOID: BSHIP_MAP(1, "sigmoid (pitched)", SigmoidOp{}, A, none, none);
                case BSHIP_TANH:    BSHIP_MAP(1, "tanh (pitched)", TanhOp{}, A, none, none);
                case BSHIP_REL:     BSHIP_MAP(1, "rel (pitched)", RelOp{}, A, none, none);
                case BSHIP_EL:      BSHIP_MAP(1, "el (pitched)", ElOp{}, A, none, none);
            }
            break;
        case BSHIP_PITCHED_DERIV:
            BSHIP_REQUIRE_PTR(a);
            BSHIP_REQUIRE_PTR(b);
            switch (op) {
                case BSHIP_SIGMOID_DERIV: BSHIP_MAP(2, "sigmoid_deriv (pitched)", SigmoidDerivOp{}, A, B, none);
                case BSHIP_TANH_DERIV:    BSHIP_MAP(2, "tanh_deriv (pitched)", TanhDerivOp{}, A, B, none);
                case BSHIP_REL_DERIV:     BSHIP_MAP(2, "rel_deriv (pitched)", RelDerivOp{}, A, B, none);
                case BSHIP_EL_DERIV:      BSHIP_MAP(2, "el_deriv (pitched)", ElDerivOp{}, A, B, none);
            }
            break;
        case BSHIP_PITCHED_CLIP:
            BSHIP_REQUIRE_PTR(a);
            BSHIP_MAP(1, "clip_t (pitched)", (ClipOp{s0, s1}), A, none, none);
        case BSHIP_PITCHED_COND:
            BSHIP_REQUIRE_PTR(b);      // the condition
            switch (op) {
                case BSHIP_COPY_IF:
                    BSHIP_REQUIRE_PTR(a);
                    BSHIP_MAP(3, "copy_to_if (pitched)", CopyIfOp{}, A, B, O);
                case BSHIP_FILL_IF:
                    BSHIP_MAP(2, "fill_if (pitched)", FillIfOp{s0}, B, O, none);
                case BSHIP_ADD_IF:
                    BSHIP_REQUIRE_PTR(a);
                    BSHIP_MAP(3, "add_into_if (pitched)", AddIfOp{}, A, B, O);
            }
            break;
        case BSHIP_PITCHED_FILL:
            BSHIP_MAP(0, "fill (pitched)", FillOp{s0}, none, none, none);
        default:
            return set_error(BSHIP_ERR_BAD_OP, "bship_elementwise_pitched_f32: unknown family %d", family);
    }
#undef BSHIP_MAP
    return set_error(BSHIP_ERR_BAD_OP, "bship_elementwise_pitched_f32: unknown op %d of family %d", op, family);
}

}  // extern "C"
