// Elementwise handler operations: one streaming kernel template, instantiated
// per operation. Every operation is HBM-bound. Measured on MI355X, the fastest
// shape for such kernels is the simplest one: each lane moves one 128-bit
// vector per operand with non-temporal accesses, a workgroup of 256 lanes
// covers one tile of 1024 floats, and the grid has one workgroup per tile
// (hundreds of thousands of short workgroups, dispatched in address order)
// rather than a few long-running ones that stride over the tiles.
//
// Arithmetic follows NumPy's float32 evaluation order exactly (each NumPy
// temporary is one float32 rounding), so products are never fused into adds.
#pragma clang fp contract(off)

#include "common.h"
#include "window.h"
#include "functors.h"

namespace bship {

constexpr size_t kTile = static_cast<size_t>(kBlock) * 4;   // floats per workgroup and vector

// F::apply(v0, v1, v2) -> result. NIN pointers are read (p0..), `out` is written.
// `out` may alias any input, so nothing here is __restrict__; a lane loads all
// of its operands before it stores. VPL = 128-bit vectors per lane: 1 for the
// cheap operations, more for the float64 transcendentals so that a wavefront
// has enough loads in flight to hide its long arithmetic phase.
// run: tiles that one XCD takes in a row (xcd_run_tile).
template <int NIN, bool AL, int VPL, typename F>
__global__ __launch_bounds__(kBlock) void ew_kernel(F f, const float* p0, const float* p1,
                                                    const float* p2, float* out, size_t n, unsigned run, bool through) {
    const size_t base = static_cast<size_t>(xcd_run_tile(run)) * (kTile * VPL) + threadIdx.x * 4;
    f4 r0[VPL], r1[VPL], r2[VPL];
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const size_t i = base + u * kTile;
        if (i + 4 <= n) {
            r0[u] = vload<4, AL>(p0 + i);
            if (NIN > 1) r1[u] = vload<4, AL>(p1 + i);
            if (NIN > 2) r2[u] = vload<4, AL>(p2 + i);
        }
    }
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const size_t i = base + u * kTile;
        if (i + 4 <= n) {
            f4 o;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                o[k] = f.apply(r0[u][k], NIN > 1 ? r1[u][k] : 0.0f, NIN > 2 ? r2[u][k] : 0.0f);
            vstore<4, AL>(out + i, o, through);
        } else {
            for (size_t j = i; j < n; ++j)     // the last, partial vector of the array
                out[j] = f.apply(p0[j], NIN > 1 ? p1[j] : 0.0f, NIN > 2 ? p2[j] : 0.0f);
        }
    }
}

template <typename F, typename = void> struct VectorsPerLane { static constexpr int value = 1; };
template <typename F> struct VectorsPerLane<F, std::void_t<decltype(F::kVectorsPerLane)>> {
    static constexpr int value = F::kVectorsPerLane;
};

template <int NIN, typename F>
int launch_ew(const char* name, F f, const float* p0, const float* p1, const float* p2,
              float* out, size_t n) {
    if (n == 0) return 0;
    constexpr int VPL = VectorsPerLane<F>::value;
    const size_t tiles = (n + kTile * VPL - 1) / (kTile * VPL);
    if (tiles > 0x7fffffffu)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: %zu elements exceed one launch", name, n);
    const dim3 grid(static_cast<unsigned>(tiles));
    const bool through = store_through(n);
    // Measured on MI355X in the sweep, 2^28 and 2^26 elements: kernels with three or more streams (two
    // inputs and the output) gain 2-2.5 % (sigmoid_deriv at 2^26: 7 %) when an XCD works on runs of
    // 512 KiB-1 MiB per stream, kernels with one input lose 2-4 % with any run length, and runs of
    // 256 KiB (which leave an XCD with addresses that agree in bits 18-20) cost every kernel 4-5 %.
    const unsigned run = NIN >= 2 ? static_cast<unsigned>(ctx().ew_run_bytes / (kTile * VPL * sizeof(float))) : 0;
    bool al = aligned16(p0) && aligned16(out) && (NIN < 2 || aligned16(p1)) &&
              (NIN < 3 || aligned16(p2));
    if (al)
        hipLaunchKernelGGL((ew_kernel<NIN, true, VPL, F>), grid, dim3(kBlock), 0, ctx().stream, f,
                           p0, p1, p2, out, n, run, through);
    else
        hipLaunchKernelGGL((ew_kernel<NIN, false, VPL, F>), grid, dim3(kBlock), 0, ctx().stream, f,
                           p0, p1, p2, out, n, run, through);
    return check_launch(name);
}

}  // namespace bship

using namespace bship;

// The elementwise entry points go through the fusing window: the checks first, then either the
// window takes the call (BSHIP_EW_WINDOW) or what earlier calls left behind is enqueued and the
// kernel launched.
#define BSHIP_EW_PROLOGUE(first, outp)        \
    BSHIP_REQUIRE_INIT_NO_FLUSH();            \
    if (n == 0) return 0;                     \
    BSHIP_REQUIRE_PTR(first);                 \
    BSHIP_REQUIRE_PTR(outp);                  \
    BSHIP_REQUIRE_F32_ALIGNED(first);         \
    BSHIP_REQUIRE_F32_ALIGNED(outp)

#define BSHIP_EW_WINDOW(op_ok, what, record)                                                     \
    do {                                                                                         \
        if (!(op_ok)) return set_error(BSHIP_ERR_BAD_OP, "%s: unknown op %d", __func__, what);   \
        if (window_takes()) return window_push(record);                                          \
        BSHIP_FLUSH_PENDING();                                                                   \
    } while (0)

extern "C" {

int bship_binary_f32(int op, const float* a, const float* b, float* out, size_t n) {
    BSHIP_EW_PROLOGUE(a, out);
    BSHIP_REQUIRE_PTR(b);
    BSHIP_REQUIRE_F32_ALIGNED(b);
    BSHIP_EW_WINDOW(op >= BSHIP_ADD && op <= BSHIP_FMOD, op, window::rec_binary(op, a, b, out, n));
    switch (op) {
        case BSHIP_ADD:  return launch_ew<2>("add_tt", AddOp{}, a, b, nullptr, out, n);
        case BSHIP_SUB:  return launch_ew<2>("subtract_tt", SubOp{}, a, b, nullptr, out, n);
        case BSHIP_MUL:  return launch_ew<2>("mult_tt", MulOp{}, a, b, nullptr, out, n);
        case BSHIP_DIV:  return launch_ew<2>("divide_tt", DivOp{}, a, b, nullptr, out, n);
        case BSHIP_FMOD: return launch_ew<2>("modulo_tt", FmodOp{}, a, b, nullptr, out, n);
    }
    return set_error(BSHIP_ERR_BAD_OP, "bship_binary_f32: unknown op %d", op);
}

int bship_mult_add_tt_f32(const float* a, const float* b, float* out, size_t n) {
    BSHIP_EW_PROLOGUE(a, out);
    BSHIP_REQUIRE_PTR(b);
    BSHIP_REQUIRE_F32_ALIGNED(b);
    BSHIP_EW_WINDOW(true, 0, window::rec_mult_add_tt(a, b, out, n));
    return launch_ew<3>("mult_add_tt", MultAddOp{}, a, b, out, out, n);
}

int bship_scalar_f32(int op, float s, const float* t, float* out, size_t n) {
    BSHIP_EW_PROLOGUE(t, out);
    BSHIP_EW_WINDOW(op >= BSHIP_ADD_ST && op <= BSHIP_MULT_ADD_ST, op, window::rec_scalar(op, s, t, out, n));
    switch (op) {
        case BSHIP_ADD_ST:      return launch_ew<1>("add_st", AddStOp{s}, t, nullptr, nullptr, out, n);
        case BSHIP_MULT_ST:     return launch_ew<1>("mult_st", MultStOp{s}, t, nullptr, nullptr, out, n);
        case BSHIP_MULT_ADD_ST: return launch_ew<2>("mult_add_st", MultAddStOp{s}, t, out, nullptr, out, n);
    }
    return set_error(BSHIP_ERR_BAD_OP, "bship_scalar_f32: unknown op %d", op);
}

int bship_unary_f32(int op, const float* x, float* y, size_t n) {
    BSHIP_EW_PROLOGUE(x, y);
    BSHIP_EW_WINDOW(op >= BSHIP_ABS && op <= BSHIP_EL, op, window::rec_unary(op, x, y, n));
    switch (op) {
        case BSHIP_ABS:     return launch_ew<1>("abs_t", AbsOp{}, x, nullptr, nullptr, y, n);
        case BSHIP_SIGN:    return launch_ew<1>("sign_t", SignOp{}, x, nullptr, nullptr, y, n);
        case BSHIP_SQRT:    return launch_ew<1>("sqrt_t", SqrtOp{}, x, nullptr, nullptr, y, n);
        case BSHIP_LOG:     return launch_ew<1>("log_t", LogOp{}, x, nullptr, nullptr, y, n);
        case BSHIP_SIGMOID: return launch_ew<1>("sigmoid", SigmoidOp{}, x, nullptr, nullptr, y, n);
        case BSHIP_TANH:    return launch_ew<1>("tanh", TanhOp{}, x, nullptr, nullptr, y, n);
        case BSHIP_REL:     return launch_ew<1>("rel", RelOp{}, x, nullptr, nullptr, y, n);
        case BSHIP_EL:      return launch_ew<1>("el", ElOp{}, x, nullptr, nullptr, y, n);
    }
    return set_error(BSHIP_ERR_BAD_OP, "bship_unary_f32: unknown op %d", op);
}

int bship_deriv_f32(int op, const float* y, const float* dy, float* dx, size_t n) {
    BSHIP_EW_PROLOGUE(y, dx);
    BSHIP_REQUIRE_PTR(dy);
    BSHIP_REQUIRE_F32_ALIGNED(dy);
    BSHIP_EW_WINDOW(op >= BSHIP_SIGMOID_DERIV && op <= BSHIP_EL_DERIV, op, window::rec_deriv(op, y, dy, dx, n));
    switch (op) {
        case BSHIP_SIGMOID_DERIV: return launch_ew<2>("sigmoid_deriv", SigmoidDerivOp{}, y, dy, nullptr, dx, n);
        case BSHIP_TANH_DERIV:    return launch_ew<2>("tanh_deriv", TanhDerivOp{}, y, dy, nullptr, dx, n);
        case BSHIP_REL_DERIV:     return launch_ew<2>("rel_deriv", RelDerivOp{}, y, dy, nullptr, dx, n);
        case BSHIP_EL_DERIV:      return launch_ew<2>("el_deriv", ElDerivOp{}, y, dy, nullptr, dx, n);
    }
    return set_error(BSHIP_ERR_BAD_OP, "bship_deriv_f32: unknown op %d", op);
}

int bship_clip_f32(const float* a, float lo, float hi, float* out, size_t n) {
    BSHIP_EW_PROLOGUE(a, out);
    BSHIP_EW_WINDOW(true, 0, window::rec_clip(a, lo, hi, out, n));
    return launch_ew<1>("clip_t", ClipOp{lo, hi}, a, nullptr, nullptr, out, n);
}

int bship_cond_f32(int op, const float* a, float val, float* out, const float* cond, size_t n) {
    BSHIP_EW_PROLOGUE(cond, out);
    BSHIP_REQUIRE_F32_ALIGNED(a);
    BSHIP_FLUSH_PENDING();          // the conditional operations belong to no layer's sequence
    switch (op) {
        case BSHIP_COPY_IF:
            BSHIP_REQUIRE_PTR(a);
            return launch_ew<3>("copy_to_if", CopyIfOp{}, a, cond, out, out, n);
        case BSHIP_FILL_IF:
            return launch_ew<2>("fill_if", FillIfOp{val}, cond, out, nullptr, out, n);
        case BSHIP_ADD_IF:
            BSHIP_REQUIRE_PTR(a);
            return launch_ew<3>("add_into_if", AddIfOp{}, a, cond, out, out, n);
    }
    return set_error(BSHIP_ERR_BAD_OP, "bship_cond_f32: unknown op %d", op);
}

}  // extern "C"
