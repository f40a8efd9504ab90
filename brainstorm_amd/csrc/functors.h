// Per-element arithmetic of the handler operations, shared by the streaming
// kernels (elementwise.hip) and the fused layer kernels (fused.hip).
//
// Every functor maps up to three input values to one result with exactly the
// float32 rounding steps NumPy performs for the reference expression (each
// NumPy temporary is one rounding; products are never fused into adds), so a
// fused kernel that chains them gives the same bits as the separate kernels.
#pragma once
#pragma clang fp contract(off)

#include "common.h"
#include "fastmath64.h"

namespace bship {

// ------------------------------- functors ---------------------------------
// Inputs arrive as (v0, v1, v2) in the order the launcher passes pointers.

struct AddOp  { __device__ float apply(float a, float b, float) const { return a + b; } };
struct SubOp  { __device__ float apply(float a, float b, float) const { return a - b; } };
struct MulOp  { __device__ float apply(float a, float b, float) const { return a * b; } };
struct DivOp  { __device__ float apply(float a, float b, float) const { return a / b; } };
struct FmodOp { __device__ float apply(float a, float b, float) const { return fmodf(a, b); } };
// (a, b, old out): out + a*b with the product rounded first
struct MultAddOp {
    __device__ float apply(float a, float b, float o) const { float p = a * b; return o + p; }
};

struct AddStOp  { float s; __device__ float apply(float t, float, float) const { return t + s; } };
struct MultStOp { float s; __device__ float apply(float t, float, float) const { return s * t; } };
// (t, old out)
struct MultAddStOp {
    float s;
    __device__ float apply(float t, float o, float) const { float p = s * t; return o + p; }
};

struct AbsOp  { __device__ float apply(float x, float, float) const { return fabsf(x); } };
// np.sign: 1, -1, 0 (also for -0.0), NaN stays NaN
struct SignOp {
    __device__ float apply(float x, float, float) const {
        return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : (x == 0.0f ? 0.0f : x));
    }
};
struct SqrtOp { __device__ float apply(float x, float, float) const { return sqrtf(x); } };
// Transcendentals are evaluated in float64 and rounded once (fastmath64.h).
#ifndef BSHIP_HEAVY_VPL
#define BSHIP_HEAVY_VPL 2
#endif
struct LogOp {
    static constexpr int kVectorsPerLane = BSHIP_HEAVY_VPL;
    __device__ float apply(float x, float, float) const { return log_f32(x); }
};
struct TanhOp {
    static constexpr int kVectorsPerLane = BSHIP_HEAVY_VPL;
    __device__ float apply(float x, float, float) const { return tanh_f32(x); }
};
struct SigmoidOp {
    static constexpr int kVectorsPerLane = BSHIP_HEAVY_VPL;
    __device__ float apply(float x, float, float) const { return sigmoid_f32(x); }
};
// numpy 277-278: x*(x>0); the mask is 1.0 or 0.0, so negatives give -0.0
struct RelOp {
    __device__ float apply(float x, float, float) const { return x > 0.0f ? x : x * 0.0f; }
};
// numpy 303-305: x*(x>=0) + (exp(x)-1)*(x<0), every step in float32
struct ElOp {
    __device__ float apply(float x, float, float) const {
        float e = exp_f32(x);
        float t1 = x * (x >= 0.0f ? 1.0f : 0.0f);
        float t2 = (e - 1.0f) * (x < 0.0f ? 1.0f : 0.0f);
        return t1 + t2;
    }
};

// derivatives take (y, dy)
struct SigmoidDerivOp {
    __device__ float apply(float y, float dy, float) const { float p = dy * y; float q = 1.0f - y; return p * q; }
};
struct TanhDerivOp {
    __device__ float apply(float y, float dy, float) const { float p = y * y; float q = 1.0f - p; return dy * q; }
};
struct RelDerivOp {
    __device__ float apply(float y, float dy, float) const { return dy * (y > 0.0f ? 1.0f : 0.0f); }
};
struct ElDerivOp {
    __device__ float apply(float y, float dy, float) const {
        float t1 = dy * (y >= 0.0f ? 1.0f : 0.0f);
        float q = y + 1.0f;
        float p = dy * q;
        float t2 = p * (y < 0.0f ? 1.0f : 0.0f);
        return t1 + t2;
    }
};

// np.clip = minimum(maximum(a, lo), hi) with NaN in `a` propagating
struct ClipOp {
    float lo, hi;
    __device__ float apply(float a, float, float) const {
        float t = (a != a || a > lo) ? a : lo;
        return (t != t || t < hi) ? t : hi;
    }
};

// conditional ops; cond != 0 is true for NaN as in NumPy
struct CopyIfOp {  // (a, cond, old out)
    __device__ float apply(float a, float c, float o) const { return c != 0.0f ? a : o; }
};
struct FillIfOp {  // (cond, old out)
    float val;
    __device__ float apply(float c, float o, float) const { return c != 0.0f ? val : o; }
};
struct AddIfOp {   // (a, cond, old out)
    __device__ float apply(float a, float c, float o) const { return c != 0.0f ? o + a : o; }
};


}  // namespace bship
