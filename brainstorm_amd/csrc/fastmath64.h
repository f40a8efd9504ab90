// float32 transcendentals evaluated in float64 and rounded once.
//
// NumPy evaluates exp/log/tanh of float32 arrays with SIMD polynomial code that
// is 1-4 ulp away from the true value, differently on different host CPUs.
// These routines aim at the true value instead: every intermediate is float64
// with a relative error below 2^-40, so the single final rounding to float32
// gives the correctly rounded result except for inputs whose true value lies
// within 2^-40 of a rounding boundary. The operation count (about 25-30 float64
// instructions per element) keeps the streaming kernels that call them close to
// their memory-bound speed, which the general-purpose float64 library routines
// (several times more instructions: full double accuracy, full range) do not.
#pragma once

#include <hip/hip_runtime.h>

namespace bship {

// 1/d with relative error below 2^-48: the hardware estimate (measured 2^-24.4
// on gfx950) plus one Newton step.
__device__ __forceinline__ double rcp64(double d) {
    double y = __builtin_amdgcn_rcp(d);
    y = __builtin_fma(__builtin_fma(-d, y, 1.0), y, y);
    return y;
}

// Range reduction of exp: y = k*ln2 + r with |r| <= ln2/2. Valid for |y| < 1000.
__device__ __forceinline__ void exp_reduce(double y, double& kd, double& r) {
    kd = __builtin_rint(y * 1.4426950408889634);          // y / ln 2
    r = __builtin_fma(-kd, 0.6931471805599453, y);
}

// q(r) = (exp(r) - 1) / r = 1 + r/2! + r^2/3! + ... + r^9/10!  for |r| <= 0.3466.
// Truncation error r^10/11! < 2^-42 relative to exp(r).
__device__ __forceinline__ double expm1_over_r(double r) {
    double q = 2.755731922398589e-07;                      // 1/10!
    q = __builtin_fma(q, r, 2.7557319223985893e-06);       // 1/9!
    q = __builtin_fma(q, r, 2.48015873015873e-05);         // 1/8!
    q = __builtin_fma(q, r, 1.984126984126984e-04);        // 1/7!
    q = __builtin_fma(q, r, 1.388888888888889e-03);        // 1/6!
    q = __builtin_fma(q, r, 8.333333333333333e-03);        // 1/5!
    q = __builtin_fma(q, r, 4.1666666666666664e-02);       // 1/4!
    q = __builtin_fma(q, r, 1.6666666666666666e-01);       // 1/3!
    q = __builtin_fma(q, r, 0.5);                          // 1/2!
    q = __builtin_fma(q, r, 1.0);                          // 1/1!
    return q;
}

// exp(y) for -1000 < y < 700 (callers clamp).
__device__ __forceinline__ double exp64(double y) {
    double kd, r;
    exp_reduce(y, kd, r);
    const double p = __builtin_fma(r, expm1_over_r(r), 1.0);
    return __builtin_ldexp(p, static_cast<int>(kd));
}

// np.exp(x) for a float32 x, rounded once (overflows to inf, underflows through denormals to 0).
__device__ __forceinline__ float exp_f32(float x) {
    const double y = __builtin_fmin(__builtin_fmax(static_cast<double>(x), -200.0), 100.0);
    const float r = static_cast<float>(exp64(y));
    return (x != x) ? x : r;
}

// Logistic function with the reference's two branches (numpy_handler.py:283-287):
// 1/(1+exp(-x)) for x >= 0, exp(x)/(1+exp(x)) for x < 0; e = exp(-|x|) serves both.
__device__ __forceinline__ float sigmoid_f32(float x) {
    const double ax = __builtin_fmin(__builtin_fabs(static_cast<double>(x)), 200.0);
    const double e = exp64(-ax);
    const double num = (x >= 0.0f) ? 1.0 : e;
    const float r = static_cast<float>(num * rcp64(1.0 + e));
    return (x != x) ? x : r;
}

// tanh(x) = em / (em + 2) with em = exp(2x) - 1. For |2x| below ln2/2 the reduced
// argument is 2x itself and em = r*q(r) keeps full relative accuracy near zero.
__device__ __forceinline__ float tanh_f32(float x) {
    const double y = __builtin_fmin(__builtin_fmax(2.0 * static_cast<double>(x), -40.0), 40.0);
    double kd, r;
    exp_reduce(y, kd, r);
    const double rq = r * expm1_over_r(r);
    const double em_big = __builtin_ldexp(1.0 + rq, static_cast<int>(kd)) - 1.0;
    const double em = (kd == 0.0) ? rq : em_big;
    const float t = static_cast<float>(em * rcp64(em + 2.0));
    return (x != x) ? x : t;
}

// ln(x): x = m * 2^e with m in [sqrt(1/2), sqrt(2)); ln m = 2 atanh(s), s = (m-1)/(m+1),
// |s| <= 0.1716, series up to s^15 (next term < 2^-44 relative).
__device__ __forceinline__ float log_f32(float x) {
    const double xd = static_cast<double>(x);              // exact, also for float32 denormals
    double m = __builtin_amdgcn_frexp_mant(xd);            // [0.5, 1)
    int e = __builtin_amdgcn_frexp_exp(xd);
    const bool low = m < 0.7071067811865476;
    m = low ? m * 2.0 : m;
    e = low ? e - 1 : e;
    const double s = (m - 1.0) * rcp64(m + 1.0);
    const double z = s * s;
    double p = 6.666666666666667e-02;                      // 1/15
    p = __builtin_fma(p, z, 7.692307692307693e-02);        // 1/13
    p = __builtin_fma(p, z, 9.090909090909091e-02);        // 1/11
    p = __builtin_fma(p, z, 1.1111111111111111e-01);       // 1/9
    p = __builtin_fma(p, z, 1.4285714285714285e-01);       // 1/7
    p = __builtin_fma(p, z, 0.2);                          // 1/5
    p = __builtin_fma(p, z, 3.3333333333333331e-01);       // 1/3
    p = p * z;
    const double two_s = s + s;
    const double ln_m = __builtin_fma(two_s, p, two_s);
    float r = static_cast<float>(__builtin_fma(static_cast<double>(e), 0.6931471805599453, ln_m));
    if (!(x > 0.0f)) r = (x == 0.0f) ? -INFINITY : NAN;    // 0 -> -inf; negative, NaN -> NaN
    if (x == INFINITY) r = INFINITY;
    return r;
}

}  // namespace bship
