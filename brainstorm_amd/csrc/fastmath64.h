// float32 transcendentals evaluated in float64 and rounded once.
//
// NumPy evaluates exp/log/tanh of float32 arrays with SIMD polynomial code that
// is 1-4 ulp away from the true value, differently on different host CPUs.
// These routines aim at the true value instead: every intermediate is float64
// with a relative error below 2^-42, so the single final rounding to float32
// gives the correctly rounded result except for inputs whose true value lies
// within 2^-42 of a rounding boundary. The operation count (about 25-30 float64
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

// Instruction budget. On gfx950 a float64 fma/add/mul issues at the rate of an unpacked float32 one,
// while float64 reciprocal, conversion, rounding, ldexp and frexp take twice as long. The
// streaming kernels that call these routines stay memory-bound only below about 28 issue slots
// per element, so: range reductions round by adding 1.5*2^52 (the integer lands in the low
// word of the sum), powers of two are built and applied with integer instructions on the
// exponent field, clamps happen in float32 before the one conversion, and the polynomials are
// near-minimax fits (Chebyshev-node interpolation computed with 60 digits) instead of longer
// Taylor sums.

constexpr double kRoundMagic = 6755399441055744.0;         // 1.5 * 2^52

// q(r) = (exp(r) - 1) / r for |r| <= ln2/2, relative error below 2^-43.
__device__ __forceinline__ double expm1_over_r(double r) {
    double q = 2.762511557828763e-06;
    q = __builtin_fma(q, r, 2.4876178959085513e-05);
    q = __builtin_fma(q, r, 1.9841208732536384e-04);
    q = __builtin_fma(q, r, 1.388882165071769e-03);
    q = __builtin_fma(q, r, 8.333333353729397e-03);
    q = __builtin_fma(q, r, 4.16666668910917e-02);
    q = __builtin_fma(q, r, 1.666666666664829e-01);
    q = __builtin_fma(q, r, 4.9999999999797773e-01);
    q = __builtin_fma(q, r, 1.0);
    return q;
}

// 2^k as a float64, -1022 <= k <= 1023.
__device__ __forceinline__ double pow2_f64(int k) {
    return __hiloint2double((k << 20) + 0x3ff00000, 0);
}

// p * 2^k for a normal p whose result is normal too: k is added to the exponent field.
__device__ __forceinline__ double scale_pow2(double p, int k) {
    return __hiloint2double(__double2hiint(p) + (k << 20), __double2loint(p));
}

// exp(y) for |y| < 700 (callers clamp): y = k*ln2 + r, |r| <= ln2/2, exp(r) = 1 + r*q(r) in [0.70, 1.42].
__device__ __forceinline__ double exp64(double y) {
    const double t = __builtin_fma(y, 1.4426950408889634, kRoundMagic);   // y / ln 2 rounded to an integer
    const int k = __double2loint(t);
    const double kd = t - kRoundMagic;
    const double r = __builtin_fma(-kd, 0.6931471805599453, y);
    const double p = __builtin_fma(r, expm1_over_r(r), 1.0);
    return scale_pow2(p, k);
}

// np.exp(x) for a float32 x, rounded once (overflows to inf, underflows through denormals to 0).
__device__ __forceinline__ float exp_f32(float x) {
    const double y = static_cast<double>(__builtin_amdgcn_fmed3f(x, -200.0f, 100.0f));
    const float r = static_cast<float>(exp64(y));
    return (x != x) ? x : r;
}

// Logistic function. The reference picks 1/(1+exp(-x)) for x >= 0 and exp(x)/(1+exp(x)) for
// x < 0 (numpy_handler.py:283-287) so that float32 exp never overflows; in float64, with |x|
// clamped to 200, the first form is accurate on both sides (exp(200) = 7e86, no cancellation),
// and both forms round to the same float32.
__device__ __forceinline__ float sigmoid_f32(float x) {
    const double xd = static_cast<double>(__builtin_amdgcn_fmed3f(x, -200.0f, 200.0f));
    const float r = static_cast<float>(rcp64(1.0 + exp64(-xd)));
    return (x != x) ? x : r;
}

// tanh(x) = em / (em + 2) with em = exp(2x) - 1 = 2^k (1 + rq) - 1, where 2x = k*ln2 + 2h,
// |h| <= ln2/4 and rq = exp(2h) - 1 = h * Q(h). For k = 0 this is rq itself, which keeps full
// relative accuracy near zero. |x| is clamped to 20 (tanh rounds to 1 from 9.02 on).
__device__ __forceinline__ float tanh_f32(float x) {
    const double xd = static_cast<double>(__builtin_amdgcn_fmed3f(x, -20.0f, 20.0f));
    const double t = __builtin_fma(xd, 2.8853900817779268, kRoundMagic);   // 2x / ln 2 rounded to an integer
    const int k = __double2loint(t);
    const double kd = t - kRoundMagic;
    const double h = __builtin_fma(-kd, 0.34657359027997264, xd);          // x - k ln2/2
    // Q(h) = (exp(2h) - 1) / h, relative error below 2^-43
    double q = 1.4144059176083267e-03;
    q = __builtin_fma(q, h, 6.3683018135258914e-03);
    q = __builtin_fma(q, h, 2.5396747177646572e-02);
    q = __builtin_fma(q, h, 8.888845856459322e-02);
    q = __builtin_fma(q, h, 2.666666673193407e-01);
    q = __builtin_fma(q, h, 6.666666702574672e-01);
    q = __builtin_fma(q, h, 1.333333333331863);
    q = __builtin_fma(q, h, 1.999999999991911);
    q = __builtin_fma(q, h, 2.0);
    const double rq = h * q;
    const double s = pow2_f64(k);
    const double em = __builtin_fma(s, rq, s - 1.0);
    const float r = static_cast<float>(em * rcp64(em + 2.0));
    // tanh is odd: the sign is the argument's (for -0.0 the fma above has produced +0.0)
    return (x != x) ? x : __builtin_copysignf(r, x);
}

// ln(x): x = m * 2^e with m in [sqrt(1/2), sqrt(2)); ln m = 2 atanh(s) = 2s (1 + z P(z)) with
// s = (m-1)/(m+1), z = s^2 <= 0.0295, P fitted to a relative error of ln m below 2^-43.
// m and e come from the high word of the float64 image of x (exact also for float32 denormals):
// subtracting the high word of sqrt(1/2) moves the split point of the mantissa there.
__device__ __forceinline__ float log_f32(float x) {
    const double xd = static_cast<double>(x);
    const int ix = __double2hiint(xd) - 0x3fe6a09e;
    const int e = ix >> 20;
    const double m = __hiloint2double((ix & 0x000fffff) + 0x3fe6a09e, __double2loint(xd));
    const double ed = __hiloint2double(0x43300000, e ^ static_cast<int>(0x80000000u)) - 4503601774854144.0;   // 2^52 + 2^31
    const double s = (m - 1.0) * rcp64(m + 1.0);
    const double z = s * s;
    double p = 9.681942493316599e-02;
    p = __builtin_fma(p, z, 1.1095668714032891e-01);
    p = __builtin_fma(p, z, 1.4285877767516472e-01);
    p = __builtin_fma(p, z, 1.9999999396220844e-01);
    p = __builtin_fma(p, z, 3.333333333368934e-01);
    p = p * z;
    const double two_s = s + s;
    const double ln_m = __builtin_fma(two_s, p, two_s);
    float r = static_cast<float>(__builtin_fma(ed, 0.6931471805599453, ln_m));
    // everything but positive finite numbers: 0 -> -inf, +inf -> +inf, negative or NaN -> NaN
    if (!__builtin_amdgcn_classf(x, 0x180)) r = (x == 0.0f) ? -INFINITY : (x == INFINITY ? INFINITY : NAN);
    return r;
}

}  // namespace bship
