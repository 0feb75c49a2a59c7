// Scalar functions of the elementwise kernel family, device side.
//
// Semantics follow the CPU lambdas of the reference, J/backend/main/implementations/fun/Scalar*.java
// (J/ = src/main/java/neureka/).  The reference evaluates most f32 activations as
// `(float) f((double) x)` (fun/api/CPUFun.java:7-9); here f32 is evaluated in f32 with formulations
// that avoid the cancellation a literal f32 transcription would suffer, so results stay within 1e-5
// relative of the reference.  Functions the reference overrides with pure float arithmetic
// (fast_gaus, softsign, gasu, fast_tanh, relu, quad, ...) are transcribed operation for operation and are
// bit-identical (the library is compiled with -ffp-contract=off and correctly rounded division).
// f64 uses the reference's own formulas.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/neureka_hip.h"

namespace nk {

template <typename T> struct Num;
template <> struct Num<float> {
    static __device__ __forceinline__ float exp(float x) { return ::expf(x); }
    static __device__ __forceinline__ float expm1(float x) { return ::expm1f(x); }
    static __device__ __forceinline__ float log(float x) { return ::logf(x); }
    static __device__ __forceinline__ float log1p(float x) { return ::log1pf(x); }
    static __device__ __forceinline__ float log10(float x) { return ::log10f(x); }
    static __device__ __forceinline__ float sin(float x) { return ::sinf(x); }
    static __device__ __forceinline__ float cos(float x) { return ::cosf(x); }
    static __device__ __forceinline__ float sqrt(float x) { return ::sqrtf(x); }
    static __device__ __forceinline__ float cbrt(float x) { return ::cbrtf(x); }
    static __device__ __forceinline__ float pow(float a, float b) { return ::powf(a, b); }
    static __device__ __forceinline__ float fmod(float a, float b) { return ::fmodf(a, b); }
    static __device__ __forceinline__ float abs(float x) { return ::fabsf(x); }
    static __device__ __forceinline__ float tanh(float x) { return ::tanhf(x); }
    static __device__ __forceinline__ float fma(float a, float b, float c) { return ::fmaf(a, b, c); }
};
__device__ __forceinline__ double log_double(double x);        // below: the natural and the decimal logarithm of a double
__device__ __forceinline__ double log10_double(double x);
template <> struct Num<double> {
    static __device__ __forceinline__ double exp(double x) { return ::exp(x); }
    static __device__ __forceinline__ double expm1(double x) { return ::expm1(x); }
    static __device__ __forceinline__ double log(double x) { return log_double(x); }
    static __device__ __forceinline__ double log1p(double x) { return ::log1p(x); }
    static __device__ __forceinline__ double log10(double x) { return log10_double(x); }
    static __device__ __forceinline__ double sin(double x) { return ::sin(x); }
    static __device__ __forceinline__ double cos(double x) { return ::cos(x); }
    static __device__ __forceinline__ double sqrt(double x) { return ::sqrt(x); }
    static __device__ __forceinline__ double cbrt(double x) { return ::cbrt(x); }
    static __device__ __forceinline__ double pow(double a, double b) { return ::pow(a, b); }
    static __device__ __forceinline__ double fmod(double a, double b) { return ::fmod(a, b); }
    static __device__ __forceinline__ double abs(double x) { return ::fabs(x); }
    static __device__ __forceinline__ double tanh(double x) { return ::tanh(x); }
    static __device__ __forceinline__ double fma(double a, double b, double c) { return ::fma(a, b, c); }
};

// a * b + c with c a wave-uniform constant that stays in scalar registers.  Written as one instruction because the
// compiler, left to itself, copies every double constant of a polynomial into a pair of vector registers right before
// its multiply-add (two more vector instructions per step; hoisting them out of the interpreter's loop instead costs
// the registers of every table entry at once).
__device__ __forceinline__ double fma_const(double a, double b, double c) {
    double d;
    asm("v_fma_f64 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "s"(c));
    return d;
}
// exp(z) in double, sized for its callers here: the float kernels that must repeat the reference's double evaluation
// ((float) f((double) x), fun/api/CPUFun.java:7-9) because its formulas cancel -- 1 - tanh^2, s (1 - s) -- so that the
// float they round to has to be the reference's float.  z = n ln2 + r with |r| <= ln2 / 2 (ln2 in two parts, n ln2_hi
// exact), e^r as the Taylor polynomial of degree 13 (the next term is below 2^-57), the power of two applied by ldexp:
// two dozen full-rate instructions, no table, no branch, an error of about one unit in the last place.  The device
// library's exp spends three times that on cases these callers never reach.
__device__ __forceinline__ double exp_reduced(double z) {        // -746 <= z <= 710, or NaN
    const double n = __builtin_rint(z * 1.4426950408889634074);
    double r = __builtin_fma(n, -6.93147180369123816490e-01, z);
    r = __builtin_fma(n, -1.90821492927058770002e-10, r);
    double p = fma_const(r, 1.6059043836821613e-10, 2.08767569878681e-09);      // 1/13!, 1/12!, ... 1/2!
    p = fma_const(p, r, 2.505210838544172e-08);
    p = fma_const(p, r, 2.755731922398589e-07);
    p = fma_const(p, r, 2.7557319223985893e-06);
    p = fma_const(p, r, 2.48015873015873e-05);
    p = fma_const(p, r, 1.984126984126984e-04);
    p = fma_const(p, r, 1.3888888888888889e-03);
    p = fma_const(p, r, 8.333333333333333e-03);
    p = fma_const(p, r, 4.1666666666666664e-02);
    p = fma_const(p, r, 1.6666666666666666e-01);
    p = __builtin_fma(p, r, 0.5);
    p = __builtin_fma(p, r, 1.0);
    p = __builtin_fma(p, r, 1.0);
    return __builtin_ldexp(p, (int)n);
}
// Arguments are clamped to where the result saturates (0 below -746, infinity above 710); a NaN fails both
// comparisons, passes through and comes out as NaN.
__device__ __forceinline__ double exp_fast(double z) {
    z = z < -746.0 ? -746.0 : z;
    z = z > 710.0 ? 710.0 : z;
    return exp_reduced(z);
}
// 1 / d for 1 <= d < 1e305 (the 1 + e^z of a logistic function): the hardware estimate and two Newton steps, a
// relative error of about 2^-52, a third of the instructions of the correctly rounded division.
__device__ __forceinline__ double rcp_fast(double d) {
    double r = __builtin_amdgcn_rcp(d);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    return r;
}
// ln x in double for the f64 kernels (ln, softplus): x = m 2^e with m in [sqrt(1/2), sqrt 2), ln m = 2 atanh((m - 1)/(m + 1))
// -- m - 1 is exact, so the result keeps its relative accuracy where x is close to 1 -- as the odd series up to s^19 (the
// next term is below 3e-17 of the sum), e ln 2 with ln 2 in two parts (e ln2_hi is exact): about 3 units in the last
// place (7e-16), some thirty full-rate instructions and one reciprocal, no table.  Math.log is specified to 1 ulp and
// not bit for bit; the device library's log costs three times as much (2^25 doubles: 116 us, bound by it, against
// 80 for a function that only moves the data).  Zero, negative numbers, infinity and NaN get Math.log's answers.
// (the reduction: x = m 2^n, returns atanh((m - 1)/(m + 1)) = ln(m) / 2 for 0 < x < infinity)
__device__ __forceinline__ double half_log_of_mantissa(double x, double& n) {
    int e;
    double m = __builtin_frexp(x, &e);                           // [0.5, 1), subnormal arguments included
    const bool low = m < 0.70710678118654752;
    m = low ? m + m : m;
    e = low ? e - 1 : e;
    n = (double)e;
    const double s = (m - 1.0) * rcp_fast(m + 1.0);
    const double s2 = s * s;
    double q = fma_const(s2, 0.052631578947368418, 0.058823529411764705);      // 1/19, 1/17, ... 1/3
    q = fma_const(q, s2, 0.066666666666666666);
    q = fma_const(q, s2, 0.076923076923076927);
    q = fma_const(q, s2, 0.090909090909090912);
    q = fma_const(q, s2, 0.1111111111111111);
    q = fma_const(q, s2, 0.14285714285714285);
    q = fma_const(q, s2, 0.2);
    q = fma_const(q, s2, 0.33333333333333331);
    return __builtin_fma(s * s2, q, s);
}
__device__ __forceinline__ double log_double(double x) {
    if (x > 0.0 && x < (double)__builtin_inff()) {
        double n;
        const double h = half_log_of_mantissa(x, n);
        return __builtin_fma(n, 6.93147180369123816490e-01, __builtin_fma(n, 1.90821492927058770002e-10, h + h));
    }
    return x == 0.0 ? -(double)__builtin_inff() : (x < 0.0 ? __builtin_nan("") : x);
}
// log10 on the same reduction: n log10(2) in two parts plus ln(m) / ln 10.  Math.log10 promises the whole number n for an
// argument that equals 10^n; the doubles that do are 10^0 ... 10^22, and a result that lands within 1e-13 of such an n is
// compared with that power (a product of exact factors) and replaced by n when the argument is the power.
__device__ __forceinline__ double log10_double(double x) {
    if (x > 0.0 && x < (double)__builtin_inff()) {
        double n;
        const double h = half_log_of_mantissa(x, n);
        double r = __builtin_fma(n, 3.01029995663611771306e-01, __builtin_fma(n, 3.69423907715893078616e-13, (h + h) * 4.34294481903251816668e-01));
        const double k = __builtin_rint(r);
        if (k >= 0.0 && k <= 22.0 && __builtin_fabs(r - k) < 1e-13) {
            double power = 1.0;
            for (int i = 0; i < (int)k; i++) power *= 10.0;      // exact up to 10^22
            r = x == power ? k : r;
        }
        return r;
    }
    return x == 0.0 ? -(double)__builtin_inff() : (x < 0.0 ? __builtin_nan("") : x);
}
// 1 / (1 + e^(k x)) for a float x, |k| <= 2.  The argument stays within +-700, so that 1 + e^z stays finite for the
// Newton steps (the answers there, 1 and 1e-304, are the saturated ones), by one float instruction on x instead of two
// double comparisons with their selects.  That clamp turns a NaN into a number: the caller puts the NaN back into its
// float result (`x != x ? x : result`).
template <int K1000>                                              // k in thousandths: -2000, -1000, -1702
__device__ __forceinline__ double logistic_of_float(float x) {
    constexpr double k = K1000 / 1000.0;
    constexpr float bound = (float)(700.0 / (K1000 < 0 ? -k : k));
    const float xc = __builtin_amdgcn_fmed3f(x, -bound, bound);
    return rcp_fast(1.0 + exp_reduced((double)xc * k));
}

// Binary operators whose f32 form the reference evaluates through double (Math.pow / Math.log take and return
// double; implementations/elementwise/CPUBiElementWisePower.java:11,21,31, CPUBiElementWiseDivision.java:31,
// CPUBiElementWiseModulo.java:31 and the broadcast twins): the intermediates neither overflow nor underflow
// where float ones would.
// The exponents that dominate in practice have exact answers that need no general pow (which costs some hundred
// double-precision instructions): Math.pow returns its first argument for an exponent of 1 and 1.0 for an exponent
// of zero by specification, and a square is the correctly rounded product (exact in double for a float base) --
// what a correctly rounded pow returns and what HotSpot substitutes for pow(x, 2.0).
// Where java.lang.Math.pow differs from C99's pow the reference's answer is kept: a NaN exponent gives NaN whatever
// the base (C: pow(1, NaN) = 1) and a base of magnitude 1 with an infinite exponent gives NaN (C: 1).
__device__ __forceinline__ double pow_double(double a, double b) {
    if (b == 2.0) return a * a;
    if (b == 1.0) return a;
    if (b == 0.0) return 1.0;
    if (b != b || (fabs(a) == 1.0 && isinf(b))) return __builtin_nan("");
    return ::pow(a, b);
}
__device__ __forceinline__ double pow_ref(double a, double b) { return pow_double(a, b); }
// f32: the reference evaluates (float) Math.pow((double) a, (double) b).  The float routine of the device library works
// on a two-float logarithm and is within 2 ulp of that (far inside 1e-5) at a fraction of the cost of the double one
// (f32 tensors: 0.6 -> 3 TB/s); Math.pow's special cases that C answers differently are taken out first, as above.
// A positive finite base and a finite exponent -- the bulk of every tensor -- take a path of about forty full-rate
// instructions: log2 of the base in double (a = m 2^e with m in [sqrt(1/2), sqrt 2), log m = 2 atanh((m - 1)/(m + 1)) as
// the odd series up to s^13, relative error 2^-34), the product with the exponent in double, and 2^p as the hardware's
// float exp2 of the fractional part scaled by ldexp.  The error of the product enters the result as p 2^-34 ln 2 <
// 1e-8 and the float conversion of the fraction as 2e-8, so the result is within 3 ulp of (float) Math.pow.
__device__ __forceinline__ double log2_of_positive(float a) {       // 0 < a < infinity
    int e;
    double m = __builtin_frexp((double)a, &e);                   // [0.5, 1)
    const bool low = m < 0.70710678118654752;
    m = low ? m + m : m;
    e = low ? e - 1 : e;
    const double s = (m - 1.0) * rcp_fast(m + 1.0);
    const double s2 = s * s;
    double q = fma_const(s2, 0.076923076923076927, 0.090909090909090912);       // 1/13, 1/11, ... 1/3
    q = fma_const(q, s2, 0.1111111111111111);
    q = fma_const(q, s2, 0.14285714285714285);
    q = fma_const(q, s2, 0.2);
    q = fma_const(q, s2, 0.33333333333333331);
    const double ln_m_half = __builtin_fma(s * s2, q, s);        // atanh(s)
    return __builtin_fma(ln_m_half, 2.8853900817779268, (double)e);             // e + 2 atanh(s) log2(e)
}
__device__ __forceinline__ float pow_positive(float a, float b) {
    double p = (double)b * log2_of_positive(a);
    p = p < -320.0 ? -320.0 : p;                                 // 2^-320 and 2^320 are 0 and infinity in float
    p = p > 320.0 ? 320.0 : p;
    const double n = __builtin_rint(p);
    const float r = __builtin_amdgcn_exp2f((float)(p - n));
    return __builtin_ldexpf(r, (int)n);
}
// a^b with the range of a double and the precision of a float (3 ulp of a float): what the float derivatives of the
// power and of the cube root need -- the reference forms them in double (b * Math.pow(a, b - 1), Math.pow(a, b) *
// Math.log(a), 1 / (3 * Math.pow(x, 2/3))) and rounds the product to float, so the power may leave the float range
// where the product does not.  l2 = log2_of_positive(a).
__device__ __forceinline__ double pow_from_log2(double l2, double b) {
    double p = b * l2;
    p = p < -1100.0 ? -1100.0 : p;                               // 2^-1100 and 2^1100 are 0 and infinity in double
    p = p > 1100.0 ? 1100.0 : p;
    const double n = __builtin_rint(p);
    const float r = __builtin_amdgcn_exp2f((float)(p - n));
    return __builtin_ldexp((double)r, (int)n);
}
// A finite base below zero: Math.pow answers with the power of |a|, negated for an odd whole exponent, and with NaN for an
// exponent that is no whole number.  The factor that carries this (floats from 2^24 on are even numbers): tensors of
// mixed sign stay on the short path instead of sending every wavefront through the library routine as well.
__device__ __forceinline__ float pow_sign_of(float a, float e) {
    const bool whole = e == __builtin_rintf(e);
    const bool odd = ::fabsf(e) < 16777216.0f && ((int)e & 1);
    const float s = whole ? (odd ? -1.0f : 1.0f) : __builtin_nanf("");
    return a < 0.0f ? s : 1.0f;
}
// ... looked at only by wavefronts that hold a negative base at all (a branch on the scalar unit): tensors of positive
// bases pay one comparison for it
__device__ __forceinline__ float pow_signed(float a, float e, float power_of_magnitude) {
    if (__builtin_amdgcn_ballot_w64(a < 0.0f) != 0) return pow_sign_of(a, e) * power_of_magnitude;
    return power_of_magnitude;
}
__device__ __forceinline__ double pow_signed(float a, float e, double power_of_magnitude) {
    if (__builtin_amdgcn_ballot_w64(a < 0.0f) != 0) return (double)pow_sign_of(a, e) * power_of_magnitude;
    return power_of_magnitude;
}
__device__ __forceinline__ float pow_ref(float a, float b) {
    if (b == 2.0f) return a * a;
    if (b == 1.0f) return a;
    if (b == 0.0f) return 1.0f;
    if (b != b || (::fabsf(a) == 1.0f && ::isinf(b))) return __builtin_nanf("");
    if (a != 0.0f && ::fabsf(a) < __builtin_inff() && ::fabsf(b) < __builtin_inff()) return pow_signed(a, b, pow_positive(::fabsf(a), b));
    return ::powf(a, b);
}
__device__ __forceinline__ double dpow_da_ref(double a, double b) { return b * pow_double(a, b - 1); }
// (exponents 0, 1 and 2 have exact answers in pow_double; everything that is not a positive finite base with a finite
// exponent -- signs, zeros, infinities, NaN -- keeps the library routine behind Math.pow's special cases)
__device__ __forceinline__ bool pow_is_plain(float a, float e) {
    return a > 0.0f && a < __builtin_inff() && ::fabsf(e) < __builtin_inff() && e != 0.0f && e != 1.0f && e != 2.0f;
}
__device__ __forceinline__ float dpow_da_ref(float a, float b) {
    const float e = b - 1.0f;
    if (pow_is_plain(::fabsf(a), e)) return (float)((double)b * pow_signed(a, e, pow_from_log2(log2_of_positive(::fabsf(a)), (double)e)));
    return (float)((double)b * pow_double((double)a, (double)e));
}
// the broadcast twin multiplies by a, not by b (implementations/broadcast/CPUBroadcastPower.java:20-21)
__device__ __forceinline__ double bcast_dpow_da_ref(double a, double b) { return a * pow_double(a, b - 1); }
__device__ __forceinline__ float bcast_dpow_da_ref(float a, float b) {
    const float e = b - 1.0f;
    if (pow_is_plain(::fabsf(a), e)) return (float)((double)a * pow_signed(a, e, pow_from_log2(log2_of_positive(::fabsf(a)), (double)e)));
    return (float)((double)a * pow_double((double)a, (double)e));
}
__device__ __forceinline__ double dpow_db_ref(double a, double b) { return pow_double(a, b) * ::log(a); }
__device__ __forceinline__ float dpow_db_ref(float a, float b) {
    if (a < 0.0f) return __builtin_nanf("");                     // the logarithm of a negative base is NaN, and so is the product
    if (a > 0.0f && a < __builtin_inff() && ::fabsf(b) < __builtin_inff()) {      // one logarithm serves the power and the factor ln a
        const double l2 = log2_of_positive(a);
        double p = pow_from_log2(l2, (double)b);
        p = b == 2.0f ? (double)a * (double)a : p;               // the exponents Math.pow answers exactly (pow_double)
        p = b == 1.0f ? (double)a : p;
        p = b == 0.0f ? 1.0 : p;
        return (float)(p * (l2 * 0.69314718055994531));
    }
    return (float)(pow_double((double)a, (double)b) * ::log((double)a));
}
// x^(2/3) as the derivative of the cube root takes it: (T) Math.pow(x, (T) (2/3)) (fun/ScalarCbrt.java:31-32)
// Math.pow's answers off the positive finite numbers, for an exponent that is positive and no whole number: NaN below
// zero, +0 for both zeros, +infinity for both infinities, NaN for NaN -- spelled out, so that a tensor of mixed sign
// does not take every wavefront through the general routine.
// f64: the square of the cube root; the exponent 2.0 / 3.0 lies 3.7e-17 below 2/3, so the two differ by that times
// |ln x| < 745, relatively: 3e-14 at the ends of the range, against the 1e-12 the JDK's unspecified pow leaves room for.
__device__ __forceinline__ double cbrt_squared_ref(double x) {
    if (x > 0.0 && x < (double)__builtin_inff()) { const double c = ::cbrt(x); return c * c; }
    if (x < 0.0 && x > -(double)__builtin_inff()) return __builtin_nan("");
    return x == 0.0 ? 0.0 : ::fabs(x);
}
__device__ __forceinline__ float cbrt_squared_ref(float x) {
    // (as branches: the same with selects over an unconditional power of |x| measured slower, 71 against 60 us for 2^25
    // elements of mixed sign)
    const double e = (double)(2.0f / 3.0f);
    if (x > 0.0f && x < __builtin_inff()) return (float)pow_from_log2(log2_of_positive(x), e);
    if (x < 0.0f && x > -__builtin_inff()) return __builtin_nanf("");
    return x == 0.0f ? 0.0f : ::fabsf(x);
}
__device__ __forceinline__ double ddiv_db_ref(double a, double b) { return -(a / (b * b)); }
__device__ __forceinline__ float ddiv_db_ref(float a, float b) { return (float)-((double)a / ((double)b * (double)b)); }   // b*b is exact in double

// FunUtil.invSqrt (fun/FunUtil.java:5-27): the bit-trick inverse square root with 4 (double) or 2
// (float) Newton steps, transcribed operation for operation.
__device__ __forceinline__ double inv_sqrt_ref(double x) {
    double xhalf = 0.5 * x;
    long long i = __double_as_longlong(x);
    i = 0x5fe6ec85e7de30daLL - (i >> 1);
    x = __longlong_as_double(i);
    x *= (1.5 - xhalf * x * x);
    x *= (1.5 - xhalf * x * x);
    x *= (1.5 - xhalf * x * x);
    x *= (1.5 - xhalf * x * x);
    return x;
}
__device__ __forceinline__ float inv_sqrt_ref(float x) {
    float xhalf = 0.5f * x;
    int i = __float_as_int(x);
    i = 0x5f3759df - (i >> 1);
    x = __int_as_float(i);
    x *= (1.5f - xhalf * x * x);
    x *= (1.5f - xhalf * x * x);
    return x;
}

// ScalarSigmoid.sig (fun/ScalarSigmoid.java:38): 1/(1+exp(-x)).
__device__ __forceinline__ double sigmoid(double x) { return 1.0 / (1.0 + ::exp(-x)); }
// f32 building blocks for the two activations of the bandwidth-critical chain (sig, tanh): the
// hardware exp2 and reciprocal (about 1 ulp each).  exp(-t) = exp2(-t * log2 e); the rounding of that product
// alone would enter the result as a relative error of t * 2^-24 (5e-6 at t = 87), so the product is carried in two
// floats -- p and what p lacks -- and the small part is applied to the result to first order.  `dt` is a
// correction of the argument the caller already knows (the rounding of x * 1.702 in gelu), 0 otherwise.
// The results stay within a few ulp of the reference's (float) f((double) x) wherever they are not saturated, and
// within 1.3e-6 relative at the far ends (|x| towards 87).
template <bool WITH_DT>
__device__ __forceinline__ float fast_exp_neg_impl(float t, float dt) {           // exp(-(t + dt)) for t >= 0
    const float L = 1.44269502162933349609375f;                  // (float) log2(e); log2(e) - L = 1.9e-8 stays out: t * 1.3e-8
    t = t > 128.0f ? 128.0f : t;                                 // exp(-128) is below the smallest float; a NaN stays
    const float p = t * L;
    float lack = __builtin_fmaf(t, L, -p);                       // (relative, 1.2e-6 at t = 87) costs less than its two operations
    if constexpr (WITH_DT) lack = lack + dt * L;                 // (adding a zero is not nothing to the compiler: -0 + 0 = +0)
    const float e = __builtin_amdgcn_exp2f(-p);
    return __builtin_fmaf(e * -0.693147182464599609375f, lack, e);               // e * 2^-lack
}
__device__ __forceinline__ float fast_exp_neg(float t, float dt) { return fast_exp_neg_impl<true>(t, dt); }
__device__ __forceinline__ float fast_exp_neg(float t) { return fast_exp_neg_impl<false>(t, 0.0f); }
// f32: the same quantity as the reference's double evaluation, evaluated on e = exp(-|x|) <= 1 so
// nothing overflows: x >= 0 -> 1/(1+e), x < 0 -> e/(1+e).  `dx` as above: sigmoid(x + dx).
__device__ __forceinline__ float sigmoid(float x, float dx) {
    const float e = fast_exp_neg(::fabsf(x), x >= 0.0f ? dx : -dx);
    const float r = __builtin_amdgcn_rcpf(1.0f + e);
    return x >= 0.0f ? r : e * r;
}
__device__ __forceinline__ float sigmoid(float x) {              // no correction of the argument: three instructions fewer
    const float e = fast_exp_neg(::fabsf(x));
    const float r = __builtin_amdgcn_rcpf(1.0f + e);
    return x >= 0.0f ? r : e * r;
}
// x * 1.702 in two floats (the reference multiplies in double: fun/ScalarGeLU.java), then the sigmoid of it
__device__ __forceinline__ float gelu_sigmoid(float x) {
    const float C = 1.70200002193450927734375f;                  // (float) 1.702
    const float y = x * C;
    const float lo = ::fabsf(y) < 1.0e30f ? __builtin_fmaf(x, C, -y) + x * -2.193450927734375e-8f : 0.0f;   // + x * (1.702 - C)
    return sigmoid(y, lo);
}
__device__ __forceinline__ double gelu_sigmoid(double x) { return sigmoid(x * 1.702); }

// ScalarTanh.tanh (fun/ScalarTanh.java:37-38): 2/(1+exp(-2x))-1.
__device__ __forceinline__ double tanh_ref(double x) { return 2.0 / (1.0 + ::exp(-x * 2.0)) - 1.0; }
__device__ __forceinline__ float tanh_ref(float x) {
    const float ax = ::fabsf(x);
    float r;
    if (ax < 0.125f) {                       // odd series, next term 62/2835 x^9 < 2e-10 relative here
        const float x2 = ax * ax;
        // (an approximation of this library, not one of the reference's float formulas: fused multiply-adds are free to use)
        const float poly = __builtin_fmaf(x2, __builtin_fmaf(x2, __builtin_fmaf(x2, -0.0539682540f, 0.133333333f), -0.333333333f), 1.0f);
        r = ax * poly;
    } else {
        // (1 - e)/(1 + e) with 1 - e >= 0.22: no cancellation, and an error of e enters the quotient scaled by 2e, so
        // the plain exp2 (relative error of e: 2|x| * 4e-8, at most 3e-8 in the quotient) needs no correction here
        const float e = __builtin_amdgcn_exp2f(-2.88539008177792682f * ax);
        r = (1.0f - e) * __builtin_amdgcn_rcpf(1.0f + e);
    }
    return ::copysignf(r, x);
}

// 1 - tanh(x)^2 (ScalarTanh derivative, fun/ScalarTanh.java:31-34)
__device__ __forceinline__ double dtanh_ref(double x) { double t = tanh_ref(x); return 1.0 - t * t; }
__device__ __forceinline__ float dtanh_ref(float x) {
    float e = ::expf(-2.0f * ::fabsf(x));       // sech^2 = 4e/(1+e)^2, no cancellation for large |x|
    float s = 1.0f + e;
    return 4.0f * e / (s * s);
}

template <typename T>
__device__ __forceinline__ T softsign(T x) { return x / (T(1) + Num<T>::abs(x)); }

// exp(-(x*x)) (fun/ScalarGaussian.java).  f32 carries the rounding error of x*x into the result so
// that it matches the reference's double evaluation to f32 accuracy.
__device__ __forceinline__ double gauss(double x) { return ::exp(-(x * x)); }
__device__ __forceinline__ float gauss(float x) {
    float hi = x * x;
    float lo = ::fmaf(x, x, -hi);
    float e = ::expf(-hi);
    return e > 0.0f ? e - e * lo : e;       // e == 0 (x*x overflowed or is huge): lo may be infinite; NaN stays NaN
}

// The evaluators below work on V values at once with the switch outside the lane loop: the op-code
// is uniform over the whole grid, so the dispatch is done once per instruction, not once per value.
// NK_ONE_BY_ONE (a constant in the function that uses the macro): the elements of a thread are evaluated one after the
// other, with a scheduling barrier between them.  The double-precision library functions behind the heavy entries need
// 28-44 registers per element in flight (pow 44, log 36, sin / cos / exp 28); interleaved over the four elements of a
// thread that alone is 176 and the kernel ends at 190-256 registers, one or two wavefronts per SIMD, and is bound by
// the few bytes it keeps in flight.
#define NK_EACH(expr)                                   \
    {                                                   \
        _Pragma("unroll") for (int v = 0; v < V; v++) { \
            const T x = a[v]; (void)x;                  \
            a[v] = (expr);                              \
            if constexpr (NK_ONE_BY_ONE) __builtin_amdgcn_sched_barrier(0); \
        }                                               \
    }                                                   \
    break

template <typename T> __device__ __forceinline__ T selu_ref(T x) {
    const double ALPHA = 1.6732632423543772848170429916717, SCALE = 1.0507009873554804934193349852946;
    if (x > T(0)) return T(SCALE) * x;
    if (x <= T(0)) {
        if (sizeof(T) == 8) return T(SCALE * ALPHA * ((double)Num<T>::exp(x) - 1.0));
        return T(SCALE * ALPHA) * Num<T>::expm1(x);
    }
    return T(NAN);
}
// Derivatives are not on any bandwidth-critical path, and several of the reference's float formulas
// cancel (1 - tanh^2, s*(1-s), -t*tanh^2 + t).  To stay within tolerance of the reference's *results*,
// the f32 derivatives below repeat its float lambdas literally, including their double intermediates.
template <typename T> __device__ __forceinline__ T dselu_ref(T x) {
    const double ALPHA = 1.6732632423543772848170429916717, SCALE = 1.0507009873554804934193349852946;
    if (x > T(0)) return T(SCALE);
    if (x <= T(0)) return T(SCALE * ALPHA * exp_fast((double)x));
    return T(NAN);
}
__device__ __forceinline__ float tanh_f32_via_f64(float x) { const float t = (float)(2.0 * logistic_of_float<-2000>(x) - 1.0); return x != x ? x : t; }
__device__ __forceinline__ float sig_f32_via_f64(float x) { const float s = (float)logistic_of_float<-1000>(x); return x != x ? x : s; }
// log(1 + exp(x)) (fun/ScalarSoftplus.java:18-22).  The reference evaluates exactly this in double, and for x below
// about -16 the sum 1 + exp(x) keeps only a few bits of exp(x): its result is exp(x) rounded to a multiple of
// 2^-52 (0 or 2.2e-16 around x = -36.7).  Parity is with those results, so the f32 kernel repeats the double
// formula there; above, log1p of the float exponential agrees with it to a few ulp.
// f32 above -13: max(x, 0) + log1p(e), e = exp(-|x|) in (0, 1] -- one evaluation for both signs -- with
// log1p(e) = 2 atanh(s), s = e / (2 + e) <= 1/3, as the odd series up to s^13 (the next term is 1.3e-8 relative at s = 1/3);
// e from the hardware exp2 with its argument's rounding error carried along (1.3e-6 relative at the far end).
__device__ __forceinline__ float softplus_f32(float x) {
    const float e = fast_exp_neg(::fabsf(x));
    const float s = e * __builtin_amdgcn_rcpf(2.0f + e);
    const float s2 = s * s;
    float p = 0.0769230798f;                                     // 1/13, 1/11, ... 1/3
    p = __builtin_fmaf(p, s2, 0.0909090936f);
    p = __builtin_fmaf(p, s2, 0.111111112f);
    p = __builtin_fmaf(p, s2, 0.142857149f);
    p = __builtin_fmaf(p, s2, 0.200000003f);
    p = __builtin_fmaf(p, s2, 0.333333343f);
    p = __builtin_fmaf(p, s2, 1.0f);
    const float r = 2.0f * s * p;
    return (x > 0.0f ? x : 0.0f) + r;                            // (a NaN arrives through r)
}
template <typename T> __device__ __forceinline__ T softplus_ref(T x) {
    using N = Num<T>;
    if constexpr (sizeof(T) == 8) return log_double(1.0 + exp_fast(x));
    else {
        if (x < T(-13)) return T(::log(1.0 + ::exp((double)x)));
        return softplus_f32(x);
    }
}
template <typename T> __device__ __forceinline__ T dgasu_ref(T x) {
    T x2 = x * x, x6 = x2 * x2 * x2;
    return T(3) * x2 / (T(2) * x2 * Num<T>::abs(x) + x6 + T(1));
}
template <typename T> __device__ __forceinline__ T dgatu_ref(T x) {      // fun/ScalarGaTU.java
    T x2 = x * x, x3 = x2 * x, temp = T(3) * x2;
    if constexpr (sizeof(T) == 8) { T t = tanh_ref(x3); return -temp * (t * t) + temp; }
    else { double t = (double)tanh_f32_via_f64(x3); float tanh2 = (float)(t * t); return -temp * tanh2 + temp; }
}
template <typename T> __device__ __forceinline__ T dfast_gaus_ref(T x) {
    T x2 = x * x;
    return T(-2) * x / (x2 * x2 + T(2) * x2 + T(1));
}
template <typename T> __device__ __forceinline__ T dgelu_ref(T x) {      // fun/ScalarGeLU.java
    T sig;
    if constexpr (sizeof(T) == 8) sig = sigmoid(x * 1.702); else { sig = (float)logistic_of_float<-1702>(x); sig = x != x ? x : sig; }
    T ds = sig * (T(1) - sig);
    return sig + ds * x * T(1.702);
}
template <typename T> __device__ __forceinline__ T sig_as_ref(T x) {
    if constexpr (sizeof(T) == 8) return sigmoid(x); else return sig_f32_via_f64(x);
}
template <typename T> __device__ __forceinline__ T dsig_ref(T x) { T s = sig_as_ref(x); return s * (T(1) - s); }
template <typename T> __device__ __forceinline__ T dsilu_ref(T x) { T s = sig_as_ref(x); return s + (x * s * (T(1) - s)); }
template <typename T> __device__ __forceinline__ T dtanh_as_ref(T x) {   // fun/ScalarTanh.java:31-34
    if constexpr (sizeof(T) == 8) return dtanh_ref(x);
    else { double t = (double)tanh_f32_via_f64(x); return (float)(1.0 - t * t); }
}
template <typename T> __device__ __forceinline__ T dfast_tanh_ref(T x) {
    T t1 = x * x, t2 = Num<T>::sqrt(T(1) + t1);
    return T(1) / (t1 * t2 + t2);
}

// FUNSET selects how much of the function table a kernel instantiation carries (register pressure):
//   1  the f32-cheap forward activations; 2  everything (sin/cos/log10/cbrt, all derivatives, fmod, pow).
template <typename T, int V, int FUNSET>
__device__ __forceinline__ void apply_fun(int id, T (&a)[V]) {
    using N = Num<T>;
    constexpr bool NK_ONE_BY_ONE = FUNSET >= 2;
    switch (id) {
        case NK_FUN_ABS: NK_EACH(N::abs(x));
        case NK_FUN_GASU: NK_EACH(softsign(x * x * x));
        case NK_FUN_GATU: NK_EACH(tanh_ref(x * x * x));
        case NK_FUN_GAUS: NK_EACH(gauss(x));
        case NK_FUN_FAST_GAUS: NK_EACH(T(1) / (T(1) + x * x));
        case NK_FUN_GELU: NK_EACH(x * gelu_sigmoid(x));
        case NK_FUN_IDY: break;
        case NK_FUN_LN: NK_EACH(N::log(x));
        case NK_FUN_QUAD: NK_EACH(x * x);
        case NK_FUN_RELU: NK_EACH(x >= T(0) ? x : x * T(.01));
        case NK_FUN_SELU: NK_EACH(selu_ref(x));
        case NK_FUN_SIG: NK_EACH(sigmoid(x));
        case NK_FUN_SILU: NK_EACH(x * sigmoid(x));
        case NK_FUN_SOFTSIGN: NK_EACH(softsign(x));
        case NK_FUN_TANH: NK_EACH(tanh_ref(x));
        case NK_FUN_FAST_TANH: NK_EACH(x * inv_sqrt_ref(T(1) + x * x));
        case NK_FUN_EXP: NK_EACH(N::exp(x));
        case NK_FUN_SQRT: NK_EACH(N::sqrt(x));
        default:
            if constexpr (FUNSET >= 2) {
                switch (id) {
                    case NK_FUN_SOFTPLUS: NK_EACH(softplus_ref(x));
                    case NK_FUN_COS: NK_EACH(N::cos(x));
                    case NK_FUN_SIN: NK_EACH(N::sin(x));
                    case NK_FUN_LOG10: NK_EACH(N::log10(x));
                    case NK_FUN_CBRT: NK_EACH(N::cbrt(x));
                    default: NK_EACH(T(NAN) + x);
                }
            } else NK_EACH(T(NAN) + x);
    }
}

// does function `id` need the full table?
constexpr bool fun_is_heavy(int id) { return id == NK_FUN_COS || id == NK_FUN_SIN || id == NK_FUN_LOG10 || id == NK_FUN_CBRT || id == NK_FUN_SOFTPLUS; }

// derivatives that call a double-precision routine of the device library (registers: evaluated one element at a time)
constexpr bool dfun_calls_library(int id) { return id == NK_FUN_COS || id == NK_FUN_SIN || id == NK_FUN_CBRT || id == NK_FUN_GASU || id == NK_FUN_GATU; }

template <typename T, int V, bool ONE_BY_ONE = true>
__device__ __forceinline__ void apply_dfun(int id, T (&a)[V]) {
    using N = Num<T>;
    constexpr bool NK_ONE_BY_ONE = ONE_BY_ONE;
    switch (id) {
        case NK_FUN_ABS: NK_EACH(x < T(0) ? T(-1) : T(1));
        case NK_FUN_COS: NK_EACH(sizeof(T) == 8 ? T(-::sin((double)x)) : T(-N::sin(x)));      // (nothing cancels: the float routine, 2 ulp, serves f32)
        case NK_FUN_GASU: NK_EACH(dgasu_ref(x));
        case NK_FUN_GATU: NK_EACH(dgatu_ref(x));
        case NK_FUN_GAUS: NK_EACH(T(-2.0 * (double)x * exp_fast(-((double)x * (double)x))));
        case NK_FUN_FAST_GAUS: NK_EACH(dfast_gaus_ref(x));
        case NK_FUN_GELU: NK_EACH(dgelu_ref(x));
        case NK_FUN_IDY: NK_EACH(T(1));
        case NK_FUN_LN: NK_EACH(T(1) / x);
        case NK_FUN_QUAD: NK_EACH(T(2) * x);
        case NK_FUN_RELU: NK_EACH(x >= T(0) ? T(1) : T(.01));
        case NK_FUN_SELU: NK_EACH(dselu_ref(x));
        case NK_FUN_SIG: NK_EACH(dsig_ref(x));
        case NK_FUN_SILU: NK_EACH(dsilu_ref(x));
        case NK_FUN_SIN: NK_EACH(sizeof(T) == 8 ? T(::cos((double)x)) : T(N::cos(x)));
        case NK_FUN_SOFTPLUS: NK_EACH(sig_as_ref(x));                   // the logistic function itself
        case NK_FUN_SOFTSIGN: NK_EACH(T(1) / (T(2) * N::abs(x) + x * x + T(1)));
        case NK_FUN_TANH: NK_EACH(dtanh_as_ref(x));
        case NK_FUN_FAST_TANH: NK_EACH(dfast_tanh_ref(x));
        case NK_FUN_EXP: NK_EACH(T(exp_fast((double)x)));
        case NK_FUN_LOG10: NK_EACH(T(1) / (x * T(2.302585092994046)));   // x * ln(10)
        case NK_FUN_SQRT: NK_EACH(T(0.5) * inv_sqrt_ref(x));
        case NK_FUN_CBRT: NK_EACH(T(1) / (T(3) * cbrt_squared_ref(x)));
        default: NK_EACH(T(NAN) + x);
    }
}
#undef NK_EACH

// binary operators: CPUBiElementWise*.java / CPUBroadcast*.java (_getFun).  a = a op b.
#define NK_EACH2(expr)                                  \
    {                                                   \
        _Pragma("unroll") for (int v = 0; v < V; v++) { \
            const T x = a[v], y = b[v]; (void)x; (void)y; \
            a[v] = (expr);                              \
            if constexpr (NK_ONE_BY_ONE) __builtin_amdgcn_sched_barrier(0); \
        }                                               \
    }                                                   \
    break

template <typename T, int V, int FUNSET, bool ONE_BY_ONE = (FUNSET >= 2)>
__device__ __forceinline__ void apply_bin(int op, T (&a)[V], const T (&b)[V]) {
    using N = Num<T>;
    constexpr bool NK_ONE_BY_ONE = ONE_BY_ONE;
    switch (op) {
        case NK_OP_ADD: NK_EACH2(x + y);
        case NK_OP_SUB: NK_EACH2(x - y);
        case NK_OP_MUL: NK_EACH2(x * y);
        case NK_OP_DIV: NK_EACH2(x / y);
        case NK_OP_IDY: NK_EACH2(y);
        default:
            if constexpr (FUNSET >= 2) {
                switch (op) {
                    case NK_OP_MOD: NK_EACH2(N::fmod(x, y));     // Java's % on floating point is C's fmod
                    case NK_OP_POW: NK_EACH2(pow_ref(x, y));
                    default: NK_EACH2(T(NAN) + x + y);
                }
            } else NK_EACH2(T(NAN) + x + y);
    }
}
constexpr bool bin_is_heavy(int op) { return op == NK_OP_MOD || op == NK_OP_POW; }

// partial derivatives: CPUBiElementWise*.java (_getDeriveAt0 / _getDeriveAt1).  a = d(a op b)/d(operand d).
template <typename T, int V, int FUNSET, bool ONE_BY_ONE = (FUNSET >= 2)>
__device__ __forceinline__ void apply_dbin(int op, int d, T (&a)[V], const T (&b)[V]) {
    using N = Num<T>;
    constexpr bool NK_ONE_BY_ONE = ONE_BY_ONE;
    switch (op * 2 + d) {
        case NK_OP_ADD * 2 + 0:
        case NK_OP_ADD * 2 + 1:
        case NK_OP_SUB * 2 + 0: NK_EACH2(T(1));
        case NK_OP_SUB * 2 + 1: NK_EACH2(T(-1));
        case NK_OP_MUL * 2 + 0: NK_EACH2(y);
        case NK_OP_MUL * 2 + 1: NK_EACH2(x);
        case NK_OP_IDY * 2 + 0:
        case NK_OP_IDY * 2 + 1: NK_EACH2(y);      // CPUScalarBroadcastIdentity.java:25-33: both derivatives are the function itself
        default:
            if constexpr (FUNSET >= 2) {
                switch (op * 2 + d) {
                    case NK_OP_DIV * 2 + 0:
                    case NK_OP_MOD * 2 + 0: NK_EACH2(T(1) / y);
                    case NK_OP_DIV * 2 + 1:
                    case NK_OP_MOD * 2 + 1: NK_EACH2(ddiv_db_ref(x, y));
                    case NK_OP_POW * 2 + 0: NK_EACH2(dpow_da_ref(x, y));
                    case NK_OP_POW * 2 + 1: NK_EACH2(dpow_db_ref(x, y));
                    default: NK_EACH2(T(NAN) + x + y);
                }
            } else NK_EACH2(T(NAN) + x + y);
    }
}
constexpr bool dbin_is_heavy(int op) { return op == NK_OP_DIV || op == NK_OP_MOD || op == NK_OP_POW; }
#undef NK_EACH2

}  // namespace nk
