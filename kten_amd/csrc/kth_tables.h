// Table-driven exp and log for the "f64 libm, round once to f32" rule of kotlin.math
// (JVMRawTensor.kt:144,395,399). Both evaluate in f64 to about 1e-16 relative error, so
// after the single rounding to fp32 they return the correctly rounded float for all but a
// vanishing fraction of inputs, while costing about twenty f64 operations, which keeps
// the elementwise kernels HBM-bound. The tables are computed on the host in extended
// precision when the library is initialised and read through LDS.
//
//   log: x = z * 2^k with z in [0.6875, 1.375); the top 7 mantissa bits of z pick a
//        centre c with invc ~ 1/c and logc = -log(invc); r = z * invc - 1 (one fma, so
//        exact up to its own rounding), |r| < 2^-7;
//        log x = k ln2 + logc + log1p(r), log1p by its Taylor series to r^7.
//        The interval starting at 1.0 has invc = 1, logc = 0: no cancellation near 1.
//   exp: k = round(x * 128 / ln2), r = x - k ln2 / 128 (two fmas with a split constant),
//        |r| <= ln2 / 256; e^x = 2^(k >> 7) * T[k & 127] * e^r, T[i] = 2^(i/128),
//        e^r by its Taylor series to r^6, scaling by ldexp (handles overflow to inf and
//        gradual underflow).
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

namespace kth {

constexpr int kLogTableEntries = 128;     // {invc, logc} pairs
constexpr int kExpTableEntries = 128;
constexpr int kAtanTableEntries = 65;     // atan(i / 64), i = 0..64

struct LogEntry { double invc, logc; };

constexpr uint64_t kLogOff = 0x3fe6000000000000ull;   // 0.6875

// log of a positive finite double (normal), to about 1e-16 relative.
__device__ __forceinline__ double table_log_d(double d, const LogEntry* tab) {
    const uint64_t ix = static_cast<uint64_t>(__double_as_longlong(d));
    const uint64_t tmp = ix - kLogOff;
    const int i = static_cast<int>(tmp >> 45) & (kLogTableEntries - 1);
    const int k = static_cast<int>(static_cast<int64_t>(tmp) >> 52);
    const double z = __longlong_as_double(static_cast<long long>(ix - (tmp & 0xfff0000000000000ull)));
    const LogEntry e = tab[i];
    const double r = fma(z, e.invc, -1.0);
    double p = fma(r, 1.0 / 7.0, -1.0 / 6.0);
    p = fma(r, p, 1.0 / 5.0);
    p = fma(r, p, -1.0 / 4.0);
    p = fma(r, p, 1.0 / 3.0);
    p = fma(r, p, -1.0 / 2.0);
    const double l1p = fma(r * r, p, r);
    return fma(static_cast<double>(k), 0.693147180559945309417232121458, e.logc) + l1p;
}

__device__ __forceinline__ float table_log(float x, const LogEntry* tab) {
    // The conversion is exact; fp32 denormals become normal doubles.
    float res = static_cast<float>(table_log_d(static_cast<double>(x), tab));
    // Math.log: NaN or negative -> NaN, +-0 -> -inf, +inf -> +inf.
    if (x == 0.0f) res = -INFINITY;
    if (x < 0.0f) res = __uint_as_float(0x7fc00000u);
    if (!(x < INFINITY)) res = x;                            // +inf and NaN pass through
    return res;
}

// e^d for d in [-120, 100], to about 1e-16 relative.
__device__ __forceinline__ double table_exp_d(double d, const double* tab) {
    const double kd = rint(d * 184.664965233787316142070359168242182);   // 128 / ln2
    const int k = static_cast<int>(kd);
    // ln2 / 128 split so that kd * hi is exact for |kd| < 2^16.
    double r = fma(kd, -0x1.62e42fefa0000p-8, d);
    r = fma(kd, -0x1.cf79abc9e3b3ap-47, r);
    const double s = tab[k & (kExpTableEntries - 1)];
    double p = fma(r, 1.0 / 720.0, 1.0 / 120.0);
    p = fma(r, p, 1.0 / 24.0);
    p = fma(r, p, 1.0 / 6.0);
    p = fma(r, p, 0.5);
    p = fma(r * r, p, r);                                    // e^r - 1
    return ldexp(fma(s, p, s), k >> 7);
}

__device__ __forceinline__ float table_exp(float x, const double* tab) {
    // Outside [-120, 100] the fp32 result is already 0 or inf; clamping keeps k in int range.
    float res = static_cast<float>(table_exp_d(fmin(fmax(static_cast<double>(x), -120.0), 100.0), tab));
    if (x != x) res = x;
    return res;
}

// 1 / d for d in [1, 1e45]: the hardware estimate and two Newton steps (error about 1e-16
// relative), without the scaling and fix-up code of an IEEE division.
__device__ __forceinline__ double newton_rcp(double d) {
    double r = __builtin_amdgcn_rcp(d);
    r = fma(fma(-d, r, 1.0), r, r);
    r = fma(fma(-d, r, 1.0), r, r);
    return r;
}

// tanh, sinh, cosh from t = e^|x| (Math.tanh / sinh / cosh of the double, rounded once).
// Below 2^-5 the odd functions use their Taylor series, so nothing cancels; above it the
// differences t - 1/t and t^2 - 1 lose at most five bits of the 53.
__device__ __forceinline__ float table_tanh(float x, const double* tab) {
    const double a = fabs(static_cast<double>(x));
    double y;
    if (a < 0.03125) {
        const double z = a * a;
        double p = fma(z, -1382.0 / 155925.0, 62.0 / 2835.0);
        p = fma(z, p, -17.0 / 315.0);
        p = fma(z, p, 2.0 / 15.0);
        p = fma(z, p, -1.0 / 3.0);
        y = fma(a * z, p, a);
    } else {
        const double t = table_exp_d(2.0 * fmin(a, 20.0), tab);     // tanh(20) rounds to 1 in f64 already
        y = (t - 1.0) * newton_rcp(t + 1.0);
    }
    float res = copysignf(static_cast<float>(y), x);
    if (x != x) res = x;
    return res;
}

__device__ __forceinline__ float table_sinh(float x, const double* tab) {
    const double a = fabs(static_cast<double>(x));
    double y;
    if (a < 0.03125) {
        const double z = a * a;
        double p = fma(z, 1.0 / 362880.0, 1.0 / 5040.0);
        p = fma(z, p, 1.0 / 120.0);
        p = fma(z, p, 1.0 / 6.0);
        y = fma(a * z, p, a);
    } else {
        const double t = table_exp_d(fmin(a, 100.0), tab);          // e^100 / 2 is beyond fp32: rounds to inf
        y = 0.5 * (t - newton_rcp(t));
    }
    float res = copysignf(static_cast<float>(y), x);
    if (x != x) res = x;
    return res;
}

__device__ __forceinline__ float table_cosh(float x, const double* tab) {
    const double t = table_exp_d(fmin(fabs(static_cast<double>(x)), 100.0), tab);
    float res = static_cast<float>(0.5 * (t + newton_rcp(t)));
    if (x != x) res = x;
    return res;
}

// Math.pow(double, double) rounded to float, for the operands the tables cover: a finite
// base other than 0 and a finite exponent. |a|^b = e^(b ln|a|); the error of b ln|a| is at
// most about 2e-14 absolute, i.e. the result is within 2e-14 relative of the exact power
// before the rounding to fp32. A negative base takes the sign of an odd integer exponent and
// gives NaN for a non-integer one (Java and C agree on these).
__device__ __forceinline__ float table_pow_finite(float a, float b, const LogEntry* log_tab, const double* exp_tab) {
    const double l = table_log_d(fabs(static_cast<double>(a)), log_tab);
    const double y = table_exp_d(fmin(fmax(static_cast<double>(b) * l, -120.0), 100.0), exp_tab);
    float res = static_cast<float>(y);
    if (a < 0.0f) {
        const float t = truncf(b);
        if (t != b) return __uint_as_float(0x7fc00000u);
        // odd integer: |b| < 2^24 and its lowest bit set (larger floats are all even)
        if (fabsf(b) < 16777216.0f && (static_cast<int>(fabsf(b)) & 1)) res = -res;
    }
    return res;
}

// ---------------------------------------------------------------- sin / cos / tan

// Arguments up to 1e6 in magnitude are reduced in f64 by k = round(x * 2/pi) and
// r = x - k * pi/2 with pi/2 split into 33 + 33 + 53 bits (k p1 and k p2 are exact products, the
// subtractions of nearly equal values are exact), so r is good to about 1e-16 relative even
// when x is the float closest to a multiple of pi/2. sin r and cos r on [-pi/4, pi/4] come from
// their Taylor series (to r^17 and r^16: truncation below 1e-18). Larger arguments need a
// multi-word reduction and take the library routine.
constexpr double kTrigFastLimit = 1.0e6;

__device__ __forceinline__ void sincos_reduced(double x, double& s, double& c, int& k) {
    const double kd = rint(x * 0x1.45f306dc9c883p-1);
    k = static_cast<int>(kd);
    double r = fma(kd, -0x1.921fb54400000p+0, x);
    r = fma(kd, -0x1.0b4611a600000p-34, r);
    r = fma(kd, -0x1.3198a2e037073p-69, r);
    if (kd == 0.0) r = x;                                    // keeps the sign of -0
    const double z = r * r;
    double p = fma(z, 1.0 / 355687428096000.0, -1.0 / 1307674368000.0);
    p = fma(z, p, 1.0 / 6227020800.0);
    p = fma(z, p, -1.0 / 39916800.0);
    p = fma(z, p, 1.0 / 362880.0);
    p = fma(z, p, -1.0 / 5040.0);
    p = fma(z, p, 1.0 / 120.0);
    p = fma(z, p, -1.0 / 6.0);
    s = fma(r * z, p, r);
    double q = fma(z, 1.0 / 20922789888000.0, -1.0 / 87178291200.0);
    q = fma(z, q, 1.0 / 479001600.0);
    q = fma(z, q, -1.0 / 3628800.0);
    q = fma(z, q, 1.0 / 40320.0);
    q = fma(z, q, -1.0 / 720.0);
    q = fma(z, q, 1.0 / 24.0);
    c = fma(z * z, q, fma(z, -0.5, 1.0));
}

// 1 / d for any normal d whose reciprocal is normal: hardware estimate and two Newton steps.
__device__ __forceinline__ double newton_rcp_any(double d) {
    double r = __builtin_amdgcn_rcp(d);
    r = fma(fma(-d, r, 1.0), r, r);
    r = fma(fma(-d, r, 1.0), r, r);
    return r;
}

__device__ __forceinline__ float table_sin(float x) {
    const double d = static_cast<double>(x);
    if (!(fabs(d) <= kTrigFastLimit)) return static_cast<float>(sin(d));      // large, inf (-> NaN), NaN
    double s, c; int k;
    sincos_reduced(d, s, c, k);
    const double y = (k & 1) ? c : s;
    return static_cast<float>((k & 2) ? -y : y);
}

__device__ __forceinline__ float table_cos(float x) {
    const double d = static_cast<double>(x);
    if (!(fabs(d) <= kTrigFastLimit)) return static_cast<float>(cos(d));
    double s, c; int k;
    sincos_reduced(d, s, c, k);
    const double y = (k & 1) ? s : c;
    return static_cast<float>(((k + 1) & 2) ? -y : y);
}

__device__ __forceinline__ float table_tan(float x) {
    const double d = static_cast<double>(x);
    if (!(fabs(d) <= kTrigFastLimit)) return static_cast<float>(tan(d));
    double s, c; int k;
    sincos_reduced(d, s, c, k);
    // cos r >= 0.7 on the reduced range; sin r of an odd quadrant is at least 1e-9 for a float argument
    const bool odd = (k & 1) != 0;                               // one reciprocal for either quadrant
    return static_cast<float>((odd ? -c : s) * newton_rcp_any(odd ? s : c));
}

// ---------------------------------------------------------------- atan / asin / acos

// atan of a in [0, 1]: c = round(64 a) / 64, t = (a - c) / (1 + a c), atan a = atan c + atan t
// with |t| <= 1/128, atan t by its Taylor series to t^9 (next term below 2^-77).
__device__ __forceinline__ double atan_unit(double a, const double* tab) {
    const double id = rint(a * 64.0);
    const double c = id * 0.015625;
    const double t = (a - c) * newton_rcp_any(fma(a, c, 1.0));
    const double z = t * t;
    double p = fma(z, 1.0 / 9.0, -1.0 / 7.0);
    p = fma(z, p, 1.0 / 5.0);
    p = fma(z, p, -1.0 / 3.0);
    return tab[static_cast<int>(id)] + fma(t * z, p, t);
}

// atan(num / den) for 0 <= num <= den, den in [1, 1e300], without forming the quotient: with u = num / den the
// same t is (num - c den) / (den + num c), so the division by den and the one inside atan_unit become one.
// c only has to be near u: the hardware's reciprocal estimate picks it.
__device__ __forceinline__ double atan_ratio(double num, double den, const double* tab) {
    const double id = rint(num * __builtin_amdgcn_rcp(den) * 64.0);
    const double c = id * 0.015625;
    const double t = fma(-c, den, num) * newton_rcp_any(fma(num, c, den));
    const double z = t * t;
    double p = fma(z, 1.0 / 9.0, -1.0 / 7.0);
    p = fma(z, p, 1.0 / 5.0);
    p = fma(z, p, -1.0 / 3.0);
    return tab[static_cast<int>(id)] + fma(t * z, p, t);
}

constexpr double kPio2Hi = 0x1.921fb54442d18p+0, kPio2Lo = 0x1.1a62633145c07p-54;

// atan of a >= 0 (finite or inf).
__device__ __forceinline__ double atan_positive(double a, const double* tab) {
    if (a <= 1.0) return atan_unit(a, tab);
    const double small = a > 1.0e300 ? 0.0 : atan_ratio(1.0, a, tab);
    return (kPio2Hi - small) + kPio2Lo;
}

__device__ __forceinline__ float table_atan(float x, const double* tab) {
    float res = copysignf(static_cast<float>(atan_positive(fabs(static_cast<double>(x)), tab)), x);
    if (x != x) res = x;
    return res;
}

// 1 / sqrt(w) for w in [2^-30, 2]: the hardware estimate and two Newton steps on the residual 1 - w y^2.
__device__ __forceinline__ double newton_rsqrt_unit(double w) {
    double y = __builtin_amdgcn_rsq(w);
    double e = fma(-w * y, y, 1.0);
    y = fma(y * e, 0.5, y);
    e = fma(-w * y, y, 1.0);
    return fma(y * e, 0.5, y);
}

// asin a = 2 atan(a / (1 + sqrt((1 - a)(1 + a)))) on [0, 1]; NaN outside [-1, 1] (Math.asin).
__device__ __forceinline__ float table_asin(float x, const double* tab) {
    const double a = fabs(static_cast<double>(x));
    if (!(a <= 1.0)) return __uint_as_float(0x7fc00000u);
    const double w = (1.0 - a) * (1.0 + a);
    const double root = w > 0.0 ? w * newton_rsqrt_unit(w) : 0.0;       // sqrt(w)
    return copysignf(static_cast<float>(2.0 * atan_ratio(a, 1.0 + root, tab)), x);
}

// acos x = 2 atan(sqrt((1 - x) / (1 + x))) on (-1, 1], pi at -1; NaN outside [-1, 1] (Math.acos).
// acos |x| = 2 atan(sqrt((1 - |x|) / (1 + |x|))), whose argument stays in [0, 1]; acos x = pi - acos |x| below zero.
__device__ __forceinline__ float table_acos(float x, const double* tab) {
    const double d = static_cast<double>(x);
    const double a = fabs(d);
    if (!(a <= 1.0)) return __uint_as_float(0x7fc00000u);
    // sqrt((1 - a) / (1 + a)) = (1 - a) / sqrt((1 - a)(1 + a)); both factors are exact for a float a >= 2^-29
    const double w = (1.0 - a) * (1.0 + a);
    const double root = w > 0.0 ? (1.0 - a) * newton_rsqrt_unit(w) : 0.0;
    const double r = 2.0 * atan_unit(root, tab);
    return static_cast<float>(d < 0.0 ? (2.0 * kPio2Hi - r) + 2.0 * kPio2Lo : r);
}

}  // namespace kth
