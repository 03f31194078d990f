// Short f64 evaluations of the transcendental maps, each good to better than 2^-44 relative,
// and the test that tells whether such a value already fixes the float it rounds to.
//
// kotlin.math's Float overloads are "f64 libm, round once to f32" (JVMRawTensor.kt:395-425).
// The routines of kth_tables.h reproduce that with about 1e-16 relative error, which costs
// 50-65 vector instructions per element, among them quarter-rate f64 reciprocals with two
// Newton steps: the maps were bound by arithmetic, not by memory. A value known to 2^-44
// decides the rounding to fp32 unless it lies within that distance of the midpoint of two
// neighbouring floats, which happens for about one input in 30 000. So every map first takes
// the short evaluation below; rounds_safely() tells the lanes whose result is decided, and the
// others (and inputs outside the short routine's domain: NaN, huge arguments, results in the
// fp32 denormal range) take the long routine. Whatever path a lane takes, it returns the float
// that the exact result rounds to, so the two paths cannot disagree where both apply.
//
// Measured on gfx950 (wave64, cycles per wave instruction per SIMD): f64 fma / add / mul / min /
// rndne / ldexp / cvt about 4.5-5.3, f32 fma and 32-bit integer ops 2.6, v_rcp_f64 and v_rsq_f64 17
// (relative error 2^-24.4 and 2^-24.2; after one Newton step 2^-48.7 and 2^-47.7), v_rcp_f32 8.7.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

#include "kth_tables.h"

namespace kth {

constexpr int kSinCosTableEntries = 64;   // {sin, cos}(j pi / 32), j = 0..63
constexpr int kAsinTableEntries = 47;     // {asin c, sqrt(1 - c^2)}, c = j / 64, j = 0..46

// Half-width, in units of the last place of the f64 value, of the band around the midpoint of two
// neighbouring floats inside which a value of relative error up to 2^-41 does not decide its rounding:
// 2^13 ulps of 2^-52 are 2^-39 of the value's binade, at least 2^-40 of the value.
constexpr uint32_t kTieBand = 1u << 13;

// True when the float nearest to y is also the float nearest to every value within 2^-41 relative of y:
// y is not in the band around a rounding midpoint and |y| is in the fp32 normal range (or exactly 0).
__device__ __forceinline__ bool rounds_safely(double y) {
    const uint32_t lo = static_cast<uint32_t>(__double2loint(y));
    const uint32_t mag = static_cast<uint32_t>(__double2hiint(y)) & 0x7fffffffu;
    // fp32 keeps 23 of the 52 mantissa bits: the midpoint of two floats is bit 28 set and bits 27..0 clear
    const bool near_tie = ((lo & 0x1fffffffu) - (0x10000000u - kTieBand)) < 2u * kTieBand;
    return !near_tie && (mag >= 0x38100000u || mag == 0u);       // 0x381: exponent of 2^-126
}

// 1 / d to 2^-48: hardware estimate and one Newton step.
__device__ __forceinline__ double rcp_fast(double d) {
    const double r = __builtin_amdgcn_rcp(d);
    return fma(fma(-d, r, 1.0), r, r);
}

// e^d = S (1 + p) for d in [-120, 100]: S = 2^(k / 128) from the table, scaled exactly; p = e^r - 1 by its
// Taylor series to r^5 (|r| <= ln2 / 256: the next term is below 2^-52 of p).
__device__ __forceinline__ void exp_parts(double d, const double* tab, double& S, double& p) {
    const double kd = rint(d * 184.664965233787316142070359168242182);   // 128 / ln2
    const int k = static_cast<int>(kd);
    double r = fma(kd, -0x1.62e42fefa0000p-8, d);
    r = fma(kd, -0x1.cf79abc9e3b3ap-47, r);
    S = ldexp(tab[k & (kExpTableEntries - 1)], k >> 7);
    double q = fma(r, 1.0 / 120.0, 1.0 / 24.0);
    q = fma(r, q, 1.0 / 6.0);
    q = fma(r, q, 0.5);
    p = fma(r * r, q, r);
}

// tanh |x| = (t - 1) / (t + 1), t = e^(2|x|) = S (1 + p). t - 1 = S p + (S - 1) has no cancellation: S - 1 is
// exact, it is 0 when k = 0 and at least 2^(1/128) - 1 otherwise.
__device__ __forceinline__ bool fast_tanh(float x, const double* tab, double& y) {
    const double a = fabs(static_cast<double>(x));
    double S, p;
    exp_parts(2.0 * fmin(a, 20.0), tab, S, p);
    y = fma(S, p, S - 1.0) * rcp_fast(fma(S, p, S + 1.0));
    return x == x;
}

// sinh |x| = (E + E / t) / 2 with E = t - 1 as above, t = e^|x|.
__device__ __forceinline__ bool fast_sinh(float x, const double* tab, double& y) {
    const double a = fabs(static_cast<double>(x));
    double S, p;
    exp_parts(fmin(a, 100.0), tab, S, p);
    const double E = fma(S, p, S - 1.0);
    y = 0.5 * fma(E, rcp_fast(fma(S, p, S)), E);
    return x == x;
}

__device__ __forceinline__ bool fast_cosh(float x, const double* tab, double& y) {
    const double a = fabs(static_cast<double>(x));
    double S, p;
    exp_parts(fmin(a, 100.0), tab, S, p);
    const double t = fma(S, p, S);
    y = 0.5 * (t + rcp_fast(t));
    return x == x;
}

// ---------------------------------------------------------------- sin / cos / tan

// For 0 <= a <= 65536: a = k pi/32 + r, |r| <= pi/64. pi/32 is split into 33 + 33 + 53 bits, so k p1 is an
// exact product (k < 2^20), a - k p1 is exact and each later step rounds once: r is good to 2^-52 relative
// even next to a multiple of pi/32. S = sin(k pi/32), C = cos(k pi/32) come from the table (exact 0 and +-1
// at the multiples of pi/2); sr = sin r to r^7 and cm1 = cos r - 1 to r^6 (truncation below 2^-50 absolute).
constexpr float kTrigShortLimit = 65536.0f;

__device__ __forceinline__ void trig_parts(double a, const double* tab, double& S, double& C, double& sr, double& cm1) {
    const double kd = rint(a * 0x1.45f306dc9c883p+3);             // 32 / pi
    const int k = static_cast<int>(kd);
    double r = fma(kd, -0x1.921fb54400000p-4, a);
    r = fma(kd, -0x1.0b4611a600000p-38, r);
    r = fma(kd, -0x1.3198a2e037073p-73, r);
    const double2 sc = reinterpret_cast<const double2*>(tab)[k & (kSinCosTableEntries - 1)];
    S = sc.x; C = sc.y;
    const double z = r * r;
    double p = fma(z, -1.0 / 5040.0, 1.0 / 120.0);
    p = fma(z, p, -1.0 / 6.0);
    sr = fma(r * z, p, r);
    double q = fma(z, -1.0 / 720.0, 1.0 / 24.0);
    q = fma(z, q, -0.5);
    cm1 = z * q;
}

// sin |x| (the caller restores the sign): S cos r + C sin r = S + (S cm1 + C sr).
__device__ __forceinline__ bool fast_sin(float x, const double* tab, double& y) {
    double S, C, sr, cm1;
    trig_parts(fabs(static_cast<double>(x)), tab, S, C, sr, cm1);
    y = S + fma(S, cm1, C * sr);
    return fabsf(x) <= kTrigShortLimit;
}

__device__ __forceinline__ bool fast_cos(float x, const double* tab, double& y) {
    double S, C, sr, cm1;
    trig_parts(fabs(static_cast<double>(x)), tab, S, C, sr, cm1);
    y = C + fma(C, cm1, -(S * sr));
    return fabsf(x) <= kTrigShortLimit;
}

// tan |x|: next to a pole C is exactly 0 and the cosine is -S sr, as accurate as sr.
__device__ __forceinline__ bool fast_tan(float x, const double* tab, double& y) {
    double S, C, sr, cm1;
    trig_parts(fabs(static_cast<double>(x)), tab, S, C, sr, cm1);
    const double s = S + fma(S, cm1, C * sr);
    const double c = C + fma(C, cm1, -(S * sr));
    y = s * rcp_fast(c);
    return fabsf(x) <= kTrigShortLimit;
}

// ---------------------------------------------------------------- asin / acos

// asin p for the smaller of (|x|, sqrt(1 - x^2)): with q the larger one, c = round(64 p) / 64 and the table's
// asin c and sqrt(1 - c^2), asin p = asin c + asin(p sqrt(1 - c^2) - c q): no division, and the argument d of
// the last term is at most 0.0113, asin d to d^7 (the next term is below 2^-56 of d). The root is
// w rsq(w) with one Newton step (2^-47.7). swap tells that p is the root, i.e. |x| > 1/sqrt 2.
__device__ __forceinline__ double asin_smaller(float a32, const double* tab, bool& swap) {
    const double A = static_cast<double>(a32);
    const double w = (1.0 - A) * (1.0 + A);
    const double y0 = __builtin_amdgcn_rsq(w);
    const double e = fma(-w * y0, y0, 1.0);
    const double root = w * fma(y0 * e, 0.5, y0);
    swap = a32 > 0.70710678f;
    const double p = swap ? root : A, q = swap ? A : root;
    const float idf = rintf(static_cast<float>(p) * 64.0f);
    const double c = static_cast<double>(idf * 0.015625f);
    const double2 e2 = reinterpret_cast<const double2*>(tab)[static_cast<int>(idf)];
    const double d = fma(p, e2.y, -(c * q));
    const double z = d * d;
    double s = fma(z, 15.0 / 336.0, 3.0 / 40.0);
    s = fma(z, s, 1.0 / 6.0);
    return e2.x + fma(d * z, s, d);
}

// asin |x| for |x| < 1.
__device__ __forceinline__ bool fast_asin(float x, const double* tab, double& y) {
    const float a32 = fabsf(x);
    bool swap;
    const double r = asin_smaller(a32, tab, swap);
    y = swap ? kPio2Hi - r : r;
    return a32 < 1.0f;
}

// acos x for |x| < 1: acos |x| = asin sqrt(1 - x^2) directly when that is the smaller one (no cancellation
// next to 1), pi/2 - asin |x| otherwise; pi - acos |x| below zero.
__device__ __forceinline__ bool fast_acos(float x, const double* tab, double& y) {
    const float a32 = fabsf(x);
    bool swap;
    const double r = asin_smaller(a32, tab, swap);
    const double pos = swap ? r : kPio2Hi - r;
    y = x < 0.0f ? 2.0 * kPio2Hi - pos : pos;
    return a32 < 1.0f;
}

// ---------------------------------------------------------------- pow

// a^b = 2^(b log2 a) for a finite base above zero and a finite exponent other than zero, in base 2 so that the
// reduction of the exponent function is exact: log2 a = k + log2 c + log2(1 + r) with the decomposition of
// table_log_d (z = a 2^-k in [0.6875, 1.375), c the centre of z's interval, r = z / c - 1 by one fma, |r| < 2^-7)
// and the table's {1 / c, log2 c}; log2(1 + r) by its series to r^7 (next term below 2^-56 of the value), good to
// 2^-51 also next to a = 1, where the table's interval has c = 1 and the series is all there is.
// w = b log2 a is then off by at most 1100 x 2^-51 absolute; 2^w = 2^m T[j] 2^q with 128 w = 128 m + j + 128 q
// exactly (q = w - round(128 w) / 128 is an exact difference), 2^q - 1 by its series to q^5 (|q| <= 2^-8: the
// next term is below 2^-55). The result is good to 2^-44 for |w| up to 128, beyond which it is 0 or inf anyway.
struct Log2Entry { double invc, log2c; };

// SHORT (the math mode "within 2 ulp"): log2(1 + r) to r^5 and 2^q - 1 to q^3. The logarithm is then good to 2^-37
// relative (worst next to a = 1, where log2 a itself is as small as |r|), w = b log2 a to 2^-30 absolute at |w| = 128,
// the power to 2^-30: the float it rounds to is the exact power's or its neighbour.
template <bool SHORT = false>
__device__ __forceinline__ bool fast_pow(float a, float b, const Log2Entry* log2_tab, const double* exp_tab, double& y) {
    const double d = static_cast<double>(a);
    const uint64_t ix = static_cast<uint64_t>(__double_as_longlong(d));
    const uint64_t tmp = ix - kLogOff;
    const int i = static_cast<int>(tmp >> 45) & (kLogTableEntries - 1);
    const int k = static_cast<int>(static_cast<int64_t>(tmp) >> 52);
    const double z = __longlong_as_double(static_cast<long long>(ix - (tmp & 0xfff0000000000000ull)));
    const Log2Entry e = log2_tab[i];
    const double r = fma(z, e.invc, -1.0);
    // log2(1 + r) = r (c1 + r (c2 + ...)), c_n = (-1)^(n+1) / (n ln 2)
    double p = 0x1.2776c50ef9bfep-2;                                         // 1/(5 ln2)
    if (!SHORT) {
        p = fma(r, 0x1.a61762a7aded9p-3, -0x1.ec709dc3a03fdp-3);            // 1/(7 ln2), -1/(6 ln2)
        p = fma(r, p, 0x1.2776c50ef9bfep-2);
    }
    p = fma(r, p, -0x1.71547652b82fep-2);                                    // -1/(4 ln2)
    p = fma(r, p, 0x1.ec709dc3a03fdp-2);                                     // 1/(3 ln2)
    p = fma(r, p, -0x1.71547652b82fep-1);                                    // -1/(2 ln2)
    p = fma(r, p, 0x1.71547652b82fep+0);                                     // 1/ln2
    const double t = fma(r, p, static_cast<double>(k) + e.log2c);
    const double w = fmin(fmax(static_cast<double>(b) * t, -1100.0), 1100.0);
    const double kd = rint(w * 128.0);
    const int j = static_cast<int>(kd);
    const double q = fma(kd, -0.0078125, w);
    // 2^q - 1 = q (l1 + q (l2 + ...)), l_n = ln2^n / n!
    double g = 0x1.c6b08d704a0c0p-5;                                         // ln2^3/6
    if (!SHORT) {
        g = fma(q, 0x1.5d87fe78a6731p-10, 0x1.3b2ab6fba4e77p-7);            // ln2^5/120, ln2^4/24
        g = fma(q, g, 0x1.c6b08d704a0c0p-5);
    }
    g = fma(q, g, 0x1.ebfbdff82c58fp-3);                                     // ln2^2/2
    g = fma(q, g, 0x1.62e42fefa39efp-1);                                     // ln2
    const double s = exp_tab[j & (kExpTableEntries - 1)];
    y = ldexp(fma(s, q * g, s), j >> 7);
    return a > 0.0f && a < INFINITY && fabsf(b) < INFINITY && b != 0.0f;
}

}  // namespace kth
