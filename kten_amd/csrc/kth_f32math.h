// The transcendental maps evaluated in fp32 (a short f64 step only where fp32 cannot carry it: the argument reduction of
// sin / cos / tan and the quotient of tan), for the math mode "within 2 ulp".
//
// kotlin.math's Float overloads are "f64 libm, round once to f32" (JVMRawTensor.kt:144,395-425). The default mode of the
// library reproduces that float bit for bit with f64 routines (kth_fast.h, kth_tables.h), which keeps the vector ALU,
// not the memory, as the bound of these maps. The routines below stay within 2 units in the last place of that float
// (the tolerance the parity rules state for transcendentals) with 25-45 fp32 instructions per element: polynomial
// kernels on reduced arguments, an error-free transformation (fma residuals, two-sums) wherever a cancellation would
// otherwise amplify a rounding, IEEE operations only (+ - * / sqrt fma rint), so that a host compiler evaluates the
// same expressions to the same bits and the error bound can be checked on the CPU over the float space
// (tests/cpp/f32math_test.cpp). sigmoid is not here: the reference's float expression 1f / (1f + exp(-x)) turns one ulp
// of its exp into three of the result where 1f + e rounds (e in [2^24, 2^25)), so it keeps the f64 exp in every mode.
//
// Compiled with -ffp-contract=off: every fused multiply-add below is written as fmaf / fma.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define KTH_F32_FN __host__ __device__ __forceinline__
#else
#define KTH_F32_FN inline
#endif

namespace kth {
namespace f32 {

KTH_F32_FN uint32_t bits_of(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
KTH_F32_FN float float_of(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }
KTH_F32_FN float with_sign(float magnitude, float sign_of) { return float_of(bits_of(magnitude) | (bits_of(sign_of) & 0x80000000u)); }
KTH_F32_FN float quiet_nan() { return float_of(0x7fc00000u); }

// 2^n, n in [-126, 127].
KTH_F32_FN float pow2i(int n) { return float_of(static_cast<uint32_t>(n + 127) << 23); }
// x 2^n for |n| <= 250 and x in [1/2, 2): two exact powers of two, so the result is rounded once (in the
// denormal range) or overflows to infinity.
KTH_F32_FN float scale2(float x, int n) { const int h = n >> 1; return (x * pow2i(h)) * pow2i(n - h); }

// 1 / d to an ulp or so, for correction terms only (a term that is 2^-24 of the result needs 2^-8 of itself): the
// hardware estimate on the device, the quotient on the host. The two differ where a result lies within 2^-45 of the
// midpoint of two floats, about once in a million inputs, and both are then within the same bound.
KTH_F32_FN float approx_rcp(float d) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_rcpf(d);
#else
    return 1.0f / d;
#endif
}

// sqrt w to an ulp or so, for callers that take the residual w - s^2 themselves (s + s_lo is then good to 2^-46
// whichever neighbour s is): the hardware's square root on the device, the IEEE one on the host.
KTH_F32_FN float approx_sqrt(float w) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_sqrtf(w);
#else
    return sqrtf(w);
#endif
}

// n / d within 0.5 + 2^-20 ulp, for normal d and a normal quotient: the estimate, its exact remainder by an fma, one
// correction (4 instructions where the IEEE quotient takes 12). On the host the IEEE quotient.
KTH_F32_FN float div_near(float n, float d) {
#if defined(__HIP_DEVICE_COMPILE__)
    const float r = __builtin_amdgcn_rcpf(d);
    const float q = n * r;
    return fmaf(fmaf(-q, d, n), r, q);
#else
    return n / d;
#endif
}

struct HiLo { float hi, lo; };

// (n_hi + n_lo) / (d_hi + d_lo), lo parts at most an ulp of their hi: an estimate of the quotient of the hi parts,
// its exact remainder by an fma, and the first-order correction with the lo parts in it.
KTH_F32_FN float div_hilo(HiLo n, HiLo d) {
    const float r = approx_rcp(d.hi);
    const float q = n.hi * r;
    const float rem = fmaf(-q, d.hi, n.hi);
    return q + (rem + fmaf(-q, d.lo, n.lo)) * r;
}

// ---------------------------------------------------------------- e^a = 2^n (1 + p)

// a = n ln2 + r, |r| <= ln2 / 2 (+ an ulp): ln2 = hi + lo with 12 trailing zero bits in hi, so a - n hi is exact.
// p = e^r - 1 = r + r^2 Q(r) as p_hi + p_lo: the final sum r + t by a fast two-sum (|t| < |r| / 4), so p is known to
// about 2^-30 of itself although it is the sum of two floats.
struct ExpParts { int n; float p, p_lo; };

KTH_F32_FN ExpParts exp_parts(float a) {
    const float nf = rintf(a * 1.44269504f);
    float r = fmaf(nf, -0.693145752f, a);                  // 0x1.62e4p-1
    r = fmaf(nf, -1.42860677e-06f, r);                     // ln2 - 0x1.62e4p-1
    float q = fmaf(r, 0.00019909059f, 0.0013940518f);
    q = fmaf(r, q, 0.008333283f);
    q = fmaf(r, q, 0.041666362f);
    q = fmaf(r, q, 0.16666667f);
    q = fmaf(r, q, 0.5f);
    const float t = (r * r) * q;
    ExpParts e;
    e.n = static_cast<int>(nf);
    e.p = r + t;
    e.p_lo = t - (e.p - r);
    return e;
}

// exp (JVMRawTensor.kt:395). 1 + p is formed with its rounding error folded back in.
KTH_F32_FN float exp_(float x) {
    const float a = fminf(fmaxf(x, -104.5f), 89.5f);
    const ExpParts e = exp_parts(a);
    const float s = 1.0f + e.p;
    const float s_lo = (e.p - (s - 1.0f)) + e.p_lo;        // 1 >= |p|: fast two-sum
    const float r = scale2(s + s_lo, e.n);
    return x != x ? x : r;
}

// tanh (JVMRawTensor.kt:397). Below 0.55: x + x^3 T(x^2). From there on 1 - 2 / (e^(2|x|) + 1): the quotient is at most
// 1/2, so its error of an ulp is half an ulp of the result. e^(2|x|) + 1 = 2^n p + (2^n + 1) in one fma.
KTH_F32_FN float tanh_(float x) {
    const float ax = fabsf(x);
    const float z = ax * ax;
    float t = fmaf(z, 0.002426026f, -0.008443189f);
    t = fmaf(z, t, 0.021793442f);
    t = fmaf(z, t, -0.053961426f);
    t = fmaf(z, t, 0.13333307f);
    t = fmaf(z, t, -0.33333334f);
    const float small = fmaf(ax * z, t, ax);
    const ExpParts e = exp_parts(2.0f * fminf(ax, 10.0f));
    const float S = pow2i(e.n);
    const float D = fmaf(S, e.p, S + 1.0f);
    const float large = 1.0f - div_near(2.0f, D);
    const float r = ax < 0.55f ? small : large;
    return x != x ? x : with_sign(r, x);
}

// t = e^a / 4 = 2^(n-2) (1 + p) for 0 <= a <= 89.5 as hi + lo (the fma's residual is exact: 2^(n-2) - t_hi is, by
// Sterbenz), and u = e^-a / 4 = (1/16) / t with its residual. Quarters, so that e^a near the overflow threshold of
// sinh and cosh (89.416, where e^a itself is beyond fp32) still fits: the result is 2 (t -+ u).
struct ExpPair { HiLo t; float u, u_lo; };
KTH_F32_FN ExpPair exp_pair(float a) {
    const ExpParts e = exp_parts(a);
    const float S = pow2i(e.n - 2);
    ExpPair r;
    r.t.hi = fmaf(S, e.p, S);
    r.t.lo = fmaf(S, e.p, S - r.t.hi) + S * e.p_lo;
    const float rt = approx_rcp(r.t.hi);
    r.u = 0.0625f * rt;
    // 1/16 = u (t_hi + t_lo) + residual: u_lo = (1/16 - u t_hi) / t_hi - u t_lo / t_hi
    r.u_lo = fmaf(-r.u, r.t.hi, 0.0625f) * rt - (r.u * rt) * r.t.lo;
    return r;
}

// sinh (JVMRawTensor.kt:401): 2 (t - u), the difference of the large terms by a fast two-sum (t >= u), the small terms
// added to its residual. t and u are each known to 2^-46 of themselves, so the difference holds down to |x| = 2^-12
// (t - u = 2 sinh |x| >= 2^-11, error 2^-45); below that sinh x rounds to x itself (x^3 / 6 < 2^-26 x).
KTH_F32_FN float sinh_(float x) {
    const float ax = fabsf(x);
    const ExpPair v = exp_pair(fminf(ax, 89.5f));
    const float d = v.t.hi - v.u;
    const float large = 2.0f * (d + (((v.t.hi - d) - v.u) + (v.t.lo - v.u_lo)));
    return x != x ? x : with_sign(ax < 0.000244140625f ? ax : large, x);
}

// cosh (JVMRawTensor.kt:403): 2 (t + u), no cancellation.
KTH_F32_FN float cosh_(float x) {
    const float ax = fabsf(x);
    const ExpPair v = exp_pair(fminf(ax, 89.5f));
    const float d = v.t.hi + v.u;
    const float r = 2.0f * (d + ((v.u - (d - v.t.hi)) + (v.t.lo + v.u_lo)));
    return x != x ? x : r;
}

// ---------------------------------------------------------------- log

// log (JVMRawTensor.kt:144). x = 2^k m with m in [sqrt(1/2), sqrt 2), f = m - 1 (exact),
// log m = f - (f^2 / 2 - f^3 P(f)); k ln2 is added as hi + lo with hi exact in the product.
KTH_F32_FN float log_(float x) {
    const bool denormal = bits_of(x) < 0x00800000u;                        // (zero included; it is set right below)
    int k = denormal ? -25 : 0;
    uint32_t u = bits_of(denormal ? x * 33554432.0f : x);                  // times 2^25
    u -= 0x3f3504f3u;                                                      // the bits of sqrt(1/2)
    k += static_cast<int>(static_cast<int32_t>(u) >> 23);                  // floor of the exponent difference
    const float m = float_of((u & 0x007fffffu) + 0x3f3504f3u);
    const float f = m - 1.0f;
    float p = fmaf(f, 0.0694301f, -0.11771368f);
    p = fmaf(f, p, 0.11849299f);
    p = fmaf(f, p, -0.12386837f);
    p = fmaf(f, p, 0.14222765f);
    p = fmaf(f, p, -0.1666919f);
    p = fmaf(f, p, 0.20001975f);
    p = fmaf(f, p, -0.24999985f);
    p = fmaf(f, p, 0.33333316f);
    const float ff = f * f;
    const float hfsq = 0.5f * ff;
    const float kf = static_cast<float>(k);
    // k ln2_hi is exact (|k| <= 150, 12 trailing zero bits in ln2_hi)
    const float tail = fmaf(ff * f, p, kf * 1.42860677e-06f);
    float r = fmaf(kf, 0.693145752f, f - (hfsq - tail));
    r = x == INFINITY ? x : r;
    r = x == 0.0f ? -INFINITY : r;
    r = x < 0.0f ? quiet_nan() : r;
    return x != x ? x : r;
}

// ---------------------------------------------------------------- sin, cos, tan

// |x| <= 65536: k = round(x 2/pi), r = x - k pi/2 in f64 with pi/2 = 33 + 53 bits (k < 2^16: the first product and
// difference are exact, the second fma leaves 2^-69 absolute), handed on as two floats r_hi + r_lo.
// sin r = r + r^3 S(z), cos r = 1 - z/2 + z^2 C(z) on |r| <= pi/4, each with its last, large addition made once.
constexpr float kTrigLimit = 65536.0f;

// sin r = r_hi + s_small, cos r = w + c_small with the large terms r_hi and w = fl(1 - z/2) exact floats and the small
// ones rounded once each: sin and cos add them, tan divides the sums as hi + lo pairs.
struct TrigParts { int k; float rh, s_small, w, c_small; };

// (The argument is |x|: sin and tan restore the sign, so that -0 stays -0 without a test in f64.)
KTH_F32_FN TrigParts trig_parts(float ax) {
    const double a = static_cast<double>(ax);
    const double kd = rint(a * 0.63661977236758138);                      // 2 / pi
    double r = fma(kd, -0x1.921fb54400000p+0, a);
    r = fma(kd, -0x1.0b4611a626331p-34, r);
    const float rh = static_cast<float>(r);
    const float rl = static_cast<float>(r - static_cast<double>(rh));
    const float z = rh * rh;
    float sp = fmaf(z, 2.7181693e-06f, -0.00019839335f);
    sp = fmaf(z, sp, 0.008333329f);
    sp = fmaf(z, sp, -0.16666667f);
    float cp = fmaf(z, -2.7241444e-07f, 2.4799965e-05f);
    cp = fmaf(z, cp, -0.0013888886f);
    cp = fmaf(z, cp, 0.041666668f);
    TrigParts t;
    t.k = static_cast<int>(kd);
    t.rh = rh;
    // sin(r_hi + r_lo) = sin r_hi + r_lo cos r_hi, cos r_hi ~ 1 - z/2
    t.s_small = fmaf(rh * z, sp, rl * fmaf(z, -0.5f, 1.0f));
    const float hz = 0.5f * z;
    t.w = 1.0f - hz;
    t.c_small = ((1.0f - t.w) - hz) + fmaf(z * z, cp, -(rh * rl));
    return t;
}

KTH_F32_FN float sin_short(float x) {
    const TrigParts t = trig_parts(fabsf(x));
    const float v = (t.k & 1) ? t.w + t.c_small : t.rh + t.s_small;
    // the quadrant's sign and the argument's, both as a flip of the sign bit
    return float_of(bits_of(v) ^ ((static_cast<uint32_t>(t.k & 2) << 30) ^ (bits_of(x) & 0x80000000u)));
}

KTH_F32_FN float cos_short(float x) {
    const TrigParts t = trig_parts(fabsf(x));
    const float v = (t.k & 1) ? t.rh + t.s_small : t.w + t.c_small;
    return ((t.k + 1) & 2) ? -v : v;
}

// tan = s / c (or -c / s in the odd quadrants): each sum by a fast two-sum (|r_hi| >= |s_small|, w >= |c_small|),
// then the compensated quotient: one rounding at the end instead of three.
KTH_F32_FN float tan_short(float x) {
    const TrigParts t = trig_parts(fabsf(x));
    HiLo s, c;
    s.hi = t.rh + t.s_small; s.lo = t.s_small - (s.hi - t.rh);
    c.hi = t.w + t.c_small;  c.lo = t.c_small - (c.hi - t.w);
    const bool odd = (t.k & 1) != 0;
    HiLo n = odd ? c : s, d = odd ? s : c;
    const float v = div_hilo(n, d);
    return float_of(bits_of(v) ^ ((odd ? 0x80000000u : 0u) ^ (bits_of(x) & 0x80000000u)));
}

// ---------------------------------------------------------------- atan, asin, acos

// atan (JVMRawTensor.kt:425): |x| against the breakpoints 7/16, 11/16, 19/16, 39/16 picks
// atan |x| = base + atan t with t = (|x| - b) / (1 + b |x|) for b = 0, 1/2, 1, 3/2, or t = -1 / |x| with base pi/2,
// so |t| < 7/16 and an error in t weighs little against the base; atan t = t + t^3 A(t^2).
KTH_F32_FN float atan_(float x) {
    const float ax = fabsf(x);
    // the range by selects: b = 0, 1/2, 1, 3/2 or "infinity" (t = -1 / |x|)
    const bool r1 = ax >= 0.4375f, r2 = ax >= 0.6875f, r3 = ax >= 1.1875f, r4 = ax >= 2.4375f;
    const float b = r3 ? 1.5f : r2 ? 1.0f : r1 ? 0.5f : 0.0f;
    const float hi = r4 ? 1.57079625f : r3 ? 0.982793689f : r2 ? 0.785398126f : r1 ? 0.463647604f : 0.0f;
    const float lo = r4 ? 7.54978942e-08f : r3 ? 3.44732172e-08f : r2 ? 3.77489471e-08f : r1 ? 5.01215813e-09f : 0.0f;
    const float num = r4 ? -1.0f : ax - b;                                // exact for b = 1/2, 1, 3/2 in their ranges
    const float den = r4 ? fminf(ax, 3.40282347e+38f) : fmaf(b, ax, 1.0f);   // (finite: the estimate of 1 / inf times inf is no number)
    const float t = div_near(num, den);
    const float z = t * t;
    float a = fmaf(z, 0.04622634f, -0.08428244f);
    a = fmaf(z, a, 0.11038711f);
    a = fmaf(z, a, -0.1428182f);
    a = fmaf(z, a, 0.19999912f);
    a = fmaf(z, a, -0.33333334f);
    const float r = hi + (t + fmaf(t * z, a, lo));
    return x != x ? x : with_sign(r, x);
}

// asin R(z): asin x = x + x^3 R(x^2) for |x| <= 1/2.
KTH_F32_FN float asin_poly(float z) {
    float r = fmaf(z, 0.03646355f, 0.015257911f);
    r = fmaf(z, r, 0.03156781f);
    r = fmaf(z, r, 0.044549387f);
    r = fmaf(z, r, 0.07500308f);
    return fmaf(z, r, 0.16666664f);
}

// asin (JVMRawTensor.kt:421) and acos (:423) share their pieces. |x| <= 1/2: asin x = x + x^3 R(x^2). Beyond:
// with w = (1 - |x|) / 2 (exact), s = sqrt w and its residual s_lo = (w - s^2) / (2 s),
// 2 asin sqrt w = 2 s + 2 (s_lo + s w R(w)), and asin |x| = pi/2 minus that, acos |x| = that, acos -|x| = pi minus
// that: the difference of the two large terms by a fast two-sum, the small ones added to its residual.
// R is evaluated once, at x^2 or at w.
struct AsinParts { float ax, poly_term, root2, root2_lo; bool small; };

KTH_F32_FN AsinParts asin_parts(float x) {
    AsinParts a;
    a.ax = fabsf(x);
    a.small = a.ax <= 0.5f;
    const float w = 0.5f * (1.0f - a.ax);
    const float s = approx_sqrt(w);
    const float arg = a.small ? a.ax * a.ax : w;
    const float base = a.small ? a.ax : s;
    a.poly_term = (base * arg) * asin_poly(arg);                          // x^3 R(x^2), or s w R(w)
    const float s_lo = fmaf(-s, s, w) * (0.5f * approx_rcp(s));
    a.root2 = 2.0f * s;
    a.root2_lo = 2.0f * (a.poly_term + (s > 0.0f ? s_lo : 0.0f));
    return a;
}

KTH_F32_FN float asin_(float x) {
    const AsinParts a = asin_parts(x);
    const float small = a.ax + a.poly_term;
    const float d = 1.57079625f - a.root2;                                // pi/2 = 1.57079625 + 7.54978942e-08
    const float d_lo = (1.57079625f - d) - a.root2;
    const float large = d + ((d_lo + 7.54978942e-08f) - a.root2_lo);
    const float r = with_sign(a.small ? small : large, x);
    return a.ax <= 1.0f ? r : x != x ? x : quiet_nan();
}

KTH_F32_FN float acos_(float x) {
    const AsinParts a = asin_parts(x);
    // |x| <= 1/2: pi/2 - asin x = pi/2_hi - (x + (asin x - x - pi/2_lo)), asin x - x = +-poly_term
    const float e = with_sign(a.poly_term, x) - 7.54978942e-08f;
    const float mid = 1.57079625f - (x + e);
    const float pos = a.root2 + a.root2_lo;
    const float d = 3.14159250f - a.root2;                                // pi = 3.14159250 + 1.50995788e-07
    const float d_lo = (3.14159250f - d) - a.root2;
    const float neg = d + ((d_lo + 1.50995788e-07f) - a.root2_lo);
    const float r = a.small ? mid : x > 0.0f ? pos : neg;
    return a.ax <= 1.0f ? r : x != x ? x : quiet_nan();
}

}  // namespace f32
}  // namespace kth
