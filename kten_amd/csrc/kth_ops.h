// Device functors for the elementwise operations, with the arithmetic rules of the
// kten-jvm backend (reference: backend/kten-jvm/.../store/JVMRawTensor.kt, cited per op):
//   - + - * / sqrt and their compositions are single IEEE roundings, never fused
//     (the library is compiled with -ffp-contract=off and correctly rounded div/sqrt);
//   - kotlin.math Float overloads are "f64 libm, round once to f32": computed here in
//     f64 as well, so results land on (or within an ulp of) the same float;
//   - java.lang.Math.max/min/round/signum/pow special cases are spelled out.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

namespace kth {

// java.lang.Math.max(float,float): NaN wins, -0 < +0. (JVMRawTensor.kt:159)
// v_max_f32 / v_min_f32 order the zeros that way themselves (max(+0, -0) = +0 whichever operand holds which) and
// return the other operand when one is a NaN, so the instruction and one unordered compare make the Java rule.
// `r` unless an operand is a NaN, then that operand (a first). Written as two selects on the bit patterns: as nested
// conditions the compiler made branches of it inside the reduction loops (four masked jumps per element).
__device__ __forceinline__ float java_nan_rule(float a, float b, float r) {
    const uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b), ur = __float_as_uint(r);
    const uint32_t with_b = (b != b) ? ub : ur;
    return __uint_as_float((a != a) ? ua : with_b);
}

__device__ __forceinline__ float jmax(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return java_nan_rule(a, b, r);
}

// java.lang.Math.min(float,float). (JVMRawTensor.kt:160)
__device__ __forceinline__ float jmin(float a, float b) {
    float r;
    asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return java_nan_rule(a, b, r);
}

// Float.pow(Float) = Math.pow(double,double).toFloat() (JVMRawTensor.kt:138-140).
// Java, unlike C99/OpenCL pow: pow(x, NaN) = NaN also for x == 1; pow(+-1, +-inf) = NaN.
__device__ __forceinline__ float jpow(float a, float b) {
    double x = static_cast<double>(a), y = static_cast<double>(b);
    if (y == 0.0) return 1.0f;
    if (y != y) return b;
    if (isinf(y) && fabs(x) == 1.0) return __uint_as_float(0x7fc00000u);
    return static_cast<float>(pow(x, y));
}

// ---- binary functors: apply(a, b, p) where p carries PlatformProvider.epsilon for eq/neq.
struct OpPlus  { static constexpr const char* name = "OpPlus"; static __device__ __forceinline__ float apply(float a, float b, float) { return a + b; } };
struct OpMinus { static constexpr const char* name = "OpMinus"; static __device__ __forceinline__ float apply(float a, float b, float) { return a - b; } };
struct OpTimes { static constexpr const char* name = "OpTimes"; static __device__ __forceinline__ float apply(float a, float b, float) { return a * b; } };
struct OpDiv   { static constexpr const char* name = "OpDiv"; static __device__ __forceinline__ float apply(float a, float b, float) { return a / b; } };
struct OpPow   { static constexpr const char* name = "OpPow"; static __device__ __forceinline__ float apply(float a, float b, float) { return jpow(a, b); } };
// JVMRawTensor.kt:355-377
struct OpLt    { static constexpr const char* name = "OpLt"; static __device__ __forceinline__ float apply(float a, float b, float) { return a <  b ? 1.0f : 0.0f; } };
struct OpLte   { static constexpr const char* name = "OpLte"; static __device__ __forceinline__ float apply(float a, float b, float) { return a <= b ? 1.0f : 0.0f; } };
struct OpGt    { static constexpr const char* name = "OpGt"; static __device__ __forceinline__ float apply(float a, float b, float) { return a >  b ? 1.0f : 0.0f; } };
struct OpGte   { static constexpr const char* name = "OpGte"; static __device__ __forceinline__ float apply(float a, float b, float) { return a >= b ? 1.0f : 0.0f; } };
struct OpEq    { static constexpr const char* name = "OpEq"; static __device__ __forceinline__ float apply(float a, float b, float eps) { return fabsf(a - b) < eps ? 1.0f : 0.0f; } };
struct OpNeq   { static constexpr const char* name = "OpNeq"; static __device__ __forceinline__ float apply(float a, float b, float eps) { return fabsf(a - b) < eps ? 0.0f : 1.0f; } };

// ---- unary functors: apply(x, p, q); p, q are only used by clamp.
#define KTH_UNARY(NAME, EXPR)                                                             \
    struct NAME { static constexpr const char* name = #NAME;                              \
        static __device__ __forceinline__ float apply(float x, float p, float q) {       \
        (void)p; (void)q; return (EXPR); } };

KTH_UNARY(OpNeg,        -x)                                             // :122
KTH_UNARY(OpReciprocal, 1.0f / x)                                       // :142
KTH_UNARY(OpLog,        static_cast<float>(log(static_cast<double>(x))))   // :144
KTH_UNARY(OpExp,        static_cast<float>(exp(static_cast<double>(x))))   // :395
KTH_UNARY(OpTanh,       static_cast<float>(tanh(static_cast<double>(x))))  // :397
KTH_UNARY(OpSinh,       static_cast<float>(sinh(static_cast<double>(x))))  // :401
KTH_UNARY(OpCosh,       static_cast<float>(cosh(static_cast<double>(x))))  // :403
KTH_UNARY(OpAbs,        fabsf(x))                                       // :405
KTH_UNARY(OpSqrt,       sqrtf(x))                                       // :413 (sqrt via double rounds to the same float)
KTH_UNARY(OpSin,        static_cast<float>(sin(static_cast<double>(x))))   // :415
KTH_UNARY(OpCos,        static_cast<float>(cos(static_cast<double>(x))))   // :417
KTH_UNARY(OpTan,        static_cast<float>(tan(static_cast<double>(x))))   // :419
KTH_UNARY(OpAsin,       static_cast<float>(asin(static_cast<double>(x))))  // :421
KTH_UNARY(OpAcos,       static_cast<float>(acos(static_cast<double>(x))))  // :423
KTH_UNARY(OpAtan,       static_cast<float>(atan(static_cast<double>(x))))  // :425
KTH_UNARY(OpFloor,      floorf(x))                                      // :427
KTH_UNARY(OpCeil,       ceilf(x))                                       // :429
KTH_UNARY(OpTrunc,      truncf(x))                                      // :433 kotlin truncate == C truncf, signed zeros included
KTH_UNARY(OpRsqrt,      1.0f / sqrtf(x))                                // :435 two roundings, not a hardware rsq
KTH_UNARY(OpSquare,     x * x)                                          // pow(x, 2f): the exact product is representable in f64
KTH_UNARY(OpIdentity,   x)                                              // pow(x, 1f)
// pow(x, c) for the exponents whose correctly rounded f64 result is one f64 operation away (Math.pow is
// within one f64 ulp of it and rounds to the same float): x^3 = (x*x)*x and x^4 = (x*x)*(x*x) with x*x exact,
// x^-1 = 1/x, x^-2 = 1/(x*x), x^0.5 = sqrt(x) except that pow(-0, 0.5) = +0 and pow(-inf, 0.5) = +inf.
__device__ __forceinline__ float pow_cube(float x)   { const double d = static_cast<double>(x); return static_cast<float>((d * d) * d); }
__device__ __forceinline__ float pow_fourth(float x) { const double d = static_cast<double>(x), q = d * d; return static_cast<float>(q * q); }
__device__ __forceinline__ float pow_half(float x) {
    if (x == 0.0f) return 0.0f;
    if (x == -INFINITY) return INFINITY;
    return sqrtf(x);                                            // (the f64 square root rounds to the same float)
}
KTH_UNARY(OpPowCube,    pow_cube(x))
KTH_UNARY(OpPowFourth,  pow_fourth(x))
KTH_UNARY(OpPowInverse, static_cast<float>(1.0 / static_cast<double>(x)))
KTH_UNARY(OpPowHalf,    pow_half(x))
KTH_UNARY(OpPowInverseSquare, static_cast<float>(1.0 / (static_cast<double>(x) * static_cast<double>(x))))
#undef KTH_UNARY

// sigmoid = 1f / (1f + exp(-1f * x)) with exp rounded to float first. (:399)
struct OpSigmoid {
    static constexpr const char* name = "OpSigmoid";
    static __device__ __forceinline__ float apply(float x, float, float) {
        float m = -1.0f * x;
        float e = static_cast<float>(exp(static_cast<double>(m)));
        float d = 1.0f + e;
        return 1.0f / d;
    }
};

// Math.signum. (:407)
struct OpSign {
    static constexpr const char* name = "OpSign";
    static __device__ __forceinline__ float apply(float x, float, float) {
        if (x != x || x == 0.0f) return x;
        return x > 0.0f ? 1.0f : -1.0f;
    }
};

// Math.round(float).toFloat() (:431): floor(x + 1/2) without the rounding error of
// x + 0.5f, NaN -> 0, saturation at the Int range, zero results are +0.
struct OpRound {
    static constexpr const char* name = "OpRound";
    static __device__ __forceinline__ float apply(float x, float, float) {
        if (x != x) return 0.0f;
        float r = floorf(x);
        float frac = x - r;                       // exact; NaN for infinities
        float v = r + (frac >= 0.5f ? 1.0f : 0.0f);
        v = fminf(fmaxf(v, -2147483648.0f), 2147483648.0f);
        return v;
    }
};

// clamp = Math.min(Math.max(x, lo), hi). (:409-411)
struct OpClamp {
    static constexpr const char* name = "OpClamp";
    static __device__ __forceinline__ float apply(float x, float lo, float hi) {
        return jmin(jmax(x, lo), hi);
    }
};

}  // namespace kth
