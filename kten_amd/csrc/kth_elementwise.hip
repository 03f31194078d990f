// Elementwise kernels: unary maps, tensor-scalar maps, same-shape and broadcast binary
// ops, fill, materialised broadcast, NaN scan. All are HBM-streaming kernels: every
// thread moves float4s, loads of a tile are issued before any arithmetic, and a
// workgroup of 256 threads (4 wave64s) covers a contiguous 4 KiB span per operand.
#include "kth_internal.h"
#include "kth_ops.h"
#include "kth_tables.h"
#include "kth_fast.h"
#include "kth_f32math.h"
#include "kth_fold.h"

#include <cmath>
#include <cstring>

using namespace kth;

namespace {

constexpr int kBlock = 256;
// float4s per thread. Measured on random data in chains of these kernels: one float4
// per thread is fastest for the contiguous maps (73 us per 268 MB copy against 75 us at
// two and 77 us at four), two for the broadcast kernels.
constexpr int kUnroll = 1;
constexpr uint32_t kTile = kBlock * kUnroll;     // float4s per workgroup
#ifndef KTH_BCAST_UNROLL
#define KTH_BCAST_UNROLL 2
#endif
constexpr int kBcastUnroll = KTH_BCAST_UNROLL;
constexpr uint32_t kBcastTile = kBlock * kBcastUnroll;
constexpr uint32_t kReuseChunkShift = 6;          // 64 tiles (of up to 8 KiB per operand) stay in L2 while the slices pass; half when both operands repeat

typedef float v4f __attribute__((ext_vector_type(4)));

// Streaming load: every full-size operand is read exactly once per kernel, so it is
// loaded with the non-temporal hint. Measured on MI355X chains of these kernels, that
// keeps the read stream from displacing the freshly written output of the previous
// kernel in the 256 MB memory-side cache; stores stay ordinary so that the next
// kernel finds them there (8.0 TB/s algorithmic against 5.8 TB/s with plain loads).
__device__ __forceinline__ float4 ld4(const float* p, uint32_t i4) {
    v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p) + i4);
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st4(float* p, uint32_t i4, float4 v) {
    reinterpret_cast<float4*>(p)[i4] = v;
}

// ---------------------------------------------------------------- contiguous maps

// out[i] = Op(a[i], p, q). out may alias a.
template <class Op>
__global__ __launch_bounds__(kBlock) void unary_kernel(const float* a, float* out, uint32_t n, float p, float q) {
    const uint32_t n4 = n >> 2;
    const uint32_t base = blockIdx.x * kTile + threadIdx.x;
    float4 v[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) v[k] = ld4(a, i);
    }
#pragma unroll
    for (int k = 0; k < kUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) {
            float4 r;
            r.x = Op::apply(v[k].x, p, q); r.y = Op::apply(v[k].y, p, q);
            r.z = Op::apply(v[k].z, p, q); r.w = Op::apply(v[k].w, p, q);
            st4(out, i, r);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        uint32_t i = (n4 << 2) + threadIdx.x;
        out[i] = Op::apply(a[i], p, q);
    }
}

// ---------------------------------------------------------------- table-driven exp / log

__device__ LogEntry g_log_table[kLogTableEntries];
__device__ double   g_exp_table[kExpTableEntries];
__device__ double   g_atan_table[kAtanTableEntries];
__device__ double   g_sincos_table[2 * kSinCosTableEntries];
__device__ double   g_asin_table[2 * kAsinTableEntries];
__device__ Log2Entry g_log2_table[kLogTableEntries];

// Copies `count` doubles of a device table into LDS, all threads of the workgroup taking part.
__device__ __forceinline__ void stage_table(double* lds, const double* table, int count) {
    for (int i = threadIdx.x; i < count; i += kBlock) lds[i] = table[i];
}

struct OpLogT {
    static constexpr const char* name = "OpLog";
    static constexpr int kTableDoubles = 2 * kLogTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, reinterpret_cast<const double*>(g_log_table), kTableDoubles); }
    static __device__ __forceinline__ float apply(float x, const double* lds) {
        return table_log(x, reinterpret_cast<const LogEntry*>(lds));
    }
    static __device__ __forceinline__ float4 apply4(float4 v, const double* lds) {
        return make_float4(apply(v.x, lds), apply(v.y, lds), apply(v.z, lds), apply(v.w, lds));
    }
};
struct OpExpT {
    static constexpr const char* name = "OpExp";
    static constexpr int kTableDoubles = kExpTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_exp_table, kTableDoubles); }
    static __device__ __forceinline__ float apply(float x, const double* lds) { return table_exp(x, lds); }
    static __device__ __forceinline__ float4 apply4(float4 v, const double* lds) {
        return make_float4(apply(v.x, lds), apply(v.y, lds), apply(v.z, lds), apply(v.w, lds));
    }
};
// sigmoid = 1f / (1f + exp(-1f * x)), exp rounded to float first (JVMRawTensor.kt:399).
struct OpSigmoidT {
    static constexpr const char* name = "OpSigmoid";
    static constexpr int kTableDoubles = kExpTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_exp_table, kTableDoubles); }
    static __device__ __forceinline__ float apply(float x, const double* lds) {
        float m = -1.0f * x;
        float e = table_exp(m, lds);
        float d = 1.0f + e;
        return 1.0f / d;
    }
    static __device__ __forceinline__ float4 apply4(float4 v, const double* lds) {
        return make_float4(apply(v.x, lds), apply(v.y, lds), apply(v.z, lds), apply(v.w, lds));
    }
};

// The maps below take the short evaluation of kth_fast.h and fall back to the long routine of
// kth_tables.h for the lanes whose rounding the short value does not decide.
__device__ __forceinline__ float with_sign_of(float magnitude_result, float x) {      // odd maps evaluated at |x|
    return __uint_as_float(__float_as_uint(magnitude_result) ^ (__float_as_uint(x) & 0x80000000u));
}

// Four elements through a short routine, then one branch for the lanes of the wave whose rounding it left open:
// the four evaluations are independent straight-line code, and the long routine is reached about once in
// several hundred waves.
#define KTH_SHORT_THEN_LONG(FAST, SIGNED, ROLLED, LONG_CALL)                                                     \
    static __device__ __forceinline__ float apply(float x, const double* lds) {                          \
        double y;                                                                                         \
        const bool ok = FAST(x, lds, y);                                                                 \
        float r = SIGNED ? with_sign_of(static_cast<float>(y), x) : static_cast<float>(y);               \
        if (!(ok && rounds_safely(y))) r = LONG_CALL;                                                    \
        return r;                                                                                         \
    }                                                                                                     \
    static __device__ __forceinline__ float4 apply4(float4 v, const double* lds) {                       \
        const float xs[4] = {v.x, v.y, v.z, v.w};                                                        \
        float rs[4];                                                                                      \
        bool open[4];                                                                                     \
        _Pragma("unroll") for (int j = 0; j < 4; j++) {                                                  \
            const float x = xs[j];                                                                        \
            double y;                                                                                     \
            const bool ok = FAST(x, lds, y);                                                             \
            rs[j] = SIGNED ? with_sign_of(static_cast<float>(y), x) : static_cast<float>(y);             \
            open[j] = !(ok && rounds_safely(y));                                                         \
        }                                                                                                 \
        if (ROLLED && (open[0] | open[1] | open[2] | open[3])) {                                         \
            /* one copy of the long routine for the four elements: the loop stays rolled, j is uniform */ \
            _Pragma("unroll 1") for (int j = 0; j < 4; j++) {                                            \
                const bool o = j == 0 ? open[0] : j == 1 ? open[1] : j == 2 ? open[2] : open[3];         \
                if (o) {                                                                                  \
                    const float x = j == 0 ? xs[0] : j == 1 ? xs[1] : j == 2 ? xs[2] : xs[3];            \
                    const float y = LONG_CALL;                                                           \
                    if (j == 0) rs[0] = y; else if (j == 1) rs[1] = y; else if (j == 2) rs[2] = y; else rs[3] = y; \
                }                                                                                         \
            }                                                                                             \
        }                                                                                                 \
        if (!ROLLED && (open[0] | open[1] | open[2] | open[3])) {                                        \
            _Pragma("unroll") for (int j = 0; j < 4; j++) {                                              \
                const float x = xs[j];                                                                    \
                if (open[j]) rs[j] = LONG_CALL;                                                          \
            }                                                                                             \
        }                                                                                                 \
        return make_float4(rs[0], rs[1], rs[2], rs[3]);                                                  \
    }

struct OpTanhT {
    static constexpr const char* name = "OpTanh";
    static constexpr int kTableDoubles = kExpTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_exp_table, kTableDoubles); }
    KTH_SHORT_THEN_LONG(fast_tanh, true, true, table_tanh(x, lds))
};
struct OpSinhT {
    static constexpr const char* name = "OpSinh";
    static constexpr int kTableDoubles = kExpTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_exp_table, kTableDoubles); }
    KTH_SHORT_THEN_LONG(fast_sinh, true, true, table_sinh(x, lds))
};
struct OpCoshT {
    static constexpr const char* name = "OpCosh";
    static constexpr int kTableDoubles = kExpTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_exp_table, kTableDoubles); }
    KTH_SHORT_THEN_LONG(fast_cosh, false, true, table_cosh(x, lds))
};

// atan keeps the long routine alone: with one reciprocal per lane it is already the cheaper one
// (100 us per 268 MB map against 111 us for the short routine with its selects).
struct OpAtanT {
    static constexpr const char* name = "OpAtan";
    static constexpr int kTableDoubles = kAtanTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_atan_table, kTableDoubles); }
    static __device__ __forceinline__ float apply(float x, const double* lds) { return table_atan(x, lds); }
    static __device__ __forceinline__ float4 apply4(float4 v, const double* lds) {
        return make_float4(apply(v.x, lds), apply(v.y, lds), apply(v.z, lds), apply(v.w, lds));
    }
};
// asin and acos: the {asin c, sqrt(1 - c^2)} table of the short routine first, then the atan table of the long one.
struct OpAsinT {
    static constexpr const char* name = "OpAsin";
    static constexpr int kTableDoubles = 2 * kAsinTableEntries + kAtanTableEntries;
    static __device__ __forceinline__ void stage(double* lds) {
        stage_table(lds, g_asin_table, 2 * kAsinTableEntries);
        stage_table(lds + 2 * kAsinTableEntries, g_atan_table, kAtanTableEntries);
    }
    KTH_SHORT_THEN_LONG(fast_asin, true, true, table_asin(x, lds + 2 * kAsinTableEntries))
};
struct OpAcosT {
    static constexpr const char* name = "OpAcos";
    static constexpr int kTableDoubles = 2 * kAsinTableEntries + kAtanTableEntries;
    static __device__ __forceinline__ void stage(double* lds) {
        stage_table(lds, g_asin_table, 2 * kAsinTableEntries);
        stage_table(lds + 2 * kAsinTableEntries, g_atan_table, kAtanTableEntries);
    }
    KTH_SHORT_THEN_LONG(fast_acos, false, true, table_acos(x, lds + 2 * kAsinTableEntries))
};
// sin, cos, tan: the short routine reads {sin, cos}(j pi / 32) through LDS; the long one needs no table.
struct OpSinT {
    static constexpr const char* name = "OpSin";
    static constexpr int kTableDoubles = 2 * kSinCosTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_sincos_table, kTableDoubles); }
    KTH_SHORT_THEN_LONG(fast_sin, true, false, table_sin(x))
};
struct OpCosT {
    static constexpr const char* name = "OpCos";
    static constexpr int kTableDoubles = 2 * kSinCosTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_sincos_table, kTableDoubles); }
    KTH_SHORT_THEN_LONG(fast_cos, false, false, table_cos(x))
};
struct OpTanT {
    static constexpr const char* name = "OpTan";
    static constexpr int kTableDoubles = 2 * kSinCosTableEntries;
    static __device__ __forceinline__ void stage(double* lds) { stage_table(lds, g_sincos_table, kTableDoubles); }
    KTH_SHORT_THEN_LONG(fast_tan, true, false, table_tan(x))
};

// pow(tensor | Float): the common operands (finite non-zero base, finite exponent) go through
// the exp / log tables, read from global memory (3 KiB, cache resident); zeros, infinities
// and NaNs take jpow's spelled-out Java rules over the library routine.
__device__ __forceinline__ float pow_with_tables(float a, float b, const LogEntry* log_tab, const double* exp_tab) {
    const bool common = (a != 0.0f) && (fabsf(a) < INFINITY) && (fabsf(b) < INFINITY) && (b != 0.0f);
    if (common) return table_pow_finite(a, b, log_tab, exp_tab);
    return jpow(a, b);
}
// The short base-2 evaluation first (a finite base above zero, a finite exponent other than zero), the routine above for
// the lanes whose rounding it leaves open and for every other operand.
__device__ __forceinline__ float pow_short_then_long(float a, float b, const Log2Entry* log2_tab, const LogEntry* log_tab, const double* exp_tab) {
    double y;
    const bool ok = fast_pow(a, b, log2_tab, exp_tab, y);
    float r = static_cast<float>(y);
    if (!(ok && rounds_safely(y))) r = pow_with_tables(a, b, log_tab, exp_tab);
    return r;
}
// The math mode "within 2 ulp": the shorter evaluation decides by itself for a finite base above zero and a finite
// exponent other than zero with a normal result; every other operand (and a result in the denormal range, where the
// rounding to fp32 is not relative) takes the routine above as before.
__device__ __forceinline__ float pow_within_2_ulp(float a, float b, const Log2Entry* log2_tab, const LogEntry* log_tab, const double* exp_tab) {
    double y;
    const bool ok = fast_pow<true>(a, b, log2_tab, exp_tab, y);
    float r = static_cast<float>(y);
    if (!(ok && y >= 0x1p-126)) r = pow_with_tables(a, b, log_tab, exp_tab);
    return r;
}
struct OpPowT {
    static constexpr const char* name = "OpPow";
    static __device__ __forceinline__ float apply(float a, float b, float) { return pow_short_then_long(a, b, g_log2_table, g_log_table, g_exp_table); }
};

// The maps of the math mode "within 2 ulp": fp32 evaluations (kth_f32math.h) through the plain unary kernel, no table
// and no LDS. sin / cos / tan beyond 65536 in magnitude take the long f64 routine in every mode.
#define KTH_F32_MAP(NAME, EXPR)                                                            \
    struct NAME { static constexpr const char* name = #NAME;                               \
        static __device__ __forceinline__ float apply(float x, float, float) { return (EXPR); } };
KTH_F32_MAP(OpExpF,  f32::exp_(x))
KTH_F32_MAP(OpLogF,  f32::log_(x))
KTH_F32_MAP(OpTanhF, f32::tanh_(x))
KTH_F32_MAP(OpSinhF, f32::sinh_(x))
KTH_F32_MAP(OpCoshF, f32::cosh_(x))
KTH_F32_MAP(OpSinF,  fabsf(x) <= f32::kTrigLimit ? f32::sin_short(x) : table_sin(x))
KTH_F32_MAP(OpCosF,  fabsf(x) <= f32::kTrigLimit ? f32::cos_short(x) : table_cos(x))
KTH_F32_MAP(OpTanF,  fabsf(x) <= f32::kTrigLimit ? f32::tan_short(x) : table_tan(x))
KTH_F32_MAP(OpAsinF, f32::asin_(x))
KTH_F32_MAP(OpAcosF, f32::acos_(x))
KTH_F32_MAP(OpAtanF, f32::atan_(x))
#undef KTH_F32_MAP

// Unary map whose op reads a small f64 table through LDS. The data loads of the tile are
// issued first, the table copy overlaps them. Four float4 per thread, so the 1-2 KiB
// table is amortised over a 16 KiB tile.
constexpr int kLdsUnroll = 4;
template <class Op>
__global__ __launch_bounds__(kBlock) void unary_lds_kernel(const float* a, float* out, uint32_t n) {
    __shared__ double tab[Op::kTableDoubles];
    const uint32_t n4 = n >> 2;
    const uint32_t base = blockIdx.x * (kBlock * kLdsUnroll) + threadIdx.x;
    float4 v[kLdsUnroll];
#pragma unroll
    for (int k = 0; k < kLdsUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) v[k] = ld4(a, i);
    }
    Op::stage(tab);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kLdsUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) st4(out, i, Op::apply4(v[k], tab));
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        uint32_t i = (n4 << 2) + threadIdx.x;
        out[i] = Op::apply(a[i], tab);
    }
}

// pow with both tables (3 KiB) in LDS: the lookups of 64 lanes go to 64 different entries, which as loads from
// global memory cost more than the arithmetic. MODE 0: out[i] = pow(a[i], c); 1: pow(c, a[i]); 2: pow(a[i], b[i]).
// out may alias a or b.
template <int MODE, bool EXACT>
__global__ __launch_bounds__(kBlock) void pow_lds_kernel(const float* a, const float* b, float* out, uint32_t n, float c) {
    constexpr int kLogDoubles = 2 * kLogTableEntries;
    __shared__ double tab[2 * kLogDoubles + kExpTableEntries];       // {1/c, ln c}, 2^(i/128), {1/c, log2 c}
    const uint32_t n4 = n >> 2;
    const uint32_t base = blockIdx.x * (kBlock * kLdsUnroll) + threadIdx.x;
    float4 v[kLdsUnroll], w[kLdsUnroll];
#pragma unroll
    for (int k = 0; k < kLdsUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) { v[k] = ld4(a, i); if (MODE == 2) w[k] = ld4(b, i); }
    }
    stage_table(tab, reinterpret_cast<const double*>(g_log_table), kLogDoubles);
    stage_table(tab + kLogDoubles, g_exp_table, kExpTableEntries);
    stage_table(tab + kLogDoubles + kExpTableEntries, reinterpret_cast<const double*>(g_log2_table), kLogDoubles);
    __syncthreads();
    const LogEntry* log_tab = reinterpret_cast<const LogEntry*>(tab);
    const double* exp_tab = tab + kLogDoubles;
    const Log2Entry* log2_tab = reinterpret_cast<const Log2Entry*>(tab + kLogDoubles + kExpTableEntries);
    auto one = [&](float x, float y) {
        const float base_ = MODE == 1 ? c : x, expo = MODE == 1 ? x : MODE == 2 ? y : c;
        return EXACT ? pow_short_then_long(base_, expo, log2_tab, log_tab, exp_tab) : pow_within_2_ulp(base_, expo, log2_tab, log_tab, exp_tab);
    };
    // four elements through the short routine, then one branch for the lanes of the wave it leaves open
    auto four = [&](float4 x, float4 y) {
        const float xs[4] = {x.x, x.y, x.z, x.w}, ys[4] = {y.x, y.y, y.z, y.w};
        float rs[4];
        bool open[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float base_ = MODE == 1 ? c : xs[j];
            const float expo = MODE == 1 ? xs[j] : MODE == 2 ? ys[j] : c;
            double val;
            const bool ok = fast_pow<!EXACT>(base_, expo, log2_tab, exp_tab, val);
            rs[j] = static_cast<float>(val);
            open[j] = EXACT ? !(ok && rounds_safely(val)) : !(ok && val >= 0x1p-126);
        }
        if (open[0] | open[1] | open[2] | open[3]) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float base_ = MODE == 1 ? c : xs[j];
                const float expo = MODE == 1 ? xs[j] : MODE == 2 ? ys[j] : c;
                if (open[j]) rs[j] = pow_with_tables(base_, expo, log_tab, exp_tab);
            }
        }
        return make_float4(rs[0], rs[1], rs[2], rs[3]);
    };
#pragma unroll
    for (int k = 0; k < kLdsUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) st4(out, i, four(v[k], MODE == 2 ? w[k] : v[k]));
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        uint32_t i = (n4 << 2) + threadIdx.x;
        out[i] = one(a[i], MODE == 2 ? b[i] : 0.0f);
    }
}

// out[i] = REV ? Op(c, a[i]) : Op(a[i], c). out may alias a.
template <class Op, bool REV>
__global__ __launch_bounds__(kBlock) void scalar_kernel(const float* a, float* out, uint32_t n, float c, float eps) {
    const uint32_t n4 = n >> 2;
    const uint32_t base = blockIdx.x * kTile + threadIdx.x;
    float4 v[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) v[k] = ld4(a, i);
    }
#pragma unroll
    for (int k = 0; k < kUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) {
            float4 r;
            if (REV) {
                r.x = Op::apply(c, v[k].x, eps); r.y = Op::apply(c, v[k].y, eps);
                r.z = Op::apply(c, v[k].z, eps); r.w = Op::apply(c, v[k].w, eps);
            } else {
                r.x = Op::apply(v[k].x, c, eps); r.y = Op::apply(v[k].y, c, eps);
                r.z = Op::apply(v[k].z, c, eps); r.w = Op::apply(v[k].w, c, eps);
            }
            st4(out, i, r);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        uint32_t i = (n4 << 2) + threadIdx.x;
        out[i] = REV ? Op::apply(c, a[i], eps) : Op::apply(a[i], c, eps);
    }
}

// out[i] = Op(a[i], b[i]). out may alias a or b.
template <class Op>
__global__ __launch_bounds__(kBlock) void binary_same_kernel(const float* a, const float* b, float* out, uint32_t n, float eps) {
    const uint32_t n4 = n >> 2;
    const uint32_t base = blockIdx.x * kTile + threadIdx.x;
    float4 va[kUnroll], vb[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) { va[k] = ld4(a, i); vb[k] = ld4(b, i); }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) {
            float4 r;
            r.x = Op::apply(va[k].x, vb[k].x, eps); r.y = Op::apply(va[k].y, vb[k].y, eps);
            r.z = Op::apply(va[k].z, vb[k].z, eps); r.w = Op::apply(va[k].w, vb[k].w, eps);
            st4(out, i, r);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        uint32_t i = (n4 << 2) + threadIdx.x;
        out[i] = Op::apply(a[i], b[i], eps);
    }
}

__global__ __launch_bounds__(kBlock) void fill_kernel(float* out, uint32_t n, float v) {
    // `out` may start at any element offset, so the float4 body begins at the first
    // 16-byte aligned element.
    const uint32_t head = static_cast<uint32_t>((4u - ((reinterpret_cast<uintptr_t>(out) >> 2) & 3u)) & 3u);
    const uint32_t h = head < n ? head : n;
    float* body = out + h;
    const uint32_t nb = n - h;
    const uint32_t n4 = nb >> 2;
    const uint32_t base = blockIdx.x * kTile + threadIdx.x;
    const float4 v4 = make_float4(v, v, v, v);
#pragma unroll
    for (int k = 0; k < kUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) st4(body, i, v4);
    }
    if (blockIdx.x == 0) {
        if (threadIdx.x < h) out[threadIdx.x] = v;
        if (threadIdx.x < (nb & 3u)) body[(n4 << 2) + threadIdx.x] = v;
    }
}

// ---------------------------------------------------------------- broadcast

// The broadcast plan travels by value in the kernel arguments. Dim 0 is the innermost
// coalesced dim. For the vector kernels dim 0 is counted in float4s and an operand's
// dim-0 stride is 4 (contiguous) or 0 (broadcast along it); all strides are in floats.
struct BcastPlan {
    int      ndim;
    uint32_t size[KTH_MAX_DIMS];
    FastDiv  div[KTH_MAX_DIMS];
    uint32_t astride[KTH_MAX_DIMS];
    uint32_t bstride[KTH_MAX_DIMS];
    bool     a_stream, b_stream;     // operand has as many elements as the output
    // Tile order of the vector kernel. 0: tiles in the order of the output. Otherwise the output is `repeats` slices of
    // `slice` units (the dims inside some dim along which an operand repeats; that dim and those outside it number the
    // slices), a slice is cut into equal chunks of chunk_tiles tiles, and the tiles run chunk by chunk: the chunk of slice 0,
    // the same chunk of slice 1, ... Each XCD takes a contiguous share of that sequence, so that the part of an operand
    // which one slice shares with the next is read from memory once and found in the XCD's L2 by the slices that follow.
    uint32_t repeats, slice, slice_tiles, tiles, per_xcd, chunk_tiles;
    FastDiv  group_div, chunk_div;   // by repeats * chunk_tiles, by chunk_tiles
};

__device__ __forceinline__ void decompose(const BcastPlan& pl, uint32_t idx, uint32_t& aoff, uint32_t& boff) {
    aoff = 0; boff = 0;
    for (int d = 0; d < pl.ndim - 1; d++) {
        uint32_t q = (__umulhi(idx, pl.div[d].mul) + idx) >> pl.div[d].shift;
        uint32_t r = idx - q * pl.size[d];
        aoff += r * pl.astride[d];
        boff += r * pl.bstride[d];
        idx = q;
    }
    aoff += idx * pl.astride[pl.ndim - 1];
    boff += idx * pl.bstride[pl.ndim - 1];
}

// STREAM: the operand is as large as the output (read once): non-temporal load.
// Otherwise it is a small broadcast operand that every workgroup re-reads: cached load.
template <bool VEC>
__device__ __forceinline__ float4 ld_operand(const float* p, uint32_t off, bool stream) {
    if (VEC) {
        if (stream) return ld4(p + off, 0);
        return *reinterpret_cast<const float4*>(p + off);
    }
    float s = p[off];
    return make_float4(s, s, s, s);
}

// out[o] = Op(a[map_a(o)], b[map_b(o)]) over n4 float4s of the output, innermost dim
// a multiple of 4. AV / BV: the operand is contiguous along the innermost dim (float4
// load) or broadcast along it (one scalar load per float4, served by L2).
template <class Op, bool AV, bool BV>
__global__ __launch_bounds__(kBlock) void binary_bcast_vec_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                                  float* __restrict__ out, uint32_t n4, float eps, BcastPlan pl) {
    uint32_t base = blockIdx.x * kBcastTile + threadIdx.x;
    if (pl.repeats) {
        const uint32_t t = (blockIdx.x & 7u) * pl.per_xcd + (blockIdx.x >> 3);
        if (t >= pl.tiles) return;
        const uint32_t chunk = (__umulhi(t, pl.group_div.mul) + t) >> pl.group_div.shift;
        const uint32_t in_group = t - chunk * pl.repeats * pl.chunk_tiles;
        const uint32_t rep = (__umulhi(in_group, pl.chunk_div.mul) + in_group) >> pl.chunk_div.shift;
        const uint32_t tile = chunk * pl.chunk_tiles + (in_group - rep * pl.chunk_tiles);
        if (tile >= pl.slice_tiles) return;                  // the last chunk of a slice may be short
        const uint32_t inner = tile * kBcastTile + threadIdx.x;
        base = rep * pl.slice + inner;
        n4 = min(n4, rep * pl.slice + pl.slice);             // the tile ends with its slice
    }
    float4 va[kBcastUnroll], vb[kBcastUnroll];
    // an operand of a small tensor (under 32 MB) is worth keeping in the caches: whoever made it or reads it next is near
    const bool big = n4 >= (2u << 20);
#pragma unroll
    for (int k = 0; k < kBcastUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) {
            uint32_t ao, bo;
            decompose(pl, i, ao, bo);
            va[k] = ld_operand<AV>(a, ao, pl.a_stream && big);
            vb[k] = ld_operand<BV>(b, bo, pl.b_stream && big);
        }
    }
#pragma unroll
    for (int k = 0; k < kBcastUnroll; k++) {
        uint32_t i = base + k * kBlock;
        if (i < n4) {
            float4 r;
            r.x = Op::apply(va[k].x, vb[k].x, eps); r.y = Op::apply(va[k].y, vb[k].y, eps);
            r.z = Op::apply(va[k].z, vb[k].z, eps); r.w = Op::apply(va[k].w, vb[k].w, eps);
            st4(out, i, r);
        }
    }
}

// Outermost dims taken off a broadcast and run as the grid's y and z: batch item (y, z) is the same problem on the
// operands and the output moved by these strides (in floats; 0 where an operand does not have the dim).
struct Batch { uint32_t a[2], b[2], out[2]; };

__device__ __forceinline__ void move_to_batch_item(const Batch& bt, const float*& a, const float*& b, float*& out) {
    a += static_cast<size_t>(blockIdx.y) * bt.a[0] + static_cast<size_t>(blockIdx.z) * bt.a[1];
    b += static_cast<size_t>(blockIdx.y) * bt.b[0] + static_cast<size_t>(blockIdx.z) * bt.b[1];
    out += static_cast<size_t>(blockIdx.y) * bt.out[0] + static_cast<size_t>(blockIdx.z) * bt.out[1];
}

// Four values of an operand at offsets off, off + stride, ... (stride in elements).
typedef float v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));
__device__ __forceinline__ void gather4(const float* __restrict__ p, uint32_t off, uint32_t stride, float (&v)[4]) {
    if (stride == 0) {
        const float x = p[off];
        v[0] = x; v[1] = x; v[2] = x; v[3] = x;
    } else if (stride == 1) {
        const v4f_unaligned x = *reinterpret_cast<const v4f_unaligned*>(p + off);
        v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    } else {
        v[0] = p[off]; v[1] = p[off + stride]; v[2] = p[off + 2 * stride]; v[3] = p[off + 3 * stride];
    }
}

// Any shapes, four consecutive outputs per (thread, k): the output and every operand that
// has the output's element count (AL / BL: it is then laid out exactly like the output) move
// as float4; a broadcast operand is gathered element by element through the plan (dim 0 in
// elements), which the caches serve. The last, partial group of four is done by elements.
template <class Op, bool AL, bool BL>
__global__ __launch_bounds__(kBlock) void binary_bcast_mixed_kernel(const float* __restrict__ a_, const float* __restrict__ b_,
                                                                   float* __restrict__ out_, uint32_t n, float eps, BcastPlan pl, Batch bt) {
    const float* a = a_; const float* b = b_; float* out = out_;
    move_to_batch_item(bt, a, b, out);          // (a batched launch has items of a multiple of 4 floats: the float4s stay aligned)
    const bool batched = bt.out[1] != 0;
    const uint32_t base = blockIdx.x * kBcastTile + threadIdx.x;
#pragma unroll
    for (int k = 0; k < kBcastUnroll; k++) {
        const uint32_t e0 = (base + k * kBlock) * 4;
        if (e0 >= n) continue;
        if (e0 + 4 <= n) {
            float va[4], vb[4];
            // an operand laid out like the output: read once in a plain launch (streaming load); in a batched one every
            // batch item reads it again, so it is loaded through the caches
            if (AL) { const float4 v = batched ? reinterpret_cast<const float4*>(a)[e0 >> 2] : ld4(a, e0 >> 2); va[0] = v.x; va[1] = v.y; va[2] = v.z; va[3] = v.w; }
            if (BL) { const float4 v = batched ? reinterpret_cast<const float4*>(b)[e0 >> 2] : ld4(b, e0 >> 2); vb[0] = v.x; vb[1] = v.y; vb[2] = v.z; vb[3] = v.w; }
            // The four outputs are neighbours along dim 0 unless they cross its end. Then a broadcast
            // operand that does not vary along dim 0 needs one load for all four, and one that is
            // contiguous there one 16-byte load from a 4-byte aligned address: four single loads at
            // lane stride 16 would each sweep the same eight cache lines.
            uint32_t ao0, bo0;
            decompose(pl, e0, ao0, bo0);
            uint32_t r0 = e0;
            if (pl.ndim > 1) r0 = e0 - ((__umulhi(e0, pl.div[0].mul) + e0) >> pl.div[0].shift) * pl.size[0];
            if (pl.ndim == 1 || r0 + 3 < pl.size[0]) {
                if (!AL) gather4(a, ao0, pl.astride[0], va);
                if (!BL) gather4(b, bo0, pl.bstride[0], vb);
            } else {
                // ... they cross its end: the offsets step along dim 0 and are worked out anew only where it ends
                uint32_t ao = ao0, bo = bo0, r = r0;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (j > 0) {
                        if (++r == pl.size[0]) { r = 0; decompose(pl, e0 + j, ao, bo); }
                        else { ao += pl.astride[0]; bo += pl.bstride[0]; }
                    }
                    if (!AL) va[j] = a[ao];
                    if (!BL) vb[j] = b[bo];
                }
            }
            float4 r;
            r.x = Op::apply(va[0], vb[0], eps); r.y = Op::apply(va[1], vb[1], eps);
            r.z = Op::apply(va[2], vb[2], eps); r.w = Op::apply(va[3], vb[3], eps);
            st4(out, e0 >> 2, r);
        } else {
            for (uint32_t e = e0; e < n; e++) {
                uint32_t ao, bo;
                decompose(pl, e, ao, bo);
                out[e] = Op::apply(a[ao], b[bo], eps);
            }
        }
    }
}

// ---------------------------------------------------------------- both operands small: out[i][j][v] = Op(row[i][v], col[j][v])

// The broadcast of two operands that are both smaller than the output, in the shape every such pair coalesces to
// when it is two- or three-dimensional: [N,1] o [1,M] (V = 1), or the same with an innermost run of V floats that
// both operands keep ([N,1,V] o [M,V]) or that the row operand alone keeps ([N,1,V] o [1,M,1]: the column operand then holds
// one value per column index, and the tile's window of them goes into LDS). The mixed kernel pays a vector-memory instruction per operand element
// there, and the address unit of a compute unit takes a wave's memory instruction for about 16 cycles whatever it
// moves: 8 loads and a store per 256 outputs hold it to 2.3-3.8 TB/s. Here a workgroup owns 4096 consecutive
// outputs, brings the slices of both operands that the span touches into LDS with 16-byte loads (the row operand's
// rows i_lo..i_hi as one range; the column operand whole when it is no longer than the span, while a longer one
// is read from memory 16 bytes per thread), and every thread then resolves the position of its four
// outputs with one division pair and steps through them, reading both operands from LDS: one store and less
// than one load instruction per 256 outputs reach the address unit.
constexpr uint32_t kOuterTile = 8192;            // outputs per workgroup
constexpr uint32_t kOuterMaxRun = 1024;          // longest innermost run V

struct OuterPlan {
    uint32_t n;                  // outputs
    uint32_t run;                // V
    uint32_t span;               // M * V: outputs per row index
    uint32_t a_is_row;           // operand a is indexed by [i][v], b by [j][v]; or the other way round
    uint32_t row_lds;            // floats of LDS for the row operand's slice; the column operand's follows
    uint32_t col_flat;           // the column operand holds one value per column index j, not a run: [N,1,V] o [1,M,1]
    uint32_t cols;               // M
    FastDiv  span_div, run_div;
};

// LDS[0 .. count) = src[first .. first + count): 16-byte loads from dword addresses, float stores into LDS
// at `at` (any offset).
__device__ __forceinline__ void stage_range(float* lds, uint32_t at, const float* __restrict__ src, uint32_t first, uint32_t count) {
    for (uint32_t u = threadIdx.x * 4; u < count; u += kBlock * 4) {
        if (u + 4 <= count) {
            const v4f_unaligned x = *reinterpret_cast<const v4f_unaligned*>(src + first + u);
            lds[at + u] = x.x; lds[at + u + 1] = x.y; lds[at + u + 2] = x.z; lds[at + u + 3] = x.w;
        } else {
            for (uint32_t j = u; j < count; j++) lds[at + j] = src[first + j];
        }
    }
}

// A_ROW: operand a is the row operand (pl.a_is_row). RUN1: V = 1 (pl.run == 1, hence not pl.col_flat): no position
// inside a run to keep track of. Both are facts of the launch; as template arguments they take the operand swap (for a
// division: the second division) and the run's bookkeeping out of the loop over a thread's outputs.
template <class Op, bool A_ROW, bool RUN1>
__global__ __launch_bounds__(kBlock) void binary_outer_kernel(const float* __restrict__ a_, const float* __restrict__ b_,
                                                             float* __restrict__ out_, float eps, OuterPlan pl, Batch bt) {
    const float* a = a_; const float* b = b_; float* out = out_;
    move_to_batch_item(bt, a, b, out);
    if (RUN1) { pl.run = 1; pl.col_flat = 0; }
    // sized at launch to what the shape needs (at most 56 KiB), so that short operands leave room for eight workgroups per CU
    extern __shared__ float outer_lds[];
    float* row_lds = outer_lds;
    float* col_lds = outer_lds + pl.row_lds;
    const float* rowp = A_ROW ? a : b;
    const float* colp = A_ROW ? b : a;
    const uint32_t s = blockIdx.x * kOuterTile;
    const uint32_t len = min(kOuterTile, pl.n - s);
    const uint32_t i_lo = (__umulhi(s, pl.span_div.mul) + s) >> pl.span_div.shift;
    const uint32_t last = s + len - 1;
    const uint32_t i_hi = (__umulhi(last, pl.span_div.mul) + last) >> pl.span_div.shift;
    stage_range(row_lds, 0, rowp, i_lo * pl.run, (i_hi - i_lo + 1) * pl.run);
    // the column operand: staged whole when it is no longer than the span; a longer one is read from memory,
    // 16 bytes per thread (its four outputs are neighbours there too, except where the span passes its end)
    const bool staged = pl.col_flat || pl.span <= len;
    // one value per column index: the indexes the tile meets are consecutive (past the last one the first follows)
    uint32_t j_lo = 0;
    if (pl.col_flat) {
        const uint32_t c_lo = s - i_lo * pl.span;
        const uint32_t window = min(pl.cols, len / pl.run + 2u);
        if (window < pl.cols) j_lo = (__umulhi(c_lo, pl.run_div.mul) + c_lo) >> pl.run_div.shift;
        for (uint32_t t = threadIdx.x; t < window; t += kBlock) col_lds[t] = colp[j_lo + t < pl.cols ? j_lo + t : j_lo + t - pl.cols];
    } else if (staged) stage_range(col_lds, 0, colp, 0, pl.span);
    // a column operand read from memory: all of a thread's loads are issued before the first is used
    constexpr uint32_t kGroups = kOuterTile / (kBlock * 4);
    v4f_unaligned ahead[kGroups];
    if (!staged) {
#pragma unroll
        for (uint32_t k = 0; k < kGroups; k++) {
            const uint32_t g = threadIdx.x * 4 + k * kBlock * 4;
            if (g < len) {
                const uint32_t e0 = s + g;
                const uint32_t i = (__umulhi(e0, pl.span_div.mul) + e0) >> pl.span_div.shift;
                const uint32_t c = e0 - i * pl.span;
                if (c + 4 <= pl.span) ahead[k] = *reinterpret_cast<const v4f_unaligned*>(colp + c);
                else {
                    float t[4];
#pragma unroll
                    for (uint32_t j = 0; j < 4; j++) t[j] = colp[c + j < pl.span ? c + j : c + j - pl.span];
                    ahead[k] = v4f_unaligned{t[0], t[1], t[2], t[3]};
                }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < kGroups; k++) {
        const uint32_t g = threadIdx.x * 4 + k * kBlock * 4;
        if (g >= len) break;
        const uint32_t e0 = s + g;
        const uint32_t i = (__umulhi(e0, pl.span_div.mul) + e0) >> pl.span_div.shift;
        uint32_t c = e0 - i * pl.span;                                     // column operand offset j * V + v
        uint32_t col = RUN1 ? c : (__umulhi(c, pl.run_div.mul) + c) >> pl.run_div.shift;   // column index j
        uint32_t v = RUN1 ? 0u : c - col * pl.run;
        uint32_t row_base = (i - i_lo) * pl.run;
        float y[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (!staged) { y[0] = ahead[k].x; y[1] = ahead[k].y; y[2] = ahead[k].z; y[3] = ahead[k].w; }
        float r[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float x = row_lds[row_base + v];
            const float yy = pl.col_flat ? col_lds[col >= j_lo ? col - j_lo : col + pl.cols - j_lo] : staged ? col_lds[c] : y[j];
            r[j] = A_ROW ? Op::apply(x, yy, eps) : Op::apply(yy, x, eps);
            c++;
            if (!RUN1) { v++; if (v == pl.run) { v = 0; col++; } }
            if (c == pl.span) { c = 0; col = 0; row_base += pl.run; }
        }
        // (16 bytes at a dword address: a batch item may start anywhere)
        if (g + 4 <= len) *reinterpret_cast<v4f_unaligned*>(out + e0) = v4f_unaligned{r[0], r[1], r[2], r[3]};
        else for (uint32_t j = 0; g + j < len; j++) out[e0 + j] = r[j];
    }
}

// The same operands when the column operand is longer than a tile (span > kOuterTile): a workgroup takes a
// block of kOuterRows row indexes by kOuterCols column offsets, so that a thread's 16 bytes of the column operand
// are loaded once and serve kOuterRows output rows, and nothing but the row index changes between its stores.
// The rows' slice of the row operand (kOuterRows * run floats) is staged in LDS. Grid: (column blocks, row blocks).
constexpr uint32_t kOuterRows = 8;
constexpr uint32_t kOuterCols = kOuterTile / kOuterRows;      // 1024 column offsets: four per thread
template <class Op, bool A_ROW>
__global__ __launch_bounds__(kBlock) void binary_outer_rows_kernel(const float* __restrict__ a_, const float* __restrict__ b_,
                                                                  float* __restrict__ out_, float eps, OuterPlan pl, uint32_t rows, Batch bt) {
    // (the grid's y counts row blocks here: one batch dim, on z)
    const float* a = a_ + static_cast<size_t>(blockIdx.z) * bt.a[1];
    const float* b = b_ + static_cast<size_t>(blockIdx.z) * bt.b[1];
    float* out = out_ + static_cast<size_t>(blockIdx.z) * bt.out[1];
    extern __shared__ float outer_rows_lds[];
    const float* rowp = A_ROW ? a : b;
    const float* colp = A_ROW ? b : a;
    const uint32_t i0 = blockIdx.y * kOuterRows;
    const uint32_t nrows = min(kOuterRows, rows - i0);
    const uint32_t c0 = blockIdx.x * kOuterCols + threadIdx.x * 4;
    float y[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t count = 0;                                        // column offsets of this thread inside the span
    if (c0 < pl.span) {
        count = min(4u, pl.span - c0);
        if (pl.col_flat) {
            for (uint32_t j = 0; j < count; j++) y[j] = colp[(__umulhi(c0 + j, pl.run_div.mul) + c0 + j) >> pl.run_div.shift];
        } else if (count == 4) {
            const v4f_unaligned t = *reinterpret_cast<const v4f_unaligned*>(colp + c0);
            y[0] = t.x; y[1] = t.y; y[2] = t.z; y[3] = t.w;
        } else {
            for (uint32_t j = 0; j < count; j++) y[j] = colp[c0 + j];
        }
    }
    stage_range(outer_rows_lds, 0, rowp, i0 * pl.run, nrows * pl.run);
    __syncthreads();
    if (count == 0) return;
    uint32_t v[4];
    v[0] = c0 - ((__umulhi(c0, pl.run_div.mul) + c0) >> pl.run_div.shift) * pl.run;
#pragma unroll
    for (int j = 1; j < 4; j++) { v[j] = v[j - 1] + 1; if (v[j] == pl.run) v[j] = 0; }
    for (uint32_t r = 0; r < nrows; r++) {
        const float* xs = outer_rows_lds + r * pl.run;
        float res[4];
#pragma unroll
        for (int j = 0; j < 4; j++) res[j] = A_ROW ? Op::apply(xs[v[j]], y[j], eps) : Op::apply(y[j], xs[v[j]], eps);
        float* to = out + static_cast<size_t>(i0 + r) * pl.span + c0;
        if (count == 4) *reinterpret_cast<v4f_unaligned*>(to) = v4f_unaligned{res[0], res[1], res[2], res[3]};
        else for (uint32_t j = 0; j < count; j++) to[j] = res[j];
    }
}

struct OpFirst { static constexpr const char* name = "OpFirst"; static __device__ __forceinline__ float apply(float a, float, float) { return a; } };
// maskedFill (JVMRawTensor.kt:537-540): the fill value rides in the third argument.
struct OpMaskedFill { static constexpr const char* name = "OpMaskedFill"; static __device__ __forceinline__ float apply(float a, float m, float value) { return m == 1.0f ? value : a; } };

// ---------------------------------------------------------------- NaN scan

__global__ __launch_bounds__(kBlock) void contains_nan_kernel(const float* __restrict__ a, uint32_t n, int* flag) {
    const uint32_t n4 = n >> 2;
    int found = 0;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n4; i += gridDim.x * kBlock) {
        float4 v = ld4(a, i);
        found |= (v.x != v.x) | (v.y != v.y) | (v.z != v.z) | (v.w != v.w);
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) {
        float v = a[(n4 << 2) + threadIdx.x];
        found |= (v != v);
    }
    // Every writer stores the same value, so plain stores need no atomics.
    if (__syncthreads_or(found) && threadIdx.x == 0) *flag = 1;
}

__global__ void clear_flag_kernel(int* flag) { *flag = 0; }

// ---------------------------------------------------------------- host side

inline uint32_t blocks_for(uint64_t vec_count) {
    uint64_t b = (vec_count + kTile - 1) / kTile;
    return static_cast<uint32_t>(b == 0 ? 1 : b);
}

// Builds the coalesced broadcast plan for out = a (op) b. Returns false when an operand
// does not broadcast to oshape (ShapeFunctions.kt:187-201).
// On return plan.size[0] is in elements; *vec_ok says whether the float4 kernels apply.
bool build_plan(const int32_t* ashape, int adims, const int32_t* bshape, int bdims,
                const int32_t* oshape, int odims, BcastPlan* plan, bool* vec_ok, bool* a_vec, bool* b_vec) {
    if (adims > odims || bdims > odims) return false;
    // Right-aligned, left-padded shapes and row-major strides with 0 on broadcast dims.
    int64_t osz[KTH_MAX_DIMS], ast[KTH_MAX_DIMS], bst[KTH_MAX_DIMS];
    int64_t arun = 1, brun = 1;
    for (int d = odims - 1; d >= 0; d--) {
        int ad = d - (odims - adims), bd = d - (odims - bdims);
        int64_t as = ad >= 0 ? ashape[ad] : 1, bs = bd >= 0 ? bshape[bd] : 1, os = oshape[d];
        if (!(as == os || as == 1) || !(bs == os || bs == 1)) return false;
        osz[d] = os;
        ast[d] = (as == 1 && os != 1) ? 0 : arun;
        bst[d] = (bs == 1 && os != 1) ? 0 : brun;
        arun *= as; brun *= bs;
    }
    // Innermost-first list without size-1 dims, then merge a dim into the one inside
    // it when both operands step through them as through one longer dim.
    int n = 0;
    int64_t sz[KTH_MAX_DIMS], sa[KTH_MAX_DIMS], sb[KTH_MAX_DIMS];
    for (int d = odims - 1; d >= 0; d--) {
        if (osz[d] == 1) continue;
        if (n > 0 && ast[d] == sa[n - 1] * sz[n - 1] && bst[d] == sb[n - 1] * sz[n - 1]) {
            sz[n - 1] *= osz[d];
        } else {
            sz[n] = osz[d]; sa[n] = ast[d]; sb[n] = bst[d]; n++;
        }
    }
    if (n == 0) { sz[0] = 1; sa[0] = 1; sb[0] = 1; n = 1; }
    plan->ndim = n;
    for (int d = 0; d < n; d++) {
        plan->size[d] = static_cast<uint32_t>(sz[d]);
        plan->astride[d] = static_cast<uint32_t>(sa[d]);
        plan->bstride[d] = static_cast<uint32_t>(sb[d]);
        plan->div[d] = make_div(plan->size[d]);
    }
    *a_vec = (sa[0] == 1);
    *b_vec = (sb[0] == 1);
    *vec_ok = (sz[0] % 4 == 0) && (sa[0] <= 1) && (sb[0] <= 1);
    return true;
}

void to_vector_units(BcastPlan* plan) {
    plan->size[0] /= 4;
    plan->div[0] = make_div(plan->size[0]);
    plan->astride[0] *= 4;
    plan->bstride[0] *= 4;
}

int check_shape(const int32_t* shape, int dims, const char* what, uint64_t* count) {
    if (dims < 0 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "%s: %d dims (max %d)", what, dims, KTH_MAX_DIMS);
    if (dims > 0 && !shape) return fail(KTH_E_ARGUMENT, "%s: null shape", what);
    uint64_t n = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0) return fail(KTH_E_ARGUMENT, "%s: negative dim %d", what, shape[i]);
        n *= static_cast<uint64_t>(shape[i]);
        if (n > kMaxElements) return fail(KTH_E_ARGUMENT, "%s: more than 2^31-1 elements", what);
    }
    *count = n;
    return KTH_OK;
}

template <class Op>
void launch_unary(const float* a, float* out, uint32_t n, float p, float q) {
    LaunchScope scope("unary_kernel", Op::name, static_cast<uint64_t>(n) * 8);
    hipLaunchKernelGGL((unary_kernel<Op>), dim3(blocks_for(n >> 2)), dim3(kBlock), 0, state().stream, a, out, n, p, q);
}

template <class Op>
void launch_unary_lds(const float* a, float* out, uint32_t n) {
    LaunchScope scope("unary_lds_kernel", Op::name, static_cast<uint64_t>(n) * 8);
    const uint64_t tile = static_cast<uint64_t>(kBlock) * kLdsUnroll;
    const uint32_t blocks = static_cast<uint32_t>(((n >> 2) + tile - 1) / tile);
    hipLaunchKernelGGL((unary_lds_kernel<Op>), dim3(blocks == 0 ? 1 : blocks), dim3(kBlock), 0, state().stream, a, out, n);
}

template <class Op>
void launch_scalar(bool rev, const float* a, float* out, uint32_t n, float c, float eps) {
    LaunchScope scope(rev ? "scalar_kernel_rev" : "scalar_kernel", Op::name, static_cast<uint64_t>(n) * 8);
    if (rev) hipLaunchKernelGGL((scalar_kernel<Op, true>), dim3(blocks_for(n >> 2)), dim3(kBlock), 0, state().stream, a, out, n, c, eps);
    else     hipLaunchKernelGGL((scalar_kernel<Op, false>), dim3(blocks_for(n >> 2)), dim3(kBlock), 0, state().stream, a, out, n, c, eps);
}

// mode 0: a ^ c, 1: c ^ a, 2: a ^ b (see pow_lds_kernel)
void launch_pow(int mode, const float* a, const float* b, float* out, uint32_t n, float c) {
    LaunchScope scope(mode == 0 ? "pow_lds_kernel_scalar" : mode == 1 ? "pow_lds_kernel_scalar_rev" : "pow_lds_kernel", "OpPow",
                      static_cast<uint64_t>(n) * (mode == 2 ? 12 : 8));
    const uint64_t tile = static_cast<uint64_t>(kBlock) * kLdsUnroll;
    const uint32_t blocks = static_cast<uint32_t>(((n >> 2) + tile - 1) / tile);
    const dim3 grid(blocks == 0 ? 1 : blocks);
    if (state().math_mode == KTH_MATH_EXACT) {
        if (mode == 0)      hipLaunchKernelGGL((pow_lds_kernel<0, true>), grid, dim3(kBlock), 0, state().stream, a, b, out, n, c);
        else if (mode == 1) hipLaunchKernelGGL((pow_lds_kernel<1, true>), grid, dim3(kBlock), 0, state().stream, a, b, out, n, c);
        else                hipLaunchKernelGGL((pow_lds_kernel<2, true>), grid, dim3(kBlock), 0, state().stream, a, b, out, n, c);
    } else {
        if (mode == 0)      hipLaunchKernelGGL((pow_lds_kernel<0, false>), grid, dim3(kBlock), 0, state().stream, a, b, out, n, c);
        else if (mode == 1) hipLaunchKernelGGL((pow_lds_kernel<1, false>), grid, dim3(kBlock), 0, state().stream, a, b, out, n, c);
        else                hipLaunchKernelGGL((pow_lds_kernel<2, false>), grid, dim3(kBlock), 0, state().stream, a, b, out, n, c);
    }
}

template <class Op>
void launch_binary_same(const float* a, const float* b, float* out, uint32_t n, float eps) {
    LaunchScope scope("binary_same_kernel", Op::name, static_cast<uint64_t>(n) * 12);
    hipLaunchKernelGGL((binary_same_kernel<Op>), dim3(blocks_for(n >> 2)), dim3(kBlock), 0, state().stream, a, b, out, n, eps);
}

// Chooses the vector kernel's tile order (BcastPlan::repeats). In the order of the output, an operand that repeats
// along dim d is swept once per index of d, and what it holds inside d has to survive in L2 from one sweep to the
// next. Consecutive workgroups go to consecutive XCDs: when a sweep is a whole number of tiles and that a multiple
// of 8, every XCD meets the same eighth of the operand in every sweep and the eight L2s hold 8 MB of it between them
// (measured: [32,2048,1024] + [1,2048,1024] runs like an operand pair of equal shapes, 81 us; with 16 MB inside the
// dim 104 us); otherwise every XCD meets all of it and 2 MB is already too much ([128,511,1020] + [1,511,1020] 97 us,
// [32,2047,1020] + [1,2047,1020] 114 us). Beyond those sizes the slices are taken chunk by chunk (88, 84 and 91 us
// for the three; [1,6,4,56860] * [23,1,4,56860] 54 -> 28 us), from the innermost dim along which an operand repeats
// and inside which a slice is a chunk or more. The chunked order costs about 5 % where the plain one already works.
constexpr uint64_t kReuseAligned = 12ull << 20;      // bytes of an operand inside the dim it repeats along: sweeps of 8 k tiles
constexpr uint64_t kReuseUnaligned = 3ull << 19;     // ... other sweeps

void order_tiles_for_reuse(BcastPlan* plan, uint32_t n4, dim3* grid) {
    plan->repeats = 0;
    uint64_t a_inside = 1, b_inside = 1, slice = 1;          // units of a, of b and of the output inside dim d
    uint64_t from_slice = 0;
    bool pays = false, a_in_group = false, b_in_group = false;
    for (int d = 0; d < plan->ndim; d++) {
        const bool a_repeats = plan->astride[d] == 0 && plan->size[d] > 1, b_repeats = plan->bstride[d] == 0 && plan->size[d] > 1;
        const uint64_t slice_tiles = (slice + kBcastTile - 1) / kBcastTile;
        if ((a_repeats || b_repeats) && from_slice == 0 && d > 0 && (slice_tiles >> kReuseChunkShift) != 0) from_slice = slice;
        if (from_slice != 0) { a_in_group = a_in_group || a_repeats; b_in_group = b_in_group || b_repeats; }
        const uint64_t enough = (slice % kBcastTile == 0 && slice_tiles % 8 == 0) ? kReuseAligned : kReuseUnaligned;
        pays = pays || (a_repeats && a_inside * (plan->astride[0] ? 16 : 4) >= enough) || (b_repeats && b_inside * (plan->bstride[0] ? 16 : 4) >= enough);
        if (plan->astride[d] != 0) a_inside *= plan->size[d];
        if (plan->bstride[d] != 0) b_inside *= plan->size[d];
        slice *= plan->size[d];
    }
    if (!pays || from_slice == 0) return;
    // with both operands repeating, the slices between two uses of a tile bring their own tiles of the other operand
    const uint64_t longest = 1ull << ((a_in_group && b_in_group) ? kReuseChunkShift - 1 : kReuseChunkShift);
    const uint64_t repeats = n4 / from_slice;
    const uint64_t slice_tiles = (from_slice + kBcastTile - 1) / kBcastTile;
    // chunks of equal length, so that the slots past a slice's last tile are few and spread evenly (a last chunk of
    // 15 tiles out of 32 left the XCDs that took it idle for an eighth of the launch)
    const uint64_t chunks = (slice_tiles + longest - 1) / longest;
    const uint64_t chunk_tiles = (slice_tiles + chunks - 1) / chunks;
    const uint64_t tiles = chunks * chunk_tiles * repeats;
    if (repeats < 6 || tiles > 0xfffffff0ull) return;        // 4 repeats of 64 MB: 117 us against 115
    plan->repeats = static_cast<uint32_t>(repeats);
    plan->chunk_tiles = static_cast<uint32_t>(chunk_tiles);
    plan->chunk_div = make_div(plan->chunk_tiles);
    plan->group_div = make_div(static_cast<uint32_t>(repeats * chunk_tiles));
    plan->slice = static_cast<uint32_t>(from_slice);
    plan->slice_tiles = static_cast<uint32_t>(slice_tiles);
    plan->tiles = static_cast<uint32_t>(tiles);
    plan->per_xcd = static_cast<uint32_t>((tiles + 7) / 8);
    *grid = dim3(plan->per_xcd * 8);
}

// Whether the d innermost dims of `plan` (d = 2 or 3) are one of the shapes the outer-product kernels take, and the
// kernel plan for n outputs if so.
bool match_outer(const BcastPlan& plan, int d, uint32_t n, OuterPlan* op, uint32_t* rows) {
    if (d != 2 && d != 3) return false;
    const bool with_run = d == 3;
    const uint32_t run = with_run ? plan.size[0] : 1u;
    // the dim next to the outermost one is the column index, the outermost the row index
    bool run_ok = !with_run || (plan.astride[0] == 1 && plan.bstride[0] == 1 && run <= kOuterMaxRun);
    bool a_row = plan.astride[d - 2] == 0 && plan.astride[d - 1] == run && plan.bstride[d - 2] == run && plan.bstride[d - 1] == 0;
    bool b_row = plan.bstride[d - 2] == 0 && plan.bstride[d - 1] == run && plan.astride[d - 2] == run && plan.astride[d - 1] == 0;
    // or the row operand alone keeps the innermost run and the column operand holds one value per column index
    bool flat = false;
    if (with_run && !run_ok && run <= kOuterMaxRun) {
        const bool a_flat_row = plan.astride[0] == 1 && plan.astride[1] == 0 && plan.astride[2] == run &&
                                plan.bstride[0] == 0 && plan.bstride[1] == 1 && plan.bstride[2] == 0;
        const bool b_flat_row = plan.bstride[0] == 1 && plan.bstride[1] == 0 && plan.bstride[2] == run &&
                                plan.astride[0] == 0 && plan.astride[1] == 1 && plan.astride[2] == 0;
        flat = run_ok = a_flat_row || b_flat_row;
        a_row = a_flat_row; b_row = b_flat_row;
    }
    if (!(run_ok && (a_row || b_row) && plan.size[d - 2] >= 2)) return false;
    *op = OuterPlan{};
    op->n = n; op->run = run; op->span = plan.size[d - 2] * run; op->a_is_row = a_row ? 1u : 0u;
    op->col_flat = flat ? 1u : 0u; op->cols = plan.size[d - 2];
    op->span_div = make_div(op->span); op->run_div = make_div(run);
    op->row_lds = (((kOuterTile - 1) / op->span + 2) * run + 3u) & ~3u;
    *rows = plan.size[d - 1];
    return true;
}

template <class Op>
void launch_outer(const float* a, const float* b, float* out, float eps, const OuterPlan& op, uint32_t rows, uint64_t bytes,
                  const Batch& bt, uint32_t batch_y, uint32_t batch_z) {
    hipStream_t st = state().stream;
    if (op.span >= 2048u && rows <= 65535u * kOuterRows && batch_y == 1) {
        LaunchScope scope("binary_outer_rows_kernel", Op::name, bytes);
        const dim3 grid((op.span + kOuterCols - 1) / kOuterCols, (rows + kOuterRows - 1) / kOuterRows, batch_z);
        if (op.a_is_row) hipLaunchKernelGGL((binary_outer_rows_kernel<Op, true>), grid, dim3(kBlock), kOuterRows * op.run * sizeof(float), st, a, b, out, eps, op, rows, bt);
        else             hipLaunchKernelGGL((binary_outer_rows_kernel<Op, false>), grid, dim3(kBlock), kOuterRows * op.run * sizeof(float), st, a, b, out, eps, op, rows, bt);
        return;
    }
    const uint32_t col_lds = op.col_flat ? std::min(op.cols, kOuterTile / op.run + 2u)
                                         : op.span <= kOuterTile ? op.span : 4u;  // a longer column operand is not staged
    LaunchScope scope("binary_outer_kernel", Op::name, bytes);
    const dim3 grid((op.n + kOuterTile - 1) / kOuterTile, batch_y, batch_z);
    const size_t lds = (op.row_lds + col_lds) * sizeof(float);
    const bool run1 = op.run == 1 && !op.col_flat;
    if (op.a_is_row) {
        if (run1) hipLaunchKernelGGL((binary_outer_kernel<Op, true, true>), grid, dim3(kBlock), lds, st, a, b, out, eps, op, bt);
        else      hipLaunchKernelGGL((binary_outer_kernel<Op, true, false>), grid, dim3(kBlock), lds, st, a, b, out, eps, op, bt);
    } else {
        if (run1) hipLaunchKernelGGL((binary_outer_kernel<Op, false, true>), grid, dim3(kBlock), lds, st, a, b, out, eps, op, bt);
        else      hipLaunchKernelGGL((binary_outer_kernel<Op, false, false>), grid, dim3(kBlock), lds, st, a, b, out, eps, op, bt);
    }
}

template <class Op>
void launch_mixed(const float* a, const float* b, float* out, uint32_t n, float eps, const BcastPlan& plan, bool al, bool bl,
                  const Batch& bt, uint32_t batch_y, uint32_t batch_z) {
    hipStream_t st = state().stream;
    const uint64_t groups = (static_cast<uint64_t>(n) + 3) / 4;
    dim3 grid(static_cast<uint32_t>((groups + kBcastTile - 1) / kBcastTile), batch_y, batch_z), block(kBlock);
    if (al && bl)  hipLaunchKernelGGL((binary_bcast_mixed_kernel<Op, true, true>), grid, block, 0, st, a, b, out, n, eps, plan, bt);
    else if (al)   hipLaunchKernelGGL((binary_bcast_mixed_kernel<Op, true, false>), grid, block, 0, st, a, b, out, n, eps, plan, bt);
    else if (bl)   hipLaunchKernelGGL((binary_bcast_mixed_kernel<Op, false, true>), grid, block, 0, st, a, b, out, n, eps, plan, bt);
    else           hipLaunchKernelGGL((binary_bcast_mixed_kernel<Op, false, false>), grid, block, 0, st, a, b, out, n, eps, plan, bt);
}

template <class Op>
void launch_binary_bcast(const float* a, const float* b, float* out, uint32_t n, float eps,
                         BcastPlan plan, bool vec_ok, bool a_vec, bool b_vec, uint64_t bytes) {
    const Batch no_batch{};
    // Both operands smaller than the output, in the two- or three-dimensional outer-product shape, and the
    // innermost dim not a multiple of 4 (a multiple of 4 has the float4 kernels): the LDS-staged kernel.
    if (!vec_ok && !plan.a_stream && !plan.b_stream && n >= 4 * kOuterTile) {
        OuterPlan op; uint32_t rows;
        if (match_outer(plan, plan.ndim, n, &op, &rows)) { launch_outer<Op>(a, b, out, eps, op, rows, bytes, no_batch, 1, 1); return; }
        // Not that shape as a whole (four dims or more, a dim both operands keep outside one that only one keeps):
        // the one or two outermost dims become the grid's z and y, when what is left inside them is that shape, or a
        // broadcast in which one operand is as large as the item (the mixed kernel then moves it and the output
        // as float4s and has one small operand to gather: its fast path).
        for (int peel = 1; peel <= 2 && plan.ndim - peel >= 2; peel++) {
            const int d = plan.ndim - peel;
            uint64_t item = 1;
            for (int k = 0; k < d; k++) item *= plan.size[k];
            const uint32_t bz = plan.size[plan.ndim - 1], by = peel == 2 ? plan.size[plan.ndim - 2] : 1u;
            if (bz > 65535u || by > 65535u || item < 256) continue;
            Batch bt{};
            bt.a[1] = plan.astride[plan.ndim - 1]; bt.b[1] = plan.bstride[plan.ndim - 1];
            bt.out[1] = static_cast<uint32_t>(item * by);
            if (peel == 2) { bt.a[0] = plan.astride[plan.ndim - 2]; bt.b[0] = plan.bstride[plan.ndim - 2]; bt.out[0] = static_cast<uint32_t>(item); }
            if (match_outer(plan, d, static_cast<uint32_t>(item), &op, &rows)) {
                launch_outer<Op>(a, b, out, eps, op, rows, bytes, bt, by, bz);
                return;
            }
            // an operand that keeps every dim of the item is laid out like the item
            bool a_full = true, b_full = true;
            uint64_t dense = 1;
            for (int k = 0; k < d; k++) {
                a_full = a_full && plan.astride[k] == dense; b_full = b_full && plan.bstride[k] == dense;
                dense *= plan.size[k];
            }
            if ((a_full || b_full) && item % 4 == 0 && item >= 4096) {
                BcastPlan inner = plan;
                inner.ndim = d;
                inner.a_stream = a_full; inner.b_stream = b_full;
                LaunchScope scope("binary_bcast_mixed_kernel_batched", Op::name, bytes);
                launch_mixed<Op>(a, b, out, static_cast<uint32_t>(item), eps, inner, a_full, b_full, bt, by, bz);
                return;
            }
        }
    }
    hipStream_t st = state().stream;
    const uint32_t n4 = n >> 2;
    dim3 vec_grid(static_cast<uint32_t>((static_cast<uint64_t>(n4) + kBcastTile - 1) / kBcastTile));
    if (vec_ok) {
        to_vector_units(&plan);
        order_tiles_for_reuse(&plan, n4, &vec_grid);
    }
    const bool chunked = vec_ok && plan.repeats != 0;
    LaunchScope scope(!vec_ok ? "binary_bcast_mixed_kernel"
                      : (a_vec && b_vec) ? (chunked ? "binary_bcast_vec_kernel_vv_chunked" : "binary_bcast_vec_kernel_vv")
                      : a_vec ? (chunked ? "binary_bcast_vec_kernel_vs_chunked" : "binary_bcast_vec_kernel_vs")
                      : b_vec ? (chunked ? "binary_bcast_vec_kernel_sv_chunked" : "binary_bcast_vec_kernel_sv")
                      : "binary_bcast_vec_kernel_ss", Op::name, bytes);
    if (vec_ok) {
        const dim3 grid = vec_grid, block(kBlock);
        if (a_vec && b_vec)  hipLaunchKernelGGL((binary_bcast_vec_kernel<Op, true, true>), grid, block, 0, st, a, b, out, n4, eps, plan);
        else if (a_vec)      hipLaunchKernelGGL((binary_bcast_vec_kernel<Op, true, false>), grid, block, 0, st, a, b, out, n4, eps, plan);
        else if (b_vec)      hipLaunchKernelGGL((binary_bcast_vec_kernel<Op, false, true>), grid, block, 0, st, a, b, out, n4, eps, plan);
        else                 hipLaunchKernelGGL((binary_bcast_vec_kernel<Op, false, false>), grid, block, 0, st, a, b, out, n4, eps, plan);
    } else {
        launch_mixed<Op>(a, b, out, n, eps, plan, plan.a_stream, plan.b_stream, no_batch, 1, 1);
    }
}

#define KTH_BINARY_DISPATCH(op, CALL)                          \
    switch (op) {                                              \
    case KTH_PLUS:  CALL(OpPlus);  break;                      \
    case KTH_MINUS: CALL(OpMinus); break;                      \
    case KTH_TIMES: CALL(OpTimes); break;                      \
    case KTH_DIV:   CALL(OpDiv);   break;                      \
    case KTH_POW:   CALL(OpPowT);  break;                      \
    case KTH_LT:    CALL(OpLt);    break;                      \
    case KTH_LTE:   CALL(OpLte);   break;                      \
    case KTH_GT:    CALL(OpGt);    break;                      \
    case KTH_GTE:   CALL(OpGte);   break;                      \
    case KTH_EQ:    CALL(OpEq);    break;                      \
    case KTH_NEQ:   CALL(OpNeq);   break;                      \
    default: break;                                            \
    }

bool is_binary_op(int op) {
    return (op >= KTH_PLUS && op <= KTH_POW) || (op >= KTH_LT && op <= KTH_NEQ);
}

// The four single-rounding operations: a tensor operand that is one constant everywhere may be
// taken as the scalar operand of the same functor, with the same bits in the result.
bool folds_a_constant(int op) { return op >= KTH_PLUS && op <= KTH_DIV; }

// out = op(a, c), or op(c, a) with rev, through the scalar kernels.
void launch_scalar_op(int op, bool rev, const float* pa, float* po, uint32_t n32, float c, float eps) {
#define S(OP) launch_scalar<OP>(rev, pa, po, n32, c, eps)
    KTH_BINARY_DISPATCH(op, S)
#undef S
}

}  // namespace

namespace kth {
void launch_fill(float* p, uint64_t n, float value) {
    if (n == 0) return;
    const uint32_t n32 = static_cast<uint32_t>(n);
    LaunchScope scope("fill_kernel", "", n * 4);
    hipLaunchKernelGGL(fill_kernel, dim3(blocks_for(n32 >> 2)), dim3(kBlock), 0, state().stream, p, n32, value);
}
}  // namespace kth

extern "C" {

int kth_fill(uint64_t handle, uint64_t offset, uint64_t n, float value) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    Store* st = lookup_unsettled(handle, "kth_fill");
    if (!st) return KTH_E_HANDLE;
    if (offset > st->n_floats || n > st->n_floats - offset)
        return fail(KTH_E_ARGUMENT, "kth_fill: range [%llu, +%llu) outside a store of %llu floats",
                    (unsigned long long)offset, (unsigned long long)n, (unsigned long long)st->n_floats);
    if (n == 0) return KTH_OK;
    if (offset == 0) {
        // A fill of the store's head is only noted: whoever reads the store next either folds the
        // constant into its own kernel or has the fill launched first (kth_internal.h, Store::fill_n).
        settle_for_overwrite(st, n);
        st->fill_n = n; st->fill_value = value;
        return KTH_OK;
    }
    settle(st);
    launch_fill(st->ptr + offset, n, value);
    KTH_LAUNCH_CHECK("fill");
    return KTH_OK;
}

int kth_set_math_mode(int mode) {
    std::lock_guard<std::mutex> g(lock());
    if (mode != KTH_MATH_EXACT && mode != KTH_MATH_WITHIN_2_ULP)
        return fail(KTH_E_ARGUMENT, "kth_set_math_mode: %d is neither KTH_MATH_EXACT nor KTH_MATH_WITHIN_2_ULP", mode);
    state().math_mode = mode;
    return KTH_OK;
}

int kth_get_math_mode(int* mode) {
    std::lock_guard<std::mutex> g(lock());
    if (!mode) return fail(KTH_E_ARGUMENT, "kth_get_math_mode: null output");
    *mode = state().math_mode;
    return KTH_OK;
}

int kth_unary(int op, uint64_t a, uint64_t out, uint64_t n) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    Store* sa = lookup(a, "kth_unary(a)", true);
    if (!sa) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_unary(out)");
    if (!so) return KTH_E_HANDLE;
    if (n > sa->n_floats || n > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_unary: n=%llu exceeds a store (%llu in, %llu out)", (unsigned long long)n,
                    (unsigned long long)sa->n_floats, (unsigned long long)so->n_floats);
    const float* pa = sa->ptr; float* po = so->ptr; uint32_t n32 = static_cast<uint32_t>(n);
#define U(OP) if (n32) launch_unary<OP>(pa, po, n32, 0.0f, 0.0f)
    // T: a transcendental map. Mode "exact": the f64 routines behind LDS tables (the float kotlin.math returns, bit
    // for bit); mode "within 2 ulp": the fp32 routine through the plain kernel.
#define T(EXACT, FAST) if (n32) { if (exact) launch_unary_lds<EXACT>(pa, po, n32); else launch_unary<FAST>(pa, po, n32, 0.0f, 0.0f); }
    const bool exact = state().math_mode == KTH_MATH_EXACT;
    switch (op) {
    case KTH_NEG: U(OpNeg); break;           case KTH_RECIPROCAL: U(OpReciprocal); break;
    case KTH_LOG: T(OpLogT, OpLogF); break;
    case KTH_EXP: T(OpExpT, OpExpF); break;
    case KTH_TANH: T(OpTanhT, OpTanhF); break;
    case KTH_SIGMOID: if (n32) launch_unary_lds<OpSigmoidT>(pa, po, n32); break;
    case KTH_SINH: T(OpSinhT, OpSinhF); break;
    case KTH_COSH: T(OpCoshT, OpCoshF); break;
    case KTH_ABS: U(OpAbs); break;           case KTH_SIGN: U(OpSign); break;
    case KTH_SQRT: U(OpSqrt); break;
    case KTH_SIN: T(OpSinT, OpSinF); break;
    case KTH_COS: T(OpCosT, OpCosF); break;
    case KTH_TAN: T(OpTanT, OpTanF); break;
    case KTH_ASIN: T(OpAsinT, OpAsinF); break;
    case KTH_ACOS: T(OpAcosT, OpAcosF); break;
    case KTH_ATAN: T(OpAtanT, OpAtanF); break;
    case KTH_FLOOR: U(OpFloor); break;
    case KTH_CEIL: U(OpCeil); break;         case KTH_ROUND: U(OpRound); break;
    case KTH_TRUNC: U(OpTrunc); break;       case KTH_RSQRT: U(OpRsqrt); break;
    default: return fail(KTH_E_ARGUMENT, "kth_unary: op %d is not a unary map", op);
    }
#undef T
#undef U
    if (n == 0) return KTH_OK;
    KTH_LAUNCH_CHECK("unary");
    return KTH_OK;
}

int kth_clamp(uint64_t a, uint64_t out, uint64_t n, float lo, float hi) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    Store* sa = lookup(a, "kth_clamp(a)", true);
    if (!sa) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_clamp(out)");
    if (!so) return KTH_E_HANDLE;
    if (n > sa->n_floats || n > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_clamp: n=%llu exceeds a store", (unsigned long long)n);
    if (n == 0) return KTH_OK;
    launch_unary<OpClamp>(sa->ptr, so->ptr, static_cast<uint32_t>(n), lo, hi);
    KTH_LAUNCH_CHECK("clamp");
    return KTH_OK;
}

int kth_scalar(int op, uint64_t a, float c, int reverse, uint64_t out, uint64_t n) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!is_binary_op(op)) return fail(KTH_E_ARGUMENT, "kth_scalar: op %d is not a binary op", op);
    Store* sa = lookup_unsettled(a, "kth_scalar(a)", true);
    if (!sa) return KTH_E_HANDLE;
    Store* so = lookup_unsettled(out, "kth_scalar(out)");
    if (!so) return KTH_E_HANDLE;
    if (n > sa->n_floats || n > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_scalar: n=%llu exceeds a store", (unsigned long long)n);
    if (n == 0) return KTH_OK;
    // A constant times (plus, ...) a constant: the broadcast seed gradient times an exponent, a fresh
    // zerosLike plus a bias. The result is owed the folded constant; nothing is read or written now.
    float folded;
    if (folds_a_constant(op) && sa->fill_n >= n && (so != sa || sa->fill_n == n) &&
        fold_constants(op, reverse ? c : sa->fill_value, reverse ? sa->fill_value : c, &folded)) {
        if (so != sa) settle_for_overwrite(so, n);
        so->fill_n = n; so->fill_value = folded;
        return KTH_OK;
    }
    settle(sa);
    if (so != sa) settle_for_overwrite(so, n);
    const bool rev = reverse != 0;
    // pow(x, 1) into a store of its own (the backward pass of a square asks for it) is a copy, and a copy is put off
    // until one of the two stores is written
    if (op == KTH_POW && !rev && c == 1.0f && so != sa && n == so->n_floats) {
        make_alias(so, sa);
        return KTH_OK;
    }
    const float* pa = sa->ptr; float* po = so->ptr; uint32_t n32 = static_cast<uint32_t>(n);
    const float eps = state().epsilon;
    // pow with an exponent whose f64 result is exact or one correctly rounded operation needs no
    // transcendental: pow(x, 2) is the exact product x*x (48 bits fit a double), pow(x, 1) is x;
    // 3, 4, -1, -2 and 0.5 likewise.
    if (op == KTH_POW && !rev && c == 2.0f)      launch_unary<OpSquare>(pa, po, n32, 0.0f, 0.0f);
    else if (op == KTH_POW && !rev && c == 1.0f) launch_unary<OpIdentity>(pa, po, n32, 0.0f, 0.0f);
    else if (op == KTH_POW && !rev && c == 3.0f)  launch_unary<OpPowCube>(pa, po, n32, 0.0f, 0.0f);
    else if (op == KTH_POW && !rev && c == 4.0f)  launch_unary<OpPowFourth>(pa, po, n32, 0.0f, 0.0f);
    else if (op == KTH_POW && !rev && c == -1.0f) launch_unary<OpPowInverse>(pa, po, n32, 0.0f, 0.0f);
    else if (op == KTH_POW && !rev && c == 0.5f)  launch_unary<OpPowHalf>(pa, po, n32, 0.0f, 0.0f);
    else if (op == KTH_POW && !rev && c == -2.0f) launch_unary<OpPowInverseSquare>(pa, po, n32, 0.0f, 0.0f);
    else if (op == KTH_POW) launch_pow(rev ? 1 : 0, pa, nullptr, po, n32, c);
    else launch_scalar_op(op, rev, pa, po, n32, c, eps);
    KTH_LAUNCH_CHECK("scalar");
    return KTH_OK;
}

int kth_binary_inplace(int op, uint64_t a, uint64_t b, uint64_t n) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!is_binary_op(op)) return fail(KTH_E_ARGUMENT, "kth_binary_inplace: op %d is not a binary op", op);
    Store* sa = lookup_unsettled(a, "kth_binary_inplace(a)");
    if (!sa) return KTH_E_HANDLE;
    Store* sb = lookup_unsettled(b, "kth_binary_inplace(b)", true);
    if (!sb) return KTH_E_HANDLE;
    if (n > sa->n_floats || n > sb->n_floats)
        return fail(KTH_E_SHAPE, "kth_binary_inplace: n=%llu exceeds a store (%llu, %llu)", (unsigned long long)n,
                    (unsigned long long)sa->n_floats, (unsigned long long)sb->n_floats);
    if (n == 0) return KTH_OK;
    float* pa = sa->ptr; const float* pb = sb->ptr; uint32_t n32 = static_cast<uint32_t>(n);
    const float eps = state().epsilon;
    // An operand that is still an owed constant (a gradient buffer fresh from zerosLike, a broadcast
    // seed) rides as the scalar operand: one stream less to read, the same bits.
    if (folds_a_constant(op) && sa != sb && sb->fill_n >= n) {
        settle(sa);
        launch_scalar_op(op, false, pa, pa, n32, sb->fill_value, eps);
        KTH_LAUNCH_CHECK("binary_inplace");
        return KTH_OK;
    }
    if (folds_a_constant(op) && sa != sb && sa->fill_n == n) {
        const float c = sa->fill_value;
        sa->fill_n = 0;
        settle(sb);
        launch_scalar_op(op, true, pb, pa, n32, c, eps);
        KTH_LAUNCH_CHECK("binary_inplace");
        return KTH_OK;
    }
    settle(sa); settle(sb);
    if (op == KTH_POW) launch_pow(2, pa, pb, pa, n32, 0.0f);
    else {
#define B(OP) launch_binary_same<OP>(pa, pb, pa, n32, eps)
        KTH_BINARY_DISPATCH(op, B)
#undef B
    }
    KTH_LAUNCH_CHECK("binary_inplace");
    return KTH_OK;
}

int kth_binary(int op,
               uint64_t a, const int32_t* ashape, int adims,
               uint64_t b, const int32_t* bshape, int bdims,
               uint64_t out, const int32_t* oshape, int odims) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!is_binary_op(op)) return fail(KTH_E_ARGUMENT, "kth_binary: op %d is not a binary op", op);
    uint64_t an, bn, on;
    if (int rc = check_shape(ashape, adims, "kth_binary(a)", &an)) return rc;
    if (int rc = check_shape(bshape, bdims, "kth_binary(b)", &bn)) return rc;
    if (int rc = check_shape(oshape, odims, "kth_binary(out)", &on)) return rc;
    Store* sa = lookup_unsettled(a, "kth_binary(a)", true);
    if (!sa) return KTH_E_HANDLE;
    Store* sb = lookup_unsettled(b, "kth_binary(b)", true);
    if (!sb) return KTH_E_HANDLE;
    Store* so = lookup_unsettled(out, "kth_binary(out)");
    if (!so) return KTH_E_HANDLE;
    if (an > sa->n_floats || bn > sb->n_floats || on > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_binary: a shape needs more elements than its store holds");
    BcastPlan plan{};
    bool vec_ok, a_vec, b_vec;
    if (!build_plan(ashape, adims, bshape, bdims, oshape, odims, &plan, &vec_ok, &a_vec, &b_vec))
        return fail(KTH_E_SHAPE, "kth_binary: operand shapes do not broadcast to the output shape");
    const bool all_same = (an == on && bn == on);
    plan.a_stream = (an == on);
    plan.b_stream = (bn == on);
    if (!all_same && (so->ptr == sa->ptr || so->ptr == sb->ptr))
        return fail(KTH_E_ARGUMENT, "kth_binary: output aliases a broadcast operand");
    if (on == 0) return KTH_OK;
    // An operand that is one owed constant over its whole shape, whatever that shape, is the scalar
    // operand of the same functor when the other operand has the output's shape.
    const bool fold_b = folds_a_constant(op) && sb->fill_n >= bn && bn > 0 && an == on && so != sb && sa != sb;
    const bool fold_a = !fold_b && folds_a_constant(op) && sa->fill_n >= an && an > 0 && bn == on && so != sa && sa != sb;
    if (!fold_a) settle(sa);
    if (!fold_b) settle(sb);
    if (so != sa && so != sb) settle_for_overwrite(so, on); else settle(so);
    const float* pa = sa->ptr; const float* pb = sb->ptr; float* po = so->ptr;
    const uint32_t n32 = static_cast<uint32_t>(on);
    const float eps = state().epsilon;
    if (fold_a || fold_b) {
        if (fold_b) launch_scalar_op(op, false, pa, po, n32, sb->fill_value, eps);
        else        launch_scalar_op(op, true, pb, po, n32, sa->fill_value, eps);
    } else if (all_same && op == KTH_POW) {
        launch_pow(2, pa, pb, po, n32, 0.0f);
    } else if (all_same) {
#define B(OP) launch_binary_same<OP>(pa, pb, po, n32, eps)
        KTH_BINARY_DISPATCH(op, B)
#undef B
    } else {
#define B(OP) launch_binary_bcast<OP>(pa, pb, po, n32, eps, plan, vec_ok, a_vec, b_vec, (an + bn + on) * 4)
        KTH_BINARY_DISPATCH(op, B)
#undef B
    }
    KTH_LAUNCH_CHECK("binary");
    return KTH_OK;
}

int kth_masked_fill(uint64_t a, const int32_t* ashape, int adims, uint64_t mask, const int32_t* mshape, int mdims,
                    float value, uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    uint64_t an, mn;
    if (int rc = check_shape(ashape, adims, "kth_masked_fill(a)", &an)) return rc;
    if (int rc = check_shape(mshape, mdims, "kth_masked_fill(mask)", &mn)) return rc;
    Store* sa = lookup(a, "kth_masked_fill(a)", true);
    if (!sa) return KTH_E_HANDLE;
    Store* sm = lookup(mask, "kth_masked_fill(mask)", true);
    if (!sm) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_masked_fill(out)");
    if (!so) return KTH_E_HANDLE;
    if (an > sa->n_floats || mn > sm->n_floats || an > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_masked_fill: a shape needs more elements than its store holds");
    BcastPlan plan{};
    bool vec_ok, a_vec, b_vec;
    if (!build_plan(ashape, adims, mshape, mdims, ashape, adims, &plan, &vec_ok, &a_vec, &b_vec))
        return fail(KTH_E_SHAPE, "kth_masked_fill: the mask does not broadcast to the tensor's shape");
    if (mn != an && (so->ptr == sm->ptr)) return fail(KTH_E_ARGUMENT, "kth_masked_fill: output aliases the broadcast mask");
    if (an == 0) return KTH_OK;
    plan.a_stream = true;
    plan.b_stream = (mn == an);
    const uint32_t n32 = static_cast<uint32_t>(an);
    if (mn == an) launch_binary_same<OpMaskedFill>(sa->ptr, sm->ptr, so->ptr, n32, value);
    else launch_binary_bcast<OpMaskedFill>(sa->ptr, sm->ptr, so->ptr, n32, value, plan, vec_ok, a_vec, b_vec, (2 * an + mn) * 4);
    KTH_LAUNCH_CHECK("masked_fill");
    return KTH_OK;
}

int kth_broadcast_to(uint64_t src, const int32_t* sshape, int sdims,
                     uint64_t dst, const int32_t* dshape, int ddims) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    uint64_t sn, dn;
    if (int rc = check_shape(sshape, sdims, "kth_broadcast_to(src)", &sn)) return rc;
    if (int rc = check_shape(dshape, ddims, "kth_broadcast_to(dst)", &dn)) return rc;
    Store* ss = lookup_unsettled(src, "kth_broadcast_to(src)", true);
    if (!ss) return KTH_E_HANDLE;
    Store* sd = lookup_unsettled(dst, "kth_broadcast_to(dst)");
    if (!sd) return KTH_E_HANDLE;
    if (sn > ss->n_floats || dn > sd->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_broadcast_to: a shape needs more elements than its store holds");
    BcastPlan plan{};
    bool vec_ok, a_vec, b_vec;
    // Planned as the binary op first(src, src): both operand maps are the source's.
    if (!build_plan(sshape, sdims, sshape, sdims, dshape, ddims, &plan, &vec_ok, &a_vec, &b_vec))
        return fail(KTH_E_SHAPE, "kth_broadcast_to: source shape does not broadcast to the target shape");
    if (ss->ptr == sd->ptr) return fail(KTH_E_ARGUMENT, "kth_broadcast_to: source and target are the same store");
    plan.a_stream = plan.b_stream = false;
    if (dn == 0) return KTH_OK;
    const bool constant_source = ss != sd && sn > 0 && ss->fill_n >= sn;
    if (!constant_source) settle(ss);
    if (ss != sd) settle_for_overwrite(sd, dn); else settle(sd);
    if (constant_source) {
        // every element of the result is the source's one constant: the result is owed the same fill
        sd->fill_n = dn; sd->fill_value = ss->fill_value;
        return KTH_OK;
    }
    if (sn == dn) {
        LaunchScope scope("memcpy_d2d", "", dn * 8);
        KTH_HIP(hipMemcpyAsync(sd->ptr, ss->ptr, dn * 4, hipMemcpyDeviceToDevice, state().stream));
    } else {
        launch_binary_bcast<OpFirst>(ss->ptr, ss->ptr, sd->ptr, static_cast<uint32_t>(dn), 0.0f, plan, vec_ok, a_vec, b_vec,
                                     (sn + dn) * 4);
        KTH_LAUNCH_CHECK("broadcast_to");
    }
    return KTH_OK;
}

int kth_contains_nan(uint64_t handle, uint64_t n, int* out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!out) return fail(KTH_E_ARGUMENT, "kth_contains_nan: null output");
    Store* st = lookup(handle, "kth_contains_nan", true);
    if (!st) return KTH_E_HANDLE;
    if (n > st->n_floats) return fail(KTH_E_ARGUMENT, "kth_contains_nan: n=%llu exceeds the store", (unsigned long long)n);
    *out = 0;
    if (n == 0) {                      // still a blocking call: it drains the stream and reports what is pending
        KTH_HIP(hipStreamSynchronize(state().stream));
        return report_deferred_index_error();
    }
    uint64_t cap;
    int* flag = reinterpret_cast<int*>(workspace_acquire(4, &cap));
    if (!flag) return fail(KTH_E_MEMORY, "kth_contains_nan: no workspace");
    State& s = state();
    hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(1), 0, s.stream, flag);
    uint32_t n32 = static_cast<uint32_t>(n);
    uint32_t blocks = blocks_for(n32 >> 2);
    uint32_t cap_blocks = static_cast<uint32_t>(s.compute_units) * 8u;
    if (blocks > cap_blocks) blocks = cap_blocks;
    {
        LaunchScope scope("contains_nan_kernel", "", n * 4);
        hipLaunchKernelGGL(contains_nan_kernel, dim3(blocks), dim3(kBlock), 0, s.stream, st->ptr, n32, flag);
    }
    int host_flag = 0;
    hipError_t e = hipMemcpyAsync(&host_flag, flag, 4, hipMemcpyDeviceToHost, s.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(s.stream);
    workspace_release(reinterpret_cast<float*>(flag), cap);
    if (e != hipSuccess) return fail(KTH_E_DEVICE, "kth_contains_nan: %s", hipGetErrorString(e));
    *out = host_flag;
    // A pending out-of-range index of deferred checking is reported here, once; *out is valid all the same.
    return report_deferred_index_error();
}

}  // extern "C"

namespace kth {

hipError_t init_math_tables() {
    LogEntry log_tab[kLogTableEntries];
    double exp_tab[kExpTableEntries];
    for (int i = 0; i < kLogTableEntries; i++) {
        // The z values with index i have bit patterns kLogOff + (i << 45) + [0, 2^45).
        uint64_t lo_bits = kLogOff + (static_cast<uint64_t>(i) << 45), hi_bits = lo_bits + (1ull << 45);
        double lo, hi;
        memcpy(&lo, &lo_bits, 8); memcpy(&hi, &hi_bits, 8);
        if (lo == 1.0) {                       // the interval that starts at 1: exact, no cancellation near 1
            log_tab[i].invc = 1.0; log_tab[i].logc = 0.0;
            continue;
        }
        const long double c = (static_cast<long double>(lo) + static_cast<long double>(hi)) / 2.0L;
        const double invc = static_cast<double>(1.0L / c);
        log_tab[i].invc = invc;
        log_tab[i].logc = static_cast<double>(-logl(static_cast<long double>(invc)));
    }
    Log2Entry log2_tab[kLogTableEntries];
    for (int i = 0; i < kLogTableEntries; i++) {
        log2_tab[i].invc = log_tab[i].invc;
        log2_tab[i].log2c = log_tab[i].invc == 1.0 ? 0.0 : static_cast<double>(-log2l(static_cast<long double>(log_tab[i].invc)));
    }
    for (int i = 0; i < kExpTableEntries; i++)
        exp_tab[i] = static_cast<double>(exp2l(static_cast<long double>(i) / kExpTableEntries));
    double atan_tab[kAtanTableEntries];
    for (int i = 0; i < kAtanTableEntries; i++) atan_tab[i] = static_cast<double>(atanl(static_cast<long double>(i) / 64.0L));
    // {sin, cos}(j pi / 32): exact 0 and +-1 at the multiples of pi / 2, which the long double routines miss by an ulp
    double sincos_tab[2 * kSinCosTableEntries];
    const long double pi = 3.14159265358979323846264338327950288419716939937510L;
    for (int j = 0; j < kSinCosTableEntries; j++) {
        sincos_tab[2 * j] = j % 32 == 0 ? 0.0 : static_cast<double>(sinl(pi * j / 32.0L));
        sincos_tab[2 * j + 1] = j % 32 == 16 ? 0.0 : static_cast<double>(cosl(pi * j / 32.0L));
    }
    sincos_tab[1] = 1.0; sincos_tab[2 * 32 + 1] = -1.0; sincos_tab[2 * 16] = 1.0; sincos_tab[2 * 48] = -1.0;
    double asin_tab[2 * kAsinTableEntries];
    for (int j = 0; j < kAsinTableEntries; j++) {
        const long double c = static_cast<long double>(j) / 64.0L;
        asin_tab[2 * j] = static_cast<double>(asinl(c));
        asin_tab[2 * j + 1] = static_cast<double>(sqrtl((1.0L - c) * (1.0L + c)));
    }
    hipError_t e = hipMemcpyToSymbol(HIP_SYMBOL(g_log_table), log_tab, sizeof(log_tab));
    if (e != hipSuccess) return e;
    e = hipMemcpyToSymbol(HIP_SYMBOL(g_exp_table), exp_tab, sizeof(exp_tab));
    if (e != hipSuccess) return e;
    e = hipMemcpyToSymbol(HIP_SYMBOL(g_log2_table), log2_tab, sizeof(log2_tab));
    if (e != hipSuccess) return e;
    e = hipMemcpyToSymbol(HIP_SYMBOL(g_sincos_table), sincos_tab, sizeof(sincos_tab));
    if (e != hipSuccess) return e;
    e = hipMemcpyToSymbol(HIP_SYMBOL(g_asin_table), asin_tab, sizeof(asin_tab));
    if (e != hipSuccess) return e;
    return hipMemcpyToSymbol(HIP_SYMBOL(g_atan_table), atan_tab, sizeof(atan_tab));
}

}  // namespace kth
