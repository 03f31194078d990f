// Axis and full reductions over a row-major tensor seen as [outer, axis, inner].
//
// These first-pass kernels cover the layouts (short rows and slabs have LDS-staged variants below):
//   rows    (inner == 1): G lanes of a wave64 (or a whole 256-thread workgroup) walk one
//           contiguous row with float4 loads, combine by xor shuffles (+ LDS across waves);
//   columns (inner >= 256, or slabs too small to stream): a wave owns 64 float4-wide (or scalar) columns so every load
//           instruction is a contiguous 1 KiB (256 B) span; the waves of a workgroup
//           take different rows and combine through LDS;
//   stream  (1 < inner < 256, or < 512 in float4 columns; slab of 2048 floats or more): a workgroup per slab, threads stay on
//           their column while the workgroup walks the slab as one contiguous span;
//   few     (axis of 2 ... 7 over wide columns): four columns per thread;
//   strided (other small inner): one thread per output element, serial walk down the axis.
// An axis of length 1 is an elementwise pass.
// When the output alone gives too few workgroups to fill 256 CUs, the axis is cut into
// S segments; each (output, segment) writes a partial and a second kernel combines the
// S partials in a fixed order. No atomics anywhere: the same input always gives the
// same bits.
//
// Sums accumulate in f64 from the first add (f64 adds are full rate on CDNA), so SUM and
// MEAN land within an ulp of the float64 reference; kten-jvm's serial float accumulation
// order (JVMRawTensor.kt:146-148,185-207) is not reproduced bit-for-bit, only bounded.
// MAX/MIN/ARG_MAX/ARG_MIN are order-independent and bit-exact (JVMRawTensor.kt:159-184).
#include "kth_internal.h"
#include "kth_ops.h"

using namespace kth;

namespace {

constexpr int kBlock = 256;
constexpr int kWave = 64;

typedef float v4f __attribute__((ext_vector_type(4)));

// The input of a reduction is read exactly once: non-temporal loads, so the stream does
// not displace other tensors from the memory-side cache.
__device__ __forceinline__ float4 ld4_stream(const float* p) {
    v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float ld1_stream(const float* p) { return __builtin_nontemporal_load(p); }
// Four consecutive floats from an address that is only 4-byte aligned: the hardware takes a
// 16-byte load from any dword address, and one such load per lane sweeps the cache lines a wave
// touches once where four single loads at lane stride 16 would sweep them four times.
typedef float v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));
__device__ __forceinline__ float4 ld4_stream_unaligned(const float* p) {
    v4f_unaligned v = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}

// ---------------------------------------------------------------- reducers

struct ArgAcc { float v; uint32_t i; };

__device__ __forceinline__ double shfl_xor_acc(double a, int m) { return __shfl_xor(a, m); }
__device__ __forceinline__ float  shfl_xor_acc(float a, int m)  { return __shfl_xor(a, m); }
__device__ __forceinline__ ArgAcc shfl_xor_acc(ArgAcc a, int m) {
    ArgAcc r;
    r.v = __shfl_xor(a.v, m);
    r.i = static_cast<uint32_t>(__shfl_xor(static_cast<int>(a.i), m));
    return r;
}

__device__ __forceinline__ double shfl_down_acc(double a, int d) { return __shfl_down(a, d); }
__device__ __forceinline__ float  shfl_down_acc(float a, int d)  { return __shfl_down(a, d); }
__device__ __forceinline__ ArgAcc shfl_down_acc(ArgAcc a, int d) {
    ArgAcc r;
    r.v = __shfl_down(a.v, d);
    r.i = static_cast<uint32_t>(__shfl_down(static_cast<int>(a.i), d));
    return r;
}

template <bool MEAN>
struct RedSumT {
    static constexpr const char* name = MEAN ? "RedMean" : "RedSum";
    using Acc = double;
    static __device__ __forceinline__ Acc init() { return 0.0; }
    static __device__ __forceinline__ void step(Acc& a, float x, uint32_t) { a += static_cast<double>(x); }
    static __device__ __forceinline__ Acc merge(Acc a, Acc b) { return a + b; }
    // MEAN divides once in f64 and rounds once. That is what the full mean() of the reference does
    // (FloatArray.average: double accumulator, JVMRawTensor.kt:150-152). Its axis SUM and MEAN are a serial float
    // accumulation, MEAN followed by a float divide (JVMRawTensor.kt:186-192): there this backend is closer to the
    // exact result rather than identical, and differs in kind where the float running sum overflows or absorbs
    // terms: [3e38, 3e38, -3e38] sums to +inf on kten-jvm and to 3e38 here.
    static __device__ __forceinline__ float finish(Acc a, uint32_t n) {
        return MEAN ? static_cast<float>(a / static_cast<double>(n)) : static_cast<float>(a);
    }
};
using RedSum = RedSumT<false>;
using RedMean = RedSumT<true>;

template <bool MAX>
struct RedExtT {
    static constexpr const char* name = MAX ? "RedMax" : "RedMin";
    using Acc = float;
    static __device__ __forceinline__ Acc init() { return MAX ? -INFINITY : INFINITY; }
    static __device__ __forceinline__ void step(Acc& a, float x, uint32_t) { a = MAX ? jmax(a, x) : jmin(a, x); }
    static __device__ __forceinline__ Acc merge(Acc a, Acc b) { return MAX ? jmax(a, b) : jmin(a, b); }
    static __device__ __forceinline__ float finish(Acc a, uint32_t) { return a; }
};
using RedMax = RedExtT<true>;
using RedMin = RedExtT<false>;

// temp starts at -/+inf, index at 0, update on strict compare only: ties keep the lowest
// index, NaNs never win, a lane with nothing strictly better yields 0 (JVMRawTensor.kt:167-184).
template <bool MAX>
struct RedArgT {
    static constexpr const char* name = MAX ? "RedArgMax" : "RedArgMin";
    using Acc = ArgAcc;
    static __device__ __forceinline__ Acc init() { Acc a; a.v = MAX ? -INFINITY : INFINITY; a.i = 0; return a; }
    static __device__ __forceinline__ void step(Acc& a, float x, uint32_t idx) {
        if (MAX ? (x > a.v) : (x < a.v)) { a.v = x; a.i = idx; }
    }
    static __device__ __forceinline__ Acc merge(Acc a, Acc b) {
        bool take_b = (MAX ? (b.v > a.v) : (b.v < a.v)) || (b.v == a.v && b.i < a.i);
        return take_b ? b : a;
    }
    static __device__ __forceinline__ float finish(Acc a, uint32_t) { return static_cast<float>(a.i); }
};
using RedArgMax = RedArgT<true>;
using RedArgMin = RedArgT<false>;

// ---------------------------------------------------------------- geometry

// One launch's view of the tensor. Segment s covers axis positions
// [s * seg_len, min((s + 1) * seg_len, axis)). With segments > 1 results go to
// `partial` laid out [outer][segments][inner].
struct Geom {
    uint32_t outer, axis, inner;
    uint32_t segments, seg_len;
};

template <class R>
__device__ __forceinline__ void emit(const Geom& g, uint32_t o, uint32_t s, uint32_t i, typename R::Acc acc,
                                     float* out, typename R::Acc* partial) {
    if (g.segments == 1) out[static_cast<size_t>(o) * g.inner + i] = R::finish(acc, g.axis);
    else partial[(static_cast<size_t>(o) * g.segments + s) * g.inner + i] = acc;
}

// ---------------------------------------------------------------- rows: inner == 1

// G lanes per row (G in {1, 2, 4, 16, 64}, or 256 = the whole workgroup).
// VEC = 4 requires axis % 4 == 0 and seg_len % 4 == 0 so every row segment is 16-byte aligned;
// VEC = 1 takes any row with 16-byte loads from dword addresses.
template <class R, int G, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_rows_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                            typename R::Acc* __restrict__ partial, Geom g) {
    using Acc = typename R::Acc;
    constexpr int kRows = kBlock / G;
    const uint32_t bid = blockIdx.x;
    const uint32_t s = bid % g.segments;
    const uint32_t row = (bid / g.segments) * kRows + threadIdx.x / G;
    const uint32_t lane = threadIdx.x % G;
    Acc acc = R::init();
    if (row < g.outer) {
        const float* base = in + static_cast<size_t>(row) * g.axis;
        const uint32_t begin = s * g.seg_len;
        const uint32_t end = min(begin + g.seg_len, g.axis);
        // Loads are issued kBatch at a time before any of them is consumed, so every
        // thread keeps kBatch requests in flight.
        constexpr uint32_t kBatch = 8;
        if (VEC == 4) {
            // every pass issues its (up to) kBatch loads before consuming any; the last pass of a lane
            // is predicated instead of falling back to one load at a time
            for (uint32_t j = begin + lane * 4; j < end; j += kBatch * G * 4) {
                float4 v[kBatch];
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (j + k * G * 4 < end) v[k] = ld4_stream(base + j + k * G * 4);
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) {
                    const uint32_t jj = j + k * G * 4;
                    if (jj < end) { R::step(acc, v[k].x, jj); R::step(acc, v[k].y, jj + 1); R::step(acc, v[k].z, jj + 2); R::step(acc, v[k].w, jj + 3); }
                }
            }
        } else {
            // Rows that do not start on 16-byte boundaries: 16-byte loads from dword addresses, then up
            // to three single floats. A lane meets its elements in ascending index order, as the arg
            // reducers require.
            const uint32_t body_end = begin + ((end - begin) & ~3u);
            for (uint32_t j = begin + lane * 4; j < body_end; j += kBatch * G * 4) {
                float4 v[kBatch];
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (j + k * G * 4 < body_end) v[k] = ld4_stream_unaligned(base + j + k * G * 4);
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) {
                    const uint32_t jj = j + k * G * 4;
                    if (jj < body_end) { R::step(acc, v[k].x, jj); R::step(acc, v[k].y, jj + 1); R::step(acc, v[k].z, jj + 2); R::step(acc, v[k].w, jj + 3); }
                }
            }
            for (uint32_t e = body_end + lane; e < end; e += G) R::step(acc, ld1_stream(base + e), e);
        }
    }
    constexpr int kLanes = G < kWave ? G : kWave;
#pragma unroll
    for (int m = kLanes / 2; m >= 1; m >>= 1) acc = R::merge(acc, shfl_xor_acc(acc, m));
    if (G == kBlock) {
        __shared__ Acc lds[kBlock / kWave];
        if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            Acc t = lds[0];
#pragma unroll
            for (int w = 1; w < kBlock / kWave; w++) t = R::merge(t, lds[w]);
            emit<R>(g, row, s, 0, t, out, partial);
        }
    } else {
        if (lane == 0 && row < g.outer) emit<R>(g, row, s, 0, acc, out, partial);
    }
}

// ---------------------------------------------------------------- short rows: inner == 1, 2 <= axis < 256

// Rows this short are contiguous in memory one after the other, so a workgroup takes a tile of
// `rows` whole rows (a power of two in 32..4096, rows * axis <= kShortTile floats) as ONE contiguous
// span: it is loaded with coalesced float4s whatever the row length, parked in LDS at an odd
// row stride (conflict-free), and then `256 / rows` lanes fold each row from LDS, in index
// order within a lane.
constexpr uint32_t kShortTile = 4096;        // floats per tile: 16 KiB of LDS (+ padding); measured against 8 and 32 KiB
constexpr uint32_t kShortLoads = kShortTile / 4 / kBlock;

struct ShortPlan {
    uint32_t outer, axis, rows, stride;      // row length (axis, or axis * inner for slabs); stride = length | 1
    uint32_t inner;                          // slabs only
    uint32_t aligned;                        // every tile starts 16-byte aligned: float4 loads
    uint32_t lanes;                          // slabs only: lanes that share one output (power of two, <= 64)
    FastDiv  axis_div, inner_div;
};

// Loads `floats` contiguous floats from `base` (16-byte aligned if pl.aligned) and parks element e at
// tile[(e / axis) * stride + e % axis].
__device__ __forceinline__ void stage_short_tile(const float* __restrict__ base, uint32_t floats, const ShortPlan& pl, float* tile) {
    float4 v[kShortLoads];
#pragma unroll
    for (uint32_t k = 0; k < kShortLoads; k++) {
        const uint32_t e = (k * kBlock + threadIdx.x) * 4;
        if (e + 4 <= floats) v[k] = pl.aligned ? ld4_stream(base + e) : ld4_stream_unaligned(base + e);
        else {
            v[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (e < floats) v[k].x = base[e];
            if (e + 1 < floats) v[k].y = base[e + 1];
            if (e + 2 < floats) v[k].z = base[e + 2];
        }
    }
#pragma unroll
    for (uint32_t k = 0; k < kShortLoads; k++) {
        const uint32_t e = (k * kBlock + threadIdx.x) * 4;
        const float vals[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        // one division for the first of the four, the others step along the row and over its end
        const uint32_t r = (__umulhi(e, pl.axis_div.mul) + e) >> pl.axis_div.shift;
        uint32_t col = e - r * pl.axis, at = r * pl.stride + col;
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) {
            if (e + j < floats) tile[at] = vals[j];
            at++;
            if (++col == pl.axis) { col = 0; at += pl.stride - pl.axis; }
        }
    }
}

template <class R, int G>
__global__ __launch_bounds__(kBlock) void reduce_short_rows_kernel(const float* __restrict__ in, float* __restrict__ out, ShortPlan pl) {
    using Acc = typename R::Acc;
    __shared__ float tile[kShortTile + kShortTile / 8 + 8];
    const uint32_t first_row = blockIdx.x * pl.rows;
    const uint32_t rows_here = min(pl.rows, pl.outer - first_row);
    const uint32_t floats = rows_here * pl.axis;
    stage_short_tile(in + static_cast<size_t>(first_row) * pl.axis, floats, pl, tile);      // rows * axis % 4 == 0: 16-byte aligned
    __syncthreads();
    // G > 1: G lanes per row, kBlock / G rows. G == 1: a thread takes rows r, r + kBlock, ...
    const uint32_t lane = threadIdx.x % G;
    for (uint32_t r = threadIdx.x / G; r < pl.rows; r += kBlock / G) {
        Acc acc = R::init();
        if (r < rows_here) {
            const float* row = tile + r * pl.stride;
            uint32_t j = lane;
            for (; j + 3 * G < pl.axis; j += 4 * G) {               // four LDS reads in flight
                const float a0 = row[j], a1 = row[j + G], a2 = row[j + 2 * G], a3 = row[j + 3 * G];
                R::step(acc, a0, j); R::step(acc, a1, j + G); R::step(acc, a2, j + 2 * G); R::step(acc, a3, j + 3 * G);
            }
            for (; j < pl.axis; j += G) R::step(acc, row[j], j);
        }
#pragma unroll
        for (int m = G / 2; m >= 1; m >>= 1) acc = R::merge(acc, shfl_xor_acc(acc, m));
        if (lane == 0 && r < rows_here) out[first_row + r] = R::finish(acc, pl.axis);
    }
}

// The same staging for a reduction over a middle axis with a small inner size: a "row" is
// the contiguous slab [axis, inner] of one outer index (pl.axis holds axis * inner), and the
// (1 to 1024 slabs per tile), and the outputs of the tile, rows * inner of them, are dealt to
// the threads in output order:
// output (r, i) folds tile[r][j * inner + i] over j.
template <class R>
__global__ __launch_bounds__(kBlock) void reduce_short_slabs_kernel(const float* __restrict__ in, float* __restrict__ out, ShortPlan pl) {
    using Acc = typename R::Acc;
    __shared__ float tile[kShortTile + kShortTile / 8 + 8];
    const uint32_t first_row = blockIdx.x * pl.rows;
    const uint32_t rows_here = min(pl.rows, pl.outer - first_row);
    stage_short_tile(in + static_cast<size_t>(first_row) * pl.axis, rows_here * pl.axis, pl, tile);
    __syncthreads();
    const uint32_t outputs = rows_here * pl.inner, steps = pl.axis / pl.inner;
    float* dst = out + static_cast<size_t>(first_row) * pl.inner;
    // pl.lanes adjacent lanes share an output when the tile has fewer outputs than threads: lane l
    // takes the axis positions l, l + lanes, ... in ascending order, then the lanes are merged.
    const uint32_t lane = threadIdx.x & (pl.lanes - 1), group = threadIdx.x / pl.lanes;
    for (uint32_t item = group; item < outputs; item += kBlock / pl.lanes) {
        const uint32_t r = (__umulhi(item, pl.inner_div.mul) + item) >> pl.inner_div.shift;
        const float* p = tile + r * pl.stride + (item - r * pl.inner);
        Acc acc = R::init();
        uint32_t j = lane;
        for (; j + 3 * pl.lanes < steps; j += 4 * pl.lanes) {       // four LDS reads in flight
            const float a0 = p[j * pl.inner], a1 = p[(j + pl.lanes) * pl.inner];
            const float a2 = p[(j + 2 * pl.lanes) * pl.inner], a3 = p[(j + 3 * pl.lanes) * pl.inner];
            R::step(acc, a0, j); R::step(acc, a1, j + pl.lanes); R::step(acc, a2, j + 2 * pl.lanes); R::step(acc, a3, j + 3 * pl.lanes);
        }
        for (; j < steps; j += pl.lanes) R::step(acc, p[j * pl.inner], j);
        for (uint32_t m = pl.lanes >> 1; m >= 1; m >>= 1) acc = R::merge(acc, shfl_xor_acc(acc, static_cast<int>(m)));
        if (lane == 0) dst[item] = R::finish(acc, steps);
    }
}

// ---------------------------------------------------------------- columns: inner >= 64

// Workgroup = 64 x WY threads over a tile of TW * 64 * VEC columns: lane x of wave y owns VEC
// adjacent columns of sub-tile y % TW (so TW waves side by side read one contiguous span of a
// row), and takes rows y / TW, y / TW + WY / TW, ... of the segment. In use: VEC = 4, TW = 1.
template <class R, int VEC, int WY, int TW>
__global__ __launch_bounds__(kWave * WY) void reduce_cols_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                                 typename R::Acc* __restrict__ partial, Geom g, uint32_t tiles) {
    using Acc = typename R::Acc;
    constexpr uint32_t WR = WY / TW;            // row lanes
    const uint32_t bid = blockIdx.x;
    const uint32_t tile = bid % tiles;
    const uint32_t rest = bid / tiles;
    const uint32_t s = rest % g.segments;
    const uint32_t o = rest / g.segments;
    const uint32_t tx = threadIdx.x, ty = threadIdx.y;
    const uint32_t sub = ty % TW, lane = ty / TW;
    const uint32_t own = ((tile * TW + sub) * kWave + tx) * VEC;       // first column this thread answers for
    const bool active = own < g.inner;
    // float4 columns of an inner size that is not a multiple of 4: the last group starts at inner - 4 and
    // overlaps its neighbour (the loads are 16 bytes from a dword address anyway); it emits only its own columns
    const uint32_t col = (VEC == 4 && active && own + 4 > g.inner) ? g.inner - 4 : own;
    Acc acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) acc[v] = R::init();
    if (active) {
        const float* base = in + static_cast<size_t>(o) * g.axis * g.inner + col;
        const uint32_t begin = s * g.seg_len;
        const uint32_t end = min(begin + g.seg_len, g.axis);
        constexpr uint32_t kBatch = 8;          // loads in flight per thread
        // every pass issues its (up to) kBatch loads before consuming any; the last pass is predicated
        for (uint32_t r = begin + lane; r < end; r += kBatch * WR) {
            if (VEC == 4) {
                float4 v[kBatch];
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (r + k * WR < end) v[k] = ld4_stream_unaligned(base + static_cast<size_t>(r + k * WR) * g.inner);
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) {
                    const uint32_t rr = r + k * WR;
                    if (rr < end) {
                        R::step(acc[0], v[k].x, rr); R::step(acc[1 % VEC], v[k].y, rr);
                        R::step(acc[2 % VEC], v[k].z, rr); R::step(acc[3 % VEC], v[k].w, rr);
                    }
                }
            } else {
                float v[kBatch];
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (r + k * WR < end) v[k] = ld1_stream(base + static_cast<size_t>(r + k * WR) * g.inner);
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (r + k * WR < end) R::step(acc[0], v[k], r + k * WR);
            }
        }
    }
    __shared__ Acc lds[WY][kWave * VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) lds[ty][tx * VEC + v] = acc[v];
    __syncthreads();
    if (lane == 0 && active) {
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            Acc t = lds[sub][tx * VEC + v];
            for (uint32_t w = 1; w < WR; w++) t = R::merge(t, lds[w * TW + sub][tx * VEC + v]);
            if (col + v >= own) emit<R>(g, o, s, col + v, t, out, partial);
        }
    }
}

// ---------------------------------------------------------------- strided: small inner

template <class R>
__global__ __launch_bounds__(kBlock) void reduce_strided_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                               typename R::Acc* __restrict__ partial, Geom g) {
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const uint64_t n_out = static_cast<uint64_t>(g.outer) * g.inner;
    if (t >= n_out * g.segments) return;
    const uint32_t i = static_cast<uint32_t>(t % g.inner);
    const uint64_t rest = t / g.inner;
    const uint32_t s = static_cast<uint32_t>(rest % g.segments);
    const uint32_t o = static_cast<uint32_t>(rest / g.segments);
    const float* base = in + static_cast<size_t>(o) * g.axis * g.inner + i;
    const uint32_t begin = s * g.seg_len;
    const uint32_t end = min(begin + g.seg_len, g.axis);
    typename R::Acc acc = R::init();
    constexpr uint32_t kBatch = 8;
    uint32_t r = begin;
    for (; r + kBatch <= end; r += kBatch) {
        float v[kBatch];
#pragma unroll
        for (uint32_t k = 0; k < kBatch; k++) v[k] = ld1_stream(base + static_cast<size_t>(r + k) * g.inner);
#pragma unroll
        for (uint32_t k = 0; k < kBatch; k++) R::step(acc, v[k], r + k);
    }
    for (; r < end; r++) R::step(acc, ld1_stream(base + static_cast<size_t>(r) * g.inner), r);
    emit<R>(g, o, s, i, acc, out, partial);
}

// ---------------------------------------------------------------- stream: small inner, long axis

// One workgroup per (outer index, segment): its slab is one contiguous span. `lanes` groups of
// inner / VEC threads walk the rows `lanes` apart, so a load instruction of the workgroup covers
// lanes * inner consecutive floats and every thread stays on its own column(s). The lanes'
// partials meet in LDS and are merged pairwise, lane l with lane l + step.
// VEC = 4: a thread owns four adjacent columns, loaded as 16 bytes from a dword address, for any inner size of
// at least 4; when inner is not a multiple of 4 the last group starts at inner - 4 and overlaps its neighbour
// (both fold the same rows, so the columns they share get the same value twice).
template <class R, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_stream_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                              typename R::Acc* __restrict__ partial, Geom g,
                                                              uint32_t lanes, FastDiv cols_div) {
    using Acc = typename R::Acc;
    __shared__ Acc fold[kBlock * VEC];
    const uint32_t s = blockIdx.x % g.segments;
    const uint32_t o = blockIdx.x / g.segments;
    const uint32_t cols = (g.inner + VEC - 1) / VEC;
    const uint32_t t = threadIdx.x;
    const uint32_t lane = (__umulhi(t, cols_div.mul) + t) >> cols_div.shift;
    const uint32_t c = t - lane * cols;
    const uint32_t col = (VEC == 4 && c * 4 + 4 > g.inner) ? g.inner - 4 : c * VEC;      // first column of this thread
    const uint32_t begin = s * g.seg_len;
    const uint32_t end = min(begin + g.seg_len, g.axis);
    Acc acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) acc[v] = R::init();
    if (lane < lanes) {
        const float* base = in + static_cast<size_t>(o) * g.axis * g.inner + col;
        constexpr uint32_t kBatch = 8;
        // every pass issues its (up to) kBatch loads before consuming any; the last pass is predicated
        for (uint32_t r = begin + lane; r < end; r += kBatch * lanes) {
            if (VEC == 4) {
                float4 w[kBatch];
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (r + k * lanes < end) w[k] = ld4_stream_unaligned(base + static_cast<size_t>(r + k * lanes) * g.inner);
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) {
                    const uint32_t rr = r + k * lanes;
                    if (rr < end) {
                        R::step(acc[0], w[k].x, rr); R::step(acc[VEC > 1 ? 1 : 0], w[k].y, rr);
                        R::step(acc[VEC > 2 ? 2 : 0], w[k].z, rr); R::step(acc[VEC > 3 ? 3 : 0], w[k].w, rr);
                    }
                }
            } else {
                float w[kBatch];
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (r + k * lanes < end) w[k] = ld1_stream(base + static_cast<size_t>(r + k * lanes) * g.inner);
#pragma unroll
                for (uint32_t k = 0; k < kBatch; k++) if (r + k * lanes < end) R::step(acc[0], w[k], r + k * lanes);
            }
        }
    }
    // fold[lane][column]: lanes * inner <= kBlock * VEC entries
    if (lane < lanes) {
#pragma unroll
        for (int v = 0; v < VEC; v++) fold[lane * g.inner + col + v] = acc[v];
    }
    __syncthreads();
    // lane l takes lane l + step, step halving: with an inner size of 4 there are 256 lanes, and one thread per column
    // merging them in turn was a third of the kernel's time
    const uint32_t total = lanes * g.inner;
    uint32_t width = 1;
    while (width < lanes) width <<= 1;
    for (uint32_t step = width >> 1; step >= 1; step >>= 1) {
        const uint32_t half = step * g.inner;
        for (uint32_t e = t; e < half; e += kBlock)
            if (e + half < total) fold[e] = R::merge(fold[e], fold[e + half]);
        __syncthreads();
    }
    for (uint32_t i = t; i < g.inner; i += kBlock) emit<R>(g, o, s, i, fold[i], out, partial);
}

// ---------------------------------------------------------------- small inputs: a wave per slab, no LDS and no barrier

// A tensor of a megabyte or two is over before a workgroup's staging, barriers and LDS fold have paid for themselves:
// what such a launch costs is its chain of dependent steps (on this part about 1.7 us for load -> store, 3.4 us
// for the slab-per-workgroup kernel on [128,56,56] -> [128,56]). Here one wave owns the slab [axis, inner] of one
// outer index: lane = r * groups + c takes the four adjacent columns of group c (16 bytes from a dword address; the
// last group of an inner size off a multiple of 4 starts at inner - 4 and overlaps its neighbour) on rows
// r, r + row_lanes, ..., all of them requested before the first is folded when the slab is short, and the row lanes
// of a column group are merged by shuffles: nothing leaves the wave until the result does.
constexpr uint32_t kSmallBatch = 16;          // loads in flight per lane
// A workgroup is one wave: the slabs spread over as many compute units as there are slabs, and a compute unit's
// share of the loads is one slab's.
template <class R>
__global__ __launch_bounds__(kWave) void reduce_wave_slabs_kernel(const float* __restrict__ in, float* __restrict__ out, Geom g,
                                                                 uint32_t groups, uint32_t row_lanes) {
    using Acc = typename R::Acc;
    const uint32_t o = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint32_t r = lane / groups, c = lane - r * groups;
    const uint32_t own = c * 4;
    const uint32_t col = own + 4 > g.inner ? g.inner - 4 : own;
    Acc acc[4];
#pragma unroll
    for (int v = 0; v < 4; v++) acc[v] = R::init();
    if (r < row_lanes) {
        const float* base = in + static_cast<size_t>(o) * g.axis * g.inner + col;
        for (uint32_t a = r; a < g.axis; a += kSmallBatch * row_lanes) {
            float4 w[kSmallBatch];
#pragma unroll
            for (uint32_t k = 0; k < kSmallBatch; k++) if (a + k * row_lanes < g.axis) w[k] = ld4_stream_unaligned(base + static_cast<size_t>(a + k * row_lanes) * g.inner);
#pragma unroll
            for (uint32_t k = 0; k < kSmallBatch; k++) {
                const uint32_t aa = a + k * row_lanes;
                if (aa < g.axis) { R::step(acc[0], w[k].x, aa); R::step(acc[1], w[k].y, aa); R::step(acc[2], w[k].z, aa); R::step(acc[3], w[k].w, aa); }
            }
        }
    }
    // row lane r takes row lane r + step (idle lanes hold the identity); row_lanes is a power of two
    for (uint32_t step = row_lanes >> 1; step >= 1; step >>= 1) {
#pragma unroll
        for (int v = 0; v < 4; v++) acc[v] = R::merge(acc[v], shfl_down_acc(acc[v], static_cast<int>(step * groups)));
    }
    if (lane < groups) {
        float* q = out + static_cast<size_t>(o) * g.inner + col;
#pragma unroll
        for (uint32_t v = 0; v < 4; v++) if (col + v >= own) q[v] = R::finish(acc[v], g.axis);
    }
}

// Two steps of a reduce-to-shape chain in one launch: [outer, axis, inner] -> [outer, inner] by R1 as above, and that
// -> [outer] by R2 (the sum or mean over what was the inner dim), for inner a multiple of 4 below 256. The first step's
// results are rounded to float as if they had been stored; the second adds them the way the small-rows plan of
// reduce_rows_kernel would: lane c holds the four floats of 16-byte unit c and adds them in order, then the lanes are
// folded by xor-shuffles (the lanes beyond the row add exact zeros), so the result has the bits of the two launches.
template <class R1, class R2>
__global__ __launch_bounds__(kWave) void reduce_wave_slabs_rows_kernel(const float* __restrict__ in, float* __restrict__ out, Geom g,
                                                                      uint32_t groups, uint32_t row_lanes) {
    using Acc = typename R1::Acc;
    const uint32_t o = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint32_t r = lane / groups, c = lane - r * groups;
    const uint32_t col = c * 4;                              // inner % 4 == 0: no overlapping last group
    Acc acc[4];
#pragma unroll
    for (int v = 0; v < 4; v++) acc[v] = R1::init();
    if (r < row_lanes) {
        const float* base = in + static_cast<size_t>(o) * g.axis * g.inner + col;
        for (uint32_t a = r; a < g.axis; a += kSmallBatch * row_lanes) {
            float4 w[kSmallBatch];
#pragma unroll
            for (uint32_t k = 0; k < kSmallBatch; k++) if (a + k * row_lanes < g.axis) w[k] = ld4_stream_unaligned(base + static_cast<size_t>(a + k * row_lanes) * g.inner);
#pragma unroll
            for (uint32_t k = 0; k < kSmallBatch; k++) {
                const uint32_t aa = a + k * row_lanes;
                if (aa < g.axis) { R1::step(acc[0], w[k].x, aa); R1::step(acc[1], w[k].y, aa); R1::step(acc[2], w[k].z, aa); R1::step(acc[3], w[k].w, aa); }
            }
        }
    }
    for (uint32_t step = row_lanes >> 1; step >= 1; step >>= 1) {
#pragma unroll
        for (int v = 0; v < 4; v++) acc[v] = R1::merge(acc[v], shfl_down_acc(acc[v], static_cast<int>(step * groups)));
    }
    typename R2::Acc second = R2::init();
    if (lane < groups) {
#pragma unroll
        for (uint32_t v = 0; v < 4; v++) R2::step(second, R1::finish(acc[v], g.axis), col + v);
    }
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) second = R2::merge(second, shfl_xor_acc(second, m));
    if (lane == 0) out[o] = R2::finish(second, g.inner);
}

// ---------------------------------------------------------------- few rows: axis of 2 ... 7 over wide columns

// With so short an axis a column gives a thread only a handful of loads, so a thread takes four
// columns (float4-wide with VEC = 4; in use: VEC = 1), 256 * VEC apart: 8 loads in flight (two axis positions
// of its four columns), each a contiguous span across the workgroup. Axis positions in ascending order.
template <class R, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_few_kernel(const float* __restrict__ in, float* __restrict__ out, Geom g, uint32_t tiles) {
    using Acc = typename R::Acc;
    constexpr int kCols = 4;
    const uint32_t o = blockIdx.x / tiles;
    const uint32_t col0 = ((blockIdx.x - o * tiles) * kCols * kBlock + threadIdx.x) * VEC;
    const float* base = in + static_cast<size_t>(o) * g.axis * g.inner;
    Acc acc[kCols][VEC];
#pragma unroll
    for (int u = 0; u < kCols; u++)
#pragma unroll
        for (int v = 0; v < VEC; v++) acc[u][v] = R::init();
    for (uint32_t a = 0; a < g.axis; a += 2) {
        float w[2][kCols][VEC];
#pragma unroll
        for (uint32_t j = 0; j < 2; j++)
#pragma unroll
            for (int u = 0; u < kCols; u++) {
                const uint32_t c = col0 + u * kBlock * VEC;
                if (a + j < g.axis && c < g.inner) {
                    const float* p = base + static_cast<size_t>(a + j) * g.inner + c;
                    if (VEC == 4) { const float4 t = ld4_stream(p); w[j][u][0] = t.x; w[j][u][1 % VEC] = t.y; w[j][u][2 % VEC] = t.z; w[j][u][3 % VEC] = t.w; }
                    else w[j][u][0] = ld1_stream(p);
                }
            }
#pragma unroll
        for (uint32_t j = 0; j < 2; j++)
#pragma unroll
            for (int u = 0; u < kCols; u++)
                if (a + j < g.axis && col0 + u * kBlock * VEC < g.inner)
#pragma unroll
                    for (int v = 0; v < VEC; v++) R::step(acc[u][v], w[j][u][v], a + j);
    }
#pragma unroll
    for (int u = 0; u < kCols; u++) {
        const uint32_t c = col0 + u * kBlock * VEC;
        if (c < g.inner) {
            float* q = out + static_cast<size_t>(o) * g.inner + c;
            if (VEC == 4) *reinterpret_cast<float4*>(q) = make_float4(R::finish(acc[u][0], g.axis), R::finish(acc[u][1 % VEC], g.axis),
                                                                      R::finish(acc[u][2 % VEC], g.axis), R::finish(acc[u][3 % VEC], g.axis));
            else *q = R::finish(acc[u][0], g.axis);
        }
    }
}

// ---------------------------------------------------------------- an axis of length 1

// Every output folds exactly one input: an elementwise pass (SUM and MEAN still give 0 + x, which
// turns -0 into +0 as the serial sum from 0f does; the arg reducers give 0).
template <class R>
__global__ __launch_bounds__(kBlock) void reduce_unit_axis_kernel(const float* __restrict__ in, float* __restrict__ out, uint32_t n) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    const uint32_t n4 = n >> 2;
    auto one = [](float x) { typename R::Acc a = R::init(); R::step(a, x, 0u); return R::finish(a, 1u); };
    if (i < n4) {
        const float4 v = ld4_stream(in + 4 * static_cast<size_t>(i));
        *reinterpret_cast<float4*>(out + 4 * static_cast<size_t>(i)) = make_float4(one(v.x), one(v.y), one(v.z), one(v.w));
    }
    if (i < (n & 3u)) out[(static_cast<size_t>(n4) << 2) + i] = one(in[(static_cast<size_t>(n4) << 2) + i]);
}

// ---------------------------------------------------------------- second pass

// Combines the `segments` partials of each output, always in the same order.
// One wave64 per output: for a handful of outputs with many partials (full reductions).
template <class R>
__global__ __launch_bounds__(kBlock) void reduce_finalize_wave_kernel(const typename R::Acc* __restrict__ partial,
                                                                     float* __restrict__ out, Geom g) {
    using Acc = typename R::Acc;
    const uint64_t n_out = static_cast<uint64_t>(g.outer) * g.inner;
    const uint64_t idx = (static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    Acc acc = R::init();
    if (idx < n_out) {
        const uint32_t o = static_cast<uint32_t>(idx / g.inner), i = static_cast<uint32_t>(idx % g.inner);
        const Acc* p = partial + (static_cast<size_t>(o) * g.segments) * g.inner + i;
        // eight partials are requested before the first is merged (a merge with branches in it would otherwise
        // wait for every load in turn)
        for (uint32_t s = lane; s < g.segments; s += 8 * kWave) {
            Acc v[8];
#pragma unroll
            for (uint32_t k = 0; k < 8; k++) if (s + k * kWave < g.segments) v[k] = p[static_cast<size_t>(s + k * kWave) * g.inner];
#pragma unroll
            for (uint32_t k = 0; k < 8; k++) if (s + k * kWave < g.segments) acc = R::merge(acc, v[k]);
        }
    }
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) acc = R::merge(acc, shfl_xor_acc(acc, m));
    if (lane == 0 && idx < n_out) out[idx] = R::finish(acc, g.axis);
}

// 64 adjacent outputs x TY segment groups per workgroup: loads are coalesced along the
// outputs, group y folds segments y, y + TY, ..., and LDS folds the TY groups in order.
template <class R, int TY>
__global__ __launch_bounds__(kWave * TY) void reduce_finalize_tile_kernel(const typename R::Acc* __restrict__ partial,
                                                                          float* __restrict__ out, Geom g) {
    using Acc = typename R::Acc;
    const uint64_t n_out = static_cast<uint64_t>(g.outer) * g.inner;
    const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kWave + threadIdx.x;
    const uint32_t ty = threadIdx.y;
    Acc acc = R::init();
    if (idx < n_out) {
        const uint32_t o = static_cast<uint32_t>(idx / g.inner), i = static_cast<uint32_t>(idx % g.inner);
        const Acc* p = partial + (static_cast<size_t>(o) * g.segments) * g.inner + i;
        for (uint32_t s = ty; s < g.segments; s += 8 * TY) {
            Acc v[8];
#pragma unroll
            for (uint32_t k = 0; k < 8; k++) if (s + k * TY < g.segments) v[k] = p[static_cast<size_t>(s + k * TY) * g.inner];
#pragma unroll
            for (uint32_t k = 0; k < 8; k++) if (s + k * TY < g.segments) acc = R::merge(acc, v[k]);
        }
    }
    if (TY > 1) {
        __shared__ Acc lds[TY][kWave];
        lds[ty][threadIdx.x] = acc;
        __syncthreads();
        if (ty == 0) {
#pragma unroll
            for (int w = 1; w < TY; w++) acc = R::merge(acc, lds[w][threadIdx.x]);
        }
    }
    if (ty == 0 && idx < n_out) out[idx] = R::finish(acc, g.axis);
}

// ---------------------------------------------------------------- static scratch

// Partials of kth_reduce_axis_static, the entry point that allocates nothing: a fixed array in
// the code object's global segment instead of a pool workspace. Every device the library runs on
// holds its own copy at its own address until the process ends. Host code never uses the array's
// name as an address: reduce_scratch_init resolves the device address once per device and the
// kernels get that pointer as their `partial` argument.
constexpr size_t kStaticScratchBytes = 4u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kScratchDevices = 64;
void* g_scratch_ptr[kScratchDevices] = {nullptr};

// ---------------------------------------------------------------- host planning

uint32_t ceil_div(uint64_t a, uint64_t b) { return static_cast<uint32_t>((a + b - 1) / b); }

// Cuts the axis into segments so that `base_blocks * segments` reaches `target` blocks,
// while every segment keeps at least `min_len` positions and is a multiple of `quantum`.
void plan_segments(Geom* g, uint64_t base_blocks, uint64_t target, uint32_t quantum, uint32_t min_len) {
    // Cutting the axis costs a second launch (about 4.5 us): only worth it when the
    // outputs alone leave more than half of the machine idle.
    uint32_t want = base_blocks * 2 > target ? 1u : ceil_div(target, base_blocks);
    // ... and when a workgroup has more than a few passes over its share of the axis (a pass: `quantum` positions, eight
    // loads in flight each, about a microsecond): six passes or fewer are over before a second launch would have started
    if (ceil_div(g->axis, quantum * 8u) <= 6u) want = 1u;
    uint32_t max_seg = g->axis / min_len;
    if (max_seg < 1) max_seg = 1;
    if (want > max_seg) want = max_seg;
    uint32_t len = ceil_div(g->axis, want);
    len = ceil_div(len, quantum) * quantum;
    g->seg_len = len;
    g->segments = ceil_div(g->axis, len);
}

// Measured: from slabs of about 2048 floats on, streaming a slab per workgroup beats one thread
// per output (6 TB/s against 1-4.5); below that the per-workgroup fold dominates.
constexpr uint64_t kStreamMinSlab = 2048;
// Inputs up to this many floats take the small-input plans.
constexpr uint64_t kSmallInputFloats = 1u << 20;
constexpr uint64_t kSmallRowsFloats = 1u << 16;

// Whether [outer, axis, inner] takes reduce_wave_slabs_kernel (a small input whose slabs a wave takes whole), and the
// kernel's lane layout if so: most lanes of the wave at work, a lane's share of the axis in a few batches, and enough
// waves that the tensor is not one wave's work.
static bool wave_slabs_plan(uint32_t outer, uint32_t axis, uint32_t inner, uint32_t* groups_out, uint32_t* row_lanes_out) {
    const uint64_t n_in = static_cast<uint64_t>(outer) * axis * inner;
    if (!(n_in <= kSmallInputFloats && inner >= 4 && inner <= 4 * kWave && axis >= 2)) return false;
    const uint32_t groups = (inner + 3) / 4;
    uint32_t row_lanes = 1;
    while (row_lanes * 2 * groups <= kWave && row_lanes * 2 <= axis) row_lanes <<= 1;
    if (!(groups * row_lanes >= kWave / 2 && static_cast<uint64_t>(axis) * inner >= 512 && ceil_div(axis, row_lanes) <= 4 * kSmallBatch &&
          (outer >= 16 || static_cast<uint64_t>(axis) * inner <= 16384))) return false;
    *groups_out = groups; *row_lanes_out = row_lanes;
    return true;
}

// use_static: partials go to the static scratch array (no pool, no events, nothing allocated);
// a plan whose partials do not fit is refused before anything is launched.
// plan_only: makes the plan, applies that refusal and returns without launching (in and out are not used).
template <class R>
int run_reduce(const float* in, float* out, uint32_t outer, uint32_t axis, uint32_t inner, bool use_static, bool plan_only) {
    using Acc = typename R::Acc;
    State& st = state();
    const bool may_profile = !use_static;
    hipStream_t stream = st.stream;
    const uint64_t target = static_cast<uint64_t>(st.compute_units) * 8;
    Geom g{outer, axis, inner, 1, axis};
    const uint64_t n_out = static_cast<uint64_t>(outer) * inner;

    if (axis == 1) {
        if (plan_only) return KTH_OK;
        const uint32_t n = static_cast<uint32_t>(n_out);
        hipError_t e;
        {
            LaunchScope scope("reduce_unit_axis_kernel", R::name, n_out * 8, may_profile);
            hipLaunchKernelGGL((reduce_unit_axis_kernel<R>), dim3(static_cast<uint32_t>(ceil_div((n >> 2) + 3, kBlock))), dim3(kBlock), 0, stream, in, out, n);
            e = hipGetLastError();
        }
        if (e != hipSuccess) return fail(KTH_E_DEVICE, "kth_reduce: launch failed: %s", hipGetErrorString(e));
        return KTH_OK;
    }

    // Small inputs (up to 4 MiB): the launch is a chain of latencies, not a stream. Rows get enough lanes each for one
    // 16-byte load per lane and no LDS tile; slabs get a wave each (reduce_wave_slabs_kernel).
    const uint64_t n_in = n_out * axis;
    const bool small_input = n_in <= kSmallInputFloats;
    {
        uint32_t groups, row_lanes;
        if (wave_slabs_plan(outer, axis, inner, &groups, &row_lanes)) {
            if (plan_only) return KTH_OK;
            hipError_t e;
            {
                LaunchScope scope("reduce_wave_slabs_kernel", R::name, (n_in + n_out) * 4, may_profile);
                hipLaunchKernelGGL((reduce_wave_slabs_kernel<R>), dim3(outer), dim3(kWave), 0, stream, in, out, g, groups, row_lanes);
                e = hipGetLastError();
            }
            if (e != hipSuccess) return fail(KTH_E_DEVICE, "kth_reduce: launch failed: %s", hipGetErrorString(e));
            return KTH_OK;
        }
    }
    const bool small_rows = small_input && inner == 1 && n_in <= kSmallRowsFloats;

    if (inner == 1 && axis >= 2 && axis < 256 && !small_rows) {
        if (plan_only) return KTH_OK;
        // rows per tile: the largest power of two with rows * axis <= kShortTile, at most kBlock
        ShortPlan pl{};
        uint32_t rows = 16 * kBlock;
        while (rows * axis > kShortTile || rows * (axis | 1u) > kShortTile + kShortTile / 8) rows >>= 1;
        pl.outer = outer; pl.axis = axis; pl.rows = rows; pl.stride = axis | 1u; pl.aligned = 1;
        pl.axis_div = make_div(axis);
        const dim3 grid(static_cast<uint32_t>(ceil_div(outer, rows)));
        hipError_t e;
        {
            LaunchScope scope("reduce_short_rows_kernel", R::name, (static_cast<uint64_t>(outer) * axis + n_out) * 4, may_profile);
#define SHORT_LAUNCH(GG) hipLaunchKernelGGL((reduce_short_rows_kernel<R, GG>), grid, dim3(kBlock), 0, stream, in, out, pl)
            switch (rows >= kBlock ? 1 : kBlock / rows) {
            case 1: SHORT_LAUNCH(1); break;   case 2: SHORT_LAUNCH(2); break;   case 4: SHORT_LAUNCH(4); break;
            case 8: SHORT_LAUNCH(8); break;   case 16: SHORT_LAUNCH(16); break; case 32: SHORT_LAUNCH(32); break;
            default: SHORT_LAUNCH(64); break;
            }
#undef SHORT_LAUNCH
            e = hipGetLastError();
        }
        if (e != hipSuccess) return fail(KTH_E_DEVICE, "kth_reduce: launch failed: %s", hipGetErrorString(e));
        return KTH_OK;
    }

    // Slabs [axis, inner] of at most a tile, and enough of them to give every CU a workgroup.
    uint32_t slab_rows = 0;
    // Measured: better than the column and strided kernels for every slab below 2048 floats
    // (5.0-5.3 TB/s against 0.7-4.7; from 2048 floats on the stream kernel is ahead), and for any
    // slab that fits a tile when the axis is short (<= 16).
    const uint64_t slab = static_cast<uint64_t>(axis) * inner;
    if (inner > 1 && axis >= 2 && (slab < kStreamMinSlab || (axis <= 16 && slab <= kShortTile))) {
        slab_rows = static_cast<uint32_t>(kShortTile / slab);
        if (slab_rows > 4 * kBlock) slab_rows = 4 * kBlock;
        // the tile parks a slab at the odd pitch slab | 1: slabs of 4 and 6 floats grow by more than the
        // tile's padding of an eighth, so fewer of them fit (kept a multiple of 4: tiles stay 16-byte aligned)
        const uint32_t padded_rows = static_cast<uint32_t>((kShortTile + kShortTile / 8) / (slab | 1u));
        if (slab_rows > padded_rows) slab_rows = padded_rows >= 8 ? (padded_rows & ~3u) : padded_rows;
        if (ceil_div(outer, slab_rows) < static_cast<uint64_t>(st.compute_units)) slab_rows = 0;
    }
    if (slab_rows > 0) {
        if (plan_only) return KTH_OK;
        ShortPlan pl{};
        const uint32_t length = axis * inner;
        const uint32_t rows = slab_rows;
        pl.outer = outer; pl.axis = length; pl.rows = rows; pl.stride = length | 1u; pl.inner = inner;
        pl.aligned = (static_cast<uint64_t>(rows) * length) % 4 == 0 ? 1 : 0;
        pl.lanes = 1;
        while (pl.lanes < 64 && static_cast<uint64_t>(rows) * inner * pl.lanes * 2 <= kBlock && pl.lanes * 2 <= axis) pl.lanes <<= 1;
        pl.axis_div = make_div(length); pl.inner_div = make_div(inner);
        hipError_t e;
        {
            LaunchScope scope("reduce_short_slabs_kernel", R::name, (static_cast<uint64_t>(outer) * length + n_out) * 4, may_profile);
            hipLaunchKernelGGL((reduce_short_slabs_kernel<R>), dim3(static_cast<uint32_t>(ceil_div(outer, rows))), dim3(kBlock), 0, stream, in, out, pl);
            e = hipGetLastError();
        }
        if (e != hipSuccess) return fail(KTH_E_DEVICE, "kth_reduce: launch failed: %s", hipGetErrorString(e));
        return KTH_OK;
    }

    // Measured against the column kernel: ahead for every inner size below 512 (5.8-6.4 TB/s against
    // 3.3-6.1); from there on the column kernel's 1 KiB spans win.
    const bool stream_fits = slab >= kStreamMinSlab && inner < 512 && outer <= 0x7fffffffu / 64;
    if (axis <= 7 && inner >= 1024 && !stream_fits && n_out >= 65536) {
        // (slabs of such an axis that fit a tile were taken above)
        // one column per lane and load, for any inner size: measured 7-9 % ahead of float4 columns here
        // (66 against 72 us on [23,2,1456700]), whose 16 accumulators per thread cost more than the wider loads gain
        const uint32_t tiles = ceil_div(inner, 4u * kBlock);
        const uint64_t few_blocks = static_cast<uint64_t>(tiles) * outer;
        if (few_blocks <= 0x7fffffffull) {
            if (plan_only) return KTH_OK;
            hipError_t e;
            {
                LaunchScope scope("reduce_few_kernel", R::name, (static_cast<uint64_t>(outer) * slab + n_out) * 4, may_profile);
                hipLaunchKernelGGL((reduce_few_kernel<R, 1>), dim3(static_cast<uint32_t>(few_blocks)), dim3(kBlock), 0, stream, in, out, g, tiles);
                e = hipGetLastError();
            }
            if (e != hipSuccess) return fail(KTH_E_DEVICE, "kth_reduce: launch failed: %s", hipGetErrorString(e));
            return KTH_OK;
        }
    }
    enum { ROWS, COLS, STRIDED, STREAM } kind;
    int G = 1, VEC = 1, WY = 4, TW = 1;
    uint32_t stream_lanes = 0;
    uint32_t tiles = 0;
    uint64_t blocks = 0;
    if (inner == 1) {
        kind = ROWS;
        VEC = (axis % 4 == 0) ? 4 : 1;
        const uint32_t per_lane = axis / 4;            // 16-byte loads per row
        G = per_lane >= 1024 ? 256 : per_lane >= 128 ? 64 : per_lane >= 32 ? 16 : per_lane >= 8 ? 4 : per_lane >= 2 ? 2 : 1;
        if (small_rows && axis < 256) {
            // a small tensor of short rows: a lane per 16 bytes of the row, so that every lane has one load to wait for
            G = 1;
            while (G < 64 && static_cast<uint32_t>(G) * 4 < axis) G <<= 1;
            if (G == 8) G = 16;                        // (the kernel is built for 1, 2, 4, 16, 64, 256 lanes per row)
            if (G == 32) G = 64;
        }
        const uint64_t base_blocks = ceil_div(outer, kBlock / G);
        plan_segments(&g, base_blocks, target / 2, G * VEC, G * VEC * 16);
        blocks = base_blocks * g.segments;
    } else if (inner >= 64 && !stream_fits) {
        kind = COLS;
        VEC = 4;                                       // (inner >= 64; an inner size off a multiple of 4 overlaps its last group)
        // (scalar columns with four waves side by side measured 51 us on [4,16384,1001], the overlapping
        // float4 groups 46.6 us; with float4 columns the tile one wave wide is the faster one)
        TW = 1;
        tiles = ceil_div(inner, kWave * VEC * TW);
        const uint64_t base_blocks = static_cast<uint64_t>(tiles) * outer;
        // Few column tiles and a long axis: 16 waves per workgroup fold 16 rows at a time
        // through LDS, which cuts the number of partials per output by four.
        WY = (base_blocks * 4 * TW < target && axis >= 2048) ? 16 : 4;
        plan_segments(&g, base_blocks, WY == 16 ? target / 4 : target, WY / TW, WY / TW * 8);
        blocks = base_blocks * g.segments;
    } else if (stream_fits) {
        // A long axis over a small inner size: one workgroup streams a whole slab (or a segment of it).
        kind = STREAM;
        VEC = inner >= 4 ? 4 : 1;
        stream_lanes = kBlock / ((inner + VEC - 1) / VEC);
        plan_segments(&g, outer, target / 2, stream_lanes, stream_lanes * 8);
        blocks = static_cast<uint64_t>(outer) * g.segments;
    } else {
        kind = STRIDED;
        const uint64_t base_blocks = ceil_div(n_out, kBlock);
        plan_segments(&g, base_blocks, target / 2, 1, 64);
        blocks = ceil_div(n_out * g.segments, kBlock);
    }
    if (blocks > 0x7fffffffull) return fail(KTH_E_ARGUMENT, "kth_reduce: grid too large");

    Acc* partial = nullptr;
    uint64_t cap = 0;
    if (g.segments > 1 && use_static) {
        const uint64_t need = n_out * g.segments * sizeof(Acc);
        if (need > kStaticScratchBytes)
            return fail(KTH_E_ARGUMENT, "kth_reduce_axis_static: [%u,%u,%u] needs %llu bytes of partials (%llu outputs x %u axis segments), "
                        "the static scratch holds %llu; use kth_reduce_axis", outer, axis, inner, (unsigned long long)need,
                        (unsigned long long)n_out, g.segments, (unsigned long long)kStaticScratchBytes);
        partial = reinterpret_cast<Acc*>(g_scratch_ptr[st.device]);
    }
    if (plan_only) return KTH_OK;
    if (g.segments > 1 && !use_static) {
        partial = reinterpret_cast<Acc*>(workspace_acquire(n_out * g.segments * sizeof(Acc), &cap));
        if (!partial) return fail(KTH_E_MEMORY, "kth_reduce: no workspace for %llu partials",
                                  (unsigned long long)(n_out * g.segments));
    }
    const dim3 grid(static_cast<uint32_t>(blocks));
    const uint64_t bytes = (static_cast<uint64_t>(outer) * axis * inner + n_out) * 4;
    hipError_t e;
    {
        LaunchScope scope(kind == ROWS ? "reduce_rows_kernel" : kind == COLS ? "reduce_cols_kernel" : kind == STREAM ? "reduce_stream_kernel" : "reduce_strided_kernel",
                          R::name, bytes, may_profile);
        if (kind == ROWS) {
#define ROWS_LAUNCH(GG, VV) hipLaunchKernelGGL((reduce_rows_kernel<R, GG, VV>), grid, dim3(kBlock), 0, stream, in, out, partial, g)
            if (VEC == 4) {
                switch (G) { case 256: ROWS_LAUNCH(256, 4); break; case 64: ROWS_LAUNCH(64, 4); break;
                             case 16: ROWS_LAUNCH(16, 4); break; case 4: ROWS_LAUNCH(4, 4); break; case 2: ROWS_LAUNCH(2, 4); break;
                             default: ROWS_LAUNCH(1, 4); }
            } else {
                switch (G) { case 256: ROWS_LAUNCH(256, 1); break; case 64: ROWS_LAUNCH(64, 1); break;
                             case 16: ROWS_LAUNCH(16, 1); break; case 4: ROWS_LAUNCH(4, 1); break; case 2: ROWS_LAUNCH(2, 1); break;
                             default: ROWS_LAUNCH(1, 1); }
            }
#undef ROWS_LAUNCH
        } else if (kind == COLS) {
#define COLS_LAUNCH(VV, YY, TT) hipLaunchKernelGGL((reduce_cols_kernel<R, VV, YY, TT>), grid, dim3(kWave, YY), 0, stream, in, out, partial, g, tiles)
            if (WY == 16) COLS_LAUNCH(4, 16, 1); else COLS_LAUNCH(4, 4, 1);
#undef COLS_LAUNCH
        } else if (kind == STREAM) {
            const FastDiv cols_div = make_div((inner + VEC - 1) / VEC);
            if (VEC == 4) hipLaunchKernelGGL((reduce_stream_kernel<R, 4>), grid, dim3(kBlock), 0, stream, in, out, partial, g, stream_lanes, cols_div);
            else          hipLaunchKernelGGL((reduce_stream_kernel<R, 1>), grid, dim3(kBlock), 0, stream, in, out, partial, g, stream_lanes, cols_div);
        } else {
            hipLaunchKernelGGL((reduce_strided_kernel<R>), grid, dim3(kBlock), 0, stream, in, out, partial, g);
        }
        e = hipGetLastError();
    }
    if (e == hipSuccess && g.segments > 1) {
        LaunchScope scope("reduce_finalize_kernel", R::name, 0, may_profile);
        if (n_out < 64)
            hipLaunchKernelGGL((reduce_finalize_wave_kernel<R>), dim3(ceil_div(n_out * kWave, kBlock)), dim3(kBlock), 0, stream,
                               partial, out, g);
        else if (g.segments >= 128 && n_out <= 16384)       // few workgroups: sixteen waves each
            hipLaunchKernelGGL((reduce_finalize_tile_kernel<R, 16>), dim3(ceil_div(n_out, kWave)), dim3(kWave, 16), 0, stream,
                               partial, out, g);
        else if (g.segments >= 8)
            hipLaunchKernelGGL((reduce_finalize_tile_kernel<R, 4>), dim3(ceil_div(n_out, kWave)), dim3(kWave, 4), 0, stream,
                               partial, out, g);
        else
            hipLaunchKernelGGL((reduce_finalize_tile_kernel<R, 1>), dim3(ceil_div(n_out, kWave)), dim3(kWave, 1), 0, stream,
                               partial, out, g);
        e = hipGetLastError();
    }
    if (partial && !use_static) workspace_release(reinterpret_cast<float*>(partial), cap);
    if (e != hipSuccess) return fail(KTH_E_DEVICE, "kth_reduce: launch failed: %s", hipGetErrorString(e));
    return KTH_OK;
}

int dispatch_reduce(int op, const float* in, float* out, uint32_t outer, uint32_t axis, uint32_t inner, bool use_static = false,
                    bool plan_only = false) {
    switch (op) {
    case KTH_SUM:     return run_reduce<RedSum>(in, out, outer, axis, inner, use_static, plan_only);
    case KTH_MEAN:    return run_reduce<RedMean>(in, out, outer, axis, inner, use_static, plan_only);
    case KTH_MAX:     return run_reduce<RedMax>(in, out, outer, axis, inner, use_static, plan_only);
    case KTH_MIN:     return run_reduce<RedMin>(in, out, outer, axis, inner, use_static, plan_only);
    case KTH_ARG_MAX: return run_reduce<RedArgMax>(in, out, outer, axis, inner, use_static, plan_only);
    case KTH_ARG_MIN: return run_reduce<RedArgMin>(in, out, outer, axis, inner, use_static, plan_only);
    default:          return fail(KTH_E_ARGUMENT, "kth_reduce: op %d is not an aggregating operation", op);
    }
}

// The argument checks of both axis entry points, then the launch.
int reduce_axis_checked(const char* who, bool use_static, int op, uint64_t in, uint64_t out, uint64_t outer, uint64_t axis, uint64_t inner) {
    if (op < KTH_SUM || op > KTH_ARG_MIN) return fail(KTH_E_ARGUMENT, "%s: op %d is not an aggregating operation", who, op);
    // (neither lookup makes a copy that was put off: the input is only read, and the output's are made below, once the
    // entry point that launches nothing when it refuses has accepted the plan)
    // (... nor do they launch a small reduction that was put off: the step after it may take it along, below)
    Store* si = lookup_unsettled(in, who, true, true);
    if (!si) return KTH_E_HANDLE;
    Store* so = lookup_unsettled(out, who, true, true);
    if (!so) return KTH_E_HANDLE;
    if (axis == 0) return fail(KTH_E_ARGUMENT, "%s: empty axis", who);
    if (outer > kMaxElements || axis > kMaxElements || inner > kMaxElements ||
        outer * axis > kMaxElements || outer * axis * inner > kMaxElements)
        return fail(KTH_E_ARGUMENT, "%s: more than 2^31-1 elements", who);
    if ((op == KTH_ARG_MAX || op == KTH_ARG_MIN) && axis > (1ull << 24))
        return fail(KTH_E_ARGUMENT, "%s: axis %llu too long for an index stored as float", who, (unsigned long long)axis);
    if (outer * axis * inner > si->n_floats || outer * inner > so->n_floats)
        return fail(KTH_E_ARGUMENT, "%s: [%llu,%llu,%llu] exceeds a store", who, (unsigned long long)outer,
                    (unsigned long long)axis, (unsigned long long)inner);
    if (si == so) return fail(KTH_E_ARGUMENT, "%s: output aliases the input", who);
    if (outer * inner == 0) return KTH_OK;
    // The entry point that creates nothing refuses a plan that does not fit its scratch before it launches anything,
    // the fill an operand may still be owed included.
    if (use_static)
        if (int rc = dispatch_reduce(op, nullptr, nullptr, static_cast<uint32_t>(outer), static_cast<uint32_t>(axis),
                                     static_cast<uint32_t>(inner), true, true)) return rc;
    const uint32_t o32 = static_cast<uint32_t>(outer), a32 = static_cast<uint32_t>(axis), i32 = static_cast<uint32_t>(inner);
    const bool sums = op == KTH_SUM || op == KTH_MEAN;
    {
        // A fill the input is still owed is launched here, one the output is owed is dropped if the result
        // covers it; for the entry point that creates nothing, without the event pair of a running profile.
        State& s = state();
        const bool profiling = s.profiling;
        if (use_static) s.profiling = false;
        break_aliases(so);                // the output is written: what was put off around it is done first
        so->index_valid_below = 0; so->index_valid_n = 0;      // (it was looked up as if only read)
        // The input is itself a small sum that was put off, and this is the next step of its chain (the same outer
        // index, over what was its inner dim): one launch over its source does both. Otherwise it is launched now.
        const Store::OwedReduce first = si->owed;
        const bool chain = !use_static && first.src != 0 && sums && first.outer == o32 && first.inner == a32 && i32 == 1;
        if (first.src != 0 && !chain) materialize(si);
        settle(si);
        settle_for_overwrite(so, outer * inner);
        s.profiling = profiling;
        if (chain) {
            Store& src = s.table[first.src - 1];
            uint32_t groups, row_lanes;
            if (!wave_slabs_plan(first.outer, first.axis, first.inner, &groups, &row_lanes))
                return fail(KTH_E_DEVICE, "%s: a reduction was put off that its kernel does not take", who);
            const Geom g{first.outer, first.axis, first.inner, 1, first.axis};
            LaunchScope scope("reduce_wave_slabs_rows_kernel", op == KTH_MEAN ? "RedMean" : "RedSum",
                              (static_cast<uint64_t>(first.outer) * first.axis * first.inner + outer) * 4);
            const dim3 grid(first.outer), block(kWave);
            hipStream_t stream = s.stream;
            if (first.op == KTH_SUM && op == KTH_SUM)        hipLaunchKernelGGL((reduce_wave_slabs_rows_kernel<RedSum, RedSum>), grid, block, 0, stream, src.ptr, so->ptr, g, groups, row_lanes);
            else if (first.op == KTH_SUM)                    hipLaunchKernelGGL((reduce_wave_slabs_rows_kernel<RedSum, RedMean>), grid, block, 0, stream, src.ptr, so->ptr, g, groups, row_lanes);
            else if (op == KTH_SUM)                          hipLaunchKernelGGL((reduce_wave_slabs_rows_kernel<RedMean, RedSum>), grid, block, 0, stream, src.ptr, so->ptr, g, groups, row_lanes);
            else                                             hipLaunchKernelGGL((reduce_wave_slabs_rows_kernel<RedMean, RedMean>), grid, block, 0, stream, src.ptr, so->ptr, g, groups, row_lanes);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return fail(KTH_E_DEVICE, "%s: launch failed: %s", who, hipGetErrorString(e));
            return KTH_OK;
        }
    }
    // A small sum or mean that the next step of a reduce-to-shape chain could take along (the plan of a wave per slab;
    // an inner dim that the small-rows plan would then fold, so that the two launches and the one give the same bits)
    // is put off: the output is owed it. Whoever reads the output first has it launched; if that is the chain's next
    // step, the two are one launch and this one's result is never written unless somebody else asks for it.
    {
        uint32_t groups, row_lanes;
        if (!use_static && sums && i32 % 4 == 0 && i32 < 256 && outer * inner <= kSmallRowsFloats && si->alias_of == 0 &&
            wave_slabs_plan(o32, a32, i32, &groups, &row_lanes)) {
            owe_reduce(so, si, op, o32, a32, i32);
            return KTH_OK;
        }
    }
    const int rc = dispatch_reduce(op, si->ptr, so->ptr, static_cast<uint32_t>(outer), static_cast<uint32_t>(axis),
                                   static_cast<uint32_t>(inner), use_static);
    // the positions ARG_MAX / ARG_MIN wrote are index values below the axis length: an indexed move that takes
    // them next (the scatter of a Max / Min backward) need not check them
    if (rc == KTH_OK && (op == KTH_ARG_MAX || op == KTH_ARG_MIN)) {
        so->index_valid_below = static_cast<uint32_t>(axis);
        so->index_valid_n = outer * inner;
    }
    return rc;
}

}  // namespace

namespace kth {

int run_owed_reduce(int op, const float* in, float* out, uint32_t outer, uint32_t axis, uint32_t inner) {
    return dispatch_reduce(op, in, out, outer, axis, inner);
}

// Called by kth_init with `device` current: resolves this device's copy of the scratch array.
hipError_t reduce_scratch_init(int device) {
    if (device < 0 || device >= kScratchDevices) return hipErrorInvalidDevice;
    if (g_scratch_ptr[device]) return hipSuccess;
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[device] = p;
    return hipSuccess;
}

}  // namespace kth

extern "C" {

int kth_reduce_axis(int op, uint64_t in, uint64_t out, uint64_t outer, uint64_t axis, uint64_t inner) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    return reduce_axis_checked("kth_reduce_axis", false, op, in, out, outer, axis, inner);
}

int kth_reduce_axis_static(int op, uint64_t in, uint64_t out, uint64_t outer, uint64_t axis, uint64_t inner) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!g_scratch_ptr[state().device]) return fail(KTH_E_DEVICE, "kth_reduce_axis_static: the scratch array of device %d was not resolved", state().device);
    return reduce_axis_checked("kth_reduce_axis_static", true, op, in, out, outer, axis, inner);
}

int kth_reduce_scratch_bytes(uint64_t* bytes) {
    if (!bytes) return fail(KTH_E_ARGUMENT, "kth_reduce_scratch_bytes: null output");
    *bytes = kStaticScratchBytes;
    return KTH_OK;
}

int kth_reduce_all(int op, uint64_t in, uint64_t n, uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (op != KTH_SUM && op != KTH_MEAN) return fail(KTH_E_ARGUMENT, "kth_reduce_all: op %d is not SUM or MEAN", op);
    Store* si = lookup(in, "kth_reduce_all(in)", true);
    if (!si) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_reduce_all(out)");
    if (!so) return KTH_E_HANDLE;
    if (n == 0) return fail(KTH_E_ARGUMENT, "kth_reduce_all: empty input");
    if (n > si->n_floats || so->n_floats < 1) return fail(KTH_E_ARGUMENT, "kth_reduce_all: n=%llu exceeds the store", (unsigned long long)n);
    if (si->ptr == so->ptr) return fail(KTH_E_ARGUMENT, "kth_reduce_all: output aliases the input");
    return dispatch_reduce(op, si->ptr, so->ptr, 1u, static_cast<uint32_t>(n), 1u);
}

}  // extern "C"
