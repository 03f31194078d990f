// Layout movers: get / set / fill by index ranges, transpose, permute
// (reference: JVMRawTensor.kt:270-315,437-466 with RangeTensorIndexing.sparseStoreRanges,
// AbstractIndexing.kt:65-88; narrow JVM:468-473 and concat
// AbstractJVMTensorOperations.kt:106-120 are range get / set on the host side).
//
// All of them are copies between a dense row-major tensor and a strided view of another:
//   - a range index selects a box of the tensor; the reference concatenates the box's store
//     ranges in order, which is the box read in row-major order;
//   - permute reads the input through permuted strides.
// When the innermost dim of the dense side is also contiguous on the strided side the copy
// is a plain coalesced move (move_kernel, float4 when offsets allow). When the permutation
// changes the innermost dim, tiles of 4096 elements go through LDS so that both the loads and
// the stores are coalesced (permute_tile_kernel; 64 x 64, or narrow along a short dim).
#include "kth_internal.h"

using namespace kth;

namespace {

constexpr int kBlock = 256;
constexpr int kMoveUnroll = 2;
constexpr int kTileElems = 4096;

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));

// The strided side of a move. Dim 0 is the innermost dim of the dense side; for the float4
// kernel size[0] is counted in float4s and stride[0] is 4. Strides and base are in floats.
struct MovePlan {
    int      ndim;
    uint32_t size[KTH_MAX_DIMS];
    FastDiv  div[KTH_MAX_DIMS];
    uint32_t stride[KTH_MAX_DIMS];
    uint32_t base;
};

__device__ __forceinline__ uint32_t strided_offset(const MovePlan& pl, uint32_t idx) {
    uint32_t off = pl.base;
    for (int d = 0; d < pl.ndim - 1; d++) {
        uint32_t q = (__umulhi(idx, pl.div[d].mul) + idx) >> pl.div[d].shift;
        off += (idx - q * pl.size[d]) * pl.stride[d];
        idx = q;
    }
    return off + idx * pl.stride[pl.ndim - 1];
}

// MODE 0: dense[i] = strided[at(i)]   (range get, permute with the innermost dim kept)
// MODE 1: strided[at(i)] = dense[i]   (range set)
// MODE 2: strided[at(i)] = value      (range fill)
// `units` counts float4s (VEC) or floats of the dense side.
template <int MODE, bool VEC>
__global__ __launch_bounds__(kBlock) void move_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                     uint32_t units, float value, MovePlan pl) {
    const uint32_t base = blockIdx.x * (kBlock * kMoveUnroll) + threadIdx.x;
    if (VEC) {
        v4f v[kMoveUnroll];
        uint32_t at[kMoveUnroll];
#pragma unroll
        for (int k = 0; k < kMoveUnroll; k++) {
            const uint32_t i = base + k * kBlock;
            if (i < units) {
                at[k] = strided_offset(pl, i);
                if (MODE == 0) v[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src + at[k]));
                else if (MODE == 1) v[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src) + i);
                else v[k] = v4f{value, value, value, value};
            }
        }
#pragma unroll
        for (int k = 0; k < kMoveUnroll; k++) {
            const uint32_t i = base + k * kBlock;
            if (i < units) {
                if (MODE == 0) reinterpret_cast<v4f*>(dst)[i] = v[k];
                else *reinterpret_cast<v4f*>(dst + at[k]) = v[k];
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < kMoveUnroll; k++) {
            const uint32_t i = base + k * kBlock;
            if (i < units) {
                const uint32_t at = strided_offset(pl, i);
                if (MODE == 0) dst[i] = src[at];
                else if (MODE == 1) dst[at] = src[i];
                else dst[at] = value;
            }
        }
    }
}

// The same moves when the strided side cannot take float4s (odd run lengths or offsets): the
// dense side still moves as float4s, 16-byte aligned from the start of its store. Where its four
// floats are neighbours on the strided side as well they move there as one 16-byte access at a
// dword address, otherwise one by one. `n` counts floats; for MODE 2 the dense side is the fill value.
typedef float v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));

// Offsets on the strided side of dense floats i+1 .. i+3, given float i's (`first`, at place r0 of
// its innermost run). Floats past `n` get `first`; their lanes are never moved.
__device__ __forceinline__ void straddling_offsets(const MovePlan& pl, uint32_t i, uint32_t n, uint32_t r0, uint32_t first,
                                                   uint32_t at[4]) {
    at[0] = first;
#pragma unroll
    for (int j = 1; j < 4; j++)
        at[j] = (pl.ndim == 1 || r0 + j < pl.size[0]) ? first + j * pl.stride[0] : (i + j < n ? strided_offset(pl, i + j) : first);
}

constexpr int kMixedUnroll = 1;              // units of four floats per thread (2 and 4 measured 3-7 % slower)

template <int MODE>
__global__ __launch_bounds__(kBlock) void move_mixed_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                           uint32_t n, float value, MovePlan pl) {
    const uint32_t base = blockIdx.x * (kBlock * kMixedUnroll) + threadIdx.x;
    uint32_t first[kMixedUnroll], place[kMixedUnroll];
    bool run4[kMixedUnroll];                  // the four floats lie next to each other on the strided side too
    v4f v[kMixedUnroll];
#pragma unroll
    for (int k = 0; k < kMixedUnroll; k++) {
        const uint32_t i = (base + k * kBlock) * 4u;
        run4[k] = false;
        if (i >= n) continue;
        // position inside the innermost run decides whether the four floats share it
        const uint32_t q0 = (__umulhi(i, pl.div[0].mul) + i) >> pl.div[0].shift;
        place[k] = i - q0 * pl.size[0];
        first[k] = strided_offset(pl, i);
        run4[k] = pl.stride[0] == 1 && (pl.ndim == 1 || place[k] + 3 < pl.size[0]) && i + 3 < n;
        if (MODE == 0) {
            if (run4[k]) {                   // one 16-byte load from a dword address
                const v4f_unaligned t = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(src + first[k]));
                v[k] = v4f{t.x, t.y, t.z, t.w};
            } else {
                uint32_t at[4];
                straddling_offsets(pl, i, n, place[k], first[k], at);
                v[k].x = src[at[0]];
                v[k].y = i + 1 < n ? src[at[1]] : 0.0f;
                v[k].z = i + 2 < n ? src[at[2]] : 0.0f;
                v[k].w = i + 3 < n ? src[at[3]] : 0.0f;
            }
        } else if (MODE == 2) {
            v[k] = v4f{value, value, value, value};
        } else if (i + 3 < n) {
            v[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src + i));
        } else {
            v[k].x = src[i]; v[k].y = i + 1 < n ? src[i + 1] : 0.0f; v[k].z = i + 2 < n ? src[i + 2] : 0.0f; v[k].w = 0.0f;
        }
    }
#pragma unroll
    for (int k = 0; k < kMixedUnroll; k++) {
        const uint32_t i = (base + k * kBlock) * 4u;
        if (i >= n) continue;
        if (MODE == 0) {
            if (i + 3 < n) *reinterpret_cast<v4f*>(dst + i) = v[k];
            else { dst[i] = v[k].x; if (i + 1 < n) dst[i + 1] = v[k].y; if (i + 2 < n) dst[i + 2] = v[k].z; }
        } else if (run4[k]) {
            *reinterpret_cast<v4f_unaligned*>(dst + first[k]) = v4f_unaligned{v[k].x, v[k].y, v[k].z, v[k].w};
        } else {
            uint32_t at[4];
            straddling_offsets(pl, i, n, place[k], first[k], at);
            dst[at[0]] = v[k].x;
            if (i + 1 < n) dst[at[1]] = v[k].y;
            if (i + 2 < n) dst[at[2]] = v[k].z;
            if (i + 3 < n) dst[at[3]] = v[k].w;
        }
    }
}

// A permutation that moves the input's contiguous dim X away from the innermost place:
// the output's innermost dim is Y (input stride y_in_stride), X lands at output stride
// x_out_stride, and every other dim is a batch dim with its own pair of strides.
// Two or three dims that lie in memory as one dim on one side of a permutation and apart on the other: index i of the
// joined dim is (i % len0) of the innermost, ((i / len0) % len1) of the middle and (i / len0 / len1) of the outermost one.
struct JoinedDims {
    uint32_t len0;                           // 0: the dim is not a joined one
    FastDiv  div0;
    uint32_t len1;                           // 0: two dims
    FastDiv  div1;
    uint32_t stride1, stride2;               // the middle and the outermost dim's strides on the other side
};

__device__ __forceinline__ uint32_t joined_offset(const JoinedDims& j, uint32_t i, uint32_t stride0) {
    if (!j.len0) return i * stride0;
    const uint32_t t = (__umulhi(i, j.div0.mul) + i) >> j.div0.shift;
    const uint32_t lo = i - t * j.len0;
    if (!j.len1) return lo * stride0 + t * j.stride1;
    const uint32_t hi = (__umulhi(t, j.div1.mul) + t) >> j.div1.shift;
    return lo * stride0 + (t - hi * j.len1) * j.stride1 + hi * j.stride2;
}

struct TilePlan {
    uint32_t x_len, y_len;
    uint32_t x_out_stride, y_in_stride;
    uint32_t x_tiles, y_tiles;
    FastDiv  x_tiles_div, y_tiles_div;
    JoinedDims xs;                           // X is two or three dims that the input holds as one run, each with its own place in the output
    JoinedDims ys;                           // ... and Y two or three dims that the output holds as one run, each with its own place in the input
    uint32_t tiles;                          // permute_tile_kernel: the grid holds this many rounded up to a multiple of 8
    uint32_t by_xcd;                         // ... and an XCD takes a contiguous eighth of them (rows that do not start on a cache line)
    int      nbatch;
    uint32_t bsize[KTH_MAX_DIMS];
    FastDiv  bdiv[KTH_MAX_DIMS];
    uint32_t b_in[KTH_MAX_DIMS], b_out[KTH_MAX_DIMS];
};

// One TX x TY tile of 4096 elements per workgroup (TX along the input's contiguous dim, TY
// along the output's). Element k * 256 + t of the tile is loaded by thread t in x-fastest
// order and stored in y-fastest order, so a wave instruction reads min(TX, 64) consecutive x
// and writes min(TY, 64) consecutive y; 64 x 64 is the square case, the narrow shapes serve a
// short x or y dim (channels-last images, small trailing dims), where consecutive rows of the
// short dim are usually adjacent in memory and the accesses stay contiguous across rows.
// The LDS row pitch TX + 1 is odd: both phases are free of bank conflicts.
// V is the element: a float, or a float2 / float4 when the permutation keeps an innermost
// dim of 2 or 4 floats in place (lengths, strides and offsets of the plan then count elements).
template <int TX, int TY, class V, bool JOINED>
__global__ __launch_bounds__(kBlock) void permute_tile_kernel(const V* __restrict__ in, V* __restrict__ out, TilePlan pl) {
    static_assert(TX * TY * sizeof(V) == kTileElems * sizeof(float), "a tile holds 16 KiB");
    __shared__ V tile[TY * (TX + 1)];
    // Workgroups go to the eight XCDs in turn. When the rows of the output or of the input do not start on a cache
    // line, each XCD takes one contiguous eighth of the tiles, so that the two tiles that share a line write it into
    // one L2, where the halves meet, and not into two, each of which would send a partial line to memory. With
    // aligned rows the tiles go round the XCDs one by one, which spreads the memory channels better (6.2 TB/s on
    // 8192 x 8192 against 3.8 by eighths).
    uint32_t t = pl.by_xcd ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    if (t >= pl.tiles) return;
    uint32_t q = (__umulhi(t, pl.x_tiles_div.mul) + t) >> pl.x_tiles_div.shift;
    const uint32_t x0 = (t - q * pl.x_tiles) * TX;
    t = q;
    q = (__umulhi(t, pl.y_tiles_div.mul) + t) >> pl.y_tiles_div.shift;
    const uint32_t y0 = (t - q * pl.y_tiles) * TY;
    t = q;
    uint32_t in_off = 0, out_off = 0;
    for (int d = 0; d < pl.nbatch; d++) {
        q = (__umulhi(t, pl.bdiv[d].mul) + t) >> pl.bdiv[d].shift;
        const uint32_t r = t - q * pl.bsize[d];
        in_off += r * pl.b_in[d];
        out_off += r * pl.b_out[d];
        t = q;
    }
    constexpr int kPasses = TX * TY / kBlock;
    V v[kPasses];
#pragma unroll
    for (int k = 0; k < kPasses; k++) {
        const uint32_t e = k * kBlock + threadIdx.x;
        const uint32_t x = x0 + e % TX, y = y0 + e / TX;
        if (x < pl.x_len && y < pl.y_len) {
            v[k] = __builtin_nontemporal_load(in + in_off + (JOINED ? joined_offset(pl.ys, y, pl.y_in_stride) : y * pl.y_in_stride) + x);
        }
    }
#pragma unroll
    for (int k = 0; k < kPasses; k++) {
        const uint32_t e = k * kBlock + threadIdx.x;
        tile[(e / TX) * (TX + 1) + e % TX] = v[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kPasses; k++) {
        const uint32_t e = k * kBlock + threadIdx.x;
        const uint32_t lx = e / TY, ly = e % TY;
        const uint32_t x = x0 + lx, y = y0 + ly;
        if (x < pl.x_len && y < pl.y_len) {
            out[out_off + (JOINED ? joined_offset(pl.xs, x, pl.x_out_stride) : x * pl.x_out_stride) + y] = tile[ly * (TX + 1) + lx];
        }
    }
}

// A permutation that keeps a short innermost run of `run` floats (3 ... 63 here) in place and
// transposes the dims outside it: the tile is T x T runs (T = 32 for runs up to 4 floats, 16 up
// to 16 floats, 8 above), read as T spans of T * run contiguous floats (x fastest) and written as T spans of
// T * run contiguous floats (y fastest). LDS holds the tile as [x][y][run] at an odd pitch per x,
// so the store phase reads it linearly. Lengths, strides and offsets of `t` count runs. The
// element V is a float4 when the run is a multiple of 4 floats (run, pitch then count float4s).
struct RunsPlan {
    TilePlan t;
    uint32_t run, tile, pitch;               // elements per run, runs per tile side, LDS elements per x
    uint32_t tiles;                          // the grid holds this many rounded up to a multiple of 8
    FastDiv  in_row_div, run_div, out_row_div;
    FastDiv  unit_row_div;                   // by the 16-byte units of one span (float runs only)
};

template <class V>
__global__ __launch_bounds__(kBlock) void permute_runs_kernel(const V* __restrict__ in, V* __restrict__ out, RunsPlan rp) {
    constexpr uint32_t kElems = kTileElems * sizeof(float) / sizeof(V);      // 16 KiB of elements
    __shared__ V tile[kElems + 64];
    const TilePlan& pl = rp.t;
    // Workgroups go to the eight XCDs in turn: give each XCD one contiguous eighth of the tiles, so
    // that the cache lines two neighbouring tiles share are fetched into one L2 and not into two.
    uint32_t t = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (t >= rp.tiles) return;
    uint32_t q = (__umulhi(t, pl.x_tiles_div.mul) + t) >> pl.x_tiles_div.shift;
    const uint32_t x0 = (t - q * pl.x_tiles) * rp.tile;
    t = q;
    q = (__umulhi(t, pl.y_tiles_div.mul) + t) >> pl.y_tiles_div.shift;
    const uint32_t y0 = (t - q * pl.y_tiles) * rp.tile;
    t = q;
    uint32_t in_off = 0, out_off = 0;
    for (int d = 0; d < pl.nbatch; d++) {
        q = (__umulhi(t, pl.bdiv[d].mul) + t) >> pl.bdiv[d].shift;
        const uint32_t r = t - q * pl.bsize[d];
        in_off += r * pl.b_in[d];
        out_off += r * pl.b_out[d];
        t = q;
    }
    const uint32_t row = rp.tile * rp.run;                   // elements of one span
    const uint32_t floats = rp.tile * row;
    const V* src = in + (static_cast<size_t>(in_off) + x0) * rp.run;
    V* dst = out + (static_cast<size_t>(out_off) + y0) * rp.run;
    const uint32_t x_floats = min(rp.tile, pl.x_len - x0) * rp.run;   // valid part of an input span
    const uint32_t y_floats = min(rp.tile, pl.y_len - y0) * rp.run;   // valid part of an output span
    if constexpr (sizeof(V) == sizeof(float)) {
        // Runs of floats: a span (a whole number of runs, a multiple of 8 floats) moves as 16-byte
        // units at dword addresses on both sides; only a unit over the valid end of a span at the
        // tensor's edge moves float by float.
        const uint32_t upr = row >> 2;
        const uint32_t units = rp.tile * upr;
        constexpr uint32_t kUnitPasses = kElems / 4 / kBlock;
        v4f v[kUnitPasses];
#pragma unroll
        for (uint32_t k = 0; k < kUnitPasses; k++) {
            const uint32_t u = k * kBlock + threadIdx.x;
            if (u < units) {
                const uint32_t y = (__umulhi(u, rp.unit_row_div.mul) + u) >> rp.unit_row_div.shift;
                const uint32_t p = (u - y * upr) * 4u;
                if (y0 + y < pl.y_len && p < x_floats) {
                    const float* g = src + static_cast<size_t>(joined_offset(pl.ys, y0 + y, pl.y_in_stride)) * rp.run + p;
                    if (p + 4 <= x_floats) {
                        const v4f_unaligned t4 = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(g));
                        v[k] = v4f{t4.x, t4.y, t4.z, t4.w};
                    } else {
                        v[k].x = g[0];
                        v[k].y = p + 1 < x_floats ? g[1] : 0.0f;
                        v[k].z = p + 2 < x_floats ? g[2] : 0.0f;
                        v[k].w = 0.0f;
                    }
                }
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < kUnitPasses; k++) {
            const uint32_t u = k * kBlock + threadIdx.x;
            if (u < units) {
                const uint32_t y = (__umulhi(u, rp.unit_row_div.mul) + u) >> rp.unit_row_div.shift;
                const uint32_t p = (u - y * upr) * 4u;
                const uint32_t x = (__umulhi(p, rp.run_div.mul) + p) >> rp.run_div.shift;
                uint32_t r = p - x * rp.run, at = x * rp.pitch + y * rp.run;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    tile[at + r] = v[k][j];
                    if (++r == rp.run) { r = 0; at += rp.pitch; }
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t k = 0; k < kUnitPasses; k++) {
            const uint32_t u = k * kBlock + threadIdx.x;
            if (u < units) {
                const uint32_t x = (__umulhi(u, rp.unit_row_div.mul) + u) >> rp.unit_row_div.shift;
                const uint32_t p = (u - x * upr) * 4u;
                if (x0 + x < pl.x_len && p < y_floats) {
                    const float* l = tile + x * rp.pitch + p;
                    float* g = dst + static_cast<size_t>(joined_offset(pl.xs, x0 + x, pl.x_out_stride)) * rp.run + p;
                    if (p + 4 <= y_floats) {
                        *reinterpret_cast<v4f_unaligned*>(g) = v4f_unaligned{l[0], l[1], l[2], l[3]};
                    } else {
                        g[0] = l[0];
                        if (p + 1 < y_floats) g[1] = l[1];
                        if (p + 2 < y_floats) g[2] = l[2];
                    }
                }
            }
        }
        return;
    } else {
        constexpr uint32_t kPasses = kElems / kBlock;
        V v[kPasses];
#pragma unroll
        for (uint32_t k = 0; k < kPasses; k++) {
            const uint32_t f = k * kBlock + threadIdx.x;
            if (f < floats) {
                const uint32_t y = (__umulhi(f, rp.in_row_div.mul) + f) >> rp.in_row_div.shift;
                const uint32_t p = f - y * row;
                if (y0 + y < pl.y_len && p < x_floats)
                    v[k] = __builtin_nontemporal_load(src + static_cast<size_t>(joined_offset(pl.ys, y0 + y, pl.y_in_stride)) * rp.run + p);
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < kPasses; k++) {
            const uint32_t f = k * kBlock + threadIdx.x;
            if (f < floats) {
                const uint32_t y = (__umulhi(f, rp.in_row_div.mul) + f) >> rp.in_row_div.shift;
                const uint32_t p = f - y * row;
                const uint32_t x = (__umulhi(p, rp.run_div.mul) + p) >> rp.run_div.shift;
                tile[x * rp.pitch + y * rp.run + (p - x * rp.run)] = v[k];
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t k = 0; k < kPasses; k++) {
            const uint32_t f = k * kBlock + threadIdx.x;
            if (f < floats) {
                const uint32_t x = (__umulhi(f, rp.out_row_div.mul) + f) >> rp.out_row_div.shift;
                const uint32_t p = f - x * row;
                if (x0 + x < pl.x_len && p < y_floats)
                    dst[static_cast<size_t>(joined_offset(pl.xs, x0 + x, pl.x_out_stride)) * rp.run + p] = tile[x * rp.pitch + p];
            }
        }
    }
}

// Many small transposes: the (x, y) slab of x_len * y_len floats is contiguous on both sides
// and so is the batch dim right outside it, so a workgroup moves a run of whole slabs: one
// contiguous span in, the same span out, the transposition done by the LDS addressing (rows
// parked at an odd pitch).
struct SlabPlan {
    uint32_t x_len, y_len, slab, pitch;      // pitch = x_len | 1: LDS position of (y, x) is y * pitch + x
    uint32_t group, groups, batch0;          // slabs per workgroup, workgroups per outer batch entry, slabs per outer entry
    FastDiv  slab_div, x_div, y_div, groups_div;
    int      nbatch;                         // batch dims outside the innermost one
    uint32_t bsize[KTH_MAX_DIMS];
    FastDiv  bdiv[KTH_MAX_DIMS];
    uint32_t b_in[KTH_MAX_DIMS], b_out[KTH_MAX_DIMS];
};

constexpr uint32_t kSlabTile = 4096;

__global__ __launch_bounds__(kBlock) void permute_slabs_kernel(const float* __restrict__ in, float* __restrict__ out, SlabPlan pl) {
    __shared__ float tile[kSlabTile + kSlabTile / 2 + 8];
    uint32_t t = blockIdx.x;
    uint32_t q = (__umulhi(t, pl.groups_div.mul) + t) >> pl.groups_div.shift;
    const uint32_t first = (t - q * pl.groups) * pl.group;
    t = q;
    uint32_t in_off = first * pl.slab, out_off = first * pl.slab;
    for (int d = 0; d < pl.nbatch; d++) {
        q = (__umulhi(t, pl.bdiv[d].mul) + t) >> pl.bdiv[d].shift;
        const uint32_t r = t - q * pl.bsize[d];
        in_off += r * pl.b_in[d];
        out_off += r * pl.b_out[d];
        t = q;
    }
    const uint32_t slabs = min(pl.group, pl.batch0 - first);
    const uint32_t floats = slabs * pl.slab, lds_slab = pl.y_len * pl.pitch;
    // The span moves as 16-byte units at dword addresses on both sides. A unit's first element is placed by two
    // divisions, the other three step from it: along x and over the ends of rows and slabs on the way in (the LDS
    // position just grows: a slab's rows follow each other at the row pitch, and so do the slabs), along y and over
    // the ends of columns and slabs on the way out.
    constexpr uint32_t kUnits = kSlabTile / 4 / kBlock;
    const float* src = in + in_off;
    float* dst = out + out_off;
    v4f v[kUnits];
#pragma unroll
    for (uint32_t k = 0; k < kUnits; k++) {
        const uint32_t e = (k * kBlock + threadIdx.x) * 4u;
        if (e + 4 <= floats) {
            const v4f_unaligned t4 = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(src + e));
            v[k] = v4f{t4.x, t4.y, t4.z, t4.w};
        } else if (e < floats) {
            v[k].x = src[e];
            v[k].y = e + 1 < floats ? src[e + 1] : 0.0f;
            v[k].z = e + 2 < floats ? src[e + 2] : 0.0f;
            v[k].w = 0.0f;
        }
    }
#pragma unroll
    for (uint32_t k = 0; k < kUnits; k++) {
        const uint32_t e = (k * kBlock + threadIdx.x) * 4u;
        if (e < floats) {                                     // input order inside a slab: (y, x), x fastest
            const uint32_t g = (__umulhi(e, pl.slab_div.mul) + e) >> pl.slab_div.shift;
            const uint32_t r = e - g * pl.slab;
            const uint32_t y = (__umulhi(r, pl.x_div.mul) + r) >> pl.x_div.shift;
            uint32_t x = r - y * pl.x_len;
            uint32_t at = g * lds_slab + y * pl.pitch + x;
#pragma unroll
            for (uint32_t j = 0; j < 4; j++) {
                if (e + j < floats) tile[at] = v[k][j];
                at++;
                if (++x == pl.x_len) { x = 0; at += pl.pitch - pl.x_len; }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < kUnits; k++) {
        const uint32_t e = (k * kBlock + threadIdx.x) * 4u;
        if (e < floats) {                                     // output order inside a slab: (x, y), y fastest
            const uint32_t g = (__umulhi(e, pl.slab_div.mul) + e) >> pl.slab_div.shift;
            const uint32_t r = e - g * pl.slab;
            uint32_t x = (__umulhi(r, pl.y_div.mul) + r) >> pl.y_div.shift;
            uint32_t y = r - x * pl.y_len;
            uint32_t column = g * lds_slab + x;               // LDS position of (y = 0, x) of this slab
            float w[4];
#pragma unroll
            for (uint32_t j = 0; j < 4; j++) {
                w[j] = e + j < floats ? tile[column + y * pl.pitch] : 0.0f;
                if (++y == pl.y_len) {
                    y = 0; column++;
                    if (++x == pl.x_len) { x = 0; column += lds_slab - pl.x_len; }
                }
            }
            if (e + 4 <= floats) {
                *reinterpret_cast<v4f_unaligned*>(dst + e) = v4f_unaligned{w[0], w[1], w[2], w[3]};
            } else {
                dst[e] = w[0];
                if (e + 1 < floats) dst[e + 1] = w[1];
                if (e + 2 < floats) dst[e + 2] = w[2];
            }
        }
    }
}

int shape_count(const int32_t* shape, int dims, const char* what, uint64_t* count) {
    if (dims < 1 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "%s: %d dims (1..%d)", what, dims, KTH_MAX_DIMS);
    if (!shape) return fail(KTH_E_ARGUMENT, "%s: null shape", what);
    uint64_t n = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0) return fail(KTH_E_ARGUMENT, "%s: negative dim %d", what, shape[i]);
        n *= static_cast<uint64_t>(shape[i]);
        if (n > kMaxElements) return fail(KTH_E_ARGUMENT, "%s: more than 2^31-1 elements", what);
    }
    *count = n;
    return KTH_OK;
}

// A dense logical tensor seen through strides: dims innermost first.
struct StridedDims {
    int      n;
    uint64_t size[KTH_MAX_DIMS];
    uint64_t stride[KTH_MAX_DIMS];
};

// Drops size-1 dims and merges a dim into the one inside it when the strided side steps
// through both as through one longer dim.
StridedDims coalesce(const StridedDims& in) {
    StridedDims out{};
    for (int d = 0; d < in.n; d++) {
        if (in.size[d] == 1) continue;
        if (out.n > 0 && in.stride[d] == out.stride[out.n - 1] * out.size[out.n - 1]) out.size[out.n - 1] *= in.size[d];
        else { out.size[out.n] = in.size[d]; out.stride[out.n] = in.stride[d]; out.n++; }
    }
    if (out.n == 0) { out.n = 1; out.size[0] = 1; out.stride[0] = 1; }
    return out;
}

// Launches move_kernel<MODE> over `count` dense elements; `dims` must have stride[0] == 1
// for the float4 form to apply.
template <int MODE>
void launch_move(const char* family, const float* src, float* dst, uint64_t count, float value,
                 const StridedDims& dims, uint64_t base, uint64_t bytes) {
    MovePlan pl{};
    pl.ndim = dims.n;
    pl.base = static_cast<uint32_t>(base);
    bool vec = dims.stride[0] == 1 && dims.size[0] % 4 == 0 && base % 4 == 0;
    for (int d = 1; d < dims.n; d++) vec = vec && dims.stride[d] % 4 == 0;
    for (int d = 0; d < dims.n; d++) {
        pl.size[d] = static_cast<uint32_t>(dims.size[d]);
        pl.stride[d] = static_cast<uint32_t>(dims.stride[d]);
    }
    uint64_t units = count;
    if (vec) { pl.size[0] /= 4; pl.stride[0] = 4; units = count / 4; }
    for (int d = 0; d < dims.n; d++) pl.div[d] = make_div(pl.size[d]);
    const uint32_t per_block = kBlock * kMoveUnroll;
    if (!vec && count >= 1024) {
        const uint32_t per_block4 = kBlock * kMixedUnroll;
        const uint32_t blocks4 = static_cast<uint32_t>(((count + 3) / 4 + per_block4 - 1) / per_block4);
        LaunchScope scope(family, "float4 dense side", bytes);
        hipLaunchKernelGGL((move_mixed_kernel<MODE>), dim3(blocks4), dim3(kBlock), 0, state().stream, src, dst,
                           static_cast<uint32_t>(count), value, pl);
        return;
    }
    const uint32_t blocks = static_cast<uint32_t>((units + per_block - 1) / per_block);
    LaunchScope scope(family, vec ? "float4" : "float", bytes);
    if (vec) hipLaunchKernelGGL((move_kernel<MODE, true>), dim3(blocks), dim3(kBlock), 0, state().stream, src, dst,
                                static_cast<uint32_t>(units), value, pl);
    else     hipLaunchKernelGGL((move_kernel<MODE, false>), dim3(blocks), dim3(kBlock), 0, state().stream, src, dst,
                                static_cast<uint32_t>(units), value, pl);
}

// concat: the output seen as rows of `row` floats, each made of one run per input (the run of input i: its axis
// length times the dims inside the axis). A thread makes 16 bytes of the output: it finds the row and the place in
// the row, picks the input whose run holds the place and loads from there -- so every line of the output is written
// once, whole, however short the runs are, where a range set per input would write each line in pieces. FORM 2: every
// run is a multiple of four floats, a unit never straddles two runs and loads as 16 aligned bytes. FORM 0: the four
// floats load one by one, each from where it lies. FORM 1, for long runs: four floats of one run load as 16 bytes
// from a dword address, the others as in FORM 0 (per 268 MB: one row of 16 777 217 floats 80 us against 96 us float
// by float, rows of 33 and 31 floats 115 us against 95 us; both forms in one kernel, chosen per unit, measured
// slower than either).
constexpr int kConcatMax = 8;
constexpr int kConcatUnroll = 2;
constexpr uint64_t kConcatLongRun = 64;      // floats of the longest run from which FORM 1 is taken

struct ConcatPlan {
    const float* in[kConcatMax];
    uint32_t from[kConcatMax];               // place in the output row where the run of input i starts
    uint32_t run[kConcatMax];
    uint32_t row;
    FastDiv  row_div;
};

// The plan's per-input values as wave-uniform registers, so that picking an input is a chain of selects between
// registers (left as indexed arrays, the compiler fetches the picked entry from the argument block per lane: two
// dependent loads before every load of data). `org` is the input's address less its place in the row, so that the
// element at place c of row r is org + 4 (r run + c).
typedef const float __attribute__((address_space(1)))* global_floats;       // an address made from integers: known to be device memory
typedef const v4f __attribute__((address_space(1)))* global_v4f;
typedef const v4f_unaligned __attribute__((address_space(1)))* global_v4f_unaligned;

template <int NI>
struct ConcatInputs {
    uint32_t from[NI], run[NI], org_lo[NI], org_hi[NI];
};

template <int NI>
__device__ __forceinline__ ConcatInputs<NI> concat_inputs(const ConcatPlan& pl) {
    ConcatInputs<NI> in;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const uint64_t org = reinterpret_cast<uint64_t>(pl.in[i]) - 4ull * pl.from[i];
        in.from[i] = __builtin_amdgcn_readfirstlane(pl.from[i]);
        in.run[i] = __builtin_amdgcn_readfirstlane(pl.run[i]);
        in.org_lo[i] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(org));
        in.org_hi[i] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(org >> 32));
    }
    return in;
}

template <int NI>
__device__ __forceinline__ global_floats concat_source(const ConcatPlan& pl, const ConcatInputs<NI>& in, uint32_t e, uint32_t& left) {
    const uint32_t r = (__umulhi(e, pl.row_div.mul) + e) >> pl.row_div.shift;
    const uint32_t c = e - r * pl.row;
    uint32_t from = 0, run = in.run[0], lo = in.org_lo[0], hi = in.org_hi[0];
#pragma unroll
    for (int i = 1; i < NI; i++) {
        const bool here = c >= in.from[i];
        from = here ? in.from[i] : from;
        run = here ? in.run[i] : run;
        lo = here ? in.org_lo[i] : lo;
        hi = here ? in.org_hi[i] : hi;
    }
    left = from + run - c;                   // floats from here to the end of the run
    const uint64_t org = (static_cast<uint64_t>(hi) << 32) | lo;
    return reinterpret_cast<global_floats>(org + 4ull * (r * run + c));
}

template <int NI, int FORM>
__global__ __launch_bounds__(kBlock) void concat_kernel(float* __restrict__ out, uint32_t n, ConcatPlan pl) {
    const uint32_t base = blockIdx.x * (kBlock * kConcatUnroll) + threadIdx.x;
    const ConcatInputs<NI> in = concat_inputs<NI>(pl);
    v4f v[kConcatUnroll];
#pragma unroll
    for (int k = 0; k < kConcatUnroll; k++) {
        const uint32_t e = (base + k * kBlock) * 4u;
        if (e >= n) continue;
        uint32_t left;
        const global_floats at = concat_source<NI>(pl, in, e, left);
        if (FORM == 2) {
            v[k] = __builtin_nontemporal_load(reinterpret_cast<global_v4f>(at));
        } else if (FORM == 1 && left >= 4 && e + 4 <= n) {
            const v4f_unaligned t = __builtin_nontemporal_load(reinterpret_cast<global_v4f_unaligned>(at));
            v[k] = v4f{t.x, t.y, t.z, t.w};
        } else {
            float w[4];
            w[0] = *at;
#pragma unroll
            for (uint32_t j = 1; j < 4; j++) {
                w[j] = 0.0f;
                if (e + j < n) {
                    uint32_t unused;
                    w[j] = j < left ? at[j] : *concat_source<NI>(pl, in, e + j, unused);
                }
            }
            v[k] = v4f{w[0], w[1], w[2], w[3]};
        }
    }
#pragma unroll
    for (int k = 0; k < kConcatUnroll; k++) {
        const uint32_t e = (base + k * kBlock) * 4u;
        if (e >= n) continue;
        if (e + 4 <= n) {
            *reinterpret_cast<v4f*>(out + e) = v[k];
        } else {
            out[e] = v[k].x;
            if (e + 1 < n) out[e + 1] = v[k].y;
            if (e + 2 < n) out[e + 2] = v[k].z;
        }
    }
}

// Validates normalised inclusive ranges and describes the selected box as the strided side
// of a move (dense side: the box in row-major order).
int box_of(const char* what, const int32_t* shape, int dims, const int32_t* first, const int32_t* last,
           StridedDims* box, uint64_t* base, uint64_t* count, uint64_t* total) {
    if (int rc = shape_count(shape, dims, what, total)) return rc;
    if (!first || !last) return fail(KTH_E_ARGUMENT, "%s: null range", what);
    StridedDims raw{};
    raw.n = dims;
    uint64_t run = 1, off = 0, n = 1;
    for (int d = dims - 1, k = 0; d >= 0; d--, k++) {
        if (first[d] < 0 || last[d] >= shape[d] || first[d] > last[d])
            return fail(KTH_E_ARGUMENT, "%s: range %d..%d does not index a dim of size %d", what, first[d], last[d], shape[d]);
        raw.size[k] = static_cast<uint64_t>(last[d] - first[d] + 1);
        raw.stride[k] = run;
        off += static_cast<uint64_t>(first[d]) * run;
        n *= raw.size[k];
        run *= static_cast<uint64_t>(shape[d]);
    }
    *box = coalesce(raw);
    if (box->n == 1 && box->size[0] == 1) box->stride[0] = 1;
    *base = off;
    *count = n;
    return KTH_OK;
}

// Permutes through LDS tiles. `v`: the output's dims innermost first with the input's strides,
// in units of `elem` floats (1, 2, 4, or a run of 3 ... 63), stride[0] != 1. Returns KTH_OK after launching,
// kTilesDeclined (nothing launched) when the tiles would be mostly empty.
constexpr int kTilesDeclined = 1;
int launch_tiles(const char* what, const StridedDims& v, int elem, const float* in, float* out, uint64_t n) {
    int px = -1;
    for (int d = 1; d < v.n; d++) if (v.stride[d] == 1) px = d;
    if (px < 0) return fail(KTH_E_DEVICE, "%s: no contiguous input dim found", what);
    const uint32_t x_len = static_cast<uint32_t>(v.size[px]), y_len = static_cast<uint32_t>(v.size[0]);
    const uint32_t y_in_stride = static_cast<uint32_t>(v.stride[0]);
    uint64_t x_out_stride = 1;
    for (int d = 0; d < px; d++) x_out_stride *= v.size[d];
    hipStream_t stream = state().stream;

    // Batch dims: every dim but X and Y, innermost first, with input and output strides.
    int nb = 0;
    uint32_t bsize[KTH_MAX_DIMS], b_in[KTH_MAX_DIMS], b_out[KTH_MAX_DIMS];
    uint64_t out_run = 1, batch = 1;
    for (int d = 0; d < v.n; d++) {
        if (d != px && d != 0) {
            bsize[nb] = static_cast<uint32_t>(v.size[d]);
            b_in[nb] = static_cast<uint32_t>(v.stride[d]);
            b_out[nb] = static_cast<uint32_t>(out_run);
            nb++;
            batch *= v.size[d];
        }
        out_run *= v.size[d];
    }

    const uint32_t slab = x_len * y_len;
    if (elem == 1 && slab <= kSlabTile / 2 && y_in_stride == x_len && x_out_stride == y_len && nb >= 1 &&
        b_in[0] == slab && b_out[0] == slab) {
        SlabPlan pl{};
        pl.x_len = x_len; pl.y_len = y_len; pl.slab = slab; pl.pitch = x_len | 1u;
        pl.batch0 = bsize[0];
        pl.group = kSlabTile / slab;
        if (pl.group > pl.batch0) pl.group = pl.batch0;
        pl.groups = (pl.batch0 + pl.group - 1) / pl.group;
        pl.slab_div = make_div(slab); pl.x_div = make_div(x_len); pl.y_div = make_div(y_len); pl.groups_div = make_div(pl.groups);
        uint64_t outer = 1;
        for (int d = 1; d < nb; d++) {
            pl.bsize[pl.nbatch] = bsize[d]; pl.bdiv[pl.nbatch] = make_div(bsize[d]);
            pl.b_in[pl.nbatch] = b_in[d]; pl.b_out[pl.nbatch] = b_out[d];
            pl.nbatch++;
            outer *= bsize[d];
        }
        const uint64_t blocks = static_cast<uint64_t>(pl.groups) * outer;
        if (blocks > kMaxElements) return fail(KTH_E_ARGUMENT, "%s: too many tiles", what);
        LaunchScope scope("permute_slabs_kernel", "", n * 8);
        hipLaunchKernelGGL(permute_slabs_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, stream, in, out, pl);
        return KTH_OK;
    }

    TilePlan pl{};
    pl.x_len = x_len; pl.y_len = y_len; pl.y_in_stride = y_in_stride;
    pl.x_out_stride = static_cast<uint32_t>(x_out_stride);
    // A short contiguous dim of the input whose neighbour in the input goes elsewhere in the output ([N,206,3] reversed:
    // rows of 618 floats of which a tile would take 3): the two are one X of 618 for the loads, and the store works
    // out the two output places from the index. A third dim joins when the two are still short ([N,189,3,3] by
    // [1,3,2,0]: X is the whole row of 1701 floats).
    for (int level = 0; level < 2 && pl.x_len < 64; level++) {
        int d = 0;
        while (d < nb && (b_in[d] != pl.x_len || static_cast<uint64_t>(pl.x_len) * bsize[d] > 0x7fffffffull)) d++;
        if (d == nb) break;
        if (level == 0) { pl.xs.len0 = pl.x_len; pl.xs.div0 = make_div(pl.x_len); pl.xs.stride1 = b_out[d]; }
        else { pl.xs.len1 = pl.x_len / pl.xs.len0; pl.xs.div1 = make_div(pl.xs.len1); pl.xs.stride2 = b_out[d]; }
        pl.x_len *= bsize[d];
        batch /= bsize[d];
        for (int k = d; k + 1 < nb; k++) { bsize[k] = bsize[k + 1]; b_in[k] = b_in[k + 1]; b_out[k] = b_out[k + 1]; }
        nb--;
    }
    // ... and a short contiguous dim of the output whose neighbours in the output come from elsewhere in the input.
    for (int level = 0; level < 2 && pl.y_len < 64; level++) {
        int d = 0;
        while (d < nb && (b_out[d] != pl.y_len || static_cast<uint64_t>(pl.y_len) * bsize[d] > 0x7fffffffull)) d++;
        if (d == nb) break;
        if (level == 0) { pl.ys.len0 = pl.y_len; pl.ys.div0 = make_div(pl.y_len); pl.ys.stride1 = b_in[d]; }
        else { pl.ys.len1 = pl.y_len / pl.ys.len0; pl.ys.div1 = make_div(pl.ys.len1); pl.ys.stride2 = b_in[d]; }
        pl.y_len *= bsize[d];
        batch /= bsize[d];
        for (int k = d; k + 1 < nb; k++) { bsize[k] = bsize[k + 1]; b_in[k] = b_in[k + 1]; b_out[k] = b_out[k + 1]; }
        nb--;
    }
    if (elem == 3 || elem > 4) {
        RunsPlan rp{};
        const bool vec = elem % 4 == 0;
        rp.run = static_cast<uint32_t>(vec ? elem / 4 : elem);
        rp.tile = elem <= 4 ? 32u : elem <= 16 ? 16u : 8u;
        if (pl.x_len < rp.tile || pl.y_len < rp.tile) return kTilesDeclined;
        rp.pitch = (rp.tile * rp.run) | 1u;
        rp.in_row_div = make_div(rp.tile * rp.run); rp.out_row_div = rp.in_row_div; rp.run_div = make_div(rp.run);
        rp.unit_row_div = make_div(rp.tile * rp.run / 4);
        pl.x_tiles = (pl.x_len + rp.tile - 1) / rp.tile;
        pl.y_tiles = (pl.y_len + rp.tile - 1) / rp.tile;
        pl.x_tiles_div = make_div(pl.x_tiles);
        pl.y_tiles_div = make_div(pl.y_tiles);
        pl.nbatch = nb;
        for (int d = 0; d < nb; d++) { pl.bsize[d] = bsize[d]; pl.bdiv[d] = make_div(bsize[d]); pl.b_in[d] = b_in[d]; pl.b_out[d] = b_out[d]; }
        rp.t = pl;
        const uint64_t blocks = static_cast<uint64_t>(pl.x_tiles) * pl.y_tiles * batch;
        if (blocks > kMaxElements - 8) return fail(KTH_E_ARGUMENT, "%s: too many tiles", what);   // (the grid is rounded up to 8)
        rp.tiles = static_cast<uint32_t>(blocks);
        const dim3 grid(static_cast<uint32_t>((blocks + 7) / 8 * 8));
        LaunchScope scope("permute_runs_kernel", vec ? "float4" : "float", n * 8);
        if (vec) hipLaunchKernelGGL((permute_runs_kernel<v4f>), grid, dim3(kBlock), 0, stream,
                                    reinterpret_cast<const v4f*>(in), reinterpret_cast<v4f*>(out), rp);
        else     hipLaunchKernelGGL((permute_runs_kernel<float>), grid, dim3(kBlock), 0, stream, in, out, rp);
        return KTH_OK;
    }
    // Tile shape: narrow along a dim shorter than 64 (the smallest power of two that holds it), square
    // otherwise; vector elements use one shape of 16 KiB.
    uint32_t tx = 64, ty = 64;
    if ((elem == 2 || elem == 4) && (pl.x_len < 16 || pl.y_len < 16)) return kTilesDeclined;
    if (elem == 4) { tx = 32; ty = 32; }
    else if (elem == 2) { tx = 64; ty = 32; }
    else if (pl.x_len < 64 && pl.x_len <= pl.y_len) { tx = 2; while (tx < pl.x_len) tx <<= 1; ty = kTileElems / tx; }
    else if (pl.y_len < 64) { ty = 2; while (ty < pl.y_len) ty <<= 1; tx = kTileElems / ty; }
    // A tile is 4096 elements, as narrow along a short dim as a power of two allows; when the input's contiguous dim
    // and the output's are both short (and have no neighbour to join), most of it hangs over: a [2,5] block transposed
    // inside 3 million batch items filled 10 of 4096 places and ran at 58 GB/s. Below an eighth full the caller's
    // element gather is the faster one (its reads stay inside the few cache lines of such a block).
    if (elem == 1) {
        const double filled = static_cast<double>(std::min(pl.x_len, tx)) / tx * static_cast<double>(std::min(pl.y_len, ty)) / ty;
        if (filled < 0.12) return kTilesDeclined;
    }
    pl.x_tiles = (pl.x_len + tx - 1) / tx;
    pl.y_tiles = (pl.y_len + ty - 1) / ty;
    pl.x_tiles_div = make_div(pl.x_tiles);
    pl.y_tiles_div = make_div(pl.y_tiles);
    pl.nbatch = nb;
    for (int d = 0; d < nb; d++) { pl.bsize[d] = bsize[d]; pl.bdiv[d] = make_div(bsize[d]); pl.b_in[d] = b_in[d]; pl.b_out[d] = b_out[d]; }
    const uint64_t blocks = static_cast<uint64_t>(pl.x_tiles) * pl.y_tiles * batch;
    if (blocks > kMaxElements - 8) return fail(KTH_E_ARGUMENT, "%s: too many tiles", what);
    pl.tiles = static_cast<uint32_t>(blocks);
    const uint32_t line = 128 / (4 * static_cast<uint32_t>(elem));                  // elements per cache line
    pl.by_xcd = (pl.x_out_stride % line != 0 || pl.y_in_stride % line != 0 || pl.xs.stride1 % line != 0 || pl.xs.stride2 % line != 0 ||
                 pl.ys.stride1 % line != 0 || pl.ys.stride2 % line != 0) ? 1u : 0u;
    for (int d = 0; d < nb; d++) if (b_in[d] % line != 0 || b_out[d] % line != 0) pl.by_xcd = 1u;
    const dim3 grid(static_cast<uint32_t>((blocks + 7) / 8 * 8));
    LaunchScope scope("permute_tile_kernel", elem == 4 ? "float4" : elem == 2 ? "float2" : "", n * 8);
    const bool joined = pl.xs.len0 != 0 || pl.ys.len0 != 0;                         // (the plain form keeps its address arithmetic free of the test)
#define KTH_TILE_V(TX, TY, V, J) hipLaunchKernelGGL((permute_tile_kernel<TX, TY, V, J>), grid, dim3(kBlock), 0, stream, reinterpret_cast<const V*>(in), \
                                                    reinterpret_cast<V*>(out), pl)
#define KTH_TILE(TX, TY) do { if (joined) KTH_TILE_V(TX, TY, float, true); else KTH_TILE_V(TX, TY, float, false); } while (0)
    if (elem == 4) {
        if (joined) KTH_TILE_V(32, 32, v4f, true); else KTH_TILE_V(32, 32, v4f, false);
    } else if (elem == 2) {
        if (joined) KTH_TILE_V(64, 32, v2f, true); else KTH_TILE_V(64, 32, v2f, false);
    } else {
        switch (tx) {
        case 2: KTH_TILE(2, 2048); break;    case 4: KTH_TILE(4, 1024); break;    case 8: KTH_TILE(8, 512); break;
        case 16: KTH_TILE(16, 256); break;   case 32: KTH_TILE(32, 128); break;   case 64: KTH_TILE(64, 64); break;
        case 128: KTH_TILE(128, 32); break;  case 256: KTH_TILE(256, 16); break;  case 512: KTH_TILE(512, 8); break;
        case 1024: KTH_TILE(1024, 4); break; default: KTH_TILE(2048, 2); break;
        }
    }
#undef KTH_TILE
#undef KTH_TILE_V
    return KTH_OK;
}

int permute_common(const char* what, uint64_t in, const int32_t* shape, int dims, const int32_t* axes, uint64_t out) {
    uint64_t n;
    if (int rc = shape_count(shape, dims, what, &n)) return rc;
    bool seen[KTH_MAX_DIMS] = {false};
    for (int d = 0; d < dims; d++) {
        if (axes[d] < 0 || axes[d] >= dims || seen[axes[d]])
            return fail(KTH_E_ARGUMENT, "%s: axes must name every dimension once", what);
        seen[axes[d]] = true;
    }
    Store* si = lookup(in, what, true);
    if (!si) return KTH_E_HANDLE;
    Store* so = lookup(out, what);
    if (!so) return KTH_E_HANDLE;
    if (n > si->n_floats || n > so->n_floats) return fail(KTH_E_ARGUMENT, "%s: the shape needs more elements than a store holds", what);
    if (si->ptr == so->ptr) return fail(KTH_E_ARGUMENT, "%s: output aliases the input", what);
    if (n == 0) return KTH_OK;
    return permute_device(what, si->ptr, so->ptr, shape, dims, axes);
}

}  // namespace

namespace kth {

// out = in with its dims reordered by `axes` (validated by the caller), both dense, n > 0 elements.
int permute_device(const char* what, const float* in, float* out, const int32_t* shape, int dims, const int32_t* axes) {
    uint64_t n = 1;
    for (int d = 0; d < dims; d++) n *= static_cast<uint64_t>(shape[d]);
    uint64_t in_stride[KTH_MAX_DIMS];
    uint64_t run = 1;
    for (int d = dims - 1; d >= 0; d--) { in_stride[d] = run; run *= static_cast<uint64_t>(shape[d]); }
    StridedDims raw{};
    raw.n = dims;
    for (int d = dims - 1, k = 0; d >= 0; d--, k++) {      // output dims, innermost first
        raw.size[k] = static_cast<uint64_t>(shape[axes[d]]);
        raw.stride[k] = in_stride[axes[d]];
    }
    const StridedDims v = coalesce(raw);
    if (v.stride[0] == 1 && (v.size[0] == 2 || v.size[0] == 4) && v.n >= 3) {
        // An innermost dim of 2 or 4 floats that stays in place: permute float2 / float4 elements
        // through tiles when the dims that do move (joined with their neighbours) are long enough to fill them.
        const uint64_t elem = v.size[0];
        StridedDims w{};
        for (int d = 1; d < v.n; d++) { w.size[w.n] = v.size[d]; w.stride[w.n] = v.stride[d] / elem; w.n++; }
        int wx = -1;
        for (int d = 1; d < w.n; d++) if (w.stride[d] == 1) wx = d;
        if (w.stride[0] != 1 && wx > 0) {
            const int rc = launch_tiles(what, w, static_cast<int>(elem), in, out, n);
            if (rc != kTilesDeclined) {
                if (rc) return rc;
                KTH_LAUNCH_CHECK("permute_tile_kernel");
                return KTH_OK;
            }
        }
    }
    if (v.stride[0] == 1 && v.size[0] >= 3 && (v.size[0] < 32 || (v.size[0] < 64 && v.size[0] % 4 != 0)) && v.n >= 3) {
        // A run of 3 ... 31 floats that stays innermost (up to 63 when it cannot move as float4s): tiles of
        // runs, when both transposed dims (joined with their neighbours) can fill one.
        const uint64_t run = v.size[0];
        StridedDims w{};
        for (int d = 1; d < v.n; d++) { w.size[w.n] = v.size[d]; w.stride[w.n] = v.stride[d] / run; w.n++; }
        int wx = -1;
        for (int d = 1; d < w.n; d++) if (w.stride[d] == 1) wx = d;
        if (w.stride[0] != 1 && wx > 0) {
            const int rc = launch_tiles(what, w, static_cast<int>(run), in, out, n);
            if (rc != kTilesDeclined) {
                if (rc) return rc;
                KTH_LAUNCH_CHECK("permute_runs_kernel");
                return KTH_OK;
            }
        }
    }
    if (v.stride[0] == 1) {
        launch_move<0>("move_kernel_permute", in, out, n, 0.0f, v, 0, n * 8);
        KTH_LAUNCH_CHECK("move_kernel");
        return KTH_OK;
    }
    // (launch_tiles declines shapes whose tiles would be mostly empty: the element gather of the range moves then)
    const int rc = launch_tiles(what, v, 1, in, out, n);
    if (rc == kTilesDeclined) {
        launch_move<0>("move_kernel_permute", in, out, n, 0.0f, v, 0, n * 8);
        KTH_LAUNCH_CHECK("move_kernel");
        return KTH_OK;
    }
    if (rc) return rc;
    KTH_LAUNCH_CHECK("permute_tile_kernel");
    return KTH_OK;
}

}  // namespace kth

extern "C" {

int kth_get_range(uint64_t in, const int32_t* shape, int dims, const int32_t* first, const int32_t* last, uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    StridedDims box; uint64_t base, count, total;
    if (int rc = box_of("kth_get_range", shape, dims, first, last, &box, &base, &count, &total)) return rc;
    Store* si = lookup(in, "kth_get_range(in)", true);
    if (!si) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_get_range(out)");
    if (!so) return KTH_E_HANDLE;
    if (total > si->n_floats || count > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_get_range: a shape needs more elements than its store holds");
    if (si->ptr == so->ptr) return fail(KTH_E_ARGUMENT, "kth_get_range: output aliases the input");
    launch_move<0>("move_kernel_get", si->ptr, so->ptr, count, 0.0f, box, base, count * 8);
    KTH_LAUNCH_CHECK("move_kernel");
    return KTH_OK;
}

int kth_set_range(uint64_t target, const int32_t* shape, int dims, const int32_t* first, const int32_t* last,
                  uint64_t value, uint64_t value_n) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    StridedDims box; uint64_t base, count, total;
    if (int rc = box_of("kth_set_range", shape, dims, first, last, &box, &base, &count, &total)) return rc;
    if (count != value_n)
        return fail(KTH_E_SHAPE, "Cannot set tensor with %llu elements to an index range of %llu elements",
                    static_cast<unsigned long long>(value_n), static_cast<unsigned long long>(count));
    Store* st = lookup(target, "kth_set_range(target)");
    if (!st) return KTH_E_HANDLE;
    Store* sv = lookup(value, "kth_set_range(value)", true);
    if (!sv) return KTH_E_HANDLE;
    if (total > st->n_floats || value_n > sv->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_set_range: a shape needs more elements than its store holds");
    if (st->ptr == sv->ptr) return fail(KTH_E_ARGUMENT, "kth_set_range: value aliases the target");
    launch_move<1>("move_kernel_set", sv->ptr, st->ptr, count, 0.0f, box, base, count * 8);
    KTH_LAUNCH_CHECK("move_kernel");
    return KTH_OK;
}

int kth_concat(const uint64_t* inputs, const int32_t* axis_lens, int n_inputs, const int32_t* out_shape, int dims, int axis,
               uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    uint64_t total;
    if (int rc = shape_count(out_shape, dims, "kth_concat", &total)) return rc;
    if (!inputs || !axis_lens || n_inputs < 1) return fail(KTH_E_ARGUMENT, "kth_concat: no inputs");
    if (axis < 0 || axis >= dims) return fail(KTH_E_ARGUMENT, "kth_concat: axis %d of %d dims", axis, dims);
    uint64_t inner = 1, outer = 1, along = 0;
    for (int d = axis + 1; d < dims; d++) inner *= static_cast<uint64_t>(out_shape[d]);
    for (int d = 0; d < axis; d++) outer *= static_cast<uint64_t>(out_shape[d]);
    for (int i = 0; i < n_inputs; i++) {
        if (axis_lens[i] < 0) return fail(KTH_E_ARGUMENT, "kth_concat: negative length %d of input %d", axis_lens[i], i);
        along += static_cast<uint64_t>(axis_lens[i]);
    }
    if (along != static_cast<uint64_t>(out_shape[axis]))
        return fail(KTH_E_SHAPE, "kth_concat: the inputs hold %llu along axis %d, the result %d",
                    static_cast<unsigned long long>(along), axis, out_shape[axis]);
    Store* so = lookup_unsettled(out, "kth_concat(out)");
    if (!so) return KTH_E_HANDLE;
    if (total > so->n_floats) return fail(KTH_E_ARGUMENT, "kth_concat: the result needs more elements than its store holds");
    std::vector<const float*> ptrs;
    std::vector<uint64_t> runs;
    for (int i = 0; i < n_inputs; i++) {
        Store* si = lookup(inputs[i], "kth_concat(input)", true);
        if (!si) return KTH_E_HANDLE;
        const uint64_t run = static_cast<uint64_t>(axis_lens[i]) * inner;
        if (outer * run > si->n_floats) return fail(KTH_E_ARGUMENT, "kth_concat: input %d needs more elements than its store holds", i);
        if (si->ptr == so->ptr) return fail(KTH_E_ARGUMENT, "kth_concat: the result aliases input %d", i);
        if (run == 0) continue;
        ptrs.push_back(si->ptr);
        runs.push_back(run);
    }
    settle_for_overwrite(so, total);
    if (total == 0) return KTH_OK;
    const uint64_t row = along * inner;
    hipStream_t stream = state().stream;
    if (ptrs.size() > static_cast<size_t>(kConcatMax)) {                // a range set per input
        uint64_t from = 0;
        for (size_t i = 0; i < ptrs.size(); i++) {
            StridedDims raw{};
            raw.n = 2;
            raw.size[0] = runs[i]; raw.stride[0] = 1;
            raw.size[1] = outer;   raw.stride[1] = row;
            launch_move<1>("move_kernel_set", ptrs[i], so->ptr, outer * runs[i], 0.0f, coalesce(raw), from, outer * runs[i] * 8);
            from += runs[i];
        }
        KTH_LAUNCH_CHECK("move_kernel");
        return KTH_OK;
    }
    ConcatPlan pl{};
    bool vec = true;
    uint64_t from = 0, longest = 0;
    for (int i = 0; i < kConcatMax; i++) {
        const bool have = static_cast<size_t>(i) < ptrs.size();
        pl.in[i] = have ? ptrs[i] : ptrs[0];
        pl.from[i] = have ? static_cast<uint32_t>(from) : 0xffffffffu;
        pl.run[i] = have ? static_cast<uint32_t>(runs[i]) : 0u;
        if (have) { vec = vec && runs[i] % 4 == 0; from += runs[i]; longest = std::max(longest, runs[i]); }
    }
    pl.row = static_cast<uint32_t>(row);
    pl.row_div = make_div(pl.row);
    const uint32_t n = static_cast<uint32_t>(total);
    const uint32_t per_block = kBlock * kConcatUnroll * 4;
    const dim3 grid(static_cast<uint32_t>((total + per_block - 1) / per_block)), block(kBlock);
    const int ni = ptrs.size() <= 2 ? 2 : ptrs.size() <= 4 ? 4 : 8;
    {
        const int form = vec ? 2 : longest >= kConcatLongRun ? 1 : 0;
        LaunchScope scope("concat_kernel", form == 2 ? "float4" : form == 1 ? "float4 result side, long runs" : "float4 result side", total * 8);
#define CONCAT_LAUNCH(NI) do { if (form == 2)      hipLaunchKernelGGL((concat_kernel<NI, 2>), grid, block, 0, stream, so->ptr, n, pl); \
                               else if (form == 1) hipLaunchKernelGGL((concat_kernel<NI, 1>), grid, block, 0, stream, so->ptr, n, pl); \
                               else                hipLaunchKernelGGL((concat_kernel<NI, 0>), grid, block, 0, stream, so->ptr, n, pl); } while (0)
        if (ni == 2) CONCAT_LAUNCH(2); else if (ni == 4) CONCAT_LAUNCH(4); else CONCAT_LAUNCH(8);
#undef CONCAT_LAUNCH
    }
    KTH_LAUNCH_CHECK("concat_kernel");
    return KTH_OK;
}

int kth_fill_range(uint64_t target, const int32_t* shape, int dims, const int32_t* first, const int32_t* last, float value) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    StridedDims box; uint64_t base, count, total;
    if (int rc = box_of("kth_fill_range", shape, dims, first, last, &box, &base, &count, &total)) return rc;
    Store* st = lookup(target, "kth_fill_range(target)");
    if (!st) return KTH_E_HANDLE;
    if (total > st->n_floats) return fail(KTH_E_ARGUMENT, "kth_fill_range: the shape needs more elements than the store holds");
    launch_move<2>("move_kernel_fill", nullptr, st->ptr, count, value, box, base, count * 4);
    KTH_LAUNCH_CHECK("move_kernel");
    return KTH_OK;
}

int kth_permute(uint64_t in, const int32_t* shape, int dims, const int32_t* axes, uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!axes) return fail(KTH_E_ARGUMENT, "kth_permute: null axes");
    if (dims < 1 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "kth_permute: %d dims", dims);
    return permute_common("kth_permute", in, shape, dims, axes, out);
}

int kth_transpose(uint64_t in, const int32_t* shape, int dims, int axis1, int axis2, uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (dims < 1 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "kth_transpose: %d dims", dims);
    if (axis1 < 0 || axis1 >= dims || axis2 < 0 || axis2 >= dims || axis1 == axis2)
        return fail(KTH_E_ARGUMENT, "Transpose requires different axes as parameters, but got %d and %d", axis1, axis2);
    int32_t axes[KTH_MAX_DIMS];
    for (int d = 0; d < dims; d++) axes[d] = d;
    axes[axis1] = axis2;
    axes[axis2] = axis1;
    return permute_common("kth_transpose", in, shape, dims, axes, out);
}

}  // extern "C"
