// Fused batch normalisation over one axis (reference:
// kten-api/.../tensor/operations/nn/BatchNormOperation.kt:5-41 and
// backend/kten-jvm/.../operations/nn/JVMBatchNorm.kt:33-183).
//
// The tensor is seen as [outer, channels, inner] around the axis. Per channel the reference
// makes serial float passes: sum -> mean, sum of squared deviations -> 1/sqrt(var + eps),
// then the affine map; backward: sum of gradOut, dot of (x - mean) with gradOut, then the
// input gradient. Here every pass over the data is one launch over all channels:
//
//   stats    one read of x (forward) or of x and gradOut (backward); two f64 sums per channel.
//            Forward sums d = x - k and d*d for k = the channel's first element, exactly in
//            f64; the sum of squared deviations from the rounded mean follows from them
//            (S2 - 2 (mean - k) S1 + n (mean - k)^2). Because k is one of the channel's own
//            elements the cancellation costs at most n * 2^-53 relative.
//   finalize one thread per channel folds the partials in a fixed order and does the scalar
//            float arithmetic of the reference (JVMBatchNorm.kt:57-82,128-137,150-152,
//            171-177) in its order, writing the per-channel parameters.
//   apply    one read (+ gradOut) and one write; the float expression of JVMBatchNorm.kt:88-90
//            / :153-164, evaluated left to right without contraction, so given equal
//            statistics the output bits equal the reference's. With long runs (NCHW images) the
//            apply kernel does the finalize step itself, per workgroup, for the few channels
//            its tile touches: two launches per pass instead of three.
//
// Sums accumulate in f64 in a fixed order: deterministic, and closer to the exact sums than
// the reference's serial float accumulation.
#include "kth_internal.h"

using namespace kth;

namespace {

constexpr int kBlock = 256;
constexpr int kBatch = 4;          // loads in flight per thread in the stats kernels
constexpr int kApplyUnroll = 2;

typedef float v4f __attribute__((ext_vector_type(4)));

struct Geometry {
    uint32_t outer, channels, inner;
    uint32_t per_channel;           // outer * inner
};

// ---------------------------------------------------------------- block fold of two doubles

__device__ __forceinline__ void block_fold2(double& a, double& b, double* lds) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        a += __shfl_xor(a, off);
        b += __shfl_xor(b, off);
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { lds[wave * 2] = a; lds[wave * 2 + 1] = b; }
    __syncthreads();
    if (threadIdx.x == 0) {
        a = lds[0]; b = lds[1];
        for (int w = 1; w < kBlock / 64; w++) { a += lds[w * 2]; b += lds[w * 2 + 1]; }
    }
}

// ---------------------------------------------------------------- stats, long runs (inner >= 64)

// Work of one channel: outer runs of `inner` contiguous floats, numbered through as units of W
// floats (W = 4 with float4 loads) and cut into chunks of kBlock units, so every lane has a unit
// whatever the run length; a workgroup takes the chunks
// [seg * chunks_per_seg, (seg + 1) * chunks_per_seg) of channel blockIdx.x / segments.
typedef float v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));

struct RunPlan {
    Geometry g;
    uint32_t segments, chunks_per_seg, total_chunks;
    uint32_t units_per_run, total_units;
    FastDiv  run_div, seg_div;               // run_div divides by units_per_run
};

// BACKWARD false: (sum of d, sum of d*d), d = x - k. BACKWARD true: (sum of g, sum of (x - mean) g).
template <bool BACKWARD, bool VEC>
__global__ __launch_bounds__(kBlock) void bn_stats_runs_kernel(const float* __restrict__ x, const float* __restrict__ go,
                                                              const float* __restrict__ mean, double* __restrict__ partial, RunPlan pl) {
    __shared__ double lds[2 * kBlock / 64];
    constexpr uint32_t W = 4;                // !VEC: runs of any length, 16-byte loads from dword addresses, ragged last unit
    const uint32_t b = blockIdx.x;
    const uint32_t c = (__umulhi(b, pl.seg_div.mul) + b) >> pl.seg_div.shift;
    const uint32_t seg = b - c * pl.segments;
    const uint32_t first = seg * pl.chunks_per_seg;
    uint32_t last = first + pl.chunks_per_seg;
    if (last > pl.total_chunks) last = pl.total_chunks;
    const double shift = BACKWARD ? static_cast<double>(mean[c]) : static_cast<double>(x[static_cast<uint64_t>(c) * pl.g.inner]);
    double s1 = 0.0, s2 = 0.0;
    for (uint32_t q0 = first; q0 < last; q0 += kBatch) {
        v4f vx[kBatch], vg[kBatch];
        bool ok[kBatch];
        uint32_t valid[kBatch], skip[kBatch];
#pragma unroll
        for (int k = 0; k < kBatch; k++) {
            const uint32_t q = q0 + k;
            ok[k] = q < last;
            valid[k] = 0; skip[k] = 0;
            if (ok[k]) {
                const uint32_t u = q * kBlock + threadIdx.x;
                if (u < pl.total_units) {
                    const uint32_t o = (__umulhi(u, pl.run_div.mul) + u) >> pl.run_div.shift;
                    const uint32_t off = (u - o * pl.units_per_run) * W;
                    const uint64_t at = (static_cast<uint64_t>(o) * pl.g.channels + c) * pl.g.inner + off;
                    if (VEC) {
                        valid[k] = 4;
                        vx[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x + at));
                        if (BACKWARD) vg[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(go + at));
                    } else {
                        // the last unit of a run is read as the run's last four floats; the ones a
                        // neighbouring unit already counted are skipped
                        const uint32_t back = off + 4 > pl.g.inner ? off + 4 - pl.g.inner : 0u;
                        valid[k] = 4; skip[k] = back;
                        const v4f_unaligned tx = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(x + at - back));
                        vx[k] = v4f{tx.x, tx.y, tx.z, tx.w};
                        if (BACKWARD) {
                            const v4f_unaligned tg = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(go + at - back));
                            vg[k] = v4f{tg.x, tg.y, tg.z, tg.w};
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kBatch; k++) {
            if (valid[k] == 0) continue;
#pragma unroll
            for (int e = 0; e < static_cast<int>(W); e++) {
                if (static_cast<uint32_t>(e) < skip[k]) continue;
                const double d = static_cast<double>(vx[k][e]) - shift;
                if (BACKWARD) { const double g = static_cast<double>(vg[k][e]); s1 += g; s2 += d * g; }
                else { s1 += d; s2 += d * d; }
            }
        }
    }
    block_fold2(s1, s2, lds);
    if (threadIdx.x == 0) {
        partial[(static_cast<uint64_t>(c) * pl.segments + seg) * 2] = s1;
        partial[(static_cast<uint64_t>(c) * pl.segments + seg) * 2 + 1] = s2;
    }
}

// ---------------------------------------------------------------- stats, short runs (inner < 64)

// The tensor as a matrix [outer, width = channels * inner]: a thread owns W adjacent columns
// (4 with float4 loads when width % 4 == 0, else 1), the 4 waves of a workgroup take rows
// r = first + wave, first + wave + 4, ...; a wave's loads are 1 KiB (256 B) of one row.
// Partials are per (segment, column).
struct ColPlan {
    Geometry g;
    uint32_t width, col_blocks, segments, rows_per_seg;
    FastDiv  col_div, inner_div;
    // a matrix narrower than a wave's 64 column groups: `groups` threads side by side and kBlock / groups rows at a
    // time, so that a wave still reads consecutive memory (16 columns of a million rows kept 4 lanes of 64 busy)
    uint32_t groups, row_lanes;
    FastDiv  groups_div;
};

template <bool BACKWARD, int W>
__global__ __launch_bounds__(kBlock) void bn_stats_cols_kernel(const float* __restrict__ x, const float* __restrict__ go,
                                                              const float* __restrict__ mean, double* __restrict__ partial, ColPlan pl) {
    __shared__ double lds[kBlock * 2 * W];
    const uint32_t b = blockIdx.x;
    const uint32_t seg = (__umulhi(b, pl.col_div.mul) + b) >> pl.col_div.shift;
    const uint32_t lane_row = (__umulhi(threadIdx.x, pl.groups_div.mul) + threadIdx.x) >> pl.groups_div.shift;
    const uint32_t group = threadIdx.x - lane_row * pl.groups;
    const uint32_t col = lane_row < pl.row_lanes ? ((b - seg * pl.col_blocks) * pl.groups + group) * W : pl.width;   // first of this thread's W columns
    double s1[W], s2[W];
#pragma unroll
    for (int e = 0; e < W; e++) { s1[e] = 0.0; s2[e] = 0.0; }
    if (col < pl.width) {
        double shift[W];
#pragma unroll
        for (int e = 0; e < W; e++) {
            const uint32_t ce = col + e;
            const uint32_t ch = (__umulhi(ce, pl.inner_div.mul) + ce) >> pl.inner_div.shift;
            shift[e] = BACKWARD ? static_cast<double>(mean[ch]) : static_cast<double>(x[static_cast<uint64_t>(ch) * pl.g.inner]);
        }
        const uint32_t first = seg * pl.rows_per_seg;
        uint32_t last = first + pl.rows_per_seg;
        if (last > pl.g.outer) last = pl.g.outer;
        for (uint32_t r0 = first + lane_row; r0 < last; r0 += pl.row_lanes * kBatch) {
            v4f vx[kBatch], vg[kBatch];
#pragma unroll
            for (int k = 0; k < kBatch; k++) {
                const uint32_t r = r0 + pl.row_lanes * k;
                if (r < last) {
                    const uint64_t at = static_cast<uint64_t>(r) * pl.width + col;
                    if (W == 4) {
                        vx[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x + at));
                        if (BACKWARD) vg[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(go + at));
                    } else {
                        vx[k].x = x[at];
                        if (BACKWARD) vg[k].x = go[at];
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < kBatch; k++) {
                if (r0 + pl.row_lanes * k < last) {
#pragma unroll
                    for (int e = 0; e < W; e++) {
                        const double d = static_cast<double>(vx[k][e]) - shift[e];
                        if (BACKWARD) { const double g = static_cast<double>(vg[k][e]); s1[e] += g; s2[e] += d * g; }
                        else { s1[e] += d; s2[e] += d * d; }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < W; e++) {
        lds[(threadIdx.x * W + e) * 2] = s1[e];
        lds[(threadIdx.x * W + e) * 2 + 1] = s2[e];
    }
    __syncthreads();
    // the threads of one column group, row_lanes of them groups apart, fold pairwise: lane l takes lane l + step
    uint32_t width = 1;
    while (width < pl.row_lanes) width <<= 1;
    for (uint32_t step = width >> 1; step >= 1; step >>= 1) {
        if (lane_row < step && lane_row + step < pl.row_lanes) {
            const uint32_t other = threadIdx.x + pl.groups * step;
#pragma unroll
            for (int e = 0; e < W * 2; e++) lds[threadIdx.x * W * 2 + e] += lds[other * W * 2 + e];
        }
        __syncthreads();
    }
    if (lane_row == 0 && col < pl.width) {
#pragma unroll
        for (int e = 0; e < W; e++) {
            partial[(static_cast<uint64_t>(seg) * pl.width + col + e) * 2] = lds[(threadIdx.x * W + e) * 2];
            partial[(static_cast<uint64_t>(seg) * pl.width + col + e) * 2 + 1] = lds[(threadIdx.x * W + e) * 2 + 1];
        }
    }
}

// ---------------------------------------------------------------- finalize

// The sums of one channel straight from the tensor, by one thread: for very many channels of a few items each
// (per_channel <= 32), where partial sums would be as many as the items themselves ([4194304,4] over axis 0 wrote and
// re-read 268 MB of them for 67 MB of input). Neighbouring threads read neighbouring channels. Forward: s1 = sum(x - k),
// s2 = sum((x - k)^2) with k the channel's first item; backward: s1 = sum(g), s2 = sum((x - mean) g).
__device__ __forceinline__ void fold_items(const float* __restrict__ x, const float* __restrict__ go, const Geometry& g, uint32_t c,
                                           bool backward, double shift, double& s1, double& s2) {
    s1 = 0.0; s2 = 0.0;
    constexpr uint32_t kAhead = 8;
    for (uint32_t t0 = 0; t0 < g.per_channel; t0 += kAhead) {
        float vx[kAhead], vg[kAhead];
#pragma unroll
        for (uint32_t k = 0; k < kAhead; k++) {
            const uint32_t t = t0 + k;
            if (t < g.per_channel) {
                const uint32_t o = t / g.inner, i = t - o * g.inner;
                const uint64_t at = (static_cast<uint64_t>(o) * g.channels + c) * g.inner + i;
                vx[k] = x[at];
                if (backward) vg[k] = go[at];
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < kAhead; k++) {
            if (t0 + k < g.per_channel) {
                const double d = static_cast<double>(vx[k]) - shift;
                if (backward) { const double gr = static_cast<double>(vg[k]); s1 += gr; s2 += d * gr; }
                else { s1 += d; s2 += d * d; }
            }
        }
    }
}


// Per-channel parameters for the apply kernels.
struct ForwardParams { float mean, stdev, gamma, beta; };
struct BackwardParams { float mean, stdev, gamma, dot_std_sq, grad_mean, pad0, pad1, pad2; };

// One wave folds the partials of channel c, always in the same order: lane l takes the items
// l, l + 64, ... (item t of a by-columns layout is segment t / inner, column c * inner + t % inner),
// then the lanes are folded by xor-shuffles. Every lane returns the totals.
// With very many channels of a few items each a wave per channel is 63 idle lanes: `alone` has one thread fold
// all items of its channel in ascending order instead.
__device__ __forceinline__ void fold_partials(const double* partial, uint32_t c, uint32_t segments, bool by_cols,
                                              uint32_t width, uint32_t inner, bool alone, double& s1, double& s2) {
    s1 = 0.0; s2 = 0.0;
    const uint32_t lane = alone ? 0u : threadIdx.x & 63;
    const uint32_t lanes = alone ? 1u : 64u;
    // eight items are requested before the first is added (the adds stay in ascending order of t): a wave that waits
    // for every item in turn spent 18 us on the 2048 segments of a [1048576,16] matrix
    constexpr uint32_t kAhead = 8;
    typedef double pair_t __attribute__((ext_vector_type(2)));
    const pair_t* pairs = reinterpret_cast<const pair_t*>(partial);
    const uint32_t items = by_cols ? segments * inner : segments;
    for (uint32_t t0 = lane; t0 < items; t0 += lanes * kAhead) {
        pair_t v[kAhead];
#pragma unroll
        for (uint32_t k = 0; k < kAhead; k++) {
            const uint32_t t = t0 + k * lanes;
            if (t < items) {
                uint64_t at;
                if (by_cols) {
                    const uint32_t seg = t / inner, i = t - seg * inner;
                    at = static_cast<uint64_t>(seg) * width + static_cast<uint64_t>(c) * inner + i;
                } else {
                    at = static_cast<uint64_t>(c) * segments + t;
                }
                v[k] = pairs[at];
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < kAhead; k++)
            if (t0 + k * lanes < items) { s1 += v[k].x; s2 += v[k].y; }
    }
    if (alone) return;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        s1 += __shfl_xor(s1, off);
        s2 += __shfl_xor(s2, off);
    }
}

// What the per-channel arithmetic of the forward pass needs beside the sums.
struct ForwardChannelArgs {
    Geometry g;
    int training;
    float momentum, epsilon;
    float* running_mean;
    float* running_var;
    const float* gamma;
    const float* beta;
    float* current_mean;
    float* current_std;
};

// The scalar float arithmetic of JVMBatchNorm.kt:57-85 for channel c from its two f64 sums, in the reference's order.
// `publish`: also write the channel's outputs (current mean / std, the running statistics, which are read and
// rewritten, so exactly one caller per channel may publish).
__device__ __forceinline__ ForwardParams forward_channel(const float* __restrict__ x, uint32_t c, double s1, double s2,
                                                         const ForwardChannelArgs& a, bool publish) {
    float mean, stdev = 0.0f;
    if (a.training) {
        const double n = static_cast<double>(a.g.per_channel);
        const double k = static_cast<double>(x[static_cast<uint64_t>(c) * a.g.inner]);
        mean = static_cast<float>(k + s1 / n);                                  // JVMBatchNorm.kt:57-58
        const double dm = static_cast<double>(mean) - k;
        double ssd = s2 - 2.0 * dm * s1 + n * dm * dm;
        if (ssd < 0.0) ssd = 0.0;
        const float sum = static_cast<float>(ssd);                              // :60-64
        const float count = static_cast<float>(a.g.per_channel);
        if (sum != 0.0f || a.epsilon != 0.0f) stdev = 1.0f / sqrtf(sum / count + a.epsilon);   // :66-68
        if (publish) {
            a.current_mean[c] = mean;
            a.current_std[c] = stdev;
            if (a.running_mean != nullptr && a.running_var != nullptr) {        // :72-76
                a.running_mean[c] = (a.momentum * mean) + ((1.0f - a.momentum) * a.running_mean[c]);
                const float unbiased = sum / static_cast<float>(a.g.per_channel - 1);
                a.running_var[c] = (a.momentum * unbiased) + ((1.0f - a.momentum) * a.running_var[c]);
            }
        }
    } else {                                                                    // :78-81
        mean = a.running_mean[c];
        stdev = 1.0f / sqrtf(a.running_var[c] + a.epsilon);
        if (publish) {
            a.current_mean[c] = 0.0f;
            a.current_std[c] = 0.0f;
        }
    }
    ForwardParams p;
    p.mean = mean; p.stdev = stdev;
    p.gamma = a.gamma != nullptr ? a.gamma[c] : 1.0f;                           // :84-85
    p.beta = a.beta != nullptr ? a.beta[c] : 0.0f;
    return p;
}

__global__ __launch_bounds__(kBlock) void bn_finalize_forward_kernel(const float* __restrict__ x, const double* __restrict__ partial,
                                                                    ForwardChannelArgs a, uint32_t segments, int by_cols,
                                                                    ForwardParams* __restrict__ params, float* __restrict__ soa, uint32_t pitch,
                                                                    int alone) {
    // one wave per channel, or one thread (alone = 1: over the partials; 2: over the channel's items themselves)
    const Geometry& g = a.g;
    const uint32_t c = alone ? blockIdx.x * kBlock + threadIdx.x : blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (c >= g.channels) return;
    double s1 = 0.0, s2 = 0.0;
    if (a.training && alone == 2) fold_items(x, nullptr, g, c, false, static_cast<double>(x[static_cast<uint64_t>(c) * g.inner]), s1, s2);
    else if (a.training) fold_partials(partial, c, segments, by_cols != 0, g.channels * g.inner, g.inner, alone != 0, s1, s2);
    if (!alone && (threadIdx.x & 63) != 0) return;
    const ForwardParams p = forward_channel(x, c, s1, s2, a, true);
    params[c] = p;
    // the same by parameter, for layouts where neighbouring elements belong to neighbouring channels
    soa[c] = p.mean; soa[pitch + c] = p.stdev; soa[2 * pitch + c] = p.gamma; soa[3 * pitch + c] = p.beta;
}

struct BackwardChannelArgs {
    Geometry g;
    int have_sums, training;
    float epsilon;
    const float* running_mean;
    const float* running_var;
    const float* current_mean;
    const float* current_std;
    const float* gamma;
    float* grad_gamma;
    float* grad_beta;
};

// Mean and 1 / std of channel c as the backward pass takes them (JVMBatchNorm.kt:131-137).
__device__ __forceinline__ void backward_channel_stats(uint32_t c, const BackwardChannelArgs& a, float& mean, float& stdev) {
    if (a.training) { mean = a.current_mean[c]; stdev = a.current_std[c]; }
    else {
        mean = a.running_mean[c];
        stdev = static_cast<float>(1.0 / sqrt(static_cast<double>(a.running_var[c] + a.epsilon)));
    }
}

// The scalar float arithmetic of JVMBatchNorm.kt:139-152,171-177 for channel c; `publish`: also write gradGamma / gradBeta.
__device__ __forceinline__ BackwardParams backward_channel(uint32_t c, float mean, float stdev, double s1, double s2,
                                                           const BackwardChannelArgs& a, bool publish) {
    float sum = 0.0f, dot = 0.0f;
    if (a.have_sums) {
        sum = static_cast<float>(s1);                                           // :139-147
        dot = static_cast<float>(s2);
    }
    const float count = static_cast<float>(a.g.per_channel);
    BackwardParams p;
    p.mean = mean; p.stdev = stdev;
    p.gamma = a.gamma != nullptr ? a.gamma[c] : 1.0f;
    p.dot_std_sq = dot * stdev * stdev / count;                                 // :151
    p.grad_mean = sum / count;                                                  // :152
    p.pad0 = p.pad1 = p.pad2 = 0.0f;
    if (publish) {
        if (a.grad_gamma != nullptr) a.grad_gamma[c] = dot * stdev;             // :171-173
        if (a.grad_beta != nullptr) a.grad_beta[c] = sum;                       // :175-177
    }
    return p;
}

__global__ __launch_bounds__(kBlock) void bn_finalize_backward_kernel(const float* __restrict__ x, const float* __restrict__ go,
                                                                     const double* __restrict__ partial, BackwardChannelArgs a,
                                                                     uint32_t segments, int by_cols, BackwardParams* __restrict__ params,
                                                                     float* __restrict__ soa, uint32_t pitch, int alone) {
    const Geometry& g = a.g;
    const uint32_t c = alone ? blockIdx.x * kBlock + threadIdx.x : blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (c >= g.channels) return;
    double s1 = 0.0, s2 = 0.0;
    float mean, stdev;
    backward_channel_stats(c, a, mean, stdev);
    if (a.have_sums && alone == 2) fold_items(x, go, g, c, true, static_cast<double>(mean), s1, s2);
    else if (a.have_sums) fold_partials(partial, c, segments, by_cols != 0, g.channels * g.inner, g.inner, alone != 0, s1, s2);
    if (!alone && (threadIdx.x & 63) != 0) return;
    const BackwardParams p = backward_channel(c, mean, stdev, s1, s2, a, true);
    params[c] = p;
    soa[c] = p.mean; soa[pitch + c] = p.stdev; soa[2 * pitch + c] = p.gamma; soa[3 * pitch + c] = p.dot_std_sq; soa[4 * pitch + c] = p.grad_mean;
}

// ---------------------------------------------------------------- apply

struct ApplyPlan {
    uint32_t units;                 // float4s (VEC) or floats
    uint32_t channels;
    const float* soa;               // parameters by kind, [kind][pitch]; used when by_channel4
    uint32_t pitch;
    uint32_t by_channel4;           // inner == 1 and channels % 4 == 0: a float4 holds four consecutive channels
    FastDiv  inner_div, channel_div;   // inner counted in the kernel's units
};

__device__ __forceinline__ uint32_t channel_of(const ApplyPlan& pl, uint32_t i) {
    const uint32_t q = (__umulhi(i, pl.inner_div.mul) + i) >> pl.inner_div.shift;
    const uint32_t r = (__umulhi(q, pl.channel_div.mul) + q) >> pl.channel_div.shift;
    return q - r * pl.channels;
}

__device__ __forceinline__ float bn_forward(float x, const ForwardParams& p) {
    return (x - p.mean) * p.stdev * p.gamma + p.beta;                           // JVMBatchNorm.kt:88-90
}
__device__ __forceinline__ float bn_backward_training(float x, float go, const BackwardParams& p) {
    const float base = (x - p.mean) * p.dot_std_sq;                             // :154-156
    return (go - p.grad_mean - base) * p.stdev * p.gamma;
}
__device__ __forceinline__ float bn_backward_inference(float go, const BackwardParams& p) {
    return go * p.stdev * p.gamma;                                              // :160-162
}

// MODE 0: forward. MODE 1: input gradient, training. MODE 2: input gradient, inference.
// VEC: one float4 per unit. UNIFORM: inner % 4 == 0, so the four lanes of a float4 share a
// channel (pl.inner_div counts float4s); otherwise each lane finds its own channel
// (pl.inner_div counts floats).
template <int MODE, bool VEC, bool UNIFORM>
__global__ __launch_bounds__(kBlock) void bn_apply_kernel(const float* __restrict__ x, const float* __restrict__ go, float* __restrict__ out,
                                                         const ForwardParams* __restrict__ fparams,
                                                         const BackwardParams* __restrict__ bparams, ApplyPlan pl) {
    const uint32_t base = blockIdx.x * (kBlock * kApplyUnroll) + threadIdx.x;
    if (VEC) {
        v4f vx[kApplyUnroll], vg[kApplyUnroll];
#pragma unroll
        for (int k = 0; k < kApplyUnroll; k++) {
            const uint32_t i = base + k * kBlock;
            if (i < pl.units) {
                if (MODE != 2) vx[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x) + i);
                if (MODE != 0) vg[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(go) + i);
            }
        }
#pragma unroll
        for (int k = 0; k < kApplyUnroll; k++) {
            const uint32_t i = base + k * kBlock;
            if (i < pl.units) {
                v4f r;
                if (!UNIFORM && pl.by_channel4) {
                    // four consecutive channels: one float4 per parameter kind instead of four structs,
                    // whose lane stride would sweep 32 or 64 cache lines per load
                    const uint32_t c0 = channel_of(pl, i * 4);
                    const v4f mean = *reinterpret_cast<const v4f*>(pl.soa + c0);
                    const v4f stdev = *reinterpret_cast<const v4f*>(pl.soa + pl.pitch + c0);
                    const v4f gamma = *reinterpret_cast<const v4f*>(pl.soa + 2 * pl.pitch + c0);
                    const v4f p3 = *reinterpret_cast<const v4f*>(pl.soa + 3 * pl.pitch + c0);      // beta | dot_std_sq
                    v4f p4 = p3;
                    if (MODE == 1) p4 = *reinterpret_cast<const v4f*>(pl.soa + 4 * pl.pitch + c0);  // grad_mean
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (MODE == 0) { ForwardParams q; q.mean = mean[e]; q.stdev = stdev[e]; q.gamma = gamma[e]; q.beta = p3[e]; r[e] = bn_forward(vx[k][e], q); }
                        else {
                            BackwardParams q; q.mean = mean[e]; q.stdev = stdev[e]; q.gamma = gamma[e]; q.dot_std_sq = p3[e]; q.grad_mean = p4[e];
                            r[e] = MODE == 1 ? bn_backward_training(vx[k][e], vg[k][e], q) : bn_backward_inference(vg[k][e], q);
                        }
                    }
                    reinterpret_cast<v4f*>(out)[i] = r;
                    continue;
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t c = UNIFORM ? channel_of(pl, i) : channel_of(pl, i * 4 + e);
                    if (MODE == 0) r[e] = bn_forward(vx[k][e], fparams[c]);
                    else if (MODE == 1) r[e] = bn_backward_training(vx[k][e], vg[k][e], bparams[c]);
                    else r[e] = bn_backward_inference(vg[k][e], bparams[c]);
                }
                reinterpret_cast<v4f*>(out)[i] = r;
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < kApplyUnroll; k++) {
            const uint32_t i = base + k * kBlock;
            if (i < pl.units) {
                const uint32_t c = channel_of(pl, i);
                if (MODE == 0) out[i] = bn_forward(x[i], fparams[c]);
                else if (MODE == 1) out[i] = bn_backward_training(x[i], go[i], bparams[c]);
                else out[i] = bn_backward_inference(go[i], bparams[c]);
            }
        }
    }
}

// The apply kernel that does the finalize step itself, for tensors whose runs are long (inner % 4 == 0, a tile of a
// workgroup inside at most kFoldChannels runs): wave w folds the partials of the w-th run the tile touches, in the
// order the finalize kernel folds them, and lane 0 does the channel's scalar arithmetic: the same functions on the same
// sums, hence the same parameters in every workgroup and the same bits as the two-launch form. The workgroup whose
// tile holds the first float of a channel's first run publishes that channel's outputs. The tile's loads are issued
// before the fold, whose few hundred bytes come from L2.
constexpr uint32_t kFoldChannels = kBlock / 64;

template <int MODE>
__global__ __launch_bounds__(kBlock) void bn_apply_folded_kernel(const float* __restrict__ x, const float* __restrict__ go, float* __restrict__ out,
                                                                const double* __restrict__ partial, uint32_t segments,
                                                                ForwardChannelArgs fa, BackwardChannelArgs ba, ApplyPlan pl) {
    __shared__ ForwardParams fpar[kFoldChannels];
    __shared__ BackwardParams bpar[kFoldChannels];
    constexpr uint32_t per_block = kBlock * kApplyUnroll;
    const uint32_t u0 = blockIdx.x * per_block;
    const uint32_t u1 = u0 + per_block < pl.units ? u0 + per_block : pl.units;
    const uint32_t base = u0 + threadIdx.x;
    v4f vx[kApplyUnroll], vg[kApplyUnroll];
#pragma unroll
    for (int k = 0; k < kApplyUnroll; k++) {
        const uint32_t i = base + k * kBlock;
        if (i < pl.units) {
            if (MODE != 2) vx[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(x) + i);
            if (MODE != 0) vg[k] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(go) + i);
        }
    }
    // runs are numbered through the tensor: run q is channel q % channels of outer index q / channels
    const uint32_t q0 = (__umulhi(u0, pl.inner_div.mul) + u0) >> pl.inner_div.shift;
    const uint32_t q1 = (__umulhi(u1 - 1, pl.inner_div.mul) + (u1 - 1)) >> pl.inner_div.shift;
    const uint32_t q = q0 + (threadIdx.x >> 6);
    if (q <= q1) {
        const uint32_t o = (__umulhi(q, pl.channel_div.mul) + q) >> pl.channel_div.shift;
        const uint32_t c = q - o * pl.channels;
        const Geometry& g = MODE == 0 ? fa.g : ba.g;
        // the run of outer index 0 starts the channel; its first unit lies in this tile unless the tile begins inside the run
        const bool publish = o == 0 && (q > q0 || q * (g.inner / 4) == u0);
        double s1 = 0.0, s2 = 0.0;
        if (MODE == 0) {
            if (fa.training) fold_partials(partial, c, segments, false, 0, 0, false, s1, s2);
            if ((threadIdx.x & 63) == 0) fpar[q - q0] = forward_channel(x, c, s1, s2, fa, publish);
        } else {
            float mean, stdev;
            backward_channel_stats(c, ba, mean, stdev);
            if (ba.have_sums) fold_partials(partial, c, segments, false, 0, 0, false, s1, s2);
            if ((threadIdx.x & 63) == 0) bpar[q - q0] = backward_channel(c, mean, stdev, s1, s2, ba, publish);
        }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kApplyUnroll; k++) {
        const uint32_t i = base + k * kBlock;
        if (i < pl.units) {
            const uint32_t at = ((__umulhi(i, pl.inner_div.mul) + i) >> pl.inner_div.shift) - q0;
            v4f r;
            if (MODE == 0) {
                const ForwardParams p = fpar[at];
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = bn_forward(vx[k][e], p);
            } else {
                const BackwardParams p = bpar[at];
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = MODE == 1 ? bn_backward_training(vx[k][e], vg[k][e], p) : bn_backward_inference(vg[k][e], p);
            }
            reinterpret_cast<v4f*>(out)[i] = r;
        }
    }
}

// ---------------------------------------------------------------- host side

int geometry_of(const char* what, const int32_t* shape, int dims, int axis, Geometry* g, uint64_t* n) {
    if (dims < 1 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "%s: %d dims", what, dims);
    if (!shape) return fail(KTH_E_ARGUMENT, "%s: null shape", what);
    if (axis < 0 || axis >= dims) return fail(KTH_E_ARGUMENT, "%s: axis %d of %d dims", what, axis, dims);
    uint64_t outer = 1, inner = 1;
    for (int d = 0; d < dims; d++) {
        if (shape[d] < 1) return fail(KTH_E_ARGUMENT, "%s: dim %d is %d", what, d, shape[d]);
        if (d < axis) outer *= static_cast<uint64_t>(shape[d]);
        if (d > axis) inner *= static_cast<uint64_t>(shape[d]);
        if (outer * inner * static_cast<uint64_t>(shape[axis]) > kMaxElements) return fail(KTH_E_ARGUMENT, "%s: more than 2^31-1 elements", what);
    }
    g->outer = static_cast<uint32_t>(outer);
    g->channels = static_cast<uint32_t>(shape[axis]);
    g->inner = static_cast<uint32_t>(inner);
    g->per_channel = static_cast<uint32_t>(outer * inner);
    *n = outer * inner * g->channels;
    return KTH_OK;
}

// A per-channel operand: 0 means "not given"; otherwise it must hold `channels` floats.
int channel_store(const char* what, uint64_t handle, uint32_t channels, float** ptr) {
    *ptr = nullptr;
    if (handle == 0) return KTH_OK;
    Store* s = lookup(handle, what);
    if (!s) return KTH_E_HANDLE;
    if (s->n_floats < channels) return fail(KTH_E_SHAPE, "%s holds %llu values, the axis has %u", what,
                                             static_cast<unsigned long long>(s->n_floats), channels);
    *ptr = s->ptr;
    return KTH_OK;
}

struct StatsLaunch {
    bool     by_cols;
    uint32_t segments;
    uint64_t partial_doubles;
    RunPlan  run;
    ColPlan  col;
    bool     vec;
};

// Very many channels of a few items each: no statistics launch, a thread per channel sums its items in the finalize.
static bool stats_direct(const Geometry& g) { return g.channels >= 16384 && g.per_channel <= 32; }

// A thread per channel folds the partials when there are very many channels of a few items each.
static bool finalize_alone(const Geometry& g, const StatsLaunch& st) {
    const uint64_t items = st.by_cols ? static_cast<uint64_t>(st.segments) * g.inner : st.segments;
    return g.channels >= 16384 && items <= 32;
}

StatsLaunch plan_stats(const Geometry& g) {
    StatsLaunch st{};
    const uint32_t target = static_cast<uint32_t>(state().compute_units > 0 ? state().compute_units : 256) * 8;
    if (g.inner >= 64) {
        st.by_cols = false;
        st.vec = g.inner % 4 == 0;
        RunPlan& p = st.run;
        p.g = g;
        p.units_per_run = (g.inner + 3) / 4;
        p.total_units = g.outer * p.units_per_run;
        p.total_chunks = (p.total_units + kBlock - 1) / kBlock;
        uint32_t segments = (target + g.channels - 1) / g.channels;
        const uint32_t max_segments = (p.total_chunks + kBatch - 1) / kBatch;      // at least one batch of chunks each
        if (segments > max_segments) segments = max_segments;
        if (segments < 1) segments = 1;
        p.chunks_per_seg = (p.total_chunks + segments - 1) / segments;
        p.segments = (p.total_chunks + p.chunks_per_seg - 1) / p.chunks_per_seg;
        p.run_div = make_div(p.units_per_run);
        p.seg_div = make_div(p.segments);
        st.segments = p.segments;
        st.partial_doubles = static_cast<uint64_t>(g.channels) * p.segments * 2;
    } else {
        st.by_cols = true;
        ColPlan& p = st.col;
        p.g = g;
        p.width = g.channels * g.inner;
        st.vec = p.width % 4 == 0;                     // every row then starts 16-byte aligned
        const uint32_t w = st.vec ? 4 : 1;
        p.groups = std::min<uint32_t>(64, (p.width + w - 1) / w);
        p.row_lanes = kBlock / p.groups;
        p.groups_div = make_div(p.groups);
        const uint32_t cols_per_block = p.groups * w;
        p.col_blocks = (p.width + cols_per_block - 1) / cols_per_block;
        uint32_t segments = (target + p.col_blocks - 1) / p.col_blocks;
        const uint32_t max_segments = (g.outer + p.row_lanes * kBatch - 1) / (p.row_lanes * kBatch);
        if (segments > max_segments) segments = max_segments;
        if (segments < 1) segments = 1;
        p.rows_per_seg = (g.outer + segments - 1) / segments;
        p.segments = (g.outer + p.rows_per_seg - 1) / p.rows_per_seg;
        p.col_div = make_div(p.col_blocks);
        p.inner_div = make_div(g.inner);
        st.segments = p.segments;
        st.partial_doubles = static_cast<uint64_t>(p.segments) * p.width * 2;
    }
    return st;
}

template <bool BACKWARD>
void launch_stats(const StatsLaunch& st, const float* x, const float* go, const float* mean, double* partial, uint64_t n) {
    hipStream_t stream = state().stream;
    const uint64_t bytes = (BACKWARD ? 2 : 1) * n * 4;
    if (st.by_cols) {
        LaunchScope scope("bn_stats_cols_kernel", BACKWARD ? "backward" : "forward", bytes);
        const dim3 grid(st.col.col_blocks * st.col.segments);
        if (st.vec) hipLaunchKernelGGL((bn_stats_cols_kernel<BACKWARD, 4>), grid, dim3(kBlock), 0, stream, x, go, mean, partial, st.col);
        else        hipLaunchKernelGGL((bn_stats_cols_kernel<BACKWARD, 1>), grid, dim3(kBlock), 0, stream, x, go, mean, partial, st.col);
    } else {
        LaunchScope scope("bn_stats_runs_kernel", BACKWARD ? "backward" : "forward", bytes);
        const dim3 grid(st.run.g.channels * st.run.segments);
        if (st.vec) hipLaunchKernelGGL((bn_stats_runs_kernel<BACKWARD, true>), grid, dim3(kBlock), 0, stream, x, go, mean, partial, st.run);
        else        hipLaunchKernelGGL((bn_stats_runs_kernel<BACKWARD, false>), grid, dim3(kBlock), 0, stream, x, go, mean, partial, st.run);
    }
}

template <int MODE>
void launch_apply(const Geometry& g, uint64_t n, const float* x, const float* go, float* out, const ForwardParams* fp, const BackwardParams* bp,
                  const float* soa, uint32_t pitch) {
    ApplyPlan pl{};
    const bool vec = n % 4 == 0, uniform = g.inner % 4 == 0;
    pl.soa = soa; pl.pitch = pitch;
    pl.by_channel4 = (g.inner == 1 && g.channels % 4 == 0) ? 1u : 0u;
    pl.units = static_cast<uint32_t>(vec ? n / 4 : n);
    pl.channels = g.channels;
    pl.inner_div = make_div(uniform ? g.inner / 4 : g.inner);
    pl.channel_div = make_div(g.channels);
    const uint32_t per_block = kBlock * kApplyUnroll;
    const dim3 grid((pl.units + per_block - 1) / per_block);
    const uint64_t bytes = (MODE == 0 ? 2 : MODE == 1 ? 3 : 2) * n * 4;
    LaunchScope scope("bn_apply_kernel", MODE == 0 ? "forward" : MODE == 1 ? "backward_training" : "backward_inference", bytes);
    if (uniform)  hipLaunchKernelGGL((bn_apply_kernel<MODE, true, true>), grid, dim3(kBlock), 0, state().stream, x, go, out, fp, bp, pl);
    else if (vec) hipLaunchKernelGGL((bn_apply_kernel<MODE, true, false>), grid, dim3(kBlock), 0, state().stream, x, go, out, fp, bp, pl);
    else          hipLaunchKernelGGL((bn_apply_kernel<MODE, false, false>), grid, dim3(kBlock), 0, state().stream, x, go, out, fp, bp, pl);
}

// The finalize step rides in the apply kernel when the tile of an apply workgroup lies inside at most kFoldChannels runs
// and a channel's partials are few enough to be folded by every workgroup that needs them.
static bool can_fold(const Geometry& g, const StatsLaunch& st, bool have_partials) {
    if (g.inner % 4 != 0 || 3 * (g.inner / 4) < static_cast<uint32_t>(kBlock * kApplyUnroll)) return false;
    if (have_partials && (st.by_cols || st.segments > 64 || finalize_alone(g, st))) return false;
    return true;
}

template <int MODE>
void launch_apply_folded(const Geometry& g, uint64_t n, const float* x, const float* go, float* out, const double* partial, uint32_t segments,
                         const ForwardChannelArgs& fa, const BackwardChannelArgs& ba) {
    ApplyPlan pl{};
    pl.units = static_cast<uint32_t>(n / 4);
    pl.channels = g.channels;
    pl.inner_div = make_div(g.inner / 4);
    pl.channel_div = make_div(g.channels);
    const uint32_t per_block = kBlock * kApplyUnroll;
    const dim3 grid((pl.units + per_block - 1) / per_block);
    const uint64_t bytes = (MODE == 0 ? 2 : MODE == 1 ? 3 : 2) * n * 4;
    LaunchScope scope("bn_apply_folded_kernel", MODE == 0 ? "forward" : MODE == 1 ? "backward_training" : "backward_inference", bytes);
    hipLaunchKernelGGL((bn_apply_folded_kernel<MODE>), grid, dim3(kBlock), 0, state().stream, x, go, out, partial, segments, fa, ba, pl);
}

uint64_t align256(uint64_t v) { return (v + 255) & ~255ull; }

}  // namespace

extern "C" {

int kth_batch_norm_forward(uint64_t in, const int32_t* shape, int dims, int axis, int training, float momentum, float epsilon,
                           uint64_t running_mean, uint64_t running_var, uint64_t gamma, uint64_t beta,
                           uint64_t out, uint64_t current_mean, uint64_t current_std) {
    std::lock_guard<std::mutex> guard(lock());
    KTH_REQUIRE_INIT();
    Geometry g; uint64_t n;
    if (int rc = geometry_of("kth_batch_norm_forward", shape, dims, axis, &g, &n)) return rc;
    if ((running_mean == 0) != (running_var == 0))
        return fail(KTH_E_ARGUMENT, "Running mean and running var must be both set or both absent");
    if (!training && running_mean == 0)
        return fail(KTH_E_ARGUMENT, "Running mean and running var must be given for inference mode");
    Store* si = lookup(in, "kth_batch_norm_forward(in)");
    if (!si) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_batch_norm_forward(out)");
    if (!so) return KTH_E_HANDLE;
    if (n > si->n_floats || n > so->n_floats) return fail(KTH_E_ARGUMENT, "kth_batch_norm_forward: the shape needs more elements than a store holds");
    float *rm, *rv, *ga, *be, *cm, *cs;
    if (int rc = channel_store("kth_batch_norm_forward(running_mean)", running_mean, g.channels, &rm)) return rc;
    if (int rc = channel_store("kth_batch_norm_forward(running_var)", running_var, g.channels, &rv)) return rc;
    if (int rc = channel_store("kth_batch_norm_forward(gamma)", gamma, g.channels, &ga)) return rc;
    if (int rc = channel_store("kth_batch_norm_forward(beta)", beta, g.channels, &be)) return rc;
    if (int rc = channel_store("kth_batch_norm_forward(current_mean)", current_mean, g.channels, &cm)) return rc;
    if (int rc = channel_store("kth_batch_norm_forward(current_std)", current_std, g.channels, &cs)) return rc;
    if (!cm || !cs) return fail(KTH_E_ARGUMENT, "kth_batch_norm_forward: current_mean and current_std are outputs and must be given");

    const bool direct = training && stats_direct(g);
    const StatsLaunch st = training && !direct ? plan_stats(g) : StatsLaunch{};
    const uint32_t pitch = (g.channels + 3u) & ~3u;
    const uint64_t aos_bytes = align256(static_cast<uint64_t>(g.channels) * sizeof(ForwardParams));
    const uint64_t params_bytes = aos_bytes + align256(4ull * pitch * sizeof(float));
    const uint64_t ws_bytes = params_bytes + st.partial_doubles * sizeof(double);
    uint64_t cap;
    char* ws = reinterpret_cast<char*>(workspace_acquire(ws_bytes, &cap));
    if (!ws) return fail(KTH_E_MEMORY, "kth_batch_norm_forward: no workspace of %llu bytes", static_cast<unsigned long long>(ws_bytes));
    ForwardParams* params = reinterpret_cast<ForwardParams*>(ws);
    float* soa = reinterpret_cast<float*>(ws + aos_bytes);
    double* partial = reinterpret_cast<double*>(ws + params_bytes);
    if (training && !direct) launch_stats<false>(st, si->ptr, nullptr, nullptr, partial, n);
    ForwardChannelArgs fa{};
    fa.g = g; fa.training = training ? 1 : 0; fa.momentum = momentum; fa.epsilon = epsilon;
    fa.running_mean = rm; fa.running_var = rv; fa.gamma = ga; fa.beta = be; fa.current_mean = cm; fa.current_std = cs;
    // (a result written over its own input keeps the two-launch form: the channel's shift is read from the input)
    if (!direct && so->ptr != si->ptr && can_fold(g, st, training != 0)) {
        launch_apply_folded<0>(g, n, si->ptr, nullptr, so->ptr, partial, st.segments, fa, BackwardChannelArgs{});
    } else {
        {
            LaunchScope scope("bn_finalize_forward_kernel", direct ? "from the items" : "", static_cast<uint64_t>(g.channels) * 32 + (direct ? n * 4 : 0));
            const int alone = direct ? 2 : finalize_alone(g, st) ? 1 : 0;
            const uint32_t per_block = alone ? kBlock : kBlock / 64;
            hipLaunchKernelGGL(bn_finalize_forward_kernel, dim3((g.channels + per_block - 1) / per_block), dim3(kBlock), 0, state().stream,
                               si->ptr, partial, fa, st.segments, st.by_cols ? 1 : 0, params, soa, pitch, alone);
        }
        launch_apply<0>(g, n, si->ptr, nullptr, so->ptr, params, nullptr, soa, pitch);
    }
    workspace_release(reinterpret_cast<float*>(ws), cap);
    KTH_LAUNCH_CHECK("batch_norm_forward");
    return KTH_OK;
}

int kth_batch_norm_backward(uint64_t in, const int32_t* shape, int dims, int axis, int training, float epsilon,
                            uint64_t running_mean, uint64_t running_var, uint64_t current_mean, uint64_t current_std,
                            uint64_t gamma, uint64_t grad_out, uint64_t grad_in, uint64_t grad_gamma, uint64_t grad_beta) {
    std::lock_guard<std::mutex> guard(lock());
    KTH_REQUIRE_INIT();
    Geometry g; uint64_t n;
    if (int rc = geometry_of("kth_batch_norm_backward", shape, dims, axis, &g, &n)) return rc;
    if (grad_in == 0 && grad_gamma == 0 && grad_beta == 0) return KTH_OK;         // JVMBatchNorm.kt:113-115
    Store* si = lookup(in, "kth_batch_norm_backward(in)");
    if (!si) return KTH_E_HANDLE;
    Store* sg = lookup(grad_out, "kth_batch_norm_backward(grad_out)");
    if (!sg) return KTH_E_HANDLE;
    Store* sgi = nullptr;
    if (grad_in != 0) { sgi = lookup(grad_in, "kth_batch_norm_backward(grad_in)"); if (!sgi) return KTH_E_HANDLE; }
    if (n > si->n_floats || n > sg->n_floats || (sgi && n > sgi->n_floats))
        return fail(KTH_E_ARGUMENT, "kth_batch_norm_backward: the shape needs more elements than a store holds");
    float *rm, *rv, *cm, *cs, *ga, *gg, *gb;
    if (int rc = channel_store("kth_batch_norm_backward(running_mean)", running_mean, g.channels, &rm)) return rc;
    if (int rc = channel_store("kth_batch_norm_backward(running_var)", running_var, g.channels, &rv)) return rc;
    if (int rc = channel_store("kth_batch_norm_backward(current_mean)", current_mean, g.channels, &cm)) return rc;
    if (int rc = channel_store("kth_batch_norm_backward(current_std)", current_std, g.channels, &cs)) return rc;
    if (int rc = channel_store("kth_batch_norm_backward(gamma)", gamma, g.channels, &ga)) return rc;
    if (int rc = channel_store("kth_batch_norm_backward(grad_gamma)", grad_gamma, g.channels, &gg)) return rc;
    if (int rc = channel_store("kth_batch_norm_backward(grad_beta)", grad_beta, g.channels, &gb)) return rc;
    if (training ? (!cm || !cs) : (!rm || !rv))
        return fail(KTH_E_ARGUMENT, "kth_batch_norm_backward: %s", training ? "current_mean and current_std are needed in training mode"
                                                                            : "running_mean and running_var are needed in inference mode");
    // The two sums feed gradGamma, gradBeta and the training-mode input gradient; the
    // inference-mode input gradient does not use them.
    const bool need_sums = training || gg != nullptr || gb != nullptr;
    const bool direct = need_sums && stats_direct(g);
    const StatsLaunch st = need_sums && !direct ? plan_stats(g) : StatsLaunch{};
    const uint32_t pitch = (g.channels + 3u) & ~3u;
    const uint64_t aos_bytes = align256(static_cast<uint64_t>(g.channels) * sizeof(BackwardParams));
    const uint64_t params_bytes = aos_bytes + align256(5ull * pitch * sizeof(float));
    const uint64_t ws_bytes = params_bytes + st.partial_doubles * sizeof(double);
    uint64_t cap;
    char* ws = reinterpret_cast<char*>(workspace_acquire(ws_bytes, &cap));
    if (!ws) return fail(KTH_E_MEMORY, "kth_batch_norm_backward: no workspace of %llu bytes", static_cast<unsigned long long>(ws_bytes));
    BackwardParams* params = reinterpret_cast<BackwardParams*>(ws);
    float* soa = reinterpret_cast<float*>(ws + aos_bytes);
    double* partial = reinterpret_cast<double*>(ws + params_bytes);
    if (need_sums && !direct) launch_stats<true>(st, si->ptr, sg->ptr, training ? cm : rm, partial, n);
    BackwardChannelArgs ba{};
    ba.g = g; ba.have_sums = need_sums ? 1 : 0; ba.training = training ? 1 : 0; ba.epsilon = epsilon;
    ba.running_mean = rm; ba.running_var = rv; ba.current_mean = cm; ba.current_std = cs; ba.gamma = ga; ba.grad_gamma = gg; ba.grad_beta = gb;
    if (sgi && !direct && can_fold(g, st, need_sums)) {
        if (training) launch_apply_folded<1>(g, n, si->ptr, sg->ptr, sgi->ptr, partial, st.segments, ForwardChannelArgs{}, ba);
        else launch_apply_folded<2>(g, n, nullptr, sg->ptr, sgi->ptr, partial, st.segments, ForwardChannelArgs{}, ba);
    } else {
        {
            LaunchScope scope("bn_finalize_backward_kernel", direct ? "from the items" : "", static_cast<uint64_t>(g.channels) * 32 + (direct ? n * 8 : 0));
            const int alone = direct ? 2 : finalize_alone(g, st) ? 1 : 0;
            const uint32_t per_block = alone ? kBlock : kBlock / 64;
            hipLaunchKernelGGL(bn_finalize_backward_kernel, dim3((g.channels + per_block - 1) / per_block), dim3(kBlock), 0, state().stream,
                               si->ptr, sg ? sg->ptr : nullptr, partial, ba, st.segments, st.by_cols ? 1 : 0, params, soa, pitch, alone);
        }
        if (sgi) {
            if (training) launch_apply<1>(g, n, si->ptr, sg->ptr, sgi->ptr, nullptr, params, soa, pitch);
            else launch_apply<2>(g, n, nullptr, sg->ptr, sgi->ptr, nullptr, params, soa, pitch);
        }
    }
    workspace_release(reinterpret_cast<float*>(ws), cap);
    KTH_LAUNCH_CHECK("batch_norm_backward");
    return KTH_OK;
}

}  // extern "C"
