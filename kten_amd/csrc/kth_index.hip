// gather / inplaceScatter / inplaceScatterAdd / inplaceScatter(Float) along an axis
// (reference: JVMRawTensor.kt:227-255,317-353 with StoreIndexing.applyAt,
// AbstractIndexing.kt:123-146). Positions run over the index tensor's shape without the
// axis. Within a position duplicates resolve exactly as on the JVM ("last write wins", "added
// in order"), and different positions never touch the same target element. Short index rows:
// one thread owns one position and walks the axis in ascending order. Long index rows: a
// workgroup owns the position, keeps its target row in LDS and orders the entries of each
// chunk through LDS tags (axes other than the innermost are permuted there and back).
// indexAdd sorts its index list so that every target row is updated by threads of its own.
// Index values are floats: Kotlin's toInt() (truncate, NaN -> 0, saturate) is what
// v_cvt_i32_f32 does. An index outside [0, axis length) is skipped and reported: the host
// turns the report into the reference's IllegalArgumentException.
#include "kth_internal.h"

using namespace kth;

namespace {

constexpr int kBlock = 256;

// Dim 0 is the innermost of the position dims (index shape without the axis).
struct IndexPlan {
    int      ndim;
    uint32_t size[KTH_MAX_DIMS];
    FastDiv  div[KTH_MAX_DIMS];
    uint32_t i_stride[KTH_MAX_DIMS];   // index tensor (and, for gather, the result)
    uint32_t a_stride[KTH_MAX_DIMS];   // gather: input; scatter: target
    uint32_t b_stride[KTH_MAX_DIMS];   // scatter: source
    uint32_t i_axis_stride, a_axis_stride, b_axis_stride;
    uint32_t i_axis_len, a_axis_len;
};

__device__ __forceinline__ void locate(const IndexPlan& pl, uint32_t pos, uint32_t& io, uint32_t& ao, uint32_t& bo) {
    io = ao = bo = 0;
    for (int d = 0; d < pl.ndim; d++) {
        uint32_t q = (__umulhi(pos, pl.div[d].mul) + pos) >> pl.div[d].shift;
        uint32_t r = pos - q * pl.size[d];
        io += r * pl.i_stride[d]; ao += r * pl.a_stride[d]; bo += r * pl.b_stride[d];
        pos = q;
    }
}

// One thread per element of the index tensor (= per element of the result, which has
// the same contiguous layout): gather has no ordering constraint. The plan's dims are all
// dims of the index shape, the input stride of the axis dim is 0 and the selected
// position along the axis is added separately.
__global__ __launch_bounds__(kBlock) void gather_kernel(const float* __restrict__ in, const float* __restrict__ index,
                                                       float* __restrict__ out, uint32_t elements, IndexPlan pl, int* bad) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= elements) return;
    uint32_t io, ao, bo;
    locate(pl, e, io, ao, bo);
    const int sel = static_cast<int>(index[e]);
    if (sel < 0 || static_cast<uint32_t>(sel) >= pl.a_axis_len) { *bad = 1; return; }
    out[e] = in[ao + static_cast<uint32_t>(sel) * pl.a_axis_stride];
}

// A contiguous row between global memory and LDS, 16 bytes per lane (the global side may start at
// any dword address), the last 1 ... 3 floats one by one.
typedef float v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));
typedef float v4f_lds __attribute__((ext_vector_type(4)));
template <int THREADS>
__device__ __forceinline__ void row_to_lds(const float* __restrict__ row, float* tile, uint32_t len) {
    const uint32_t body = len & ~3u;
    for (uint32_t j = threadIdx.x * 4; j < body; j += THREADS * 4) {
        const v4f_unaligned v = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(row + j));
        *reinterpret_cast<v4f_lds*>(tile + j) = v4f_lds{v.x, v.y, v.z, v.w};
    }
    if (threadIdx.x < len - body) tile[body + threadIdx.x] = row[body + threadIdx.x];
}
template <int THREADS>
__device__ __forceinline__ void lds_to_row(const float* tile, float* __restrict__ row, uint32_t len) {
    const uint32_t body = len & ~3u;
    for (uint32_t j = threadIdx.x * 4; j < body; j += THREADS * 4) {
        const v4f_lds v = *reinterpret_cast<const v4f_lds*>(tile + j);
        *reinterpret_cast<v4f_unaligned*>(row + j) = v4f_unaligned{v.x, v.y, v.z, v.w};
    }
    if (threadIdx.x < len - body) row[body + threadIdx.x] = tile[body + threadIdx.x];
}

// gather along the innermost axis when the index rows are long: one workgroup per position reads
// the input row into LDS as one contiguous span and serves out[r] = row[index[r]] from there, so
// both the reads and the writes of global memory are contiguous. The plan is the scatter form:
// position dims without the axis, i_stride for the index, a_stride for the input, b_stride for
// the result (indexSelect along the innermost axis is the same with one index row for all: i_stride 0).
template <int THREADS>
__global__ __launch_bounds__(THREADS) void gather_rows_lds_kernel(const float* __restrict__ in, const float* __restrict__ index,
                                                                 float* __restrict__ out, IndexPlan pl, int* bad) {
    extern __shared__ __attribute__((aligned(16))) float gather_row[];
    const uint32_t tid = threadIdx.x;
    uint32_t io, ao, bo;
    locate(pl, blockIdx.x, io, ao, bo);
    const float* arow = in + ao;
    const float* irow = index + io;
    float* orow = out + bo;
    row_to_lds<THREADS>(arow, gather_row, pl.a_axis_len);
    __syncthreads();
    constexpr uint32_t kBatch = 4;
    for (uint32_t r0 = tid; r0 < pl.i_axis_len; r0 += kBatch * THREADS) {
        float fi[kBatch];
#pragma unroll
        for (uint32_t k = 0; k < kBatch; k++) if (r0 + k * THREADS < pl.i_axis_len) fi[k] = __builtin_nontemporal_load(irow + r0 + k * THREADS);
#pragma unroll
        for (uint32_t k = 0; k < kBatch; k++) {
            if (r0 + k * THREADS < pl.i_axis_len) {
                const int sel = static_cast<int>(fi[k]);
                if (sel < 0 || static_cast<uint32_t>(sel) >= pl.a_axis_len) { *bad = 1; continue; }
                orow[r0 + k * THREADS] = gather_row[sel];
            }
        }
    }
}

// MODE 0: assign from src, 1: add from src, 2: assign the constant.
template <int MODE>
__global__ __launch_bounds__(kBlock) void scatter_kernel(float* __restrict__ target, const float* __restrict__ index,
                                                        const float* __restrict__ src, float value, uint32_t positions,
                                                        IndexPlan pl, int* bad) {
    const uint32_t pos = blockIdx.x * kBlock + threadIdx.x;
    if (pos >= positions) return;
    uint32_t io, ao, bo;
    locate(pl, pos, io, ao, bo);
    // The index and source values of kScatterBatch steps are loaded before the first of their
    // stores, so the loads overlap; the stores stay in ascending order of i.
    constexpr uint32_t kScatterBatch = 8;
    for (uint32_t i0 = 0; i0 < pl.i_axis_len; i0 += kScatterBatch) {
        float fi[kScatterBatch], fv[kScatterBatch];
#pragma unroll
        for (uint32_t k = 0; k < kScatterBatch; k++) {
            if (i0 + k < pl.i_axis_len) {
                fi[k] = index[io + (i0 + k) * pl.i_axis_stride];
                if (MODE != 2) fv[k] = src[bo + (i0 + k) * pl.b_axis_stride];
            }
        }
        if (MODE == 1 && i0 + kScatterBatch <= pl.i_axis_len) {
            // a full batch of adds whose eight entries are valid and name eight different elements: the elements
            // are read together and written together. (A repeated element needs its adds one after the other,
            // through memory: the loop below.)
            uint32_t sel[kScatterBatch];
            bool apart = true;
#pragma unroll
            for (uint32_t k = 0; k < kScatterBatch; k++) {
                const int v = static_cast<int>(fi[k]);
                sel[k] = static_cast<uint32_t>(v);
                apart = apart && v >= 0 && sel[k] < pl.a_axis_len;
#pragma unroll
                for (uint32_t j = 0; j < k; j++) apart = apart && sel[j] != sel[k];
            }
            if (apart) {
                float cur[kScatterBatch];
#pragma unroll
                for (uint32_t k = 0; k < kScatterBatch; k++) cur[k] = target[ao + sel[k] * pl.a_axis_stride];
#pragma unroll
                for (uint32_t k = 0; k < kScatterBatch; k++) target[ao + sel[k] * pl.a_axis_stride] = cur[k] + fv[k];
                continue;
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < kScatterBatch; k++) {
            if (i0 + k < pl.i_axis_len) {
                const int sel = static_cast<int>(fi[k]);
                if (sel < 0 || static_cast<uint32_t>(sel) >= pl.a_axis_len) { *bad = 1; continue; }
                float* to = target + ao + static_cast<uint32_t>(sel) * pl.a_axis_stride;
                if (MODE == 2) *to = value;
                else if (MODE == 1) *to = *to + fv[k];
                else *to = fv[k];
            }
        }
    }
}

// Scatter along the innermost axis, a wave per position: its lanes take 64 consecutive entries of the index row at
// a time (coalesced reads of index and source, 64 elements of the target in flight), where scatter_kernel has one
// thread walk the row. Entries of one step that name the same element find each other by a ballot per bit of the
// element number. An assignment is then made by the highest lane of each such group (the last entry wins). For an add
// the group's first lane reads the element, the sum goes from lane to lane in lane order (one shuffle per round, as
// many rounds as the step's most frequent element occurs: nearly always none) and the last lane writes it. Steps
// follow each other in the order of the row, a step's writes made visible to the wave before the next one's reads;
// the next step's index and source values are requested before that wait.
template <int MODE>
__global__ __launch_bounds__(kBlock) void scatter_wave_kernel(float* __restrict__ target, const float* __restrict__ index,
                                                             const float* __restrict__ src, float value, uint32_t positions,
                                                             IndexPlan pl, int* bad, int element_bits) {
    const uint32_t pos = blockIdx.x * (kBlock / 64) + threadIdx.x / 64;
    const uint32_t lane = threadIdx.x & 63u;
    if (pos >= positions) return;                              // the whole wave
    uint32_t io, ao, bo;
    locate(pl, pos, io, ao, bo);
    float fi_next = lane < pl.i_axis_len ? __builtin_nontemporal_load(index + io + lane) : 0.0f;
    float fv_next = (MODE != 2 && lane < pl.i_axis_len) ? __builtin_nontemporal_load(src + bo + lane * pl.b_axis_stride) : 0.0f;
    for (uint32_t i0 = 0; i0 < pl.i_axis_len; i0 += 64) {
        const bool have = i0 + lane < pl.i_axis_len;
        const float fi = fi_next, fv = fv_next;
        const uint32_t ahead = i0 + 64 + lane;
        if (ahead < pl.i_axis_len) {
            fi_next = __builtin_nontemporal_load(index + io + ahead);
            if (MODE != 2) fv_next = __builtin_nontemporal_load(src + bo + ahead * pl.b_axis_stride);
        }
        const int sel = static_cast<int>(fi);
        const bool ok = have && sel >= 0 && static_cast<uint32_t>(sel) < pl.a_axis_len;
        if (have && !ok) *bad = 1;
        unsigned long long same = __ballot(ok);
        for (int bit = 0; bit < element_bits; bit++) {
            const bool set = (sel >> bit) & 1;
            const unsigned long long with = __ballot(ok && set);
            same &= set ? with : ~with;
        }
        float* to = target + ao + static_cast<uint32_t>(ok ? sel : 0);
        const bool last = ok && ((same >> lane) >> 1) == 0;    // no later entry of the step names the element
        if (MODE != 1) {
            if (last) *to = MODE == 2 ? value : fv;
        } else {
            const unsigned long long before = same & ((1ull << lane) - 1ull);
            const uint32_t rank = ok ? __popcll(before) : 0u;
            const int from = before ? 63 - __clzll(static_cast<long long>(before)) : static_cast<int>(lane);
            float sum = 0.0f;
            if (ok && rank == 0) sum = *to + fv;
            for (uint32_t round = 1; __ballot(ok && rank >= round) != 0; round++) {
                const float carried = __shfl(sum, from);
                if (ok && rank == round) sum = carried + fv;
            }
            if (last) *to = sum;
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
    }
}

// The tail of the add form of scatter_rows_lds_kernel: the waves of the workgroup take turns, in the order of the row, over the
// entries that are still pending. A wave's pending entries find the others for their element by a ballot per bit of the
// element number, the first lane of such a group reads the element, the sum goes from lane to lane by a shuffle per further
// entry, and the last lane writes it. Not inlined: inside the kernel's loop of rounds it cost rows that never need it a
// tenth of their time (278 -> 305 us on rows of 16384 uniformly spread entries).
template <int THREADS>
__device__ __attribute__((noinline)) void settle_by_turns(float* tile, uint32_t sel, float v, bool pending, uint32_t band_len) {
    const uint32_t tid = threadIdx.x;
    __syncthreads();                                          // the winners' adds of the last round have landed
    const uint32_t lane = tid & 63u;
    const int element_bits = 32 - __clz(static_cast<int>(band_len - 1u) | 1);
    for (uint32_t w = 0; w < THREADS / 64; w++) {
        if (tid / 64 == w && __ballot(pending) != 0) {
            unsigned long long same = __ballot(pending);
            for (int bit = 0; bit < element_bits; bit++) {
                const bool set = (sel >> bit) & 1u;
                const unsigned long long with = __ballot(pending && set);
                same &= set ? with : ~with;
            }
            const unsigned long long before = same & ((1ull << lane) - 1ull);
            const uint32_t rank = pending ? __popcll(before) : 0u;
            const int from = before ? 63 - __clzll(static_cast<long long>(before)) : static_cast<int>(lane);
            const bool last = pending && ((same >> lane) >> 1) == 0;
            float sum = 0.0f;
            if (pending && rank == 0) sum = tile[sel] + v;
            for (uint32_t step = 1; __ballot(pending && rank >= step) != 0; step++) {
                const float carried = __shfl(sum, from);
                if (pending && rank == step) sum = carried + v;
            }
            if (last) tile[sel] = sum;
        }
        __syncthreads();
    }
}

// Scatter along the innermost axis when the index rows are long: one workgroup per position
// keeps the target row in LDS, so the scattered accesses never leave the CU and the row goes
// back to memory as one contiguous span. The index row is taken THREADS entries at a time, in
// order; inside such a chunk, entries that name the same target element are put in order
// through an LDS tag per element:
//   assign: the element is cleared, every contender raises it to its lane number + 1 with an
//           atomic max, and the highest lane (the last entry) then stores its value there (the
//           same scheme with tags of their own and one barrier per chunk measured 20 % slower:
//           twice the LDS per workgroup);
//   add:    contenders lower the element's tag to (round number, lane) with an atomic min; the
//           lowest lane adds its value and leaves, and the round repeats until nobody is left
//           (as many rounds as the most frequent index of the chunk occurs), one barrier a round.
// LDS: band_len floats (the whole row when it fits), plus band_len tags for MODE 1. THREADS = 1024 for rows above 32 KiB of
// LDS, which leave room for few workgroups on a CU: the chunk is then 1024 entries.
template <int MODE, int THREADS>
__global__ __launch_bounds__(THREADS) void scatter_rows_lds_kernel(float* __restrict__ target, const float* __restrict__ index,
                                                                 const float* __restrict__ src, float value, IndexPlan pl, int* bad,
                                                                 uint32_t band_len, uint32_t from_constant, float constant,
                                                                 uint32_t tag_slots, FastDiv tag_div) {
    extern __shared__ __attribute__((aligned(16))) float row_lds[];
    constexpr uint32_t kFirstEpoch = 0x3ffffeu;               // 22 bits above the 10 bits of a thread id
    constexpr uint32_t kTailFrom = 8;                         // MODE 1: rounds of a chunk before the waves take turns
    static_assert(THREADS <= 1024, "a bid keeps the thread id in 10 bits");
    __shared__ uint32_t any_pending[3];
    float* tile = row_lds;
    uint32_t* tile_bits = reinterpret_cast<uint32_t*>(row_lds);
    uint32_t* tag = reinterpret_cast<uint32_t*>(row_lds) + band_len;          // MODE 1 only
    const uint32_t tid = threadIdx.x;
    uint32_t io, ao, bo;
    locate(pl, blockIdx.x, io, ao, bo);
    const float* irow = index + io;
    const float* srow = src + bo;
    // A target row longer than the LDS holds is taken in bands of band_len elements (a multiple of 4):
    // each band walks the whole index row and applies the entries that fall into it. Entries for one
    // element are all in the same band, so their order is kept.
    for (uint32_t band0 = 0; band0 < pl.a_axis_len; band0 += band_len) {
        const uint32_t band = min(band_len, pl.a_axis_len - band0);
        float* trow = target + ao + band0;
        if (band0 > 0) __syncthreads();                       // the previous band has left the tile
        // from_constant: the target is owed a fill with `constant` that was never launched; the rows start from it
        if (from_constant) { for (uint32_t j = tid; j < band; j += THREADS) tile[j] = constant; }
        else row_to_lds<THREADS>(trow, tile, band);
        if (MODE == 1) for (uint32_t j = tid; j < tag_slots; j += THREADS) tag[j] = 0xffffffffu;
        if (MODE == 1 && tid < 3) any_pending[tid] = 0u;
        uint32_t epoch = kFirstEpoch;                         // MODE 1: the round counter, uniform over the workgroup
        // the first chunk's entries are fetched while the row arrives
        float next_i = 0.0f, next_v = value;
        if (tid < pl.i_axis_len) { next_i = __builtin_nontemporal_load(irow + tid); if (MODE != 2) next_v = __builtin_nontemporal_load(srow + tid); }
        __syncthreads();
        for (uint32_t r0 = 0; r0 < pl.i_axis_len; r0 += THREADS) {
            const uint32_t r = r0 + tid;
            bool have = r < pl.i_axis_len;
            const int sel_raw = static_cast<int>(next_i);
            const float v = MODE == 1 ? next_v * value : next_v;  // add form: value is the factor on the source (1 for scatterAdd)
            if (r + THREADS < pl.i_axis_len) { next_i = __builtin_nontemporal_load(irow + r + THREADS); if (MODE != 2) next_v = __builtin_nontemporal_load(srow + r + THREADS); }
            if (have && (sel_raw < 0 || static_cast<uint32_t>(sel_raw) >= pl.a_axis_len)) { *bad = 1; have = false; }
            if (have && (static_cast<uint32_t>(sel_raw) < band0 || static_cast<uint32_t>(sel_raw) >= band0 + band)) have = false;
            const uint32_t sel = have ? static_cast<uint32_t>(sel_raw) - band0 : 0u;
            if (MODE == 2) {
                if (have) tile[sel] = value;               // equal values: the order of the stores is immaterial
            } else if (MODE == 0) {
                if (have) tile_bits[sel] = 0u;
                __syncthreads();
                if (have) atomicMax(&tile_bits[sel], tid + 1u);
                __syncthreads();
                const bool last = have && tile_bits[sel] == tid + 1u;
                __syncthreads();
                if (last) tile[sel] = v;
                __syncthreads();
            } else {
                // Entries for one element are added in index order, one per round: every pending entry
                // bids (round, tid) for its element with atomicMin, the lowest tid of the round wins and
                // adds. Rounds count down, so a bid of a later round always beats what earlier rounds
                // left in the tag and the tags are never reset; one barrier per round, with a flag that tells
                // whether anything was pending. A winner that reads its tag after a faster loser has
                // already bid for the next round sees that bid, stays pending and wins the next round
                // (same round, lower tid): the order is kept.
                if (epoch < 2u * THREADS + 4u) {              // (only after millions of rounds on one band)
                    __syncthreads();
                    for (uint32_t j = tid; j < tag_slots; j += THREADS) tag[j] = 0xffffffffu;
                    if (tid < 3) any_pending[tid] = 0u;
                    epoch = kFirstEpoch;
                    __syncthreads();
                }
                bool pending = have;
                // fewer tags than elements (tag_slots < band_len): elements share a tag by their remainder. Entries
                // for one element still meet at one tag; entries for different elements that meet there only wait
                // a round for each other.
                const uint32_t at = tag_slots >= band_len ? sel : sel - ((__umulhi(sel, tag_div.mul) + sel) >> tag_div.shift) * tag_slots;
                for (uint32_t rounds = 0;; rounds++) {
                    const uint32_t bid = (epoch << 10) | tid;
                    const uint32_t slot = epoch % 3u;
                    if (pending) { atomicMin(&tag[at], bid); any_pending[slot] = 1u; }
                    // three flags in turn: this round's is read after the barrier; the next round's, last
                    // read two rounds ago (before the previous barrier), is cleared now. The last round's may
                    // still be being read by a slow thread and is left alone. Every round, the last one of a
                    // chunk included, moves on to the next flag.
                    if (tid == 0) any_pending[(slot + 2u) % 3u] = 0u;
                    __syncthreads();
                    const bool more = any_pending[slot] != 0u;
                    epoch--;
                    if (!more) break;
                    if (pending && tag[at] == bid) {       // one lane per tag gets here
                        tile[sel] = tile[sel] + v;
                        pending = false;
                    }
                    // Entries are still pending after kTailFrom rounds: some element is named many times (a round
                    // retires one entry of it, at a barrier each). The rounds have retired the first entries of every
                    // element, in order; the waves now take turns, in the order of the row, over what is left.
                    if (rounds + 1 >= kTailFrom) {
                        settle_by_turns<THREADS>(tile, sel, v, pending, band_len);
                        break;
                    }
                }
            }
        }
        __syncthreads();
        lds_to_row<THREADS>(tile, trow, band);
    }
}

// indexSelect / indexAdd (JVMRawTensor.kt:484-516): the index is one list of k rows along the
// axis, shared by every position. The tensor is seen as [outer, axis, inner].
struct RowsPlan {
    uint32_t axis_len, k, inner;       // inner in the kernel's units (float4s for the vector form)
    FastDiv  inner_div, k_div;
    uint32_t heads;                    // indexAdd through the sorted list: no more runs than this (min(k, axis_len + 1))
    FastDiv  heads_div;
    uint32_t long_from;                // ... and runs of this many entries or more are left to the long-run kernel
};

// One thread per unit of the result [outer, k, inner]: out[o, i, :] = in[o, index[i], :].
template <bool VEC>
__global__ __launch_bounds__(kBlock) void index_select_kernel(const float* __restrict__ in, const float* __restrict__ index,
                                                             float* __restrict__ out, uint32_t units, RowsPlan pl, int* bad) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= units) return;
    const uint32_t row = (__umulhi(e, pl.inner_div.mul) + e) >> pl.inner_div.shift;       // o * k + i
    const uint32_t col = e - row * pl.inner;
    const uint32_t o = (__umulhi(row, pl.k_div.mul) + row) >> pl.k_div.shift;
    const int sel = static_cast<int>(index[row - o * pl.k]);
    if (sel < 0 || static_cast<uint32_t>(sel) >= pl.axis_len) { *bad = 1; return; }
    const uint32_t from = (o * pl.axis_len + static_cast<uint32_t>(sel)) * pl.inner + col;
    if (VEC) {
        const v4f_lds v = __builtin_nontemporal_load(reinterpret_cast<const v4f_lds*>(in) + from);
        reinterpret_cast<v4f_lds*>(out)[e] = v;
    } else out[e] = __builtin_nontemporal_load(in + from);
}

// The same for rows whose length is not a multiple of 4 (but at least 4): a row is covered by
// ceil(inner / 4) units of four floats at dword addresses, the last one moved back so that it ends
// with the row (it rewrites up to three floats with the values they already have). pl.inner counts units.
__global__ __launch_bounds__(kBlock) void index_select_ragged_kernel(const float* __restrict__ in, const float* __restrict__ index,
                                                                    float* __restrict__ out, uint32_t units, uint32_t row_floats,
                                                                    RowsPlan pl, int* bad) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= units) return;
    const uint32_t row = (__umulhi(e, pl.inner_div.mul) + e) >> pl.inner_div.shift;       // o * k + i
    const uint32_t unit = e - row * pl.inner;
    const uint32_t o = (__umulhi(row, pl.k_div.mul) + row) >> pl.k_div.shift;
    const int sel = static_cast<int>(index[row - o * pl.k]);
    if (sel < 0 || static_cast<uint32_t>(sel) >= pl.axis_len) { *bad = 1; return; }
    const uint32_t off = min(unit * 4u, row_floats - 4u);
    const size_t from = (static_cast<size_t>(o) * pl.axis_len + static_cast<uint32_t>(sel)) * row_floats + off;
    const size_t to = static_cast<size_t>(row) * row_floats + off;
    *reinterpret_cast<v4f_unaligned*>(out + to) = *reinterpret_cast<const v4f_unaligned*>(in + from);
}

// One thread per position (o, column): target[o, index[i], column] += src[o, i, column] * alpha
// for i ascending, so repeated indices accumulate in index order as on the JVM.
__global__ __launch_bounds__(kBlock) void index_add_kernel(float* __restrict__ target, const float* __restrict__ index,
                                                          const float* __restrict__ src, float alpha, uint32_t positions,
                                                          RowsPlan pl, int* bad) {
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= positions) return;
    const uint32_t o = (__umulhi(p, pl.inner_div.mul) + p) >> pl.inner_div.shift;
    const uint32_t col = p - o * pl.inner;
    float* t = target + static_cast<size_t>(o) * pl.axis_len * pl.inner + col;
    const float* s = src + static_cast<size_t>(o) * pl.k * pl.inner + col;
    constexpr uint32_t kBatch = 8;
    for (uint32_t i0 = 0; i0 < pl.k; i0 += kBatch) {
        float fi[kBatch], fv[kBatch];
#pragma unroll
        for (uint32_t j = 0; j < kBatch; j++)
            if (i0 + j < pl.k) { fi[j] = index[i0 + j]; fv[j] = s[static_cast<size_t>(i0 + j) * pl.inner]; }
#pragma unroll
        for (uint32_t j = 0; j < kBatch; j++) {
            if (i0 + j < pl.k) {
                const int sel = static_cast<int>(fi[j]);
                if (sel < 0 || static_cast<uint32_t>(sel) >= pl.axis_len) { *bad = 1; continue; }
                float* to = t + static_cast<size_t>(sel) * pl.inner;
                *to = *to + fv[j] * alpha;
            }
        }
    }
}

// ---- indexAdd through a sorted index list ------------------------------------------------
// keys[i] = the target row of source row i (axis_len for a value out of range, which is also
// reported); vals[i] = i. After a stable sort by key, the source rows that add into one target
// row stand next to each other in their original order.
__global__ __launch_bounds__(kBlock) void index_keys_kernel(const float* __restrict__ index, uint32_t k, uint32_t axis_len,
                                                           uint32_t* __restrict__ keys, uint32_t* __restrict__ vals, int* bad,
                                                           uint32_t* __restrict__ long_count) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i == 0) *long_count = 0;
    if (i >= k) return;
    const int sel = static_cast<int>(index[i]);
    const bool ok = sel >= 0 && static_cast<uint32_t>(sel) < axis_len;
    if (!ok) *bad = 1;
    keys[i] = ok ? static_cast<uint32_t>(sel) : axis_len;
    vals[i] = i;
}

// flags[i] = 1 where a run of equal keys starts in the sorted list. The invalid entries (key axis_len) stand at
// the end as a run of their own, so that every run ends where the next one starts (or at k).
__global__ __launch_bounds__(kBlock) void index_heads_kernel(const uint32_t* __restrict__ keys, uint32_t k, uint8_t* __restrict__ flags) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= k) return;
    flags[i] = (i == 0 || keys[i - 1] != keys[i]) ? 1 : 0;
}

// A long run is not walked by one thread per element (a batch of the walk costs a memory latency, and one hot row
// holds up the whole launch): it goes on a list for index_add_long_runs_kernel. The walk streams the source at the
// memory's rate as long as there are threads enough and no thread walks for longer than the whole source takes to
// read, so "long" is a 2^18-th of the source's elements, no less than kLongRunMin and no more than kLongRunMax.
constexpr uint32_t kLongRunMin = 256, kLongRunMax = 4096;
constexpr uint32_t kLongWaves = 16, kLongEntries = 32;
struct LongRuns {
    uint32_t* start;        // where the run starts in the sorted list
    uint32_t* len;
    uint32_t* key;          // its target row
    uint32_t* count;
};
// Called by the one thread of a walking kernel that meets the run's first element: the run goes on the list.
__device__ __forceinline__ void list_long_run(const LongRuns& runs, uint32_t start, uint32_t len, uint32_t key) {
    const uint32_t slot = atomicAdd(runs.count, 1u);
    runs.start[slot] = start; runs.len[slot] = len; runs.key[slot] = key;
}

// row_first[r] = where target row r's run starts in the sorted list, ~0u for a row no entry names.
__global__ __launch_bounds__(kBlock) void index_row_first_clear_kernel(uint32_t* __restrict__ row_first, uint32_t axis_len) {
    const uint32_t r = blockIdx.x * kBlock + threadIdx.x;
    if (r < axis_len) row_first[r] = 0xffffffffu;
}
// ... and row_end[r] = one past where it ends (only read for rows that have a first position).
__global__ __launch_bounds__(kBlock) void index_row_first_kernel(const uint32_t* __restrict__ keys, uint32_t k, uint32_t axis_len,
                                                                uint32_t* __restrict__ row_first, uint32_t* __restrict__ row_end) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= k) return;
    const uint32_t key = keys[i];
    if (key >= axis_len) return;
    if (i == 0 || keys[i - 1] != key) row_first[key] = i;
    if (i + 1 == k || keys[i + 1] != key) row_end[key] = i + 1;
}

// acc + rows[vals[first]] * alpha + rows[vals[first + 1]] * alpha + ... up to `end`, one rounding per product and per
// sum, in list order. The run's length is known, so up to kWalkBatch row numbers and then as many source loads are in
// flight before the adds that wait for them: a thread that walks a run pays the memory latency once per batch.
constexpr uint32_t kWalkBatch = 8;
template <class T>
__device__ __forceinline__ T walk_run(T acc, const T* __restrict__ s, size_t row_stride, const uint32_t* __restrict__ vals,
                                      uint32_t first, uint32_t end, float alpha) {
    for (uint32_t r = first; r < end; r += kWalkBatch) {
        const uint32_t m = min(kWalkBatch, end - r);
        uint32_t rows[kWalkBatch];
        T v[kWalkBatch];
#pragma unroll
        for (uint32_t j = 0; j < kWalkBatch; j++) if (j < m) rows[j] = vals[r + j];
#pragma unroll
        for (uint32_t j = 0; j < kWalkBatch; j++) if (j < m) v[j] = __builtin_nontemporal_load(s + static_cast<size_t>(rows[j]) * row_stride);
#pragma unroll
        for (uint32_t j = 0; j < kWalkBatch; j++) if (j < m) acc = acc + v[j] * alpha;
    }
    return acc;
}

// indexAdd into a target that is owed one constant everywhere and holds nothing yet (fresh from
// zerosLike): one thread per unit (float or float4) of the whole target [outer, axis, inner]. A row that
// the list names starts from the constant and takes its run's source rows in order, as below; any
// other row is the constant. Every element is written once and none is read. Rows with a long run are left
// to index_add_long_runs_kernel.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void index_add_filled_kernel(float* __restrict__ target, const float* __restrict__ src,
                                                                 const uint32_t* __restrict__ vals, const uint32_t* __restrict__ row_first,
                                                                 const uint32_t* __restrict__ row_end, float alpha, float constant,
                                                                 uint32_t units, RowsPlan pl, FastDiv axis_div, LongRuns runs) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= units) return;
    const uint32_t row = (__umulhi(e, pl.inner_div.mul) + e) >> pl.inner_div.shift;       // o * axis_len + r
    const uint32_t col = e - row * pl.inner;
    const uint32_t o = (__umulhi(row, axis_div.mul) + row) >> axis_div.shift;
    const uint32_t key = row - o * pl.axis_len;
    const uint32_t first = row_first[key];
    const uint32_t end = first != 0xffffffffu ? row_end[key] : 0u;
    if (first != 0xffffffffu && end - first >= pl.long_from) {
        if (o == 0 && col == 0) list_long_run(runs, first, end - first, key);
        return;
    }
    const size_t s_base = static_cast<size_t>(o) * pl.k * pl.inner + col;
    if (VEC) {
        v4f_lds acc = {constant, constant, constant, constant};
        if (first != 0xffffffffu) acc = walk_run(acc, reinterpret_cast<const v4f_lds*>(src) + s_base, pl.inner, vals, first, end, alpha);
        reinterpret_cast<v4f_lds*>(target)[e] = acc;
    } else {
        float acc = constant;
        if (first != 0xffffffffu) acc = walk_run(acc, src + s_base, pl.inner, vals, first, end, alpha);
        target[e] = acc;
    }
}

// The runs of equal keys are the touched target rows; their first positions (`heads`, *head_count
// of them) come from a compaction of the sorted list. One thread per unit (float or float4) of
// [outer, touched row, inner]: it adds the run's source rows in order, target = target + src * alpha
// each time (two roundings, as JVMRawTensor.kt:515). The grid covers min(k, axis_len + 1) rows per outer index (there
// cannot be more runs); threads past the number of touched rows leave at once, and so do those of a long run (index_add_long_runs_kernel
// takes it) and of the run of invalid entries. No two threads write the same element.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void index_add_sorted_kernel(float* __restrict__ target, const float* __restrict__ src,
                                                                 const uint32_t* __restrict__ keys, const uint32_t* __restrict__ vals,
                                                                 const uint32_t* __restrict__ heads, const uint32_t* __restrict__ head_count,
                                                                 float alpha, uint32_t units, RowsPlan pl, LongRuns runs) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= units) return;
    const uint32_t row = (__umulhi(e, pl.inner_div.mul) + e) >> pl.inner_div.shift;       // o * heads + h
    const uint32_t col = e - row * pl.inner;
    const uint32_t o = (__umulhi(row, pl.heads_div.mul) + row) >> pl.heads_div.shift;
    const uint32_t h = row - o * pl.heads;                 // the h-th touched target row
    const uint32_t n_heads = *head_count;
    if (h >= n_heads) return;
    const uint32_t first = heads[h];
    const uint32_t end = h + 1 < n_heads ? heads[h + 1] : pl.k;
    const uint32_t key = keys[first];
    if (key >= pl.axis_len) return;
    if (end - first >= pl.long_from) {
        if (o == 0 && col == 0) list_long_run(runs, first, end - first, key);
        return;
    }
    const size_t t_at = (static_cast<size_t>(o) * pl.axis_len + key) * pl.inner + col;
    const size_t s_base = static_cast<size_t>(o) * pl.k * pl.inner + col;
    if (VEC) {
        v4f_lds* t = reinterpret_cast<v4f_lds*>(target) + t_at;
        *t = walk_run(*t, reinterpret_cast<const v4f_lds*>(src) + s_base, pl.inner, vals, first, end, alpha);
    } else {
        float* t = target + t_at;
        *t = walk_run(*t, src + s_base, pl.inner, vals, first, end, alpha);
    }
}

// The same for rows whose length is not a multiple of 4 (but more than 4): a row is ceil(inner / 4)
// units; a full unit moves as 16 bytes at a dword address, the last one as its 1 ... 3 floats.
// pl.inner counts units, row_floats the floats of a row.
__global__ __launch_bounds__(kBlock) void index_add_sorted_ragged_kernel(float* __restrict__ target, const float* __restrict__ src,
                                                                        const uint32_t* __restrict__ keys, const uint32_t* __restrict__ vals,
                                                                        const uint32_t* __restrict__ heads, const uint32_t* __restrict__ head_count,
                                                                        float alpha, uint32_t units, uint32_t row_floats, RowsPlan pl, LongRuns runs) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= units) return;
    const uint32_t row = (__umulhi(e, pl.inner_div.mul) + e) >> pl.inner_div.shift;       // o * heads + h
    const uint32_t off = (e - row * pl.inner) * 4u;
    const uint32_t o = (__umulhi(row, pl.heads_div.mul) + row) >> pl.heads_div.shift;
    const uint32_t h = row - o * pl.heads;                 // the h-th touched target row
    const uint32_t n_heads = *head_count;
    if (h >= n_heads) return;
    const uint32_t first = heads[h];
    const uint32_t end = h + 1 < n_heads ? heads[h + 1] : pl.k;
    const uint32_t key = keys[first];
    if (key >= pl.axis_len) return;
    if (end - first >= pl.long_from) {
        if (o == 0 && off == 0) list_long_run(runs, first, end - first, key);
        return;
    }
    float* t = target + (static_cast<size_t>(o) * pl.axis_len + key) * row_floats + off;
    const float* s = src + static_cast<size_t>(o) * pl.k * row_floats + off;
    const uint32_t cnt = min(4u, row_floats - off);
    if (cnt == 4) {
        v4f_unaligned* t4 = reinterpret_cast<v4f_unaligned*>(t);
        // the row stride is counted in floats here: units of one float, read as four at a dword address
        v4f_unaligned acc = *t4;
        for (uint32_t r = first; r < end; r += kWalkBatch) {
            const uint32_t m = min(kWalkBatch, end - r);
            uint32_t rows[kWalkBatch];
            v4f_unaligned v[kWalkBatch];
#pragma unroll
            for (uint32_t j = 0; j < kWalkBatch; j++) if (j < m) rows[j] = vals[r + j];
#pragma unroll
            for (uint32_t j = 0; j < kWalkBatch; j++) if (j < m) v[j] = *reinterpret_cast<const v4f_unaligned*>(s + static_cast<size_t>(rows[j]) * row_floats);
#pragma unroll
            for (uint32_t j = 0; j < kWalkBatch; j++) if (j < m) acc = acc + v[j] * alpha;
        }
        *t4 = acc;
    } else {
        for (uint32_t j = 0; j < cnt; j++) t[j] = walk_run(t[j], s + j, row_floats, vals, first, end, alpha);
    }
}

// A long run (RowsPlan::long_from entries or more into one target row), by a workgroup of WAVES waves per 64 positions
// (outer index and column) of that row. The adds into one element are a chain that nothing can shorten (4 cycles
// each), but the loads they wait for need not stand in it. A round is WAVES x E entries: every wave holds its E
// source values in registers (a lane per position, so a round has WAVES x E x 256 bytes in flight), and then the
// waves take turns, in list order, adding their values to the 64 sums, which stand in LDS between turns. The
// values of the next round and the row numbers of the one after it are requested before the turns begin (a wave
// reads its E row numbers as one word per lane and hands them out with v_readlane), so a round costs its
// turns and the memory latency is paid once per run. Workgroups take (run, 64 positions) items in a strided loop
// until the list is done.
constexpr uint32_t kWave = 64;
template <uint32_t WAVES, uint32_t E>
__global__ __launch_bounds__(WAVES * kWave) void index_add_long_runs_kernel(float* __restrict__ target, const float* __restrict__ src,
                                                                           const uint32_t* __restrict__ vals, LongRuns runs, float alpha,
                                                                           uint32_t from_constant, float constant, uint32_t positions,
                                                                           RowsPlan pl) {
    static_assert(E <= kWave, "a wave reads its row numbers one per lane");
    constexpr uint32_t kRound = WAVES * E;
    __shared__ float carry[kWave];
    const uint32_t lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    const uint32_t mine = w * E;                               // where this wave's entries start in a round
    const uint32_t chunks = (positions + kWave - 1) / kWave;
    const uint64_t n_items = static_cast<uint64_t>(*runs.count) * chunks;
    for (uint64_t item = blockIdx.x; item < n_items; item += gridDim.x) {
        const uint32_t slot = static_cast<uint32_t>(item / chunks);
        const uint32_t p = static_cast<uint32_t>(item - static_cast<uint64_t>(slot) * chunks) * kWave + lane;     // o * inner + column
        const bool active = p < positions;
        const uint32_t o = active ? (__umulhi(p, pl.inner_div.mul) + p) >> pl.inner_div.shift : 0u;
        const uint32_t col = active ? p - o * pl.inner : 0u;
        const uint32_t first = runs.start[slot], len = runs.len[slot], key = runs.key[slot];
        float* t = target + (static_cast<size_t>(o) * pl.axis_len + key) * pl.inner + col;
        const float* s = src + static_cast<size_t>(o) * pl.k * pl.inner + col;
        if (w == 0) carry[lane] = (active && !from_constant) ? *t : constant;
        // the wave's row numbers of the round that starts at `base`: lane j holds entry j's (0 past the run's end)
        auto rows_of = [&](uint32_t base) -> uint32_t {
            const uint32_t at = base + mine + lane;
            return (lane < E && at < len) ? vals[first + at] : 0u;
        };
        auto count_of = [&](uint32_t base) -> uint32_t {
            const uint32_t at = base + mine;
            return at < len ? min(E, len - at) : 0u;
        };
        float v[E], v_next[E];
        uint32_t rows_next = rows_of(0);
#pragma unroll
        for (uint32_t j = 0; j < E; j++) v_next[j] = 0.0f;
        {
            const uint32_t cnt = count_of(0);
#pragma unroll
            for (uint32_t j = 0; j < E; j++) {
                const uint32_t row = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(rows_next), static_cast<int>(j)));
                if (j < cnt && active) v_next[j] = __builtin_nontemporal_load(s + static_cast<size_t>(row) * pl.inner);
            }
        }
        rows_next = rows_of(kRound);
        for (uint32_t base = 0; base < len; base += kRound) {
#pragma unroll
            for (uint32_t j = 0; j < E; j++) v[j] = v_next[j];
            const uint32_t cnt = count_of(base);
            // what the later rounds need goes out before this one's turns: the next round's values first (their row
            // numbers arrived a round ago), then the row numbers of the round after it
            {
                const uint32_t cnt_next = count_of(base + kRound);
#pragma unroll
                for (uint32_t j = 0; j < E; j++) {
                    const uint32_t row = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(rows_next), static_cast<int>(j)));
                    v_next[j] = 0.0f;
                    if (j < cnt_next && active) v_next[j] = __builtin_nontemporal_load(s + static_cast<size_t>(row) * pl.inner);
                }
            }
            rows_next = rows_of(base + 2 * kRound);
#pragma unroll
            for (uint32_t j = 0; j < E; j++) v[j] = v[j] * alpha;
            const uint32_t in_round = min(kRound, len - base);
            const uint32_t turns = (in_round + E - 1) / E;
            for (uint32_t turn = 0; turn < turns; turn++) {
                if (w == turn) {
                    float acc = carry[lane];
                    if (cnt == E) {                             // a full batch: nothing but the chain of adds
#pragma unroll
                        for (uint32_t j = 0; j < E; j++) acc = acc + v[j];
                    } else {
#pragma unroll
                        for (uint32_t j = 0; j < E; j++) if (j < cnt) acc = acc + v[j];
                    }
                    carry[lane] = acc;
                }
                __syncthreads();
            }
        }
        if (w == 0 && active) *t = carry[lane];
    }
}

// The same long runs when the tensor has one or two positions beside the axis (a flat tensor: one): the kernel above gives a
// position a lane and a run's entries to the lanes' registers one after the other, which leaves 63 lanes idle and costs a
// barrier per 32 entries (9.1 ns an entry). Here a wave owns one (run, position): its lanes fetch 256 entries at a time
// (the next 256 are on their way meanwhile), park them in LDS, and lane 0 reads them back 64 at a time as sixteen
// 16-byte words and adds them in order. Nothing crosses a wave, so there is no barrier; the waves of a workgroup take different items.
constexpr uint32_t kChainWaves = 4;
constexpr uint32_t kChainPositions = 2;                   // positions up to which a run is taken this way (with 8 or 16 and many runs the 4-byte fetches cost more than the barriers: [1024,16] with 2 million rows 437 us against 101)
__global__ __launch_bounds__(kChainWaves * kWave) void index_add_chain_kernel(float* __restrict__ target, const float* __restrict__ src,
                                                                             const uint32_t* __restrict__ vals, LongRuns runs, float alpha,
                                                                             uint32_t from_constant, float constant, uint32_t positions,
                                                                             RowsPlan pl, FastDiv positions_div) {
    constexpr uint32_t kDeep = 4;                            // batches of 64 entries in flight: a batch is added in less time than a gather takes
    constexpr uint32_t kSpan = kDeep * kWave;
    __shared__ __attribute__((aligned(16))) float staged[kChainWaves][kSpan];
    const uint32_t lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    const uint64_t n_items = static_cast<uint64_t>(*runs.count) * positions;
    for (uint64_t item = static_cast<uint64_t>(blockIdx.x) * kChainWaves + w; item < n_items; item += static_cast<uint64_t>(gridDim.x) * kChainWaves) {
        const uint32_t it = static_cast<uint32_t>(item);                       // (runs * positions stays below 2^32: both are bounded by the entries)
        const uint32_t slot = (__umulhi(it, positions_div.mul) + it) >> positions_div.shift;
        const uint32_t p = it - slot * positions;
        const uint32_t o = (__umulhi(p, pl.inner_div.mul) + p) >> pl.inner_div.shift;
        const uint32_t col = p - o * pl.inner;
        const uint32_t first = runs.start[slot], len = runs.len[slot], key = runs.key[slot];
        float* t = target + (static_cast<size_t>(o) * pl.axis_len + key) * pl.inner + col;
        const float* s = src + static_cast<size_t>(o) * pl.k * pl.inner + col;
        float acc = from_constant ? constant : *t;
        constexpr uint32_t kNone = 0xffffffffu;
        auto row_at = [&](uint32_t at) -> uint32_t { return at < len ? vals[first + at] : kNone; };
        auto value_of = [&](uint32_t row) -> float { return row != kNone ? __builtin_nontemporal_load(s + static_cast<size_t>(row) * pl.inner) : 0.0f; };
        uint32_t row_next[kDeep];
        float v_next[kDeep];
#pragma unroll
        for (uint32_t d = 0; d < kDeep; d++) row_next[d] = row_at(d * kWave + lane);
#pragma unroll
        for (uint32_t d = 0; d < kDeep; d++) v_next[d] = value_of(row_next[d]);
#pragma unroll
        for (uint32_t d = 0; d < kDeep; d++) row_next[d] = row_at(kSpan + d * kWave + lane);
        for (uint32_t base = 0; base < len; base += kSpan) {
#pragma unroll
            for (uint32_t d = 0; d < kDeep; d++) staged[w][d * kWave + lane] = v_next[d] * alpha;
#pragma unroll
            for (uint32_t d = 0; d < kDeep; d++) v_next[d] = value_of(row_next[d]);
#pragma unroll
            for (uint32_t d = 0; d < kDeep; d++) row_next[d] = row_at(base + 2 * kSpan + d * kWave + lane);
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");               // the wave's stores before lane 0's loads
            __builtin_amdgcn_wave_barrier();
            if (lane == 0) {
#pragma unroll
                for (uint32_t d = 0; d < kDeep; d++) {
                    const uint32_t at = base + d * kWave;
                    if (at + kWave <= len) {
                        const float4* q = reinterpret_cast<const float4*>(staged[w] + d * kWave);
                        float4 f[kWave / 4];
#pragma unroll
                        for (uint32_t j = 0; j < kWave / 4; j++) f[j] = q[j];
#pragma unroll
                        for (uint32_t j = 0; j < kWave / 4; j++) { acc = acc + f[j].x; acc = acc + f[j].y; acc = acc + f[j].z; acc = acc + f[j].w; }
                    } else if (at < len) {
                        for (uint32_t j = 0; j < len - at; j++) acc = acc + staged[w][d * kWave + j];
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");               // ... and its loads before the next stores
            __builtin_amdgcn_wave_barrier();
        }
        if (lane == 0) *t = acc;
    }
}

// Launches the kernel that takes the listed long runs: by waves of their own when the positions are few.
static void launch_long_runs(dim3 long_grid, uint64_t long_items, hipStream_t stream, float* target, const float* src, const uint32_t* vals,
                             const LongRuns& runs, float alpha, uint32_t from_constant, float constant, uint32_t positions, const RowsPlan& pl) {
    if (positions <= kChainPositions) {
        const uint64_t waves = long_items * positions;
        const uint64_t most = 8ull * static_cast<uint64_t>(state().compute_units);
        const dim3 grid(static_cast<uint32_t>(std::max<uint64_t>(1, std::min<uint64_t>((waves + kChainWaves - 1) / kChainWaves, most))));
        hipLaunchKernelGGL(index_add_chain_kernel, grid, dim3(kChainWaves * kWave), 0, stream, target, src, vals, runs, alpha, from_constant, constant,
                           positions, pl, make_div(positions));
        return;
    }
    hipLaunchKernelGGL((index_add_long_runs_kernel<kLongWaves, kLongEntries>), long_grid, dim3(kLongWaves * kWave), 0, stream, target, src, vals, runs, alpha,
                       from_constant, constant, positions, pl);
}


// ---- scatter through a sorted list of its entries -----------------------------------------
// A scatter with few positions and long index rows (a flat tensor, a long axis next to a handful of columns) gives
// the kernels above one row walker per position and nothing else to do: a flat tensor of 16 million elements with as
// many entries took seconds. Every entry of the index tensor becomes a pair (target element, source element) instead,
// in the index tensor's memory order, which lists the entries of one position in the order of the axis. After the
// stable sort by target element, the entries that fall on one element stand together in that order: an assignment
// takes the last one of each run, an add takes them all in order (the sorted indexAdd kernels, with rows of one float).
struct EntryPlan {
    int      ndim;                         // the dims of the index shape, innermost first
    uint32_t size[KTH_MAX_DIMS];
    FastDiv  div[KTH_MAX_DIMS];
    uint32_t t_stride[KTH_MAX_DIMS];       // target elements per step of the dim (0 at the axis)
    uint32_t s_stride[KTH_MAX_DIMS];       // source elements per step of the dim
    uint32_t t_axis_stride, a_axis_len;
};
__global__ __launch_bounds__(kBlock) void scatter_keys_kernel(const float* __restrict__ index, uint32_t n, EntryPlan pl, uint32_t invalid,
                                                             uint32_t* __restrict__ keys, uint32_t* __restrict__ vals, int* bad,
                                                             uint32_t* __restrict__ long_count) {
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e == 0) *long_count = 0;
    if (e >= n) return;
    uint32_t rest = e, t = 0, sc = 0;
    for (int d = 0; d < pl.ndim; d++) {
        const uint32_t q = (__umulhi(rest, pl.div[d].mul) + rest) >> pl.div[d].shift;
        const uint32_t c = rest - q * pl.size[d];
        t += c * pl.t_stride[d]; sc += c * pl.s_stride[d];
        rest = q;
    }
    const int sel = static_cast<int>(__builtin_nontemporal_load(index + e));
    const bool ok = sel >= 0 && static_cast<uint32_t>(sel) < pl.a_axis_len;
    if (!ok) *bad = 1;
    keys[e] = ok ? t + static_cast<uint32_t>(sel) * pl.t_axis_stride : invalid;
    vals[e] = sc;
}
// One thread per run: the element takes the run's last entry (or the constant).
__global__ __launch_bounds__(kBlock) void scatter_sorted_assign_kernel(float* __restrict__ target, const float* __restrict__ src,
                                                                      const uint32_t* __restrict__ keys, const uint32_t* __restrict__ vals,
                                                                      const uint32_t* __restrict__ heads, const uint32_t* __restrict__ head_count,
                                                                      uint32_t k, uint32_t invalid, float value, uint32_t fill) {
    const uint32_t h = blockIdx.x * kBlock + threadIdx.x;
    const uint32_t n = *head_count;
    if (h >= n) return;
    const uint32_t first = heads[h];
    const uint32_t end = h + 1 < n ? heads[h + 1] : k;
    const uint32_t key = keys[first];
    if (key >= invalid) return;
    target[key] = fill ? value : __builtin_nontemporal_load(src + vals[end - 1]);
}

int shape_count(const int32_t* shape, int dims, const char* what, uint64_t* count) {
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

// Strides of `shape` for the position dims (all dims but the axis, innermost first) and for the axis.
void strides_without_axis(const int32_t* shape, int dims, int axis, uint32_t* pos_strides, uint32_t* axis_stride) {
    uint64_t run = 1;
    int n = 0;
    for (int d = dims - 1; d >= 0; d--) {
        if (d == axis) *axis_stride = static_cast<uint32_t>(run);
        else pos_strides[n++] = static_cast<uint32_t>(run);
        run *= static_cast<uint64_t>(shape[d]);
    }
}

// Names the index operand of the move its entry point is about to launch, until that entry point returns
// (whichever way: a plan that fails before the check must not leave the store's address behind).
struct IndexUseScope {
    explicit IndexUseScope(const IndexUse& use) { state().index_use = use; }
    ~IndexUseScope() { state().index_use = IndexUse{}; }
    IndexUseScope(const IndexUseScope&) = delete;
    IndexUseScope& operator=(const IndexUseScope&) = delete;
};

// Runs `launch(flag)` with a cleared device flag and reports a set flag as an argument error.
template <class F>
int with_index_check(const char* what, F launch) {
    State& s = state();
    if (!s.index_check_immediate) {
        // deferred: the kernels set the persistent flag, the next blocking call reports it; nothing waits here
        s.index_use = IndexUse{};
        launch(s.deferred_index_flag);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fail(KTH_E_DEVICE, "%s: %s", what, hipGetErrorString(e));
        return KTH_OK;
    }
    // immediate: the kernels write a word of pinned host memory, read here once the stream has drained (the
    // word is zero whenever no indexed move is in flight: only this function lets kernels at it, and it waits).
    // An index store that an earlier move (or ARG_MAX / ARG_MIN) has left marked as holding only values below
    // this axis length, and that nothing has touched since, cannot raise the flag: nothing waits for it.
    const IndexUse use = s.index_use;
    s.index_use = IndexUse{};
    const bool known = use.store && use.store->index_valid_below != 0 && use.store->index_valid_below <= use.axis_len &&
                       use.store->index_valid_n >= use.n;
    launch(s.host_index_flag_device);
    hipError_t e = hipGetLastError();
    if (known) {
        if (e != hipSuccess) return fail(KTH_E_DEVICE, "%s: %s", what, hipGetErrorString(e));
        return KTH_OK;
    }
    if (e == hipSuccess) e = hipStreamSynchronize(s.stream);
    const int host_flag = *s.host_index_flag;
    *s.host_index_flag = 0;
    if (e != hipSuccess) return fail(KTH_E_DEVICE, "%s: %s", what, hipGetErrorString(e));
    if (host_flag) return fail(KTH_E_ARGUMENT, "%s got invalid index, an index value is out of bounds at the axis", what);
    if (use.store) {
        use.store->index_valid_below = use.axis_len; use.store->index_valid_n = use.n;
        // a copy that was put off reads its source's memory: the same holds for the source's first values
        // (unsqueeze of a targets tensor makes such a copy every step, and the next step's copy inherits the record)
        if (use.store->alias_of != 0) {
            Store& src = s.table[use.store->alias_of - 1];
            src.index_valid_below = use.axis_len; src.index_valid_n = use.n;
        }
    }
    return KTH_OK;
}

// The limits of scatter_rows_lds_kernel: the innermost axis, a target row that fits the LDS a
// workgroup may have (with its tags in the add form), index rows long enough that moving the
// whole row pays.
// A workgroup may use 64 KiB of dynamic LDS unless the kernel is granted more; gfx950 has 160 KiB
// per CU, so the row kernels ask for 128 KiB once and fall back to 64 KiB if refused.
static uint32_t rows_lds_limit() {
    static const uint32_t limit = [] {
        const int want = 131072;
        bool ok = true;
        const void* wide[] = {reinterpret_cast<const void*>(&scatter_rows_lds_kernel<0, 1024>),
                              reinterpret_cast<const void*>(&scatter_rows_lds_kernel<1, 1024>),
                              reinterpret_cast<const void*>(&scatter_rows_lds_kernel<2, 1024>)};
        ok = hipFuncSetAttribute(reinterpret_cast<const void*>(&gather_rows_lds_kernel<1024>), hipFuncAttributeMaxDynamicSharedMemorySize, want) == hipSuccess;
        for (const void* f : wide) ok = ok && hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, want) == hipSuccess;
        if (!ok) (void)hipGetLastError();
        // without the raised limit a launch holds 64 KiB of static and dynamic LDS together: leave room for
        // the scatter kernel's few static words
        return ok ? 131072u : 65536u - 256u;
    }();
    return limit;
}

// How a target row of a_axis_len floats sits in LDS: band_len floats of the row at a time (all of it when it
// fits) and, for the add form, tag_slots tags behind them. A row of up to 8192 floats has a tag per element
// (64 KiB together: two workgroups on a CU). A longer one is taken up to 16384 floats at a time with
// kSharedTags tags that its elements share by remainder: 80 KiB less a little, so that two workgroups still fit
// the CU's 160 KiB and one's rounds of LDS traffic fill the other's waits.
constexpr uint32_t kSharedTags = 3968;
static void rows_lds_plan(int mode, uint32_t a_axis_len, uint32_t* band_len, uint32_t* tag_slots, uint32_t* lds_bytes) {
    const uint32_t limit = rows_lds_limit();
    if (mode != 1) {
        *band_len = a_axis_len;
        if (static_cast<uint64_t>(a_axis_len) * 4u > limit) *band_len = (limit / 4u) & ~3u;
        *tag_slots = 0;
        *lds_bytes = *band_len * 4u;
        return;
    }
    if (static_cast<uint64_t>(a_axis_len) * 8u <= 65536u || limit < 131072u) {
        *band_len = a_axis_len;
        if (static_cast<uint64_t>(a_axis_len) * 8u > limit) *band_len = (limit / 8u) & ~3u;
        *tag_slots = *band_len;
    } else {
        *band_len = a_axis_len < 16384u ? a_axis_len : 16384u;
        *tag_slots = kSharedTags;
    }
    *lds_bytes = (*band_len + *tag_slots) * 4u;
}

static bool gather_rows_fit_lds(uint32_t a_axis_len, uint32_t i_axis_len) {
    return static_cast<uint64_t>(a_axis_len) * 4u <= rows_lds_limit() && i_axis_len >= 64 && i_axis_len >= a_axis_len / 8;
}

static bool scatter_rows_fit_lds(int /*mode*/, uint32_t a_axis_len, uint32_t i_axis_len) {
    return i_axis_len >= 64 && i_axis_len >= a_axis_len / 8;      // longer target rows go in bands
}

// Plans and launches a gather on device pointers; shapes are validated by the caller.
static int gather_launch(const float* in, const int32_t* in_shape, const float* index, const int32_t* index_shape, float* out,
                         int dims, int axis, uint64_t idx_n) {
    if (gather_rows_fit_lds(static_cast<uint32_t>(in_shape[axis]), static_cast<uint32_t>(index_shape[axis])) && axis == dims - 1) {
        IndexPlan rp{};
        rp.ndim = dims - 1;
        uint64_t positions = 1;
        for (int d = dims - 2, n = 0; d >= 0; d--, n++) {
            rp.size[n] = static_cast<uint32_t>(index_shape[d]);
            rp.div[n] = make_div(rp.size[n]);
            positions *= rp.size[n];
        }
        strides_without_axis(index_shape, dims, axis, rp.i_stride, &rp.i_axis_stride);
        strides_without_axis(index_shape, dims, axis, rp.b_stride, &rp.b_axis_stride);
        strides_without_axis(in_shape, dims, axis, rp.a_stride, &rp.a_axis_stride);
        rp.i_axis_len = static_cast<uint32_t>(index_shape[axis]);
        rp.a_axis_len = static_cast<uint32_t>(in_shape[axis]);
        const uint32_t lds_bytes = rp.a_axis_len * 4u;
        return with_index_check("Gather", [&](int* flag) {
            LaunchScope scope("gather_rows_lds_kernel", "", (positions * rp.a_axis_len + 2 * idx_n) * 4);
            const dim3 grid(static_cast<uint32_t>(positions));
            if (lds_bytes > 32768u)
                hipLaunchKernelGGL((gather_rows_lds_kernel<1024>), grid, dim3(1024), lds_bytes, state().stream, in, index, out, rp, flag);
            else
                hipLaunchKernelGGL((gather_rows_lds_kernel<256>), grid, dim3(256), lds_bytes, state().stream, in, index, out, rp, flag);
        });
    }
    IndexPlan pl{};
    pl.ndim = dims;
    uint64_t in_run = 1;
    for (int d = dims - 1, n = 0; d >= 0; d--, n++) {
        pl.size[n] = static_cast<uint32_t>(index_shape[d]);
        pl.div[n] = make_div(pl.size[n]);
        pl.a_stride[n] = d == axis ? 0u : static_cast<uint32_t>(in_run);
        if (d == axis) pl.a_axis_stride = static_cast<uint32_t>(in_run);
        in_run *= static_cast<uint64_t>(in_shape[d]);
    }
    pl.a_axis_len = static_cast<uint32_t>(in_shape[axis]);
    const uint32_t blocks = static_cast<uint32_t>((idx_n + kBlock - 1) / kBlock);
    return with_index_check("Gather", [&](int* flag) {
        LaunchScope scope("gather_kernel", "", 3 * idx_n * 4);
        hipLaunchKernelGGL(gather_kernel, dim3(blocks), dim3(kBlock), 0, state().stream, in, index, out,
                           static_cast<uint32_t>(idx_n), pl, flag);
    });
}

// A gather along an axis that is not the innermost reads one 4-byte element out of every 32-byte sector it
// touches when the index is random (1.15 ms for a full-size index on [16384,4096] along axis 0). When the axis
// is long, the row form applies and the input is not much larger than the index, it is cheaper to bring the
// axis to the innermost place with the permute kernels (input and index), gather rows there through LDS and
// permute the result back.
static bool gather_pays_transposing(const int32_t* in_shape, const int32_t* index_shape, int dims, int axis, uint64_t in_n, uint64_t idx_n) {
    if (axis == dims - 1) return false;
    const uint32_t a_len = static_cast<uint32_t>(in_shape[axis]), i_len = static_cast<uint32_t>(index_shape[axis]);
    if (i_len < 256 || !gather_rows_fit_lds(a_len, i_len)) return false;
    return idx_n >= (1u << 18) && in_n <= 2 * idx_n && idx_n / i_len <= 0x7fffffffull;
}

static int gather_transposed(const float* in, const int32_t* in_shape, const float* index, const int32_t* index_shape, float* out,
                             int dims, int axis, uint64_t in_n, uint64_t idx_n) {
    int32_t to_last[KTH_MAX_DIMS], from_last[KTH_MAX_DIMS];          // axis -> innermost, and back
    int32_t a_shape[KTH_MAX_DIMS], i_shape[KTH_MAX_DIMS];
    for (int d = 0, k = 0; d < dims; d++) if (d != axis) to_last[k++] = d;
    to_last[dims - 1] = axis;
    for (int d = 0; d < dims; d++) {
        from_last[to_last[d]] = d;
        a_shape[d] = in_shape[to_last[d]];
        i_shape[d] = index_shape[to_last[d]];
    }
    uint64_t a_cap = 0, i_cap = 0, o_cap = 0;
    float* a_moved = workspace_acquire(in_n * 4, &a_cap);
    float* i_moved = a_moved ? workspace_acquire(idx_n * 4, &i_cap) : nullptr;
    float* o_moved = i_moved ? workspace_acquire(idx_n * 4, &o_cap) : nullptr;
    int rc = KTH_E_MEMORY;
    if (a_moved && i_moved && o_moved) {
        rc = permute_device("kth_gather", in, a_moved, in_shape, dims, to_last);
        if (rc == KTH_OK) rc = permute_device("kth_gather", index, i_moved, index_shape, dims, to_last);
        if (rc == KTH_OK) rc = gather_launch(a_moved, a_shape, i_moved, i_shape, o_moved, dims, dims - 1, idx_n);
        if (rc == KTH_OK) rc = permute_device("kth_gather", o_moved, out, i_shape, dims, from_last);
    }
    if (o_moved) workspace_release(o_moved, o_cap);
    if (i_moved) workspace_release(i_moved, i_cap);
    if (a_moved) workspace_release(a_moved, a_cap);
    return rc;
}

}  // namespace

extern "C" {

int kth_gather(uint64_t in, const int32_t* in_shape, uint64_t index, const int32_t* index_shape,
               int dims, int axis, uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (dims < 1 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "kth_gather: %d dims", dims);
    if (axis < 0 || axis >= dims) return fail(KTH_E_ARGUMENT, "kth_gather: axis %d of %d dims", axis, dims);
    uint64_t in_n, idx_n;
    if (int rc = shape_count(in_shape, dims, "kth_gather(in)", &in_n)) return rc;
    if (int rc = shape_count(index_shape, dims, "kth_gather(index)", &idx_n)) return rc;
    for (int d = 0; d < dims; d++)
        if (d != axis && index_shape[d] > in_shape[d])
            return fail(KTH_E_SHAPE, "kth_gather: index dim %d (%d) exceeds the input's (%d)", d, index_shape[d], in_shape[d]);
    Store* si = lookup(in, "kth_gather(in)", true);
    if (!si) return KTH_E_HANDLE;
    Store* sx = lookup_index(index, "kth_gather(index)");
    if (!sx) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_gather(out)");
    if (!so) return KTH_E_HANDLE;
    if (in_n > si->n_floats || idx_n > sx->n_floats || idx_n > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_gather: a shape needs more elements than its store holds");
    if (so->ptr == si->ptr || so->ptr == sx->ptr) return fail(KTH_E_ARGUMENT, "kth_gather: output aliases an input");
    if (idx_n == 0) return KTH_OK;
    const IndexUseScope index_use(IndexUse{sx, static_cast<uint32_t>(in_shape[axis]), idx_n});
    if (gather_pays_transposing(in_shape, index_shape, dims, axis, in_n, idx_n))
        if (int rc = gather_transposed(si->ptr, in_shape, sx->ptr, index_shape, so->ptr, dims, axis, in_n, idx_n); rc != KTH_E_MEMORY)
            return rc;                                   // no room for the transposed copies: the element form below
    return gather_launch(si->ptr, in_shape, sx->ptr, index_shape, so->ptr, dims, axis, idx_n);
}

// Whether the scatter takes the row kernel, which rewrites every target row an index position names.
static bool scatter_takes_rows(int mode, const int32_t* target_shape, const int32_t* index_shape, int dims, int axis) {
    uint64_t positions = 1;
    for (int d = 0; d < dims; d++) if (d != axis) positions *= static_cast<uint64_t>(index_shape[d]);
    return axis == dims - 1 && positions <= 0x7fffffffull &&
           scatter_rows_fit_lds(mode, static_cast<uint32_t>(target_shape[axis]), static_cast<uint32_t>(index_shape[axis]));
}

// Plans and launches on device pointers; shapes are validated by the caller. With `constant` the target is
// taken to hold *constant everywhere without being read (only where scatter_takes_rows holds and the index
// covers the target off the axis, so that every row is rewritten).
static int scatter_launch(int mode, float* target, const int32_t* target_shape, const float* index, const int32_t* index_shape,
                          const float* psrc, const int32_t* src_shape, int dims, int axis, float value, uint64_t idx_n,
                          const float* constant = nullptr) {
    IndexPlan pl{};
    pl.ndim = dims - 1;
    uint64_t positions = 1;
    int n = 0;
    for (int d = dims - 1; d >= 0; d--) {
        if (d == axis) continue;
        pl.size[n] = static_cast<uint32_t>(index_shape[d]);
        pl.div[n] = make_div(pl.size[n]);
        positions *= pl.size[n];
        n++;
    }
    strides_without_axis(index_shape, dims, axis, pl.i_stride, &pl.i_axis_stride);
    strides_without_axis(target_shape, dims, axis, pl.a_stride, &pl.a_axis_stride);
    if (mode != 2) strides_without_axis(src_shape, dims, axis, pl.b_stride, &pl.b_axis_stride);
    pl.i_axis_len = static_cast<uint32_t>(index_shape[axis]);
    pl.a_axis_len = static_cast<uint32_t>(target_shape[axis]);
    const uint32_t blocks = static_cast<uint32_t>((positions + kBlock - 1) / kBlock);
    const uint64_t bytes = (mode == 2 ? 2 : mode == 1 ? 4 : 3) * idx_n * 4;
    if (axis == dims - 1 && scatter_rows_fit_lds(mode, pl.a_axis_len, pl.i_axis_len) && positions <= 0x7fffffffull) {
        uint32_t band_len, tag_slots, lds_bytes;
        rows_lds_plan(mode, pl.a_axis_len, &band_len, &tag_slots, &lds_bytes);
        const FastDiv tag_div = make_div(tag_slots ? tag_slots : 1u);
        const uint64_t bands = (pl.a_axis_len + band_len - 1) / band_len;
        const uint64_t row_bytes = ((constant ? 1ull : 2ull) * pl.a_axis_len * positions + bands * (mode == 2 ? 1 : 2) * idx_n) * 4;
        const uint32_t from_constant = constant ? 1u : 0u;
        const float start = constant ? *constant : 0.0f;
        return with_index_check("Scatter", [&](int* flag) {
            LaunchScope scope("scatter_rows_lds_kernel", mode == 0 ? "set" : mode == 1 ? "add" : "fill", row_bytes);
            const dim3 grid(static_cast<uint32_t>(positions));
            hipStream_t stream = state().stream;
            const float factor = mode == 1 ? 1.0f : value;
#define ROWS_LAUNCH(MM, TT) hipLaunchKernelGGL((scatter_rows_lds_kernel<MM, TT>), grid, dim3(TT), lds_bytes, stream, target, index, psrc, factor, pl, flag, band_len, from_constant, start, tag_slots, tag_div)
            if (lds_bytes > 32768u) { if (mode == 0) ROWS_LAUNCH(0, 1024); else if (mode == 1) ROWS_LAUNCH(1, 1024); else ROWS_LAUNCH(2, 1024); }
            else                    { if (mode == 0) ROWS_LAUNCH(0, 256);  else if (mode == 1) ROWS_LAUNCH(1, 256);  else ROWS_LAUNCH(2, 256); }
#undef ROWS_LAUNCH
        });
    }
    if (constant) return fail(KTH_E_ARGUMENT, "kth_scatter: internal: the serial form cannot start from a constant");
    // along the innermost axis, with index rows of half a wave or more: a wave per position
    if (axis == dims - 1 && pl.i_axis_len >= 32 && positions <= 0x3fffffffull) {
        int element_bits = 1;
        while (element_bits < 31 && (1u << element_bits) < pl.a_axis_len) element_bits++;
        return with_index_check("Scatter", [&](int* flag) {
            LaunchScope scope("scatter_wave_kernel", mode == 0 ? "set" : mode == 1 ? "add" : "fill", bytes);
            const uint32_t p32 = static_cast<uint32_t>(positions);
            const dim3 grid((p32 + kBlock / 64 - 1) / (kBlock / 64)), block(kBlock);
            hipStream_t stream = state().stream;
            if (mode == 0)      hipLaunchKernelGGL((scatter_wave_kernel<0>), grid, block, 0, stream, target, index, psrc, value, p32, pl, flag, element_bits);
            else if (mode == 1) hipLaunchKernelGGL((scatter_wave_kernel<1>), grid, block, 0, stream, target, index, psrc, value, p32, pl, flag, element_bits);
            else                hipLaunchKernelGGL((scatter_wave_kernel<2>), grid, block, 0, stream, target, index, psrc, value, p32, pl, flag, element_bits);
        });
    }
    return with_index_check("Scatter", [&](int* flag) {
        LaunchScope scope("scatter_kernel", mode == 0 ? "set" : mode == 1 ? "add" : "fill", bytes);
        const dim3 grid(blocks), block(kBlock);
        const uint32_t p32 = static_cast<uint32_t>(positions);
        hipStream_t stream = state().stream;
        if (mode == 0)      hipLaunchKernelGGL((scatter_kernel<0>), grid, block, 0, stream, target, index, psrc, value, p32, pl, flag);
        else if (mode == 1) hipLaunchKernelGGL((scatter_kernel<1>), grid, block, 0, stream, target, index, psrc, value, p32, pl, flag);
        else                hipLaunchKernelGGL((scatter_kernel<2>), grid, block, 0, stream, target, index, psrc, value, p32, pl, flag);
    });
}

// A scatter along an axis that is not the innermost walks that axis serially per position, about
// 0.4 us a step once the positions no longer hide the latency. When the axis is long and the row
// form above applies, it is cheaper to bring the axis to the innermost place with the permute
// kernels (target, index and source), scatter rows there and permute the target back:
// (4 target + 4 index + 2 source) elements of streaming traffic at about 5 TB/s.
static bool scatter_pays_transposing(int mode, const int32_t* target_shape, const int32_t* index_shape, int dims, int axis,
                                     uint64_t t_n, uint64_t idx_n, uint64_t src_n) {
    if (axis == dims - 1) return false;
    const uint32_t a_len = static_cast<uint32_t>(target_shape[axis]), i_len = static_cast<uint32_t>(index_shape[axis]);
    if (i_len < 256 || !scatter_rows_fit_lds(mode, a_len, i_len)) return false;
    const double positions = static_cast<double>(idx_n) / i_len;
    const double serial_us = 0.4 * i_len * (positions > 5e5 ? positions / 5e5 : 1.0);
    const double moved_us = 40.0 + (4.0 * t_n + 4.0 * idx_n + 2.0 * src_n) * 4.0 / 5e6;
    return serial_us > 2.0 * moved_us;
}

static int scatter_transposed(int mode, float* target, const int32_t* target_shape, const float* index, const int32_t* index_shape,
                              const float* psrc, const int32_t* src_shape, int dims, int axis, float value,
                              uint64_t t_n, uint64_t idx_n, uint64_t src_n, const float* constant) {
    int32_t to_last[KTH_MAX_DIMS], from_last[KTH_MAX_DIMS];          // axis -> innermost, and back
    int32_t t_shape[KTH_MAX_DIMS], i_shape[KTH_MAX_DIMS], s_shape[KTH_MAX_DIMS];
    for (int d = 0, k = 0; d < dims; d++) if (d != axis) to_last[k++] = d;
    to_last[dims - 1] = axis;
    for (int d = 0; d < dims; d++) {
        from_last[to_last[d]] = d;
        t_shape[d] = target_shape[to_last[d]];
        i_shape[d] = index_shape[to_last[d]];
        if (mode != 2) s_shape[d] = src_shape[to_last[d]];
    }
    uint64_t t_cap = 0, i_cap = 0, s_cap = 0;
    float* t_moved = workspace_acquire(t_n * 4, &t_cap);
    float* i_moved = t_moved ? workspace_acquire(idx_n * 4, &i_cap) : nullptr;
    float* s_moved = (i_moved && mode != 2) ? workspace_acquire(src_n * 4, &s_cap) : nullptr;
    int rc = KTH_E_MEMORY;
    if (t_moved && i_moved && (mode == 2 || s_moved)) {
        // a target that is one owed constant has nothing to bring along: its rows start from the constant
        rc = constant ? KTH_OK : permute_device("kth_scatter", target, t_moved, target_shape, dims, to_last);
        if (rc == KTH_OK) rc = permute_device("kth_scatter", index, i_moved, index_shape, dims, to_last);
        if (rc == KTH_OK && mode != 2) rc = permute_device("kth_scatter", psrc, s_moved, src_shape, dims, to_last);
        if (rc == KTH_OK) {
            rc = scatter_launch(mode, t_moved, t_shape, i_moved, i_shape, s_moved, s_shape, dims, dims - 1, value, idx_n, constant);
            // also after a reported index: the valid entries have been applied, as in the serial form
            if (rc == KTH_OK || rc == KTH_E_ARGUMENT) {
                const int back = permute_device("kth_scatter", t_moved, target, t_shape, dims, from_last);
                if (back != KTH_OK) rc = back;
            }
        }
    }
    if (s_moved) workspace_release(s_moved, s_cap);
    if (i_moved) workspace_release(i_moved, i_cap);
    if (t_moved) workspace_release(t_moved, t_cap);
    return rc;
}

// What the walk of the index rows costs on the path the scatter would take, against what sorting its entries costs.
// The walkers run side by side, so the time is one row's: per chunk of 1024 entries and band of the target row in the
// rows-through-LDS kernel (measured 0.35 us for an assignment, 0.8 us for an add, 0.23 us for a constant), per step of
// 64 entries for a wave (1.4 us), per entry for a thread (30 to 85 ns with neighbouring positions sharing cache lines);
// times the rounds it takes to seat all positions. The sort and what follows it cost about a tenth of a nanosecond
// per entry (16.7 million entries: 1.2 ms sorted, 1.5 ms in all) and some 100 us of launches.
static bool scatter_pays_sorting(int mode, const int32_t* target_shape, const int32_t* index_shape, int dims, int axis,
                                 uint64_t t_n, uint64_t idx_n, bool transposing) {
    const uint64_t i_len = static_cast<uint64_t>(index_shape[axis]), a_len = static_cast<uint64_t>(target_shape[axis]);
    if (i_len < 4096 || idx_n > 0x7fffffffull || t_n > 0x7ffffffeull) return false;
    const double positions = static_cast<double>(idx_n) / static_cast<double>(i_len);
    double walk_us;
    if (transposing || scatter_takes_rows(mode, target_shape, index_shape, dims, axis)) {
        const double bands = static_cast<double>((a_len + 16383) / 16384);
        const double unit_us = mode == 1 ? 0.8 : mode == 0 ? 0.35 : 0.23;
        walk_us = bands * static_cast<double>((i_len + 1023) / 1024) * unit_us * std::ceil(positions / 256.0);
    } else if (axis == dims - 1) {
        walk_us = static_cast<double>((i_len + 63) / 64) * 1.4 * std::ceil(positions / 8192.0);
    } else {
        walk_us = static_cast<double>(i_len) * (mode == 1 ? 0.085 : 0.04) * std::ceil(positions / 524288.0);
    }
    const double sort_us = 100.0 + static_cast<double>(idx_n) * 0.0001;
    return walk_us > 1.5 * sort_us;
}

static int scatter_sorted(int mode, float* target, const int32_t* target_shape, const float* index, const int32_t* index_shape,
                          const float* psrc, const int32_t* src_shape, int dims, int axis, float value, uint64_t t_n, uint64_t idx_n) {
    EntryPlan ep{};
    ep.ndim = dims;
    uint64_t t_run = 1, s_run = 1;
    for (int d = dims - 1, k = 0; d >= 0; d--, k++) {
        ep.size[k] = static_cast<uint32_t>(index_shape[d]);
        ep.div[k] = make_div(ep.size[k]);
        ep.t_stride[k] = d == axis ? 0u : static_cast<uint32_t>(t_run);
        ep.s_stride[k] = mode == 2 ? 0u : static_cast<uint32_t>(s_run);
        if (d == axis) ep.t_axis_stride = static_cast<uint32_t>(t_run);
        t_run *= static_cast<uint64_t>(target_shape[d]);
        if (mode != 2) s_run *= static_cast<uint64_t>(src_shape[d]);
    }
    ep.a_axis_len = static_cast<uint32_t>(target_shape[axis]);
    const uint32_t k = static_cast<uint32_t>(idx_n), invalid = static_cast<uint32_t>(t_n);
    int end_bit = 1;
    while (end_bit < 32 && (1ull << end_bit) <= t_n) end_bit++;              // keys run up to t_n inclusive
    RowsPlan pl{};
    pl.axis_len = invalid; pl.k = k; pl.inner = 1;
    pl.inner_div = make_div(1); pl.k_div = make_div(k);
    pl.heads = static_cast<uint32_t>(std::min<uint64_t>(idx_n, t_n + 1)); pl.heads_div = make_div(pl.heads);
    pl.long_from = kLongRunMin;                                              // rows of one float: a thread per run walks alone
    const uint64_t k_pad = (idx_n + 63) & ~63ull;
    const uint64_t long_pad = (idx_n / pl.long_from + 64) & ~63ull;
    hipStream_t stream = state().stream;
    size_t temp_bytes = 0, select_bytes = 0;
    if (sort_pairs_u32(nullptr, &temp_bytes, nullptr, nullptr, nullptr, nullptr, k, end_bit, stream) != hipSuccess ||
        select_flagged_positions(nullptr, &select_bytes, nullptr, nullptr, nullptr, k, stream) != hipSuccess) {
        (void)hipGetLastError();
        return KTH_E_MEMORY;
    }
    if (select_bytes > temp_bytes) temp_bytes = select_bytes;
    temp_bytes = (temp_bytes + 255) & ~static_cast<size_t>(255);
    uint64_t cap = 0;
    uint32_t* keys = reinterpret_cast<uint32_t*>(workspace_acquire(5 * k_pad * 4 + 2 * 64 * 4 + 3 * long_pad * 4 + k_pad + temp_bytes, &cap));
    if (!keys) { (void)hipGetLastError(); return KTH_E_MEMORY; }
    uint32_t* vals = keys + k_pad;
    uint32_t* keys_sorted = vals + k_pad;
    uint32_t* vals_sorted = keys_sorted + k_pad;
    uint32_t* heads = vals_sorted + k_pad;
    uint32_t* head_count = heads + k_pad;
    LongRuns runs{};
    runs.count = head_count + 64;
    runs.start = runs.count + 64; runs.len = runs.start + long_pad; runs.key = runs.len + long_pad;
    void* temp = runs.key + long_pad;
    uint8_t* flags = reinterpret_cast<uint8_t*>(temp) + temp_bytes;
    const uint64_t long_items = idx_n / pl.long_from;                        // at most; one position: one chunk of lanes per run
    const dim3 long_grid(static_cast<uint32_t>(std::min<uint64_t>(long_items, 2ull * static_cast<uint64_t>(state().compute_units))));
    const dim3 per_entry((k + kBlock - 1) / kBlock), per_head((pl.heads + kBlock - 1) / kBlock);
    hipError_t sort_status = hipSuccess;
    const int rc = with_index_check("Scatter", [&](int* flag) {
        {
            LaunchScope scope("scatter_sort", "", idx_n * 4 * 7);
            hipLaunchKernelGGL(scatter_keys_kernel, per_entry, dim3(kBlock), 0, stream, index, k, ep, invalid, keys, vals, flag, runs.count);
            size_t scratch = temp_bytes;
            sort_status = sort_pairs_u32(temp, &scratch, keys, keys_sorted, vals, vals_sorted, k, end_bit, stream);
            if (sort_status != hipSuccess) return;
            hipLaunchKernelGGL(index_heads_kernel, per_entry, dim3(kBlock), 0, stream, keys_sorted, k, flags);
            scratch = temp_bytes;
            sort_status = select_flagged_positions(temp, &scratch, flags, heads, head_count, k, stream);
            if (sort_status != hipSuccess) return;
        }
        if (mode != 1) {
            LaunchScope scope("scatter_sorted_assign_kernel", mode == 0 ? "set" : "fill", idx_n * (mode == 0 ? 8 : 4));
            hipLaunchKernelGGL(scatter_sorted_assign_kernel, per_head, dim3(kBlock), 0, stream, target, psrc, keys_sorted, vals_sorted, heads, head_count, k, invalid,
                               value, mode == 2 ? 1u : 0u);
            return;
        }
        {
            LaunchScope scope("index_add_sorted_kernel", "scatter", idx_n * 12);
            hipLaunchKernelGGL((index_add_sorted_kernel<false>), per_head, dim3(kBlock), 0, stream, target, psrc, keys_sorted, vals_sorted, heads, head_count, 1.0f,
                               pl.heads, pl, runs);
        }
        if (long_items > 0) {
            LaunchScope scope("index_add_long_runs_kernel", "scatter", 0);
            launch_long_runs(long_grid, long_items, stream, target, psrc, vals_sorted, runs, 1.0f, 0u, 0.0f, 1u, pl);
        }
    });
    workspace_release(reinterpret_cast<float*>(keys), cap);
    if (sort_status != hipSuccess) return fail(KTH_E_DEVICE, "kth_scatter: sorting the entries failed: %s", hipGetErrorString(sort_status));
    return rc;
}

static int scatter_common(int mode, uint64_t target, const int32_t* target_shape, uint64_t index, const int32_t* index_shape,
                          uint64_t src, const int32_t* src_shape, int dims, int axis, float value) {
    KTH_REQUIRE_INIT();
    if (dims < 1 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "kth_scatter: %d dims", dims);
    if (axis < 0 || axis >= dims) return fail(KTH_E_ARGUMENT, "kth_scatter: axis %d of %d dims", axis, dims);
    uint64_t t_n, idx_n, src_n = 0;
    if (int rc = shape_count(target_shape, dims, "kth_scatter(target)", &t_n)) return rc;
    if (int rc = shape_count(index_shape, dims, "kth_scatter(index)", &idx_n)) return rc;
    if (mode != 2) { if (int rc = shape_count(src_shape, dims, "kth_scatter(src)", &src_n)) return rc; }
    // ShapeFunctions.kt:346-371: index must fit the source everywhere and the target off the axis.
    for (int d = 0; d < dims; d++) {
        if (mode != 2 && index_shape[d] > src_shape[d])
            return fail(KTH_E_SHAPE, "Scatter requires that index.shape[a] <= src.shape[a] for all axis 'a'");
        if (d != axis && index_shape[d] > target_shape[d])
            return fail(KTH_E_SHAPE, "Scatter requires that index.shape[a] <= target.shape[a] for all axis 'a' except the specified axis");
    }
    Store* st = lookup_unsettled(target, "kth_scatter(target)");
    if (!st) return KTH_E_HANDLE;
    Store* sx = lookup_index(index, "kth_scatter(index)");
    if (!sx) return KTH_E_HANDLE;
    Store* ss = nullptr;
    if (mode != 2) { ss = lookup(src, "kth_scatter(src)", true); if (!ss) return KTH_E_HANDLE; }
    if (t_n > st->n_floats || idx_n > sx->n_floats || (ss && src_n > ss->n_floats))
        return fail(KTH_E_ARGUMENT, "kth_scatter: a shape needs more elements than its store holds");
    if (st->ptr == sx->ptr || (ss && st->ptr == ss->ptr)) return fail(KTH_E_ARGUMENT, "kth_scatter: target aliases an input");
    if (idx_n == 0) return KTH_OK;
    const IndexUseScope index_use(IndexUse{sx, static_cast<uint32_t>(target_shape[axis]), idx_n});
    const float* psrc = ss ? ss->ptr : nullptr;
    // A target that is still an owed constant (fresh from zerosLike) need not be filled and read back
    // when the row kernel rewrites all of it: the index covers every position off the axis.
    const bool transposing = scatter_pays_transposing(mode, target_shape, index_shape, dims, axis, t_n, idx_n, src_n);
    if (scatter_pays_sorting(mode, target_shape, index_shape, dims, axis, t_n, idx_n, transposing)) {
        settle(st);
        const int rc = scatter_sorted(mode, st->ptr, target_shape, sx->ptr, index_shape, psrc, src_shape, dims, axis, value, t_n, idx_n);
        if (rc != KTH_E_MEMORY) return rc;                       // no room for the sorted lists: the walk below
    }
    bool from_constant = st->fill_n == t_n && (transposing || scatter_takes_rows(mode, target_shape, index_shape, dims, axis));
    for (int d = 0; d < dims; d++) if (d != axis && index_shape[d] != target_shape[d]) from_constant = false;
    const float constant = st->fill_value;
    if (!from_constant) settle(st);
    if (transposing) {
        const int rc = scatter_transposed(mode, st->ptr, target_shape, sx->ptr, index_shape, psrc, src_shape, dims, axis, value,
                                          t_n, idx_n, src_n, from_constant ? &constant : nullptr);
        if (rc != KTH_E_MEMORY) { if (from_constant) st->fill_n = 0; return rc; }
        if (from_constant) { settle(st); from_constant = false; }      // no room for the transposed copies: the serial form below
    }
    if (from_constant) st->fill_n = 0;
    return scatter_launch(mode, st->ptr, target_shape, sx->ptr, index_shape, psrc, src_shape, dims, axis, value, idx_n,
                          from_constant ? &constant : nullptr);
}

int kth_scatter(int add, uint64_t target, const int32_t* target_shape, uint64_t index, const int32_t* index_shape,
                uint64_t src, const int32_t* src_shape, int dims, int axis) {
    std::lock_guard<std::mutex> g(lock());
    return scatter_common(add ? 1 : 0, target, target_shape, index, index_shape, src, src_shape, dims, axis, 0.0f);
}

int kth_scatter_fill(uint64_t target, const int32_t* target_shape, uint64_t index, const int32_t* index_shape,
                     int dims, int axis, float value) {
    std::lock_guard<std::mutex> g(lock());
    return scatter_common(2, target, target_shape, index, index_shape, 0, nullptr, dims, axis, value);
}

static int rows_geometry(const char* what, const int32_t* shape, int dims, int axis, uint64_t* outer, uint64_t* inner, uint64_t* total) {
    if (dims < 1 || dims > KTH_MAX_DIMS) return fail(KTH_E_ARGUMENT, "%s: %d dims", what, dims);
    if (axis < 0 || axis >= dims) return fail(KTH_E_ARGUMENT, "%s: axis %d of %d dims", what, axis, dims);
    if (int rc = shape_count(shape, dims, what, total)) return rc;
    *outer = 1; *inner = 1;
    for (int d = 0; d < axis; d++) *outer *= static_cast<uint64_t>(shape[d]);
    for (int d = axis + 1; d < dims; d++) *inner *= static_cast<uint64_t>(shape[d]);
    return KTH_OK;
}

int kth_index_select(uint64_t in, const int32_t* shape, int dims, int axis, uint64_t index, uint64_t k, uint64_t out) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    uint64_t outer, inner, total;
    if (int rc = rows_geometry("kth_index_select", shape, dims, axis, &outer, &inner, &total)) return rc;
    const uint64_t n_out = outer * k * inner;
    if (n_out > kMaxElements) return fail(KTH_E_ARGUMENT, "kth_index_select: more than 2^31-1 result elements");
    Store* si = lookup(in, "kth_index_select(in)", true);
    if (!si) return KTH_E_HANDLE;
    Store* sx = lookup_index(index, "kth_index_select(index)");
    if (!sx) return KTH_E_HANDLE;
    Store* so = lookup(out, "kth_index_select(out)");
    if (!so) return KTH_E_HANDLE;
    if (total > si->n_floats || k > sx->n_floats || n_out > so->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_index_select: a shape needs more elements than its store holds");
    if (so->ptr == si->ptr || so->ptr == sx->ptr) return fail(KTH_E_ARGUMENT, "kth_index_select: output aliases an input");
    if (n_out == 0) return KTH_OK;
    const IndexUseScope index_use(IndexUse{sx, static_cast<uint32_t>(shape[axis]), k});
    if (inner == 1 && gather_rows_fit_lds(static_cast<uint32_t>(shape[axis]), static_cast<uint32_t>(k))) {
        // columns picked from contiguous rows: the gather row kernel with one index row for every position
        IndexPlan rp{};
        rp.ndim = 1;
        rp.size[0] = static_cast<uint32_t>(outer); rp.div[0] = make_div(rp.size[0]);
        rp.i_stride[0] = 0; rp.a_stride[0] = static_cast<uint32_t>(shape[axis]); rp.b_stride[0] = static_cast<uint32_t>(k);
        rp.i_axis_stride = rp.a_axis_stride = rp.b_axis_stride = 1;
        rp.i_axis_len = static_cast<uint32_t>(k); rp.a_axis_len = static_cast<uint32_t>(shape[axis]);
        const uint32_t lds_bytes = rp.a_axis_len * 4u;
        return with_index_check("Index select", [&](int* flag) {
            LaunchScope scope("gather_rows_lds_kernel", "indexSelect", (total + n_out + k) * 4);
            const dim3 grid(static_cast<uint32_t>(outer));
            if (lds_bytes > 32768u)
                hipLaunchKernelGGL((gather_rows_lds_kernel<1024>), grid, dim3(1024), lds_bytes, state().stream, si->ptr, sx->ptr, so->ptr, rp, flag);
            else
                hipLaunchKernelGGL((gather_rows_lds_kernel<256>), grid, dim3(256), lds_bytes, state().stream, si->ptr, sx->ptr, so->ptr, rp, flag);
        });
    }
    if (inner % 4 != 0 && inner > 4) {
        RowsPlan rp{};
        rp.axis_len = static_cast<uint32_t>(shape[axis]); rp.k = static_cast<uint32_t>(k);
        rp.inner = static_cast<uint32_t>((inner + 3) / 4);
        rp.inner_div = make_div(rp.inner); rp.k_div = make_div(rp.k);
        const uint64_t units64 = outer * k * rp.inner;
        if (units64 <= kMaxElements) {
            const uint32_t units = static_cast<uint32_t>(units64);
            return with_index_check("Index select", [&](int* flag) {
                LaunchScope scope("index_select_kernel", "float4 at dword addresses", 2 * n_out * 4 + k * 4);
                hipLaunchKernelGGL(index_select_ragged_kernel, dim3((units + kBlock - 1) / kBlock), dim3(kBlock), 0, state().stream,
                                   si->ptr, sx->ptr, so->ptr, units, static_cast<uint32_t>(inner), rp, flag);
            });
        }
    }
    const bool vec = inner % 4 == 0;
    RowsPlan pl{};
    pl.axis_len = static_cast<uint32_t>(shape[axis]); pl.k = static_cast<uint32_t>(k);
    pl.inner = static_cast<uint32_t>(vec ? inner / 4 : inner);
    pl.inner_div = make_div(pl.inner); pl.k_div = make_div(pl.k);
    const uint32_t units = static_cast<uint32_t>(vec ? n_out / 4 : n_out);
    const uint32_t blocks = (units + kBlock - 1) / kBlock;
    return with_index_check("Index select", [&](int* flag) {
        LaunchScope scope("index_select_kernel", vec ? "float4" : "float", 2 * n_out * 4 + k * 4);
        if (vec) hipLaunchKernelGGL((index_select_kernel<true>), dim3(blocks), dim3(kBlock), 0, state().stream, si->ptr, sx->ptr, so->ptr, units, pl, flag);
        else     hipLaunchKernelGGL((index_select_kernel<false>), dim3(blocks), dim3(kBlock), 0, state().stream, si->ptr, sx->ptr, so->ptr, units, pl, flag);
    });
}

int kth_index_add(uint64_t target, const int32_t* shape, int dims, int axis, uint64_t index, uint64_t k, uint64_t src, float alpha) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    uint64_t outer, inner, total;
    if (int rc = rows_geometry("kth_index_add", shape, dims, axis, &outer, &inner, &total)) return rc;
    const uint64_t n_src = outer * k * inner;
    if (n_src > kMaxElements) return fail(KTH_E_ARGUMENT, "kth_index_add: more than 2^31-1 source elements");
    Store* st = lookup_unsettled(target, "kth_index_add(target)");
    if (!st) return KTH_E_HANDLE;
    Store* sx = lookup_index(index, "kth_index_add(index)");
    if (!sx) return KTH_E_HANDLE;
    Store* ss = lookup(src, "kth_index_add(src)", true);
    if (!ss) return KTH_E_HANDLE;
    if (total > st->n_floats || k > sx->n_floats || n_src > ss->n_floats)
        return fail(KTH_E_ARGUMENT, "kth_index_add: a shape needs more elements than its store holds");
    if (st->ptr == sx->ptr || st->ptr == ss->ptr) return fail(KTH_E_ARGUMENT, "kth_index_add: target aliases an input");
    const uint64_t positions = outer * inner;
    if (positions == 0 || k == 0) return KTH_OK;
    const IndexUseScope index_use(IndexUse{sx, static_cast<uint32_t>(shape[axis]), k});
    // A target that is one owed constant (fresh from zerosLike) and a list long enough to be sorted: the
    // rows are written from the constant, nothing of the target is read. Every other case has the fill launched.
    const bool vec_inner = inner % 4 == 0;
    const bool from_constant = st->fill_n == total && k >= 64 && total / (vec_inner ? 4 : 1) <= kMaxElements;
    const float constant = st->fill_value;
    if (!from_constant) settle(st);
    RowsPlan pl{};
    pl.axis_len = static_cast<uint32_t>(shape[axis]); pl.k = static_cast<uint32_t>(k); pl.inner = static_cast<uint32_t>(inner);
    pl.inner_div = make_div(pl.inner); pl.k_div = make_div(pl.k);
    hipStream_t stream = state().stream;

    // (a workgroup per outer position walks the whole list: with fewer positions than compute units a long list is
    // better sorted, so that every touched element has a thread of its own: a vector of a million elements with a
    // list of 1.1 million takes 43 ms here and a few hundred microseconds sorted)
    const bool rows_pay = outer >= static_cast<uint64_t>(state().compute_units) || k < 4096;
    if (inner == 1 && rows_pay && scatter_rows_fit_lds(1, pl.axis_len, pl.k)) {
        if (from_constant) st->fill_n = 0;                   // every row of the target is rewritten from the constant
        // columns added into contiguous rows: the scatter row kernel in its add form, one index row for
        // every position and alpha as the factor on the source
        IndexPlan rp{};
        rp.ndim = 1;
        rp.size[0] = static_cast<uint32_t>(outer); rp.div[0] = make_div(rp.size[0]);
        rp.i_stride[0] = 0; rp.a_stride[0] = pl.axis_len; rp.b_stride[0] = pl.k;
        rp.i_axis_stride = rp.a_axis_stride = rp.b_axis_stride = 1;
        rp.i_axis_len = pl.k; rp.a_axis_len = pl.axis_len;
        uint32_t band_len, tag_slots, lds_bytes;
        rows_lds_plan(1, rp.a_axis_len, &band_len, &tag_slots, &lds_bytes);
        const FastDiv tag_div = make_div(tag_slots);
        return with_index_check("Index Add", [&](int* flag) {
            LaunchScope scope("scatter_rows_lds_kernel", "indexAdd", (2 * total + n_src + k) * 4);
            const dim3 grid(static_cast<uint32_t>(outer));
            if (lds_bytes > 32768u)
                hipLaunchKernelGGL((scatter_rows_lds_kernel<1, 1024>), grid, dim3(1024), lds_bytes, stream, st->ptr, sx->ptr, ss->ptr, alpha, rp, flag, band_len, from_constant ? 1u : 0u, constant, tag_slots, tag_div);
            else
                hipLaunchKernelGGL((scatter_rows_lds_kernel<1, 256>), grid, dim3(256), lds_bytes, stream, st->ptr, sx->ptr, ss->ptr, alpha, rp, flag, band_len, from_constant ? 1u : 0u, constant, tag_slots, tag_div);
        });
    }

    // A short list: one thread per (outer, column) position walks it in order. The walk is serial,
    // about half a microsecond per entry, so from kSortedFrom entries on the list is sorted instead
    // and every touched target row is updated by its own threads.
    constexpr uint64_t kSortedFrom = 64;
    uint32_t* keys = nullptr;
    uint64_t cap = 0;
    size_t temp_bytes = 0;
    int end_bit = 1;
    while (end_bit < 32 && (1ull << end_bit) <= pl.axis_len) end_bit++;      // keys run up to axis_len inclusive
    const uint64_t k_pad = (k + 63) & ~63ull;                                // keeps the four arrays 256-byte aligned
    // (the walk needs a couple of waves on every SIMD to keep the memory busy, and rows whose length is not a multiple
    // of 4 walk at a quarter of the rate: with fewer than 100 000 threads, or such rows, the smallest threshold)
    const uint64_t walk_threads = outer * std::min<uint64_t>(k, pl.axis_len) * ((inner + 3) / 4);
    pl.long_from = static_cast<uint32_t>(std::min<uint64_t>(std::max<uint64_t>(n_src >> 18, kLongRunMin), kLongRunMax));
    if (walk_threads < 100000 || (inner % 4 != 0 && inner > 4)) pl.long_from = kLongRunMin;
    const uint64_t long_pad = (k / pl.long_from + 64) & ~63ull;              // no more runs than that can be long
    size_t select_bytes = 0;
    if (k >= kSortedFrom &&
        sort_pairs_u32(nullptr, &temp_bytes, nullptr, nullptr, nullptr, nullptr, pl.k, end_bit, stream) == hipSuccess &&
        select_flagged_positions(nullptr, &select_bytes, nullptr, nullptr, nullptr, pl.k, stream) == hipSuccess) {
        if (select_bytes > temp_bytes) temp_bytes = select_bytes;           // the two passes share their scratch
        temp_bytes = (temp_bytes + 255) & ~static_cast<size_t>(255);
        // keys, vals, sorted keys, sorted vals, heads: k_pad each; two counts: 64 each; start, length and target row of
        // the long runs: long_pad each; the passes' scratch; flags: k_pad bytes; then, for a target written from a
        // constant, the first and the one-past-last list position of every target row
        keys = reinterpret_cast<uint32_t*>(workspace_acquire(5 * k_pad * 4 + 2 * 64 * 4 + 3 * long_pad * 4 + k_pad + temp_bytes +
                                                             (from_constant ? 2 * (static_cast<uint64_t>(pl.axis_len) + 64) * 4 : 0), &cap));
    }
    if (!keys) {
        (void)hipGetLastError();
        if (from_constant) settle(st);
        const uint32_t blocks = static_cast<uint32_t>((positions + kBlock - 1) / kBlock);
        return with_index_check("Index Add", [&](int* flag) {
            LaunchScope scope("index_add_kernel", "", 3 * n_src * 4 + k * 4);
            hipLaunchKernelGGL(index_add_kernel, dim3(blocks), dim3(kBlock), 0, stream, st->ptr, sx->ptr, ss->ptr, alpha,
                               static_cast<uint32_t>(positions), pl, flag);
        });
    }
    uint32_t* vals = keys + k_pad;
    uint32_t* keys_sorted = vals + k_pad;
    uint32_t* vals_sorted = keys_sorted + k_pad;
    uint32_t* heads = vals_sorted + k_pad;
    uint32_t* head_count = heads + k_pad;
    LongRuns runs{};
    runs.count = head_count + 64;
    runs.start = runs.count + 64; runs.len = runs.start + long_pad; runs.key = runs.len + long_pad;
    void* temp = runs.key + long_pad;
    uint8_t* flags = reinterpret_cast<uint8_t*>(temp) + temp_bytes;
    // the long runs: a lane per float position of the row, whatever unit the walking kernel takes
    RowsPlan long_pl = pl;
    const uint32_t long_chunks = static_cast<uint32_t>((positions + kWave - 1) / kWave);
    const uint64_t long_items = (k / pl.long_from) * long_chunks;           // at most
    const dim3 long_grid(static_cast<uint32_t>(std::min<uint64_t>(long_items, 2ull * static_cast<uint64_t>(state().compute_units))));
    if (from_constant) {
        uint32_t* row_first = reinterpret_cast<uint32_t*>(flags + k_pad);
        uint32_t* row_end = row_first + pl.axis_len + 64;
        if (vec_inner) { pl.inner = static_cast<uint32_t>(inner / 4); pl.inner_div = make_div(pl.inner); }
        const uint32_t units = static_cast<uint32_t>(total / (vec_inner ? 4 : 1));
        hipError_t sort_status = hipSuccess;
        int rc = with_index_check("Index Add", [&](int* flag) {
            {
                LaunchScope scope("index_sort", "", k * 4 * 7);
                hipLaunchKernelGGL(index_keys_kernel, dim3((pl.k + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, sx->ptr, pl.k,
                                   pl.axis_len, keys, vals, flag, runs.count);
                size_t scratch = temp_bytes;
                sort_status = sort_pairs_u32(temp, &scratch, keys, keys_sorted, vals, vals_sorted, pl.k, end_bit, stream);
                if (sort_status != hipSuccess) return;
                hipLaunchKernelGGL(index_row_first_clear_kernel, dim3((pl.axis_len + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, row_first, pl.axis_len);
                hipLaunchKernelGGL(index_row_first_kernel, dim3((pl.k + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, keys_sorted, pl.k, pl.axis_len, row_first, row_end);
            }
            {
                LaunchScope scope("index_add_filled_kernel", vec_inner ? "float4" : "float", (total + n_src) * 4 + k * 4);
                const dim3 grid((units + kBlock - 1) / kBlock);
                const FastDiv axis_div = make_div(pl.axis_len);
                if (vec_inner) hipLaunchKernelGGL((index_add_filled_kernel<true>), grid, dim3(kBlock), 0, stream, st->ptr, ss->ptr, vals_sorted, row_first, row_end, alpha, constant, units, pl, axis_div, runs);
                else           hipLaunchKernelGGL((index_add_filled_kernel<false>), grid, dim3(kBlock), 0, stream, st->ptr, ss->ptr, vals_sorted, row_first, row_end, alpha, constant, units, pl, axis_div, runs);
            }
            if (long_items > 0) {
                LaunchScope scope("index_add_long_runs_kernel", "from a constant", 0);
                launch_long_runs(long_grid, long_items, stream, st->ptr, ss->ptr, vals_sorted, runs, alpha, 1u, constant, static_cast<uint32_t>(positions), long_pl);
            }
        });
        workspace_release(reinterpret_cast<float*>(keys), cap);
        if (sort_status != hipSuccess) { return fail(KTH_E_DEVICE, "kth_index_add: sorting the index list failed: %s", hipGetErrorString(sort_status)); }
        st->fill_n = 0;
        return rc;
    }
    const bool vec = inner % 4 == 0;
    const bool ragged = !vec && inner > 4 && outer * k * ((inner + 3) / 4) <= kMaxElements;
    if (vec) { pl.inner = static_cast<uint32_t>(inner / 4); pl.inner_div = make_div(pl.inner); }
    if (ragged) { pl.inner = static_cast<uint32_t>((inner + 3) / 4); pl.inner_div = make_div(pl.inner); }
    pl.heads = static_cast<uint32_t>(std::min<uint64_t>(k, static_cast<uint64_t>(pl.axis_len) + 1));
    pl.heads_div = make_div(pl.heads);
    const uint32_t units = static_cast<uint32_t>(outer * pl.heads * pl.inner);
    hipError_t sort_status = hipSuccess;
    int rc = with_index_check("Index Add", [&](int* flag) {
        {
            LaunchScope scope("index_sort", "", k * 4 * 7);
            hipLaunchKernelGGL(index_keys_kernel, dim3((pl.k + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, sx->ptr, pl.k,
                               pl.axis_len, keys, vals, flag, runs.count);
            size_t scratch = temp_bytes;
            sort_status = sort_pairs_u32(temp, &scratch, keys, keys_sorted, vals, vals_sorted, pl.k, end_bit, stream);
            if (sort_status == hipSuccess) {
                hipLaunchKernelGGL(index_heads_kernel, dim3((pl.k + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, keys_sorted, pl.k, flags);
                scratch = temp_bytes;
                sort_status = select_flagged_positions(temp, &scratch, flags, heads, head_count, pl.k, stream);
            }
        }
        if (sort_status != hipSuccess) return;
        {
            LaunchScope scope("index_add_sorted_kernel", vec ? "float4" : ragged ? "float4 at dword addresses" : "float", 3 * n_src * 4 + k * 4);
            const dim3 grid((units + kBlock - 1) / kBlock);
            if (ragged) hipLaunchKernelGGL(index_add_sorted_ragged_kernel, grid, dim3(kBlock), 0, stream, st->ptr, ss->ptr, keys_sorted, vals_sorted, heads, head_count, alpha, units,
                                           static_cast<uint32_t>(inner), pl, runs);
            else if (vec) hipLaunchKernelGGL((index_add_sorted_kernel<true>), grid, dim3(kBlock), 0, stream, st->ptr, ss->ptr, keys_sorted, vals_sorted, heads, head_count, alpha, units, pl, runs);
            else     hipLaunchKernelGGL((index_add_sorted_kernel<false>), grid, dim3(kBlock), 0, stream, st->ptr, ss->ptr, keys_sorted, vals_sorted, heads, head_count, alpha, units, pl, runs);
        }
        if (long_items > 0) {
            LaunchScope scope("index_add_long_runs_kernel", "", 0);
            launch_long_runs(long_grid, long_items, stream, st->ptr, ss->ptr, vals_sorted, runs, alpha, 0u, 0.0f, static_cast<uint32_t>(positions), long_pl);
        }
    });
    workspace_release(reinterpret_cast<float*>(keys), cap);
    if (sort_status != hipSuccess) return fail(KTH_E_DEVICE, "kth_index_add: sorting the index list failed: %s", hipGetErrorString(sort_status));
    return rc;
}

}  // extern "C"
