// Stable sort of (key, value) pairs of 32-bit unsigned integers by key, and the compaction of flagged
// positions, on a given stream. The index lists of indexAdd are sorted with it so that every target
// row finds the source rows that add into it as one run, in their original order: the order of the
// floating-point adds of JVMRawTensor.kt:503-516 rests on the sort being stable.
//
// Least-significant-digit radix sort, 8 bits per pass over the low `end_bit` bits of the key. A pass is
//   1. a histogram of the digit per tile of 4096 pairs (LDS counters), stored digit-major [256][tiles];
//   2. an exclusive scan over that table, which turns it into the first output position of every
//      (digit, tile): all of digit 0 in tile order, then all of digit 1, ...;
//   3. a scatter: a tile's pairs are taken 256 at a time in input order; inside a wave the lanes holding
//      the same digit find each other with 8 ballots, the waves' counts are prefixed in wave order through
//      LDS, and every pair gets the position base + (pairs with its digit before it in the tile).
// No atomics decide an output position, so equal keys keep their input order and the result is the same
// on every run. The scan is its own small set of kernels (one workgroup for up to 8192 entries,
// chunk sums + their scan + a rescan above), shared with the compaction, which is a scan of the flags
// and a scatter of the flagged positions.
#include "kth_internal.h"

namespace kth {

namespace {

constexpr uint32_t kThreads = 256;
constexpr uint32_t kWaves = kThreads / 64;
constexpr uint32_t kItems = 16;                          // pairs per thread and tile
constexpr uint32_t kTile = kThreads * kItems;            // 4096
constexpr uint32_t kRadix = 256;
constexpr uint32_t kScanChunk = kThreads * 8;            // entries per workgroup of the scan kernels
constexpr uint32_t kScanSingle = 8192;                   // up to here one workgroup scans everything

// Exclusive scan of one value per thread over the workgroup; *total gets the sum. `lds` holds kWaves + 1 words.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t x, uint32_t* lds, uint32_t* total) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t incl = x;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(incl, d);
        if (lane >= static_cast<uint32_t>(d)) incl += up;
    }
    if (lane == 63) lds[wave] = incl;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (uint32_t w = 0; w < kWaves; w++) { const uint32_t t = lds[w]; lds[w] = run; run += t; }
        lds[kWaves] = run;
    }
    __syncthreads();
    const uint32_t res = lds[wave] + incl - x;
    *total = lds[kWaves];
    __syncthreads();                                     // lds may be reused by the caller's next round
    return res;
}

// out[i] = sum of in[0 .. i) for i < m, by one workgroup (m up to kScanSingle and beyond, it just walks).
// With count != nullptr also *count = sum of all m entries. With positions != nullptr the entries are flags and
// the scan is not stored: positions[sum of in[0 .. i)] = i for every i with in[i] != 0 (a compaction in one launch).
template <class T>
__global__ __launch_bounds__(kThreads) void scan_single_kernel(const T* in, uint32_t* out, uint32_t m, uint32_t* count,
                                                               uint32_t* __restrict__ positions) {
    __shared__ uint32_t lds[kWaves + 1];
    uint32_t carry = 0;
    for (uint32_t base = 0; base < m; base += kScanChunk) {
        uint32_t v[8], sum = 0;
#pragma unroll
        for (uint32_t j = 0; j < 8; j++) {
            const uint32_t i = base + threadIdx.x * 8 + j;
            v[j] = i < m ? static_cast<uint32_t>(in[i]) : 0u;
            sum += v[j];
        }
        uint32_t total;
        uint32_t run = carry + block_exclusive_scan(sum, lds, &total);
#pragma unroll
        for (uint32_t j = 0; j < 8; j++) {
            const uint32_t i = base + threadIdx.x * 8 + j;
            if (i < m) {
                if (!positions) out[i] = run;
                else if (v[j]) positions[run] = i;
            }
            run += v[j];
        }
        carry += total;
    }
    if (count && threadIdx.x == 0) *count = carry;
}

// sums[b] = sum of chunk b of `in`.
template <class T>
__global__ __launch_bounds__(kThreads) void scan_sums_kernel(const T* __restrict__ in, uint32_t m, uint32_t* __restrict__ sums) {
    __shared__ uint32_t lds[kWaves + 1];
    const uint32_t base = blockIdx.x * kScanChunk;
    uint32_t sum = 0;
#pragma unroll
    for (uint32_t j = 0; j < 8; j++) {
        const uint32_t i = base + threadIdx.x * 8 + j;
        if (i < m) sum += static_cast<uint32_t>(in[i]);
    }
    uint32_t total;
    (void)block_exclusive_scan(sum, lds, &total);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// Chunk b rescanned from the scanned chunk sums: out[i] = sums[b] + sum of in[chunk start .. i).
template <class T>
__global__ __launch_bounds__(kThreads) void scan_apply_kernel(const T* in, uint32_t* out, uint32_t m, const uint32_t* __restrict__ sums) {
    __shared__ uint32_t lds[kWaves + 1];
    const uint32_t base = blockIdx.x * kScanChunk;
    uint32_t v[8], sum = 0;
#pragma unroll
    for (uint32_t j = 0; j < 8; j++) {
        const uint32_t i = base + threadIdx.x * 8 + j;
        v[j] = i < m ? static_cast<uint32_t>(in[i]) : 0u;
        sum += v[j];
    }
    uint32_t total;
    uint32_t run = sums[blockIdx.x] + block_exclusive_scan(sum, lds, &total);
#pragma unroll
    for (uint32_t j = 0; j < 8; j++) {
        const uint32_t i = base + threadIdx.x * 8 + j;
        if (i < m) out[i] = run;
        run += v[j];
    }
}

uint32_t scan_chunks(uint32_t m) { return (m + kScanChunk - 1) / kScanChunk; }

// Words of scratch exclusive_scan needs for m entries.
size_t scan_scratch_words(uint32_t m) { return m <= kScanSingle ? 0 : static_cast<size_t>(scan_chunks(m)) + 1; }

// out = exclusive scan of in (m entries; out may be `in` when T is uint32_t); *count = the total, if asked for.
template <class T>
hipError_t exclusive_scan(const T* in, uint32_t* out, uint32_t m, uint32_t* scratch, uint32_t* count, hipStream_t stream) {
    if (m <= kScanSingle) {
        hipLaunchKernelGGL((scan_single_kernel<T>), dim3(1), dim3(kThreads), 0, stream, in, out, m, count, static_cast<uint32_t*>(nullptr));
        return hipGetLastError();
    }
    const uint32_t chunks = scan_chunks(m);
    hipLaunchKernelGGL((scan_sums_kernel<T>), dim3(chunks), dim3(kThreads), 0, stream, in, m, scratch);
    hipLaunchKernelGGL((scan_single_kernel<uint32_t>), dim3(1), dim3(kThreads), 0, stream, scratch, scratch, chunks, count, static_cast<uint32_t*>(nullptr));
    hipLaunchKernelGGL((scan_apply_kernel<T>), dim3(chunks), dim3(kThreads), 0, stream, in, out, m, scratch);
    return hipGetLastError();
}

// The number of pairs of each tile whose key has a given digit at `shift`: hist[digit * tiles + tile] (digit-major,
// the order the scan needs), or hist[tile * 256 + digit] when TILE_MAJOR (the order the fused scatter reads best).
template <bool TILE_MAJOR>
__global__ __launch_bounds__(kThreads) void sort_histogram_kernel(const uint32_t* __restrict__ keys, uint32_t n, uint32_t shift,
                                                                  uint32_t* __restrict__ hist, uint32_t tiles) {
    __shared__ uint32_t h[kRadix];
    h[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t base = blockIdx.x * kTile;
#pragma unroll 4
    for (uint32_t j = 0; j < kItems; j++) {
        const uint32_t i = base + j * kThreads + threadIdx.x;
        if (i < n) atomicAdd(&h[(keys[i] >> shift) & (kRadix - 1)], 1u);       // a count: the order of the adds does not matter
    }
    __syncthreads();
    hist[TILE_MAJOR ? blockIdx.x * kRadix + threadIdx.x : threadIdx.x * tiles + blockIdx.x] = h[threadIdx.x];
}

// SCANNED: first[digit * tiles + tile] = output position of the tile's first pair with that digit. Otherwise `first`
// is the raw tile-major histogram of a list of at most kFusedTiles tiles and every workgroup derives its own positions
// from it (the pairs of smaller digits, plus those of its digit in earlier tiles): 1 KiB per tile read by every
// workgroup, which for lists of up to two million pairs is cheaper than the launches of a scan.
constexpr uint32_t kFusedTiles = 512;
template <bool SCANNED>
__global__ __launch_bounds__(kThreads) void sort_scatter_kernel(const uint32_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in,
                                                                uint32_t* __restrict__ keys_out, uint32_t* __restrict__ vals_out,
                                                                uint32_t n, uint32_t shift, const uint32_t* __restrict__ first, uint32_t tiles) {
    __shared__ uint32_t wave_count[kWaves][kRadix];
    __shared__ uint32_t next[kRadix];
    __shared__ uint32_t scan_lds[kWaves + 1];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint64_t below = (1ull << lane) - 1ull;
    if (SCANNED) {
        next[threadIdx.x] = first[threadIdx.x * tiles + blockIdx.x];
    } else {
        uint32_t of_digit = 0, earlier = 0;
#pragma unroll 8
        for (uint32_t t = 0; t < tiles; t++) {
            const uint32_t c = first[t * kRadix + threadIdx.x];
            if (t < blockIdx.x) earlier += c;
            of_digit += c;
        }
        uint32_t total;
        next[threadIdx.x] = block_exclusive_scan(of_digit, scan_lds, &total) + earlier;
    }
    const uint32_t base = blockIdx.x * kTile;
    // the tile's pairs are loaded before the rounds, so their latency is paid once
    uint32_t keys[kItems], vals[kItems];
#pragma unroll
    for (uint32_t j = 0; j < kItems; j++) {
        const uint32_t i = base + j * kThreads + threadIdx.x;
        keys[j] = i < n ? keys_in[i] : 0u;
        vals[j] = i < n ? vals_in[i] : 0u;
    }
#pragma unroll
    for (uint32_t j = 0; j < kItems; j++) {
#pragma unroll
        for (uint32_t w = 0; w < kWaves; w++) wave_count[w][threadIdx.x] = 0;
        __syncthreads();
        const uint32_t i = base + j * kThreads + threadIdx.x;
        const bool valid = i < n;
        const uint32_t key = keys[j];
        const uint32_t val = vals[j];
        const uint32_t digit = (key >> shift) & (kRadix - 1);
        // the lanes of this wave that hold a pair with the same digit
        uint64_t peers = __ballot(valid);
#pragma unroll
        for (uint32_t b = 0; b < 8; b++) {
            const bool bit = (digit >> b) & 1u;
            const uint64_t with_bit = __ballot(bit);
            peers &= bit ? with_bit : ~with_bit;
        }
        const uint32_t rank = static_cast<uint32_t>(__popcll(peers & below));
        if (valid && rank == 0) wave_count[wave][digit] = static_cast<uint32_t>(__popcll(peers));
        __syncthreads();
        {   // thread d: the waves' counts of digit d become their first positions, in wave order
            uint32_t run = next[threadIdx.x];
#pragma unroll
            for (uint32_t w = 0; w < kWaves; w++) {
                const uint32_t t = wave_count[w][threadIdx.x];
                wave_count[w][threadIdx.x] = run;
                run += t;
            }
            next[threadIdx.x] = run;
        }
        __syncthreads();
        if (valid) {
            const uint32_t pos = wave_count[wave][digit] + rank;
            keys_out[pos] = key;
            vals_out[pos] = val;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(kThreads) void select_scatter_kernel(const uint8_t* __restrict__ flags, const uint32_t* __restrict__ before,
                                                                  uint32_t* __restrict__ positions, uint32_t n) {
    const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
    if (i < n && flags[i]) positions[before[i]] = i;
}

size_t align_words(size_t words) { return (words + 63) & ~static_cast<size_t>(63); }

}  // namespace

// Stable sort by the low `end_bit` bits of the key. With temp == nullptr only *temp_bytes is set, to the scratch needed.
hipError_t sort_pairs_u32(void* temp, size_t* temp_bytes, const uint32_t* keys_in, uint32_t* keys_out,
                          const uint32_t* vals_in, uint32_t* vals_out, uint32_t n, int end_bit, hipStream_t stream) {
    const uint32_t tiles = n == 0 ? 1u : (n + kTile - 1) / kTile;
    const uint64_t table64 = static_cast<uint64_t>(kRadix) * tiles;
    if (table64 > 0xffffffffull) return hipErrorInvalidValue;
    const uint32_t table = static_cast<uint32_t>(table64);
    const size_t table_words = align_words(table), scan_words = align_words(scan_scratch_words(table)), pair_words = align_words(n);
    const size_t need = (table_words + scan_words + 2 * pair_words) * sizeof(uint32_t);
    if (!temp) { *temp_bytes = need; return hipSuccess; }
    if (*temp_bytes < need) return hipErrorInvalidValue;
    if (n == 0) return hipSuccess;
    uint32_t* hist = static_cast<uint32_t*>(temp);
    uint32_t* scan_scratch = hist + table_words;
    uint32_t* alt_keys = scan_scratch + scan_words;
    uint32_t* alt_vals = alt_keys + pair_words;
    int passes = (end_bit + 7) / 8;
    if (passes < 1) passes = 1;
    if (passes > 4) passes = 4;
    // the last pass must write keys_out / vals_out: an odd number of passes starts into them, an even one into the spare pair
    const uint32_t* src_k = keys_in; const uint32_t* src_v = vals_in;
    bool into_out = (passes % 2) == 1;
    for (int p = 0; p < passes; p++) {
        uint32_t* dst_k = into_out ? keys_out : alt_keys;
        uint32_t* dst_v = into_out ? vals_out : alt_vals;
        const uint32_t shift = static_cast<uint32_t>(8 * p);
        hipError_t e = hipSuccess;
        if (tiles <= kFusedTiles) {
            hipLaunchKernelGGL((sort_histogram_kernel<true>), dim3(tiles), dim3(kThreads), 0, stream, src_k, n, shift, hist, tiles);
            hipLaunchKernelGGL((sort_scatter_kernel<false>), dim3(tiles), dim3(kThreads), 0, stream, src_k, src_v, dst_k, dst_v, n, shift, hist, tiles);
        } else {
            hipLaunchKernelGGL((sort_histogram_kernel<false>), dim3(tiles), dim3(kThreads), 0, stream, src_k, n, shift, hist, tiles);
            e = exclusive_scan<uint32_t>(hist, hist, table, scan_scratch, nullptr, stream);
            if (e != hipSuccess) return e;
            hipLaunchKernelGGL((sort_scatter_kernel<true>), dim3(tiles), dim3(kThreads), 0, stream, src_k, src_v, dst_k, dst_v, n, shift, hist, tiles);
        }
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        src_k = dst_k; src_v = dst_v;
        into_out = !into_out;
    }
    return hipSuccess;
}

// The positions i in [0, n) with flags[i] != 0, in ascending order, and how many there are.
// With temp == nullptr only *temp_bytes is set.
hipError_t select_flagged_positions(void* temp, size_t* temp_bytes, const uint8_t* flags, uint32_t* positions, uint32_t* count,
                                    uint32_t n, hipStream_t stream) {
    const size_t before_words = align_words(n), scan_words = align_words(scan_scratch_words(n));
    const size_t need = (before_words + scan_words) * sizeof(uint32_t);
    if (!temp) { *temp_bytes = need; return hipSuccess; }
    if (*temp_bytes < need) return hipErrorInvalidValue;
    uint32_t* before = static_cast<uint32_t*>(temp);
    if (n <= kScanSingle) {          // one workgroup scans the flags and writes the positions as it goes
        hipLaunchKernelGGL((scan_single_kernel<uint8_t>), dim3(1), dim3(kThreads), 0, stream, flags, before, n, count, positions);
        return hipGetLastError();
    }
    hipError_t e = exclusive_scan<uint8_t>(flags, before, n, before + before_words, count, stream);
    if (e != hipSuccess || n == 0) return e;
    hipLaunchKernelGGL(select_scatter_kernel, dim3((n + kThreads - 1) / kThreads), dim3(kThreads), 0, stream, flags, before, positions, n);
    return hipGetLastError();
}

}  // namespace kth
