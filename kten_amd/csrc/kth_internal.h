// Shared host-side state and helpers of libkten_hip.so (not part of the public ABI).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <mutex>
#include <tuple>
#include <utility>
#include <vector>

#include "../../include/kten_hip.h"
#include "../../include/kten_hip_bench.h"
#include "kth_fastdiv.h"

namespace kth {

// One device-resident fp32 store. `cap_bytes` is the pool size class it was cut from.
struct Store {
    float*   ptr = nullptr;
    uint64_t n_floats = 0;
    uint64_t cap_bytes = 0;
    uint32_t refs = 0;
    uint32_t generation = 0;   // bumped on release so stale handles are detected
    // A fill that has not been launched yet: floats [0, fill_n) are to hold fill_value (0 = nothing owed).
    // kth_fill over a store's head and the upload of one value leave this note instead of a kernel;
    // `settle` launches the fill, `lookup` settles before it returns, and the few callers that can fold the
    // constant into their own kernel (a binary op takes it as a scalar operand, a scatter starts its rows from it,
    // a broadcast passes it on) take the store with `lookup_unsettled` and clear or keep the note themselves.
    uint64_t fill_n = 0;
    float    fill_value = 0.0f;
    // Set when an indexed move has checked floats [0, index_valid_n) of this store as index values and found every
    // one inside [0, index_valid_below), or when ARG_MAX / ARG_MIN wrote them: the next indexed move with an axis at
    // least that long skips the check and its wait for the stream. Every lookup other than `lookup_index` and those
    // whose caller only reads the store clears it, so anything that could have changed the store's contents makes the
    // next use check again.
    uint32_t index_valid_below = 0;
    uint64_t index_valid_n = 0;
    // A copy that has not been made yet (copy on write). alias_of != 0: this store's n_floats values are those of the
    // store in table slot alias_of - 1 (the source, which holds at least as many); `ptr` points at the source's memory,
    // `own_ptr` keeps this store's own buffer, which nothing has touched. Whoever only reads the store reads through
    // `ptr` and needs to know nothing. Before either side is written the copy is made (`break_aliases`, which every
    // lookup does unless its caller says that it only reads); when the source is released first, a store that
    // aliases it takes over its buffer. `dependents` counts the stores that alias this one. A whole-store kth_copy and
    // pow with the exponent 1 (the backward pass of a square) create aliases instead of copies.
    uint32_t alias_of = 0;
    float*   own_ptr = nullptr;
    uint32_t dependents = 0;
    // A small axis SUM / MEAN that has not been launched yet: this store's first outer * inner values are owed the
    // reduction of the store in table slot owed.src - 1 seen as [outer, axis, inner]. The step of a reduce-to-shape
    // chain that follows (the same outer index, over what was the inner dim) is then one launch over the source instead
    // of two, and an intermediate nobody else reads is never computed. The note holds the source (`holds`: the source's
    // buffer outlives its handle's last release if need be; the handle itself is invalid from then on) and counts among
    // its `dependents`:
    // a write to the source launches the reduction first, like a copy that was put off. Whoever needs this store's
    // values gets them through `lookup`, which launches the reduction unless its caller asks for the note itself.
    struct OwedReduce { uint32_t src = 0; int op = 0; uint32_t outer = 0, axis = 0, inner = 0; } owed;
    uint32_t holds = 0;        // notes on other stores that need this one's values: it is freed when refs and holds are both 0
};

// The index operand of the indexed move that is about to be launched (set by its entry point, taken by the check).
struct IndexUse {
    Store*   store = nullptr;
    uint32_t axis_len = 0;
    uint64_t n = 0;
};

// One profiled launch: which kernel, the algorithmic bytes it moved, and the event pair that the launch itself
// carries (hipExtLaunchKernel's start and stop events: the dispatch's own begin and end, no marker of its own on
// the stream).
struct LaunchRecord {
    const char* family;
    const char* op;
    uint64_t    bytes;
    hipEvent_t  begin, end;
};

// The launch bracket that is open (LaunchScope): the kernels launched inside it are recorded under its name.
struct OpenScope {
    bool        active = false;
    const char* family = nullptr;
    const char* op = nullptr;
    uint64_t    bytes = 0;          // counted for the first launch of the scope
};

struct State {
    bool        ready = false;
    int         device = -1;
    hipStream_t stream = nullptr;
    hipEvent_t  ev_begin = nullptr, ev_end = nullptr;
    bool        timer_open = false;

    char     name[256] = {0};
    uint64_t total_mem = 0;
    int      compute_units = 0;
    int      wave_size = 0;

    float  epsilon = 1e-7f;
    double mem_hint = 0.85;
    int    math_mode = KTH_MATH_WITHIN_2_ULP;   // kth_set_math_mode

    std::vector<Store>    table;       // handle index -> store
    std::vector<uint32_t> free_slots;
    std::map<uint64_t, std::vector<float*>> pool;   // size class (bytes) -> idle buffers

    uint64_t live_bytes = 0, pool_bytes = 0, launches = 0, bytes_moved = 0;

    // Pinned staging slots for asynchronous small uploads; slot i may be refilled once
    // stage_done[i] has completed.
    static constexpr int kStageSlots = 8;
    static constexpr uint64_t kStageBytes = 1ull << 20;
    char*      stage[kStageSlots] = {nullptr};
    hipEvent_t stage_done[kStageSlots] = {nullptr};
    bool       stage_used[kStageSlots] = {false};
    int        stage_next = 0;

    // Out-of-range index values of the indexed moves: with index_check_immediate every such op waits for its own
    // flag; otherwise the kernels set this persistent device word and the next blocking call reports it.
    bool index_check_immediate = true;
    int* deferred_index_flag = nullptr;
    // immediate checking: a word of pinned host memory that the kernels write directly (and its device address),
    // so that the check costs one wait for the stream and neither a clearing kernel nor a copy back
    volatile int* host_index_flag = nullptr;
    int*          host_index_flag_device = nullptr;
    IndexUse      index_use;

    std::vector<hipEvent_t> laps;           // kth_timer_lap events not yet read by kth_timer_laps

    bool profiling = false;
    OpenScope scope;
    std::vector<LaunchRecord> records;      // launches of the current / last profile
    std::vector<hipEvent_t>   event_pool;   // idle events, reused across profiles
};

State&      state();
std::mutex& lock();

// Records the message for kth_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);

// Handle -> store, or nullptr (with the error recorded). A fill the store is owed is launched first. Copies that were
// put off (Store::alias_of) are made first on both sides, the store's own and those of the stores that alias it,
// unless `only_reads` says that the caller will not write the store's memory: it then reads through `ptr` as ever.
// A caller that passes only_reads takes `ptr` of its stores after all its lookups (a later lookup may move it).
Store* lookup(uint64_t handle, const char* what, bool only_reads = false);
// The same without launching an owed fill: for callers that fold, overwrite or drop it. `no_values`: the caller reads
// no values either (it counts references, or takes an owed reduction as a note): a reduction the store is owed stays owed.
Store* lookup_unsettled(uint64_t handle, const char* what, bool only_reads = false, bool no_values = false);
// Launches what `st` put off: the copy of its source, or the reduction it is owed.
void materialize(Store* st);
// `out` (looked up for writing; no notes left on it) is owed the SUM / MEAN `op` of `in` seen as [outer, axis, inner].
void owe_reduce(Store* out, Store* in, int op, uint32_t outer, uint32_t axis, uint32_t inner);
// The reduction itself, on the library's stream (kth_reduce.hip): out = op over the axis of in[outer, axis, inner].
int run_owed_reduce(int op, const float* in, float* out, uint32_t outer, uint32_t axis, uint32_t inner);
// Makes the copies that were put off around `st`: its own, if it aliases another store, and those of its dependents.
void break_aliases(Store* st);
// dst (no alias, no dependents, no owed fill: looked up for writing, and about to be overwritten whole) becomes a copy
// of the first dst->n_floats values of src without a kernel. src holds at least as many values and is owed no fill.
void make_alias(Store* dst, Store* src);
// `lookup` for the index operand of an indexed move, which is only read: keeps the store's record of having been
// checked as an index.
Store* lookup_index(uint64_t handle, const char* what);
// Launches the fill the store is owed, if any, on the library's stream.
void settle(Store* st);
// The store is about to be written over floats [0, n) by a kernel that reads none of them: an owed
// fill that this covers is dropped, a longer one is launched first.
void settle_for_overwrite(Store* st, uint64_t n);
// fill_kernel over p[0, n) on the library's stream (kth_elementwise.hip).
void launch_fill(float* p, uint64_t n, float value);

// Pool-backed raw device memory for kernels' own workspaces (partials of two-pass
// reductions). Stream-ordered: a workspace returned to the pool may be reused by a
// later launch because every launch is on the one in-order stream.
float* workspace_acquire(uint64_t bytes, uint64_t* cap_bytes);
void   workspace_release(float* p, uint64_t cap_bytes);

// The ascending positions i in [0, n) with flags[i] != 0 and their number, on `stream` (kth_sort.hip).
// With temp == nullptr only *temp_bytes is set, to the scratch size needed.
hipError_t select_flagged_positions(void* temp, size_t* temp_bytes, const uint8_t* flags, uint32_t* positions, uint32_t* count,
                                    uint32_t n, hipStream_t stream);

// out = in with its dims reordered: out dim d is in dim axes[d] (kth_layout.hip). Device pointers
// to dense tensors of the same, non-zero element count; `axes` names every dim once.
int permute_device(const char* what, const float* in, float* out, const int32_t* shape, int dims, const int32_t* axes);

// Stable sort of n (key, value) pairs by the low `end_bit` bits of the key, on `stream`
// (kth_sort.hip). With temp == nullptr only *temp_bytes is set, to the scratch size needed.
hipError_t sort_pairs_u32(void* temp, size_t* temp_bytes, const uint32_t* keys_in, uint32_t* keys_out,
                          const uint32_t* vals_in, uint32_t* vals_out, uint32_t n, int end_bit, hipStream_t stream);

// Resolves the device address of the static scratch array of kth_reduce_axis_static for
// `device`, which must be the current device (kth_reduce.hip). Called once from kth_init.
hipError_t reduce_scratch_init(int device);

// In deferred index checking: reads and clears the persistent flag (the stream must be drained) and returns
// KTH_E_ARGUMENT if an indexed move since the last report met an index outside its axis, KTH_OK otherwise.
int report_deferred_index_error();

// Computes the exp / log tables on the host (extended precision) and copies them into the
// device symbols of the elementwise kernels. Called once from kth_init.
hipError_t init_math_tables();

// Brackets the launches of one entry point's kernel: counts it for kth_metrics and, while a profile is
// being recorded, names the launches inside it, each of which then carries its own start and stop events
// (events_for_launch; they are created on demand, and may_profile = false leaves them out for callers that
// must not create anything).
class LaunchScope {
public:
    LaunchScope(const char* family, const char* op, uint64_t algorithmic_bytes, bool may_profile = true);
    ~LaunchScope();
    LaunchScope(const LaunchScope&) = delete;
    LaunchScope& operator=(const LaunchScope&) = delete;
};

// The event pair for the kernel that is about to be launched, or two nulls: inside an open LaunchScope of a profile
// that is being recorded, a new record under the scope's name (kth_runtime.hip).
void events_for_launch(hipEvent_t* begin, hipEvent_t* end);

// Every kernel of the library is launched through this (the macro below puts it in hipLaunchKernelGGL's place): the
// arguments are converted to the kernel's parameter types and handed to hipExtLaunchKernel, with the event pair of
// a running profile as the launch's own start and stop events. Outside a profile it is a plain launch.
template <class... P, class... A, size_t... I>
inline void launch_kernel_impl(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                               std::index_sequence<I...>, A&&... args) {
    std::tuple<P...> params{static_cast<P>(std::forward<A>(args))...};
    void* ptrs[sizeof...(P) > 0 ? sizeof...(P) : 1] = {static_cast<void*>(&std::get<I>(params))...};
    hipEvent_t begin = nullptr, end = nullptr;
    events_for_launch(&begin, &end);
    (void)hipExtLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds, stream, begin, end, 0);
}
template <class... P, class... A>
inline void launch_kernel(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t stream, A&&... args) {
    static_assert(sizeof...(P) == sizeof...(A), "kernel launched with the wrong number of arguments");
    launch_kernel_impl(kernel, grid, block, lds, stream, std::index_sequence_for<P...>{}, std::forward<A>(args)...);
}

#define KTH_REQUIRE_INIT()                                                         \
    do {                                                                           \
        if (!kth::state().ready) return kth::fail(KTH_E_NOT_INIT, "kth_init has not been called"); \
    } while (0)

#define KTH_HIP(call)                                                              \
    do {                                                                           \
        hipError_t e__ = (call);                                                   \
        if (e__ != hipSuccess)                                                     \
            return kth::fail(KTH_E_DEVICE, "%s failed: %s", #call, hipGetErrorString(e__)); \
    } while (0)

// After a kernel launch: surface launch-configuration errors immediately.
#define KTH_LAUNCH_CHECK(name)                                                     \
    do {                                                                           \
        hipError_t e__ = hipGetLastError();                                        \
        if (e__ != hipSuccess)                                                     \
            return kth::fail(KTH_E_DEVICE, "launch of %s failed: %s", name, hipGetErrorString(e__)); \
    } while (0)

constexpr uint64_t kMaxElements = 0x7fffffffull;   // store size is a Kotlin Int

}  // namespace kth

#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
    kth::launch_kernel(kernel, grid, block, lds, stream, __VA_ARGS__)
