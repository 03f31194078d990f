// Platform bring-up, the store table, the reuse pool, host<->device transfers.
#include "kth_internal.h"

#include <cstring>

namespace kth {

State& state() { static State s; return s; }
std::mutex& lock() { static std::mutex m; return m; }

static thread_local char tl_error[512] = {0};

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(tl_error, sizeof(tl_error), fmt, ap);
    va_end(ap);
    return code;
}

// Counts kth_init calls that brought the library up. A new table slot starts its generation at
// epoch << 20, so a handle from before a kth_shutdown does not validate against the stores of a
// later session (unless a slot saw a million releases).
static uint32_t g_epoch = 0;

static inline uint64_t make_handle(uint32_t index, uint32_t generation) {
    return (static_cast<uint64_t>(generation) << 32) | static_cast<uint64_t>(index + 1);
}

static void launch_store_copy(const float* src, float* dst, uint64_t n);

static void free_store(Store* st);

// A note (an owed reduction) no longer needs `st`: a store whose handle was released in the meantime is freed now.
static void drop_hold(Store* st) {
    st->holds -= 1;
    if (st->refs == 0 && st->holds == 0) free_store(st);
}

// What `d` put off is done now, on the library's stream, ahead of whatever is launched next: d's own buffer receives
// the copy of its source's values, or the reduction it is owed.
void materialize(Store* d) {
    State& s = state();
    if (d->alias_of != 0) {
        Store& src = s.table[d->alias_of - 1];
        d->ptr = d->own_ptr; d->own_ptr = nullptr; d->alias_of = 0;
        src.dependents -= 1;
        launch_store_copy(src.ptr, d->ptr, d->n_floats);
    } else if (d->owed.src != 0) {
        Store& src = s.table[d->owed.src - 1];
        const Store::OwedReduce o = d->owed;
        d->owed = Store::OwedReduce{};
        src.dependents -= 1;
        (void)run_owed_reduce(o.op, src.ptr, d->ptr, o.outer, o.axis, o.inner);
        drop_hold(&src);
    }
}

void owe_reduce(Store* out, Store* in, int op, uint32_t outer, uint32_t axis, uint32_t inner) {
    State& s = state();
    out->owed.src = static_cast<uint32_t>(in - s.table.data()) + 1;
    out->owed.op = op; out->owed.outer = outer; out->owed.axis = axis; out->owed.inner = inner;
    in->dependents += 1;
    in->holds += 1;
}

void break_aliases(Store* st) {
    State& s = state();
    if (st->alias_of != 0 || st->owed.src != 0) materialize(st);
    if (st->dependents != 0) {
        const uint32_t me = static_cast<uint32_t>(st - s.table.data()) + 1;
        for (Store& d : s.table)
            if ((d.refs > 0 || d.holds > 0) && (d.alias_of == me || d.owed.src == me)) materialize(&d);
    }
}

// The last reference to `st` is gone: its notes are dropped, the stores that alias it are served, its buffer goes back
// to the pool and its table slot is free for the next kth_alloc (a later generation).
static void free_store(Store* st) {
    State& s = state();
    if (st->alias_of != 0) {
        s.table[st->alias_of - 1].dependents -= 1;
        st->ptr = st->own_ptr; st->own_ptr = nullptr; st->alias_of = 0;
    }
    if (st->owed.src != 0) {
        Store& src = s.table[st->owed.src - 1];
        st->owed = Store::OwedReduce{};
        src.dependents -= 1;
        drop_hold(&src);
    }
    if (st->dependents != 0) {
        // The stores that alias this one need its values: the first whose own buffer is of this one's size class
        // takes this buffer over and gives its untouched one back in its place; the others get their copies now.
        // (A store that is owed a reduction of this one holds a reference to it: none is left when the last goes.)
        const uint32_t me = static_cast<uint32_t>(st - s.table.data()) + 1;
        Store* heir = nullptr;
        for (Store& d : s.table) {
            if ((d.refs == 0 && d.holds == 0) || d.alias_of != me) continue;
            if (!heir && d.cap_bytes == st->cap_bytes) heir = &d;
            else materialize(&d);
        }
        if (heir) {
            float* values = st->ptr;
            st->ptr = heir->own_ptr;
            heir->ptr = values; heir->own_ptr = nullptr; heir->alias_of = 0;
            st->dependents -= 1;
        }
    }
    s.pool[st->cap_bytes].push_back(st->ptr);
    s.live_bytes -= st->cap_bytes;
    s.pool_bytes += st->cap_bytes;
    st->ptr = nullptr;
    st->fill_n = 0;
    st->generation += 1;
    s.free_slots.push_back(static_cast<uint32_t>(st - s.table.data()));
}

void make_alias(Store* dst, Store* src) {
    State& s = state();
    if (src->alias_of != 0) src = &s.table[src->alias_of - 1];      // an alias of an alias is an alias of its source
    dst->own_ptr = dst->ptr;
    dst->ptr = src->ptr;
    dst->alias_of = static_cast<uint32_t>(src - s.table.data()) + 1;
    src->dependents += 1;
    // the same values: what is known of the source as an index tensor holds for the copy
    dst->index_valid_below = src->index_valid_below;
    dst->index_valid_n = src->index_valid_n < dst->n_floats ? src->index_valid_n : dst->n_floats;
}

Store* lookup_unsettled(uint64_t handle, const char* what, bool only_reads, bool no_values) {
    State& s = state();
    uint32_t low = static_cast<uint32_t>(handle & 0xffffffffu);
    uint32_t gen = static_cast<uint32_t>(handle >> 32);
    if (low == 0 || low > s.table.size()) {
        fail(KTH_E_HANDLE, "%s: unknown handle 0x%llx", what, (unsigned long long)handle);
        return nullptr;
    }
    Store& st = s.table[low - 1];
    if (st.refs == 0 || st.generation != gen) {
        fail(KTH_E_HANDLE, "%s: handle 0x%llx was released", what, (unsigned long long)handle);
        return nullptr;
    }
    if (!only_reads) {
        st.index_valid_below = 0;      // whoever takes the store may write it: its values are unknown again
        st.index_valid_n = 0;
        if (st.alias_of != 0 || st.dependents != 0 || st.owed.src != 0) break_aliases(&st);
    } else if (!no_values && st.owed.src != 0) {
        materialize(&st);              // a reader needs the values
    }
    return &st;
}

void settle(Store* st) {
    if (st->fill_n == 0) return;
    const uint64_t n = st->fill_n;
    st->fill_n = 0;
    launch_fill(st->ptr, n, st->fill_value);
}

void settle_for_overwrite(Store* st, uint64_t n) {
    if (st->fill_n <= n) st->fill_n = 0;
    else settle(st);
}

Store* lookup(uint64_t handle, const char* what, bool only_reads) {
    Store* st = lookup_unsettled(handle, what, only_reads);
    if (st) settle(st);
    return st;
}

Store* lookup_index(uint64_t handle, const char* what) {
    // the index operand is only read: the store keeps what is known of it, and a copy it has put off stays put off
    return lookup(handle, what, true);
}

// Size classes: 512-byte granules up to 1 MiB, then 1/8-octave steps (at most 12.5 %
// slack), so the differently-sized tensors of one graph reuse each other's buffers.
static uint64_t size_class(uint64_t bytes) {
    if (bytes == 0) bytes = 4;
    if (bytes <= (1ull << 20)) return (bytes + 511) & ~511ull;
    int top = 63 - __builtin_clzll(bytes);
    uint64_t step = 1ull << (top - 3);
    return (bytes + step - 1) & ~(step - 1);
}

static void trim_pool() {
    State& s = state();
    for (auto& kv : s.pool) {
        for (float* p : kv.second) {
            (void)hipFree(p);
            s.pool_bytes -= kv.first;
        }
        kv.second.clear();
    }
    s.pool.clear();
}

static float* pool_take(uint64_t cap) {
    State& s = state();
    auto it = s.pool.find(cap);
    if (it != s.pool.end() && !it->second.empty()) {
        float* p = it->second.back();
        it->second.pop_back();
        s.pool_bytes -= cap;
        return p;
    }
    uint64_t budget = static_cast<uint64_t>(s.mem_hint * static_cast<double>(s.total_mem));
    if (s.live_bytes + s.pool_bytes + cap > budget) {
        // Freeing must not race with kernels still using pooled buffers' old contents.
        (void)hipStreamSynchronize(s.stream);
        trim_pool();
        if (s.live_bytes + cap > budget) return nullptr;
    }
    void* p = nullptr;
    if (hipMalloc(&p, cap) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipStreamSynchronize(s.stream);
        trim_pool();
        if (hipMalloc(&p, cap) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
    }
    return static_cast<float*>(p);
}

float* workspace_acquire(uint64_t bytes, uint64_t* cap_bytes) {
    uint64_t cap = size_class(bytes);
    float* p = pool_take(cap);
    if (p) { *cap_bytes = cap; state().live_bytes += cap; }
    return p;
}

void workspace_release(float* p, uint64_t cap_bytes) {
    State& s = state();
    s.pool[cap_bytes].push_back(p);
    s.live_bytes -= cap_bytes;
    s.pool_bytes += cap_bytes;
}

constexpr int kConstFloats = 16;
struct ConstFloats { float v[kConstFloats]; };

__global__ void store_consts_kernel(float* dst, int n, ConstFloats c) {
    if (static_cast<int>(threadIdx.x) < n) dst[threadIdx.x] = c.v[threadIdx.x];
}

static hipEvent_t take_event() {
    State& s = state();
    if (!s.event_pool.empty()) { hipEvent_t e = s.event_pool.back(); s.event_pool.pop_back(); return e; }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    return e;
}

LaunchScope::LaunchScope(const char* family, const char* op, uint64_t algorithmic_bytes, bool may_profile) {
    State& s = state();
    s.launches += 1;
    s.bytes_moved += algorithmic_bytes;
    if (!s.profiling || !may_profile) return;
    s.scope.active = true; s.scope.family = family; s.scope.op = op; s.scope.bytes = algorithmic_bytes;
}

void events_for_launch(hipEvent_t* begin, hipEvent_t* end) {
    State& s = state();
    *begin = nullptr; *end = nullptr;
    if (!s.profiling || !s.scope.active) return;
    LaunchRecord r{s.scope.family, s.scope.op, s.scope.bytes, take_event(), take_event()};
    if (!r.begin || !r.end) {
        if (r.begin) s.event_pool.push_back(r.begin);
        if (r.end) s.event_pool.push_back(r.end);
        return;
    }
    s.scope.bytes = 0;                       // a scope's bytes are those of all its launches together
    s.records.push_back(r);
    *begin = r.begin; *end = r.end;
}

int report_deferred_index_error() {
    State& s = state();
    if (s.index_check_immediate || !s.deferred_index_flag) return KTH_OK;
    int host_flag = 0;
    KTH_HIP(hipMemcpyAsync(&host_flag, s.deferred_index_flag, 4, hipMemcpyDeviceToHost, s.stream));
    KTH_HIP(hipStreamSynchronize(s.stream));
    if (!host_flag) return KTH_OK;
    KTH_HIP(hipMemsetAsync(s.deferred_index_flag, 0, 4, s.stream));
    return fail(KTH_E_ARGUMENT, "an indexed move since the last blocking call got an invalid index, an index value is out of "
                                "bounds at the axis (its target was updated up to that entry)");
}

LaunchScope::~LaunchScope() { state().scope.active = false; }

}  // namespace kth

using namespace kth;

extern "C" {

const char* kth_last_error(void) { return tl_error; }

// Frees everything kth_init and the calls after it created and leaves a fresh State. Shared by kth_shutdown and
// by a kth_init that fails part-way, so that a second kth_init starts from nothing and leaks nothing.
static void teardown() {
    State& s = state();
    if (s.stream) (void)hipStreamSynchronize(s.stream);
    for (Store& st : s.table) {
        float* mine = st.alias_of != 0 ? st.own_ptr : st.ptr;       // an aliasing store's `ptr` is its source's buffer
        if ((st.refs > 0 || st.holds > 0) && mine) (void)hipFree(mine);
    }
    s.table.clear();
    s.free_slots.clear();
    trim_pool();
    if (s.deferred_index_flag) (void)hipFree(s.deferred_index_flag);
    if (s.host_index_flag) (void)hipHostFree(const_cast<int*>(s.host_index_flag));
    s.host_index_flag = nullptr; s.host_index_flag_device = nullptr;
    for (LaunchRecord& r : s.records) { (void)hipEventDestroy(r.begin); (void)hipEventDestroy(r.end); }
    for (hipEvent_t e : s.event_pool) (void)hipEventDestroy(e);
    for (hipEvent_t e : s.laps) (void)hipEventDestroy(e);
    for (int i = 0; i < State::kStageSlots; i++) {
        if (s.stage[i]) (void)hipHostFree(s.stage[i]);
        if (s.stage_done[i]) (void)hipEventDestroy(s.stage_done[i]);
    }
    if (s.ev_begin) (void)hipEventDestroy(s.ev_begin);
    if (s.ev_end) (void)hipEventDestroy(s.ev_end);
    if (s.stream) (void)hipStreamDestroy(s.stream);
    s = State();
}

// The fallible part of kth_init after the device was chosen; on any failure the caller tears down.
static int bring_up(int device) {
    State& s = state();
    KTH_HIP(hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking));
    KTH_HIP(hipEventCreate(&s.ev_begin));
    KTH_HIP(hipEventCreate(&s.ev_end));
    KTH_HIP(init_math_tables());
    KTH_HIP(reduce_scratch_init(device));
    KTH_HIP(hipMalloc(reinterpret_cast<void**>(&s.deferred_index_flag), 256));
    KTH_HIP(hipMemset(s.deferred_index_flag, 0, 256));
    void* host = nullptr; void* dev = nullptr;
    KTH_HIP(hipHostMalloc(&host, 256, hipHostMallocDefault));
    s.host_index_flag = static_cast<volatile int*>(host);
    KTH_HIP(hipHostGetDevicePointer(&dev, host, 0));
    s.host_index_flag_device = static_cast<int*>(dev);
    *s.host_index_flag = 0;
    return KTH_OK;
}

int kth_init(int device) {
    std::lock_guard<std::mutex> g(lock());
    State& s = state();
    if (s.ready) {
        if (s.device == device) return KTH_OK;
        return fail(KTH_E_ARGUMENT, "already initialised on device %d", s.device);
    }
    int count = 0;
    KTH_HIP(hipGetDeviceCount(&count));
    if (device < 0 || device >= count)
        return fail(KTH_E_ARGUMENT, "device %d out of range (%d visible)", device, count);
    KTH_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    KTH_HIP(hipGetDeviceProperties(&prop, device));
    snprintf(s.name, sizeof(s.name), "%s (%s)", prop.name, prop.gcnArchName);
    s.total_mem = prop.totalGlobalMem;
    s.compute_units = prop.multiProcessorCount;
    s.wave_size = prop.warpSize;
    if (s.wave_size != 64)
        return fail(KTH_E_DEVICE, "kernels are written for wave64; device reports wave %d", s.wave_size);
    if (int rc = bring_up(device)) {
        teardown();                      // keeps the message `fail` recorded; the next kth_init starts clean
        return rc;
    }
    s.device = device;
    s.ready = true;
    g_epoch += 1;
    return KTH_OK;
}

int kth_shutdown(void) {
    std::lock_guard<std::mutex> g(lock());
    if (!state().ready) return KTH_OK;
    teardown();
    return KTH_OK;
}

int kth_device_info(char* name, size_t cap, uint64_t* total_mem, int* compute_units, int* wave_size) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    if (name && cap > 0) { strncpy(name, s.name, cap - 1); name[cap - 1] = 0; }
    if (total_mem) *total_mem = s.total_mem;
    if (compute_units) *compute_units = s.compute_units;
    if (wave_size) *wave_size = s.wave_size;
    return KTH_OK;
}

int kth_set_epsilon(float eps) {
    std::lock_guard<std::mutex> g(lock());
    state().epsilon = eps;
    return KTH_OK;
}

int kth_set_memory_scale_hint(double fraction) {
    std::lock_guard<std::mutex> g(lock());
    if (!(fraction > 0.0 && fraction <= 1.0))
        return fail(KTH_E_ARGUMENT, "memory scale hint %g outside (0, 1]", fraction);
    state().mem_hint = fraction;
    return KTH_OK;
}

int kth_alloc(uint64_t n_floats, uint64_t* handle) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!handle) return fail(KTH_E_ARGUMENT, "kth_alloc: null handle pointer");
    if (n_floats > kMaxElements)
        return fail(KTH_E_ARGUMENT, "kth_alloc: %llu elements exceed the 2^31-1 store limit",
                    (unsigned long long)n_floats);
    State& s = state();
    uint64_t cap = size_class(n_floats * 4);
    float* p = pool_take(cap);
    if (!p)
        return fail(KTH_E_MEMORY, "kth_alloc: cannot allocate %llu bytes (live %llu, hint %.2f of %llu)",
                    (unsigned long long)cap, (unsigned long long)s.live_bytes, s.mem_hint,
                    (unsigned long long)s.total_mem);
    uint32_t idx;
    if (!s.free_slots.empty()) { idx = s.free_slots.back(); s.free_slots.pop_back(); }
    else { idx = static_cast<uint32_t>(s.table.size()); s.table.emplace_back(); s.table.back().generation = g_epoch << 20; }
    Store& st = s.table[idx];
    st.ptr = p; st.n_floats = n_floats; st.cap_bytes = cap; st.refs = 1; st.fill_n = 0; st.index_valid_below = 0; st.index_valid_n = 0;
    st.alias_of = 0; st.own_ptr = nullptr; st.dependents = 0; st.owed = Store::OwedReduce{}; st.holds = 0;
    s.live_bytes += cap;
    *handle = make_handle(idx, st.generation);
    return KTH_OK;
}

int kth_retain(uint64_t handle) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    Store* st = lookup_unsettled(handle, "kth_retain", true, true);
    if (!st) return KTH_E_HANDLE;
    st->refs += 1;
    return KTH_OK;
}

int kth_release(uint64_t handle) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    // (a fill nobody read is never launched, a copy nobody read never made, a reduction nobody read never run)
    Store* st = lookup_unsettled(handle, "kth_release", true, true);
    if (!st) return KTH_E_HANDLE;
    st->refs -= 1;
    if (st->refs == 0) {
        // The handle is invalid from here on. A store that notes on other stores still hold keeps its values until
        // they are done with it.
        if (st->holds == 0) free_store(st);
        else if (st->alias_of != 0 || st->owed.src != 0) materialize(st);      // (a held store has its values; to be safe)
    }
    return KTH_OK;
}

static int check_range(const Store* st, uint64_t off, uint64_t n, const char* what) {
    if (off > st->n_floats || n > st->n_floats - off)
        return fail(KTH_E_ARGUMENT, "%s: range [%llu, +%llu) outside a store of %llu floats", what,
                    (unsigned long long)off, (unsigned long long)n, (unsigned long long)st->n_floats);
    return KTH_OK;
}

int kth_upload(uint64_t handle, uint64_t offset, const float* src, uint64_t n) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    Store* st = lookup_unsettled(handle, "kth_upload");
    if (!st) return KTH_E_HANDLE;
    if (int rc = check_range(st, offset, n, "kth_upload")) return rc;
    if (n == 0) return KTH_OK;
    if (!src) return fail(KTH_E_ARGUMENT, "kth_upload: null source");
    State& s = state();
    if (offset == 0) settle_for_overwrite(st, n); else settle(st);
    if (n == 1 && offset == 0) {
        // One value (a [1]-shaped seed gradient, a scalar operand) is a fill of one float: noted, and
        // launched only if somebody reads the store as memory.
        st->fill_n = 1; st->fill_value = src[0];
        return KTH_OK;
    }
    if (n <= kConstFloats) {
        // A few values (a [1]-shaped seed gradient, a scalar operand): they ride in the
        // kernel arguments, so nothing blocks and no staging memory is involved.
        ConstFloats c;
        for (uint64_t i = 0; i < n; i++) c.v[i] = src[i];
        LaunchScope scope("store_consts_kernel", "", n * 4);
        hipLaunchKernelGGL(store_consts_kernel, dim3(1), dim3(kConstFloats), 0, s.stream, st->ptr + offset, static_cast<int>(n), c);
        KTH_LAUNCH_CHECK("store_consts");
        return KTH_OK;
    }
    if (n * 4 <= State::kStageBytes) {
        // Small uploads go through a pinned slot and return as soon as the copy is enqueued.
        const int slot = s.stage_next;
        s.stage_next = (slot + 1) % State::kStageSlots;
        if (!s.stage[slot]) {
            KTH_HIP(hipHostMalloc(reinterpret_cast<void**>(&s.stage[slot]), State::kStageBytes, hipHostMallocDefault));
            KTH_HIP(hipEventCreateWithFlags(&s.stage_done[slot], hipEventDisableTiming));
        }
        if (s.stage_used[slot]) KTH_HIP(hipEventSynchronize(s.stage_done[slot]));
        memcpy(s.stage[slot], src, n * 4);
        KTH_HIP(hipMemcpyAsync(st->ptr + offset, s.stage[slot], n * 4, hipMemcpyHostToDevice, s.stream));
        KTH_HIP(hipEventRecord(s.stage_done[slot], s.stream));
        s.stage_used[slot] = true;
        return KTH_OK;
    }
    KTH_HIP(hipMemcpyAsync(st->ptr + offset, src, n * 4, hipMemcpyHostToDevice, s.stream));
    KTH_HIP(hipStreamSynchronize(s.stream));
    return KTH_OK;
}

int kth_download(float* dst, uint64_t handle, uint64_t offset, uint64_t n) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    Store* st = lookup(handle, "kth_download", true);
    if (!st) return KTH_E_HANDLE;
    if (int rc = check_range(st, offset, n, "kth_download")) return rc;
    if (n != 0 && !dst) return fail(KTH_E_ARGUMENT, "kth_download: null destination");
    State& s = state();
    if (n != 0) KTH_HIP(hipMemcpyAsync(dst, st->ptr + offset, n * 4, hipMemcpyDeviceToHost, s.stream));
    KTH_HIP(hipStreamSynchronize(s.stream));
    // A pending out-of-range index of deferred checking is reported here, once; dst has been filled all the same.
    return report_deferred_index_error();
}

int kth_read_scalar(uint64_t handle, uint64_t index, float* out) {
    if (!out) return fail(KTH_E_ARGUMENT, "kth_read_scalar: null output");
    return kth_download(out, handle, index, 1);
}

namespace {

typedef float copy_v4f __attribute__((ext_vector_type(4)));

// Store-to-store copy of n floats between 16-byte aligned addresses: one float4 per thread,
// non-temporal load, ordinary store (the copy stays in the memory-side cache for the kernel
// that reads it next); the last n % 4 floats are moved by workgroup 0.
__global__ __launch_bounds__(256) void copy_kernel(const float* __restrict__ src, float* __restrict__ dst, uint32_t n) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const uint32_t n4 = n >> 2;
    if (i < n4) reinterpret_cast<copy_v4f*>(dst)[i] = __builtin_nontemporal_load(reinterpret_cast<const copy_v4f*>(src) + i);
    if (blockIdx.x == 0 && threadIdx.x < (n & 3u)) dst[(n4 << 2) + threadIdx.x] = src[(n4 << 2) + threadIdx.x];
}

// The same between any two dword addresses: 16-byte accesses on both sides (the hardware takes them
// at any dword address); the destination side is brought to a 16-byte boundary first so that its
// stores are the aligned ones. `head` = floats before that boundary (0 ... 3), moved by workgroup 0
// together with the tail.
typedef float copy_v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));
__global__ __launch_bounds__(256) void copy_any_kernel(const float* __restrict__ src, float* __restrict__ dst, uint32_t n, uint32_t head) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const uint32_t body = (n - head) >> 2;
    if (i < body) {
        const copy_v4f_unaligned v = __builtin_nontemporal_load(reinterpret_cast<const copy_v4f_unaligned*>(src + head) + i);
        reinterpret_cast<copy_v4f*>(dst + head)[i] = copy_v4f{v.x, v.y, v.z, v.w};
    }
    if (blockIdx.x == 0) {
        if (threadIdx.x < head) dst[threadIdx.x] = src[threadIdx.x];
        const uint32_t done = head + (body << 2);
        if (threadIdx.x >= 64 && threadIdx.x - 64 < n - done) dst[done + threadIdx.x - 64] = src[done + threadIdx.x - 64];
    }
}

}  // namespace

extern "C++" {
namespace kth {
static void launch_store_copy(const float* src, float* dst, uint64_t n) {
    if (n == 0) return;
    LaunchScope scope("copy_kernel", "copy on write", n * 8);
    const uint32_t blocks = static_cast<uint32_t>(((n >> 2) + 255) / 256);
    hipLaunchKernelGGL(copy_kernel, dim3(blocks == 0 ? 1 : blocks), dim3(256), 0, state().stream, src, dst, static_cast<uint32_t>(n));
}
}  // namespace kth
}

int kth_copy(uint64_t dst, uint64_t dst_offset, uint64_t src, uint64_t src_offset, uint64_t n) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    Store* d = lookup_unsettled(dst, "kth_copy(dst)");
    if (!d) return KTH_E_HANDLE;
    Store* sst = lookup_unsettled(src, "kth_copy(src)", true);
    if (!sst) return KTH_E_HANDLE;
    if (int rc = check_range(d, dst_offset, n, "kth_copy(dst)")) return rc;
    if (int rc = check_range(sst, src_offset, n, "kth_copy(src)")) return rc;
    if (n == 0) return KTH_OK;
    if (d != sst && dst_offset == 0 && sst->fill_n >= src_offset + n) {
        // a copy of floats that are all one owed constant: the head of the destination is owed it too
        settle_for_overwrite(d, n);
        d->fill_n = n; d->fill_value = sst->fill_value;
        return KTH_OK;
    }
    settle(sst);
    if (d != sst && dst_offset == 0) settle_for_overwrite(d, n); else settle(d);
    if (d != sst && dst_offset == 0 && src_offset == 0 && n == d->n_floats) {
        // the whole destination from the head of the source (copy(shallow = false)): put off until one of the two is written
        make_alias(d, sst);
        return KTH_OK;
    }
    if (d->ptr == sst->ptr) {
        uint64_t lo = dst_offset < src_offset ? dst_offset : src_offset;
        uint64_t hi = dst_offset < src_offset ? src_offset : dst_offset;
        if (hi - lo < n) return fail(KTH_E_ARGUMENT, "kth_copy: overlapping ranges in one store");
    }
    State& s = state();
    if (dst_offset % 4 == 0 && src_offset % 4 == 0 && n <= kMaxElements) {
        LaunchScope scope("copy_kernel", "", n * 8);
        const uint32_t blocks = static_cast<uint32_t>(((n >> 2) + 255) / 256);
        hipLaunchKernelGGL(copy_kernel, dim3(blocks == 0 ? 1 : blocks), dim3(256), 0, s.stream, sst->ptr + src_offset,
                           d->ptr + dst_offset, static_cast<uint32_t>(n));
        KTH_LAUNCH_CHECK("copy_kernel");
        return KTH_OK;
    }
    if (n <= kMaxElements) {
        uint32_t head = static_cast<uint32_t>((4 - dst_offset % 4) % 4);
        if (head > n) head = static_cast<uint32_t>(n);
        LaunchScope scope("copy_kernel", "dword addresses", n * 8);
        const uint32_t blocks = static_cast<uint32_t>((((n - head) >> 2) + 255) / 256);
        hipLaunchKernelGGL(copy_any_kernel, dim3(blocks == 0 ? 1 : blocks), dim3(256), 0, s.stream, sst->ptr + src_offset,
                           d->ptr + dst_offset, static_cast<uint32_t>(n), head);
        KTH_LAUNCH_CHECK("copy_kernel");
        return KTH_OK;
    }
    LaunchScope scope("memcpy_d2d", "", n * 8);
    KTH_HIP(hipMemcpyAsync(d->ptr + dst_offset, sst->ptr + src_offset, n * 4, hipMemcpyDeviceToDevice, s.stream));
    return KTH_OK;
}

int kth_sync(void) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    KTH_HIP(hipStreamSynchronize(state().stream));
    return report_deferred_index_error();
}

int kth_set_index_check(int immediate) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    if (!s.index_check_immediate && immediate) {        // leaving deferred mode: report what is pending first
        KTH_HIP(hipStreamSynchronize(s.stream));
        if (int rc = report_deferred_index_error()) { s.index_check_immediate = true; return rc; }
    }
    s.index_check_immediate = immediate != 0;
    return KTH_OK;
}

int kth_metrics(uint64_t* live_bytes, uint64_t* pool_bytes, uint64_t* launches, uint64_t* bytes_moved) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    if (live_bytes) *live_bytes = s.live_bytes;
    if (pool_bytes) *pool_bytes = s.pool_bytes;
    if (launches) *launches = s.launches;
    if (bytes_moved) *bytes_moved = s.bytes_moved;
    return KTH_OK;
}

int kth_timer_begin(void) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    KTH_HIP(hipEventRecord(s.ev_begin, s.stream));
    s.timer_open = true;
    return KTH_OK;
}

int kth_timer_end(float* milliseconds) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    if (!milliseconds) return fail(KTH_E_ARGUMENT, "kth_timer_end: null output");
    if (!s.timer_open) return fail(KTH_E_ARGUMENT, "kth_timer_end without kth_timer_begin");
    KTH_HIP(hipEventRecord(s.ev_end, s.stream));
    KTH_HIP(hipEventSynchronize(s.ev_end));
    KTH_HIP(hipEventElapsedTime(milliseconds, s.ev_begin, s.ev_end));
    s.timer_open = false;
    return KTH_OK;
}

constexpr size_t kMaxPendingLaps = 1u << 16;       // events held until kth_timer_laps reads them

int kth_timer_lap(void) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    if (s.laps.size() >= kMaxPendingLaps)
        return fail(KTH_E_ARGUMENT, "kth_timer_lap: %zu laps are pending; read them with kth_timer_laps first", s.laps.size());
    hipEvent_t e = take_event();
    if (!e) return fail(KTH_E_DEVICE, "kth_timer_lap: no event");
    KTH_HIP(hipEventRecord(e, s.stream));
    s.laps.push_back(e);
    return KTH_OK;
}

int kth_timer_laps(float* milliseconds, int capacity, int* count, float* total_ms) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    if (!count) return fail(KTH_E_ARGUMENT, "kth_timer_laps: null count");
    const int intervals = s.laps.empty() ? 0 : static_cast<int>(s.laps.size()) - 1;
    *count = intervals;
    if (total_ms) *total_ms = 0.0f;
    int rc = KTH_OK;
    if (!s.laps.empty()) {
        hipError_t e = hipEventSynchronize(s.laps.back());
        if (e != hipSuccess) rc = fail(KTH_E_DEVICE, "kth_timer_laps: %s", hipGetErrorString(e));
        for (int i = 0; rc == KTH_OK && i < intervals && i < capacity && milliseconds; i++) {
            e = hipEventElapsedTime(&milliseconds[i], s.laps[i], s.laps[i + 1]);
            if (e != hipSuccess) rc = fail(KTH_E_DEVICE, "kth_timer_laps: %s", hipGetErrorString(e));
        }
        if (rc == KTH_OK && total_ms && intervals > 0) {
            e = hipEventElapsedTime(total_ms, s.laps.front(), s.laps.back());
            if (e != hipSuccess) rc = fail(KTH_E_DEVICE, "kth_timer_laps: %s", hipGetErrorString(e));
        }
    }
    for (hipEvent_t ev : s.laps) s.event_pool.push_back(ev);
    s.laps.clear();
    return rc;
}

int kth_measure_copy(uint64_t n_floats, int reps, float* memcpy_ms, float* kernel_ms) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (n_floats == 0 || n_floats > kMaxElements || n_floats % 4 != 0 || reps < 1)
        return fail(KTH_E_ARGUMENT, "kth_measure_copy: need a multiple of 4 floats below 2^31 and at least one repetition");
    State& s = state();
    // Its own event pair: the stopwatch's pair may be open around this call.
    hipEvent_t ev0 = take_event(), ev1 = take_event();
    if (!ev0 || !ev1) {
        if (ev0) s.event_pool.push_back(ev0);
        if (ev1) s.event_pool.push_back(ev1);
        return fail(KTH_E_DEVICE, "kth_measure_copy: no event");
    }
    uint64_t cap_a = 0, cap_b = 0;
    float* a = workspace_acquire(n_floats * 4, &cap_a);
    float* b = a ? workspace_acquire(n_floats * 4, &cap_b) : nullptr;
    int rc = KTH_OK;
    if (!a || !b) rc = fail(KTH_E_MEMORY, "kth_measure_copy: no room for two buffers of %llu floats", (unsigned long long)n_floats);
    auto timed = [&](bool kernel, float* out_ms) -> hipError_t {
        const uint32_t n = static_cast<uint32_t>(n_floats);
        const uint32_t blocks = (n / 4 + 255) / 256;
        for (int i = -1; i < reps; i++) {              // one untimed pass first
            if (i == 0) { hipError_t e = hipEventRecord(ev0, s.stream); if (e != hipSuccess) return e; }
            if (kernel) hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, s.stream, a, b, n);
            else { hipError_t e = hipMemcpyAsync(b, a, n_floats * 4, hipMemcpyDeviceToDevice, s.stream); if (e != hipSuccess) return e; }
        }
        hipError_t e = hipEventRecord(ev1, s.stream);
        if (e == hipSuccess) e = hipEventSynchronize(ev1);
        float ms = 0.0f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, ev0, ev1);
        if (out_ms) *out_ms = ms / static_cast<float>(reps);
        return e;
    };
    if (rc == KTH_OK) {
        hipError_t e = hipMemsetAsync(a, 0x3c, n_floats * 4, s.stream);     // finite floats, not zeros
        if (e == hipSuccess) e = timed(false, memcpy_ms);
        if (e == hipSuccess) e = timed(true, kernel_ms);
        if (e != hipSuccess) rc = fail(KTH_E_DEVICE, "kth_measure_copy: %s", hipGetErrorString(e));
    }
    if (b) workspace_release(b, cap_b);
    if (a) workspace_release(a, cap_a);
    s.event_pool.push_back(ev0);
    s.event_pool.push_back(ev1);
    return rc;
}

int kth_profile_begin(void) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    for (LaunchRecord& r : s.records) { s.event_pool.push_back(r.begin); s.event_pool.push_back(r.end); }
    s.records.clear();
    s.profiling = true;
    return KTH_OK;
}

int kth_profile_end(void) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    State& s = state();
    s.profiling = false;
    KTH_HIP(hipStreamSynchronize(s.stream));
    return KTH_OK;
}

// Aggregates the recorded launches by (kernel family, op) in first-seen order.
static int profile_aggregate(std::vector<LaunchRecord>* keys, std::vector<uint64_t>* launches,
                             std::vector<uint64_t>* bytes, std::vector<double>* ms) {
    State& s = state();
    for (const LaunchRecord& r : s.records) {
        size_t k = 0;
        for (; k < keys->size(); k++)
            if (!strcmp((*keys)[k].family, r.family) && !strcmp((*keys)[k].op, r.op)) break;
        if (k == keys->size()) { keys->push_back(r); launches->push_back(0); bytes->push_back(0); ms->push_back(0.0); }
        float t = 0.0f;
        KTH_HIP(hipEventElapsedTime(&t, r.begin, r.end));
        (*launches)[k] += 1; (*bytes)[k] += r.bytes; (*ms)[k] += t;
    }
    return KTH_OK;
}

int kth_profile_count(int* count) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (!count) return fail(KTH_E_ARGUMENT, "kth_profile_count: null output");
    if (state().profiling) return fail(KTH_E_ARGUMENT, "kth_profile_count: a profile is still being recorded");
    std::vector<LaunchRecord> keys; std::vector<uint64_t> l, b; std::vector<double> ms;
    if (int rc = profile_aggregate(&keys, &l, &b, &ms)) return rc;
    *count = static_cast<int>(keys.size());
    return KTH_OK;
}

int kth_profile_entry(int index, char* name, size_t cap, uint64_t* launches, uint64_t* bytes, double* total_ms) {
    std::lock_guard<std::mutex> g(lock());
    KTH_REQUIRE_INIT();
    if (state().profiling) return fail(KTH_E_ARGUMENT, "kth_profile_entry: a profile is still being recorded");
    std::vector<LaunchRecord> keys; std::vector<uint64_t> l, b; std::vector<double> ms;
    if (int rc = profile_aggregate(&keys, &l, &b, &ms)) return rc;
    if (index < 0 || index >= static_cast<int>(keys.size()))
        return fail(KTH_E_ARGUMENT, "kth_profile_entry: index %d of %zu", index, keys.size());
    if (name && cap > 0) {
        if (keys[index].op[0]) snprintf(name, cap, "%s<%s>", keys[index].family, keys[index].op);
        else snprintf(name, cap, "%s", keys[index].family);
    }
    if (launches) *launches = l[index];
    if (bytes) *bytes = b[index];
    if (total_ms) *total_ms = ms[index];
    return KTH_OK;
}

}  // extern "C"
