// Runtime half of the C ABI: init/probe, error text, device buffers, streams and events.
// Mirrors crates/st-backend-hip/src/lib.rs:148-207 (init once, shared by all threads) and the RAII
// wrappers of crates/st-backend-hip/src/real.rs:190-220,649-697, flattened to C handles.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "common.h"
#include "kernels.h"

namespace sthip {

namespace {
thread_local std::string g_last_error;

struct Runtime {
    std::mutex mutex;
    bool ready = false;
    int status = ST_HIP_ERR_NOT_ENABLED;
    std::string error;
    std::vector<hipDeviceProp_t> devices;
};

Runtime &runtime()
{
    static Runtime instance;
    return instance;
}
}  // namespace

int fail(int code, const char *fmt, ...)
{
    char buffer[512];
    va_list args;
    va_start(args, fmt);
    vsnprintf(buffer, sizeof buffer, fmt, args);
    va_end(args);
    g_last_error = buffer;
    return code;
}

int hip_fail(hipError_t rc, const char *ctx)
{
    (void)hipGetLastError();  // clear the sticky flag so the next call starts clean
    return fail(ST_HIP_ERR_RUNTIME, "%s: %s (%d) - %s", ctx, hipGetErrorName(rc), static_cast<int>(rc),
                hipGetErrorString(rc));
}

void clear_error() { g_last_error.clear(); }

int ensure_init()
{
    Runtime &rt = runtime();
    std::lock_guard<std::mutex> lock(rt.mutex);
    if (rt.ready) return ST_HIP_OK;
    int count = 0;
    hipError_t rc = hipGetDeviceCount(&count);
    if (rc != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(ST_HIP_ERR_NOT_ENABLED, "HIP not enabled (no usable HIP device: %s)",
                    rc == hipSuccess ? "device count is 0" : hipGetErrorString(rc));
    }
    std::vector<hipDeviceProp_t> devices(static_cast<size_t>(count));
    for (int i = 0; i < count; ++i) {
        rc = hipGetDeviceProperties(&devices[static_cast<size_t>(i)], i);
        if (rc != hipSuccess) return hip_fail(rc, "hipGetDeviceProperties");
    }
    if (std::strncmp(devices[0].gcnArchName, "gfx950", 6) != 0) {
        return fail(ST_HIP_ERR_NOT_ENABLED,
                    "HIP not enabled (device 0 is %s; this library carries gfx950 code only)",
                    devices[0].gcnArchName);
    }
    // Set-up of the allocation-free entry point: the device address of its static scratch array on the current
    // GPU (other GPUs resolve theirs on their first call with that device current).
    void *scratch_address = nullptr;
    rc = noalloc_scratch(&scratch_address);
    if (rc != hipSuccess) return hip_fail(rc, "hipGetSymbolAddress(scratch)");
    rt.devices.swap(devices);
    rt.ready = true;
    return ST_HIP_OK;
}

namespace {
std::atomic<unsigned long long> g_transfers[4];  // h2d copies, h2d bytes, d2h copies, d2h bytes
}  // namespace

void count_transfer(bool to_device, size_t bytes)
{
    g_transfers[to_device ? 0 : 2].fetch_add(1, std::memory_order_relaxed);
    g_transfers[to_device ? 1 : 3].fetch_add(bytes, std::memory_order_relaxed);
}

namespace {
// Scratch is keyed by (stream, host thread, slot): launches on one stream from one thread are ordered, so they never
// use the buffer at the same time; two host threads that share a stream (every caller that passes none shares the
// NULL stream) each get a buffer of their own, so one thread growing its scratch can never free memory that a
// kernel the other thread has just been handed is about to use.
//
// Lifetime: an entry lives until its stream is destroyed (st_hip_stream_destroy) or st_hip_release_scratch is called
// for the stream.  When its host thread exits, the entry is not freed (kernels of that thread may still be queued) but
// orphaned, and the next thread that asks for scratch on that stream and slot adopts it: work on one stream is
// ordered and the former owner can no longer be between receiving the pointer and launching, so a pool of short-lived
// threads keeps re-using the same few buffers instead of leaking one per thread.
struct WorkspaceEntry {
    hipStream_t stream;
    std::thread::id owner;  // std::thread::id() once the owning thread has exited
    void *ptr;
    size_t capacity;
    int slot;
    bool growing;  // its owner is replacing the buffer outside the lock
};
// Never destroyed: threads may exit (and orphan their entries) while the process is shutting down.
std::mutex &workspace_mutex()
{
    static std::mutex *mutex = new std::mutex;
    return *mutex;
}
std::vector<WorkspaceEntry> &workspace_entries()
{
    static std::vector<WorkspaceEntry> *entries = new std::vector<WorkspaceEntry>;
    return *entries;
}

struct ThreadScratchGuard {
    bool armed = false;
    ~ThreadScratchGuard()
    {
        if (!armed) return;
        const std::thread::id me = std::this_thread::get_id();
        std::lock_guard<std::mutex> lock(workspace_mutex());
        for (WorkspaceEntry &e : workspace_entries())
            if (e.owner == me) e.owner = std::thread::id();
    }
};
thread_local ThreadScratchGuard thread_scratch_guard;

WorkspaceEntry *find_entry(hipStream_t stream, std::thread::id owner, int slot)
{
    for (WorkspaceEntry &e : workspace_entries())
        if (e.stream == stream && e.owner == owner && e.slot == slot) return &e;
    return nullptr;
}
}  // namespace

hipError_t stream_workspace(hipStream_t stream, size_t bytes, void **out) { return stream_workspace_slot(stream, 0, bytes, out); }

hipError_t stream_workspace_slot(hipStream_t stream, int slot, size_t bytes, void **out)
{
    const std::thread::id me = std::this_thread::get_id();
    const size_t wanted = bytes ? bytes : 256;
    void *old = nullptr;
    bool adopted_or_own = false;
    {
        std::lock_guard<std::mutex> lock(workspace_mutex());
        thread_scratch_guard.armed = true;
        WorkspaceEntry *e = find_entry(stream, me, slot);
        if (!e) {
            e = find_entry(stream, std::thread::id(), slot);  // a buffer whose thread has exited
            if (e) e->owner = me;
        }
        if (e) {
            if (e->ptr != nullptr && e->capacity >= wanted) {
                *out = e->ptr;
                return hipSuccess;
            }
            // Grow: outside the lock (the wait for the stream must not stall other threads' launches).  The entry stays
            // in the table, owned by this thread and empty, so nobody else touches it meanwhile.
            old = e->ptr;
            e->ptr = nullptr;
            e->capacity = 0;
            e->growing = true;
            adopted_or_own = true;
        }
    }
    if (adopted_or_own && old) {
        // earlier launches on this stream may still be using the old buffer
        hipError_t rc = hipStreamSynchronize(stream);
        if (rc == hipSuccess) rc = hipFree(old);
        if (rc != hipSuccess) {
            std::lock_guard<std::mutex> lock(workspace_mutex());
            if (WorkspaceEntry *e = find_entry(stream, me, slot)) e->growing = false;
            return rc;
        }
    }
    void *fresh = nullptr;
    const hipError_t rc = hipMalloc(&fresh, wanted);
    std::lock_guard<std::mutex> lock(workspace_mutex());
    WorkspaceEntry *e = find_entry(stream, me, slot);
    if (rc != hipSuccess) {
        if (e) e->growing = false;
        return rc;
    }
    if (e) {
        e->ptr = fresh;
        e->capacity = wanted;
        e->growing = false;
    } else {
        workspace_entries().push_back(WorkspaceEntry{stream, me, fresh, wanted, slot, false});
    }
    *out = fresh;
    return hipSuccess;
}

// Called after the stream has been drained (before it is destroyed, or by st_hip_release_scratch).
void release_stream_workspace(hipStream_t stream)
{
    std::vector<void *> doomed;
    {
        std::lock_guard<std::mutex> lock(workspace_mutex());
        std::vector<WorkspaceEntry> &entries = workspace_entries();
        for (size_t i = entries.size(); i-- > 0;) {
            if (entries[i].stream != stream || entries[i].growing) continue;
            if (entries[i].ptr) doomed.push_back(entries[i].ptr);
            entries.erase(entries.begin() + static_cast<long>(i));
        }
    }
    for (void *ptr : doomed) (void)hipFree(ptr);
}

size_t stream_workspace_entry_count()
{
    std::lock_guard<std::mutex> lock(workspace_mutex());
    return workspace_entries().size();
}

}  // namespace sthip

using namespace sthip;

extern "C" {

int st_hip_init(void) { return ensure_init(); }

int st_hip_real_backend_compiled(void) { return 1; }

int st_hip_device_count(void)
{
    if (ensure_init() != ST_HIP_OK) return 0;
    return static_cast<int>(runtime().devices.size());
}

int st_hip_device_name(int index, char *buf, size_t len)
{
    ST_HIP_CHECK(ensure_init());
    if (index < 0 || static_cast<size_t>(index) >= runtime().devices.size() || !buf || len == 0)
        return fail(ST_HIP_ERR_INVALID, "device index %d out of range", index);
    const hipDeviceProp_t &p = runtime().devices[static_cast<size_t>(index)];
    snprintf(buf, len, "%s", p.name[0] ? p.name : p.gcnArchName);
    return ST_HIP_OK;
}

int st_hip_device_properties(int index, st_hip_device_props *out)
{
    ST_HIP_CHECK(ensure_init());
    if (index < 0 || static_cast<size_t>(index) >= runtime().devices.size() || !out)
        return fail(ST_HIP_ERR_INVALID, "device index %d out of range", index);
    const hipDeviceProp_t &p = runtime().devices[static_cast<size_t>(index)];
    std::memset(out, 0, sizeof *out);
    out->compute_units = p.multiProcessorCount;
    out->clock_khz = p.clockRate;
    out->memory_clock_khz = p.memoryClockRate;
    out->memory_bus_bits = p.memoryBusWidth;
    out->wavefront_size = p.warpSize;
    out->lds_bytes_per_block = static_cast<int>(p.sharedMemPerBlock);
    out->l2_bytes = p.l2CacheSize;
    out->total_memory_bytes = p.totalGlobalMem;
    snprintf(out->arch, sizeof out->arch, "%s", p.gcnArchName);
    return ST_HIP_OK;
}

int st_hip_probe(st_hip_probe_result *out)
{
    if (!out) return fail(ST_HIP_ERR_INVALID, "st_hip_probe received a null out-pointer");
    std::memset(out, 0, sizeof *out);
    int count = 0;
    const hipError_t rc = hipGetDeviceCount(&count);
    if (rc != hipSuccess) (void)hipGetLastError();
    out->available = rc == hipSuccess && count > 0;
    out->device_count = rc == hipSuccess ? count : 0;
    if (ensure_init() == ST_HIP_OK) {
        out->initialized = 1;
    } else {
        snprintf(out->error, sizeof out->error, "%s", g_last_error.c_str());
    }
    return ST_HIP_OK;
}

size_t st_hip_last_error_message(char *buf, size_t len)
{
    if (buf && len > 0) snprintf(buf, len, "%s", g_last_error.c_str());
    return g_last_error.size();
}

int st_hip_malloc(void **device_ptr, size_t bytes)
{
    ST_HIP_CHECK(ensure_init());
    if (!device_ptr) return fail(ST_HIP_ERR_INVALID, "st_hip_malloc received a null out-pointer");
    *device_ptr = nullptr;
    ST_HIP_TRY(hipMalloc(device_ptr, bytes ? bytes : 1), "hipMalloc");  // real.rs:652 max(1)
    return ST_HIP_OK;
}

int st_hip_free(void *device_ptr)
{
    if (!device_ptr) return ST_HIP_OK;
    ST_HIP_TRY(hipFree(device_ptr), "hipFree");
    return ST_HIP_OK;
}

int st_hip_memcpy_h2d(void *device_dst, const void *host_src, size_t bytes, void *stream)
{
    if (bytes == 0) return ST_HIP_OK;
    count_transfer(true, bytes);
    ST_HIP_TRY(hipMemcpyAsync(device_dst, host_src, bytes, hipMemcpyHostToDevice, as_stream(stream)),
               "hipMemcpyAsync(H2D)");
    ST_HIP_TRY(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize");
    return ST_HIP_OK;
}

int st_hip_memcpy_d2h(void *host_dst, const void *device_src, size_t bytes, void *stream)
{
    if (bytes == 0) return ST_HIP_OK;
    count_transfer(false, bytes);
    ST_HIP_TRY(hipMemcpyAsync(host_dst, device_src, bytes, hipMemcpyDeviceToHost, as_stream(stream)),
               "hipMemcpyAsync(D2H)");
    ST_HIP_TRY(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize");
    return ST_HIP_OK;
}

int st_hip_memset_zero(void *device_dst, size_t bytes, void *stream)
{
    if (bytes == 0) return ST_HIP_OK;
    ST_HIP_TRY(hipMemsetAsync(device_dst, 0, bytes, as_stream(stream)), "hipMemsetAsync");
    return ST_HIP_OK;
}

int st_hip_transfer_counters(uint64_t counters[4], int reset)
{
    if (!counters) return fail(ST_HIP_ERR_INVALID, "st_hip_transfer_counters received a null out-pointer");
    for (int i = 0; i < 4; ++i)
        counters[i] = reset ? g_transfers[i].exchange(0, std::memory_order_relaxed) : g_transfers[i].load(std::memory_order_relaxed);
    return ST_HIP_OK;
}

int st_hip_stream_create(void **stream)
{
    ST_HIP_CHECK(ensure_init());
    if (!stream) return fail(ST_HIP_ERR_INVALID, "st_hip_stream_create received a null out-pointer");
    hipStream_t raw = nullptr;
    ST_HIP_TRY(hipStreamCreate(&raw), "hipStreamCreate");
    *stream = raw;
    return ST_HIP_OK;
}

int st_hip_stream_synchronize(void *stream)
{
    ST_HIP_TRY(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize");
    return ST_HIP_OK;
}

int st_hip_stream_destroy(void *stream)
{
    if (!stream) return ST_HIP_OK;
    // Same order as HipStream::drop (real.rs:207-214): drain, then release.
    (void)hipStreamSynchronize(as_stream(stream));
    release_stream_workspace(as_stream(stream));
    ST_HIP_TRY(hipStreamDestroy(as_stream(stream)), "hipStreamDestroy");
    return ST_HIP_OK;
}

int st_hip_release_scratch(void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_TRY(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize");
    release_stream_workspace(as_stream(stream));
    return ST_HIP_OK;
}

size_t st_hip_scratch_buffer_count(void) { return stream_workspace_entry_count(); }

int st_hip_device_synchronize(void)
{
    ST_HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return ST_HIP_OK;
}

int st_hip_event_create(void **event)
{
    ST_HIP_CHECK(ensure_init());
    if (!event) return fail(ST_HIP_ERR_INVALID, "st_hip_event_create received a null out-pointer");
    hipEvent_t raw = nullptr;
    ST_HIP_TRY(hipEventCreate(&raw), "hipEventCreate");
    *event = raw;
    return ST_HIP_OK;
}

int st_hip_event_record(void *event, void *stream)
{
    ST_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)), "hipEventRecord");
    return ST_HIP_OK;
}

int st_hip_event_synchronize(void *event)
{
    ST_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)), "hipEventSynchronize");
    return ST_HIP_OK;
}

int st_hip_event_elapsed_ms(void *start, void *stop, float *milliseconds)
{
    if (!milliseconds) return fail(ST_HIP_ERR_INVALID, "st_hip_event_elapsed_ms received a null out-pointer");
    ST_HIP_TRY(hipEventElapsedTime(milliseconds, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)),
               "hipEventElapsedTime");
    return ST_HIP_OK;
}

int st_hip_event_destroy(void *event)
{
    if (!event) return ST_HIP_OK;
    ST_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)), "hipEventDestroy");
    return ST_HIP_OK;
}

}  // extern "C"
