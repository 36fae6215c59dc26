// Runtime entry points: status reporting, device selection, stream sync.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <unordered_map>

#include "common.h"

namespace rumus {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return RUMUS_HIP_OK;
    return set_error(RUMUS_HIP_EHIP, "%s: %s", what, hipGetErrorString(e));
}

// ---- workspace: one device buffer per (device, stream), grown on demand -----------------
// Kernels that split the reduction axis over workgroups park their partial sums here.
// Calls on one stream run in order, so they can share a buffer; different streams get
// different buffers.  Growing is the only time the library allocates: it waits for the
// stream, frees the old buffer and allocates the new size.
namespace {
struct Arena {
    void* ptr = nullptr;
    size_t bytes = 0;
    std::recursive_mutex in_use;     // held by a WorkspaceLease
};
struct ArenaKey {
    int device;
    hipStream_t stream;
    int kind;                        // 0: the workspace of the kernels, 1: staging buffers of the half-precision entry points
    bool operator==(const ArenaKey& o) const { return device == o.device && stream == o.stream && kind == o.kind; }
};
struct ArenaKeyHash {
    size_t operator()(const ArenaKey& k) const {
        return std::hash<const void*>()(k.stream) ^ (std::hash<int>()(k.device * 2 + k.kind) * 0x9e3779b97f4a7c15ull);
    }
};
std::mutex g_arena_mutex;
std::unordered_map<ArenaKey, Arena, ArenaKeyHash> g_arenas;
}  // namespace

static thread_local size_t g_nest_offset = 0;
WorkspaceNest::WorkspaceNest(size_t offset) : prev_(g_nest_offset) { g_nest_offset = offset; }
WorkspaceNest::~WorkspaceNest() { g_nest_offset = prev_; }

WorkspaceLease::~WorkspaceLease() {
    if (arena_) static_cast<Arena*>(arena_)->in_use.unlock();
}

static thread_local void* g_fixed_ptr = nullptr;
static thread_local size_t g_fixed_bytes = 0;
WorkspaceFixed::WorkspaceFixed(void* ptr, size_t bytes) : prev_ptr_(g_fixed_ptr), prev_bytes_(g_fixed_bytes) {
    g_fixed_ptr = ptr;
    g_fixed_bytes = bytes;
}
WorkspaceFixed::~WorkspaceFixed() {
    g_fixed_ptr = prev_ptr_;
    g_fixed_bytes = prev_bytes_;
}

int arena_get(int kind, hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease);

int workspace_get(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease) {
    return arena_get(0, stream, bytes, out, lease);
}

int staging_get(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease) {
    return arena_get(1, stream, bytes, out, lease);
}

int arena_get(int kind, hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease) {
    int device = 0;
    if (int rc = check_hip(hipGetDevice(&device), "hipGetDevice")) return rc;
    if (lease.arena_) return set_error(RUMUS_HIP_EINVAL, "workspace lease used twice");
    Arena* found = nullptr;
    {
        // the table lock covers the lookup only; entries of an unordered_map do not move
        std::lock_guard<std::mutex> lock(g_arena_mutex);
        found = &g_arenas[ArenaKey{device, stream, kind}];
    }
    found->in_use.lock();            // from here on this thread alone queues work that uses the buffer
    lease.arena_ = found;
    Arena& a = *found;
    if (kind == 0 && g_fixed_ptr) {  // a buffer of fixed size stands in for the stream's own: nothing is allocated
        const size_t offset = g_nest_offset;
        if (offset + bytes > g_fixed_bytes)
            return set_error(RUMUS_HIP_EINVAL, "this call needs %zu bytes of scratch memory, the fixed buffer holds %zu",
                             offset + bytes, g_fixed_bytes);
        *out = static_cast<uint8_t*>(g_fixed_ptr) + offset;
        return RUMUS_HIP_OK;
    }
    if (const size_t offset = kind == 0 ? g_nest_offset : 0) {
        if (a.bytes < offset + bytes)
            return set_error(RUMUS_HIP_EINVAL, "nested workspace of %zu bytes behind %zu does not fit the %zu reserved", bytes,
                             offset, a.bytes);
        *out = static_cast<uint8_t*>(a.ptr) + offset;
        return RUMUS_HIP_OK;
    }
    if (a.bytes < bytes) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (stream && hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
            return set_error(RUMUS_HIP_EINVAL,
                             "%s of %zu bytes needed while the stream is capturing: call %s before the capture",
                             kind ? "staging memory" : "workspace", bytes,
                             kind ? "rumus_hip_f16_staging_reserve" : "rumus_hip_workspace_reserve");
        if (a.ptr) {
            if (int rc = check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize")) return rc;
            if (int rc = check_hip(hipFree(a.ptr), "hipFree(workspace)")) return rc;
            a.ptr = nullptr;
            a.bytes = 0;
        }
        const size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);   // whole MiB
        if (int rc = check_hip(hipMalloc(&a.ptr, want), "hipMalloc(workspace)")) return rc;
        a.bytes = want;
    }
    *out = a.ptr;
    return RUMUS_HIP_OK;
}

static int workspace_release_all() {
    std::lock_guard<std::mutex> lock(g_arena_mutex);
    int rc = RUMUS_HIP_OK;
    for (auto& kv : g_arenas) {
        if (!kv.second.ptr) continue;
        int cur = 0;
        (void)hipGetDevice(&cur);
        (void)hipSetDevice(kv.first.device);
        if (int e = check_hip(hipFree(kv.second.ptr), "hipFree(workspace)")) rc = e;
        (void)hipSetDevice(cur);
    }
    g_arenas.clear();
    return rc;
}

}  // namespace rumus

extern "C" {

int rumus_hip_workspace_reserve(rumus_hip_stream_t stream, uint64_t bytes) {
    void* p = nullptr;
    if (bytes == 0) return RUMUS_HIP_OK;
    rumus::WorkspaceLease lease;
    return rumus::workspace_get(rumus::as_stream(stream), (size_t)bytes, &p, lease);
}

int rumus_hip_f16_staging_reserve(rumus_hip_stream_t stream, uint64_t bytes) {
    void* p = nullptr;
    if (bytes == 0) return RUMUS_HIP_OK;
    rumus::WorkspaceLease lease;
    return rumus::staging_get(rumus::as_stream(stream), (size_t)bytes, &p, lease);
}

int rumus_hip_shutdown(void) { return rumus::workspace_release_all(); }

int rumus_hip_init(int device) {
    int count = 0;
    if (int rc = rumus::check_hip(hipGetDeviceCount(&count), "hipGetDeviceCount")) return rc;
    RUMUS_REQUIRE(device >= 0 && device < count, "rumus_hip_init: device %d of %d", device, count);
    if (int rc = rumus::check_hip(hipSetDevice(device), "hipSetDevice")) return rc;
    hipDeviceProp_t prop;
    if (int rc = rumus::check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties"))
        return rc;
    // The kernels are built for gfx950 only; refuse anything else up front
    // instead of failing at the first launch.
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return rumus::set_error(RUMUS_HIP_EINVAL, "rumus_hip_init: device is %s, library is gfx950 only",
                                prop.gcnArchName);
    return RUMUS_HIP_OK;
}

const char* rumus_hip_last_error(void) { return rumus::g_err; }

const char* rumus_hip_version(void) { return "rumus-hip 0.1.0 gfx950"; }

int rumus_hip_sync(rumus_hip_stream_t stream) {
    return rumus::check_hip(hipStreamSynchronize(rumus::as_stream(stream)), "hipStreamSynchronize");
}

}  // extern "C"
