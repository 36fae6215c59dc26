// Shared helpers for the gfx950 kernels of librumus_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rumus_hip.h"

namespace rumus {

// Records a thread-local message and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Converts a HIP status into a return code (0 when hipSuccess).
int check_hip(hipError_t e, const char* what);

// Exclusive use of one stream's workspace, from workspace_get until the holder goes out of scope.  A call that
// queues several kernels which talk to each other through the workspace keeps its lease until the last of them
// is queued: another host thread on the same stream then cannot slip launches of its own between them (they
// would overwrite the partial results), and cannot grow - that is, free - the buffer under them.  The lock
// behind it is per (device, stream) and recursive, so calls on different streams never wait for each other and
// an entry point may call another one while it holds the lease.
class WorkspaceLease {
  public:
    WorkspaceLease() = default;
    ~WorkspaceLease();
    WorkspaceLease(const WorkspaceLease&) = delete;
    WorkspaceLease& operator=(const WorkspaceLease&) = delete;
  private:
    friend int workspace_get(hipStream_t, size_t, void**, WorkspaceLease&);
    void* arena_ = nullptr;
};

// Device workspace of at least `bytes` for work queued on `stream` (runtime.hip); `lease` then holds the
// stream's workspace lock.
int workspace_get(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease);
// A call that holds workspace memory and then calls another entry point that takes workspace of its own on the
// same stream (the Q8 matmul around the int8 GEMM) asks for both sizes at once and keeps one of these alive over
// the inner call: workspace_get then hands out the part of the buffer behind `offset`, and fails instead of
// growing (growing would free what the outer call still uses).
struct WorkspaceNest {
    explicit WorkspaceNest(size_t offset);
    ~WorkspaceNest();
    WorkspaceNest(const WorkspaceNest&) = delete;
    WorkspaceNest& operator=(const WorkspaceNest&) = delete;
  private:
    size_t prev_;
};

// While one of these lives on a thread, workspace_get on that thread hands out `ptr` (a caller-provided buffer
// of `bytes`) instead of the stream's own buffer, and fails with EINVAL instead of allocating when a request
// does not fit.  For entry points that must not allocate.
struct WorkspaceFixed {
    WorkspaceFixed(void* ptr, size_t bytes);
    ~WorkspaceFixed();
    WorkspaceFixed(const WorkspaceFixed&) = delete;
    WorkspaceFixed& operator=(const WorkspaceFixed&) = delete;
  private:
    void* prev_ptr_;
    size_t prev_bytes_;
};

// hipGetLastError() after a kernel launch.
inline int check_launch(const char* kernel) { return check_hip(hipGetLastError(), kernel); }

inline hipStream_t as_stream(rumus_hip_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

constexpr int kWave = 64;       // CDNA wavefront width
constexpr int kXcds = 8;        // MI355X: 8 accelerator dies, each with its own L2

inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// Workgroups are handed to the 8 XCDs round-robin (workgroup b runs on XCD
// b % 8).  This maps b to a logical tile index so that each XCD owns one
// contiguous range of tiles: neighbouring tiles then share an L2.
__device__ __forceinline__ uint32_t xcd_contiguous(uint32_t b, uint32_t total) {
    uint32_t x = b % kXcds, l = b / kXcds;
    uint32_t q = total / kXcds, r = total % kXcds;
    return x * q + (x < r ? x : r) + l;
}

}  // namespace rumus

#define RUMUS_REQUIRE(cond, ...)                                         \
    do {                                                                 \
        if (!(cond)) return ::rumus::set_error(RUMUS_HIP_EINVAL, __VA_ARGS__); \
    } while (0)
