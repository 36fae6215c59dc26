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
    friend int arena_get(int, hipStream_t, size_t, void**, WorkspaceLease&);
    void* arena_ = nullptr;
};

// Device workspace of at least `bytes` for work queued on `stream` (runtime.hip); `lease` then holds the
// stream's workspace lock.
int workspace_get(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease);
// A second buffer per (device, stream), for entry points that wrap another entry point between two conversions
// (the half-precision ones): what they stage must outlive the inner call, whose workspace may grow - that is, be
// freed - under it.  Never nested, never replaced by a fixed buffer.
int staging_get(hipStream_t stream, size_t bytes, void** out, WorkspaceLease& lease);
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

// Reductions over the 64 lanes of a wave, the result in every lane, without a trip through the LDS crossbar
// (__shfl_xor is ds_bpermute): four DPP exchanges inside the rows of 16 lanes, then v_permlane16_swap and
// v_permlane32_swap across them.  The pairs that meet are those of the xor butterfly with offsets 1, 2, 4, 8,
// 16, 32 (lane i meets 7 - i and 15 - i instead of i ^ 4 and i ^ 8, which hold the same partial results), so a
// commutative `op` gives the same bits as that butterfly, in every lane.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_lane(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <typename T, typename F>
__device__ __forceinline__ T wave_all_reduce(T value, F op) {
    static_assert(sizeof(T) == 4, "32-bit values");
    auto bits = [](T t) { return __builtin_bit_cast(uint32_t, t); };
    auto val = [](uint32_t u) { return __builtin_bit_cast(T, u); };
    T v = value;
    v = op(v, val(dpp_lane<0xB1>(bits(v))));       // quad_perm [1,0,3,2]
    v = op(v, val(dpp_lane<0x4E>(bits(v))));       // quad_perm [2,3,0,1]
    v = op(v, val(dpp_lane<0x141>(bits(v))));      // row_half_mirror: the other quad of the 8
    v = op(v, val(dpp_lane<0x140>(bits(v))));      // row_mirror: the other 8 of the row
    const auto r = __builtin_amdgcn_permlane16_swap(bits(v), bits(v), false, false);   // rows 0 | 1, 2 | 3
    v = op(val(r[0]), val(r[1]));
    const auto h = __builtin_amdgcn_permlane32_swap(bits(v), bits(v), false, false);   // the halves
    return op(val(h[0]), val(h[1]));
}
__device__ __forceinline__ float wave_sum(float v) { return wave_all_reduce(v, [](float a, float b) { return a + b; }); }
__device__ __forceinline__ int32_t wave_sum(int32_t v) { return wave_all_reduce(v, [](int32_t a, int32_t b) { return a + b; }); }
__device__ __forceinline__ float wave_max(float v) { return wave_all_reduce(v, [](float a, float b) { return fmaxf(a, b); }); }
__device__ __forceinline__ uint32_t wave_max(uint32_t v) { return wave_all_reduce(v, [](uint32_t a, uint32_t b) { return a > b ? a : b; }); }

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
