// Half-precision activations for the two quantized matmuls.
//
// The reference's kernels are typed `scalar`, f32 or f16 as the activations are
// (rumus/src/backend/gpu/shaders/matmul_q8.wgsl:1-5,26-28, rumus-vision/src/shaders/qmatmul_int4.wgsl:33-38,
// picked at rumus/src/ext/mod.rs:132-150): in f16 mode they read f16 activations, sum in f16 and write f16.
// Here the f16 entry points are the f32 ones between two conversions: the activations are widened (exact), the
// product runs in the f32 kernels with their accuracy, and the result is rounded to f16 once, to nearest even
// (finite values beyond 65504 become infinities, as any f16 store would make them).  That is at least as
// accurate as an f16 running sum and deterministic.  The weights' metadata (scales, zero-points, bias) stays
// f32: it is converted once when a checkpoint is loaded (rumus_hip_f16_to_f32), not per call.
#include "common.h"

namespace rumus {

// 8 values per thread: one 16-byte load, two 16-byte stores (or the other way round)
__global__ __launch_bounds__(256) void f16_widen_kernel(const _Float16* __restrict__ in, float* __restrict__ out, uint64_t numel) {
    const uint64_t i = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i + 8 <= numel && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 v = *reinterpret_cast<const h8*>(in + i);
        float4 lo = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]}, hi = {(float)v[4], (float)v[5], (float)v[6], (float)v[7]};
        *reinterpret_cast<float4*>(out + i) = lo;
        *reinterpret_cast<float4*>(out + i + 4) = hi;
        return;
    }
    for (uint64_t j = i; j < numel && j < i + 8; j++) out[j] = (float)in[j];
}

__global__ __launch_bounds__(256) void f16_narrow_kernel(const float* __restrict__ in, _Float16* __restrict__ out, uint64_t numel) {
    const uint64_t i = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i + 8 <= numel && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const float4 lo = *reinterpret_cast<const float4*>(in + i), hi = *reinterpret_cast<const float4*>(in + i + 4);
        h8 v;
        v[0] = (_Float16)lo.x; v[1] = (_Float16)lo.y; v[2] = (_Float16)lo.z; v[3] = (_Float16)lo.w;
        v[4] = (_Float16)hi.x; v[5] = (_Float16)hi.y; v[6] = (_Float16)hi.z; v[7] = (_Float16)hi.w;
        *reinterpret_cast<h8*>(out + i) = v;
        return;
    }
    for (uint64_t j = i; j < numel && j < i + 8; j++) out[j] = (_Float16)in[j];
}

static inline size_t round_256(size_t b) { return (b + 255) & ~size_t(255); }

// f32 copies of the activations and of the result, in the stream's staging buffer
struct F16Stage {
    WorkspaceLease lease;
    float* a = nullptr;
    float* c = nullptr;
};

static int f16_stage(const uint16_t* a16, uint64_t a_numel, uint64_t c_numel, hipStream_t s, F16Stage& st, const char* who) {
    RUMUS_REQUIRE(a_numel < (1ull << 38) && c_numel < (1ull << 38), "%s: operand beyond the grid limit", who);
    void* ws = nullptr;
    const size_t a_bytes = round_256(a_numel * sizeof(float));
    if (int rc = staging_get(s, a_bytes + round_256(c_numel * sizeof(float)), &ws, st.lease)) return rc;
    st.a = static_cast<float*>(ws);
    st.c = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + a_bytes);
    if (a_numel) {
        hipLaunchKernelGGL(f16_widen_kernel, dim3((uint32_t)((a_numel + 2047) / 2048)), dim3(256), 0, s,
                           reinterpret_cast<const _Float16*>(a16), st.a, a_numel);
        if (int rc = check_launch("f16_widen_kernel")) return rc;
    }
    return RUMUS_HIP_OK;
}

static int f16_finish(const F16Stage& st, uint16_t* c16, uint64_t c_numel, hipStream_t s) {
    if (c_numel == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(f16_narrow_kernel, dim3((uint32_t)((c_numel + 2047) / 2048)), dim3(256), 0, s, st.c,
                       reinterpret_cast<_Float16*>(c16), c_numel);
    return check_launch("f16_narrow_kernel");
}

}  // namespace rumus

using namespace rumus;

extern "C" {

int rumus_hip_matmul_q8_f16(const uint16_t* a, const uint32_t* b, uint16_t* c, uint32_t m, uint32_t k, uint32_t n,
                            uint32_t block_size, rumus_hip_stream_t stream) {
    // nothing to compute, or nothing to compute on: the f32 entry point's own checks give the answer
    if (m == 0 || n == 0 || !a || !c) return rumus_hip_matmul_q8(nullptr, b, nullptr, m, k, n, block_size, stream);
    F16Stage st;
    if (int rc = f16_stage(a, (uint64_t)m * k, (uint64_t)m * n, as_stream(stream), st, "matmul_q8_f16")) return rc;
    if (int rc = rumus_hip_matmul_q8(st.a, b, st.c, m, k, n, block_size, stream)) return rc;
    return f16_finish(st, c, (uint64_t)m * n, as_stream(stream));
}

int rumus_hip_qmatmul_int4_f16(const uint16_t* x, const uint32_t* packed, const float* scales, const float* zero_points,
                               const float* bias, const int32_t* g_idx, uint16_t* y, uint32_t m, uint32_t k, uint32_t n,
                               uint32_t padded_k, uint32_t group_size, uint32_t num_groups, rumus_hip_stream_t stream) {
    if (m == 0 || n == 0 || !x || !y)
        return rumus_hip_qmatmul_int4(nullptr, packed, scales, zero_points, bias, g_idx, nullptr, m, k, n, padded_k, group_size,
                                      num_groups, stream);
    F16Stage st;
    if (int rc = f16_stage(x, (uint64_t)m * k, (uint64_t)m * n, as_stream(stream), st, "qmatmul_int4_f16")) return rc;
    if (int rc = rumus_hip_qmatmul_int4(st.a, packed, scales, zero_points, bias, g_idx, st.c, m, k, n, padded_k, group_size,
                                        num_groups, stream))
        return rc;
    return f16_finish(st, y, (uint64_t)m * n, as_stream(stream));
}

}  // extern "C"
