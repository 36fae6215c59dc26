// Internal interface between the INT4 matmul kernels and their dispatcher.
#pragma once

#include "common.h"

namespace rumus {

// Arguments of one fused INT4 dequant-matmul, y[m,n] = x[m,k] . dequant(W).
// `perm` (or null) gathers the activation column for sorted row j; `g_idx`
// (or null) picks the metadata row per original row (generic kernel only).
struct W4Args {
    const float* x;
    const uint32_t* packed;
    const float* scales;
    const float* zp;
    const float* bias;
    const int32_t* g_idx;
    const int32_t* perm;
    float* y;
    uint32_t m, k, n, padded_k, group_size, num_groups;
    // AWQ storage (or null): integer zero-points, eight per word along n, column col in bits
    // 4*(col%8) of word g*(n/8) + col/8; `zp` is null then and n % 8 == 0
    const uint32_t* zp4 = nullptr;
    // decode layout (w4_gemv_dot8 only): packed, scales and zp are tile-major copies, tile = 16
    // columns: packed_t[(c*word_rows + r)*16 + j] = packed[r*n + 16*c + j], likewise the metadata
    bool tiled = false;
    // w4_gemv_dot8 only: x holds rows of 2k floats, gate | up; the activations are silu(gate) * up
    bool glu = false;
    // w4_gemm_tile only (set by its launcher): activations split into hi and lo f16 planes in
    // A-fragment order, block (row tile of 32, step of 16 k) = 64 lanes x 16 bytes, and the f32
    // sum of every row's 16 values per step; xsteps = steps allocated per row tile
    const uint8_t* xh = nullptr;
    const uint8_t* xl = nullptr;
    const float* xs = nullptr;
    uint32_t xsteps = 0;
    // w4_gemm_tile only (set by its launcher): a power of two per row that brings the row's largest magnitude into
    // [2^14, 2^15) before the split into f16 planes (rinv), and its reciprocal for the results (rfac)
    const float* rinv = nullptr;
    const float* rfac = nullptr;
    // w4_gemm_tile only (set by its launcher; f32 zero-points): kZpFlagWords words, nonzero where a part of the
    // zero-point table holds a value that is no integer (w4_zp_scan_kernel)
    const uint32_t* zflags = nullptr;
};

// zero-points of 4 (col % 4 == 0) or 2 (col % 2 == 0) adjacent columns from the packed form
__device__ __forceinline__ float4 w4_zp4_unpack4(uint32_t v) {   // the four low nibbles
    return make_float4((float)(v & 15u), (float)((v >> 4) & 15u), (float)((v >> 8) & 15u), (float)((v >> 12) & 15u));
}
__device__ __forceinline__ float4 w4_zp4_load4(const uint32_t* zp4, uint32_t g, uint32_t n, uint32_t col) {
    return w4_zp4_unpack4(zp4[(uint64_t)g * (n / 8) + col / 8] >> ((col & 4u) * 4u));
}
__device__ __forceinline__ float2 w4_zp4_load2(const uint32_t* zp4, uint32_t g, uint32_t n, uint32_t col) {
    const uint32_t v = zp4[(uint64_t)g * (n / 8) + col / 8] >> ((col & 6u) * 4u);
    return make_float2((float)(v & 15u), (float)((v >> 4) & 15u));
}
__device__ __forceinline__ float w4_zp4_load1(const uint32_t* zp4, uint64_t g, uint32_t n, uint32_t col) {
    return (float)((zp4[g * (n / 8) + col / 8] >> ((col & 7u) * 4u)) & 15u);
}

// Reference-order kernel: any shape, g_idx and perm; one thread per column.
int w4_launch_generic(const W4Args& a, hipStream_t s);

// Bandwidth kernel for m <= 8 (needs n % 4 == 0, 16-byte aligned buffers,
// m * padded_k floats of LDS, no g_idx).
bool w4_gemv_supported(const W4Args& a);
int w4_launch_gemv(const W4Args& a, hipStream_t s);

// Decode kernel on v_dot8_u32_u4 (m <= 8, group_size % 64 == 0, n % 4 == 0,
// 16-byte aligned buffers, no g_idx); preferred over the f32 bandwidth kernel.
bool w4_gemv_dot8_supported(const W4Args& a);
int w4_launch_gemv_dot8(const W4Args& a, hipStream_t s);
// the decoder block's forms (decode layout, f32 zero-points, no perm): input through RMSNorm with `norm_w` (or null),
// or through SwiGLU (a.glu), `resid` (or null) added to the result
int w4_launch_gemv_dot8_block(const W4Args& a, const float* norm_w, float eps, const float* resid, hipStream_t s);

// f16 MFMA kernel for larger m (needs group_size 32, 64 or a multiple of 128,
// n % 4 == 0, 16-byte aligned buffers, no g_idx).
bool w4_gemm_supported(const W4Args& a);
uint32_t w4_decode_max_rows(uint32_t padded_k, uint32_t n);   // w4_gemv.hip
int w4_launch_gemm(const W4Args& a, hipStream_t s);

// int8 matrix cores for up to 128 rows (w4_gemm_i8.hip): group_size % 64 == 0, n % 4 == 0, 16-byte aligned
// buffers, no g_idx.
bool w4_gemm_i8_supported(const W4Args& a);
int w4_launch_gemm_i8(const W4Args& a, hipStream_t s);

// grad_x on the f16 matrix cores (w4_gemm_t.hip): group_size 32, 64 or a multiple of 128, n % 4 == 0, k % 4 == 0,
// 16-byte aligned buffers.
bool w4_gemm_t_supported(uint32_t m, uint32_t k, uint32_t n, uint32_t group_size, const void* gy, const void* packed,
                         const void* scales, const void* zp, const void* out);
int w4_launch_gemm_t(const float* gy, const uint32_t* packed, const float* scales, const float* zp, float* out,
                     uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k, uint32_t group_size, uint32_t num_groups,
                     hipStream_t s);

}  // namespace rumus
