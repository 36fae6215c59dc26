// Pieces shared by the INT8 GEMM kernels: operand types, the LDS row swizzle
// and the rescale/bias epilogue.
#pragma once

#include <type_traits>

#include "common.h"

namespace rumus {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;  // K bytes per LDS stage

typedef const void __attribute__((address_space(1)))* gptr_t;
typedef void __attribute__((address_space(3)))* lptr_t;

// s_waitcnt with only vmcnt set (gfx9 encoding: vmcnt[3:0] | expcnt 7 | lgkmcnt 15 | vmcnt[5:4] << 14)
#define RUMUS_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x70 | 0xF00)

// Wide-block kernel (i8_gemm_wide.hip): 256 x 32*tn blocks, tn = 8..12.  fold4: see i8_epilogue.
int i8_gemm_launch_wide(int tn, const int8_t* A, const int8_t* B, const float* sx, const float* sw,
                        const float* bias, int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N,
                        hipStream_t s, bool fold4 = false);

// The W8A8 GEMM on four interleaved digit planes per activation row with the planes added in the epilogue
// (i8_epilogue, FOLD4): m4 = 4 * rows, y [m4 / 4, n].  Only the kernels of large shapes have that epilogue:
// i8_gemm_fold4 returns EINVAL where i8_gemm_fold4_supported says no.
bool i8_gemm_fold4_supported(uint32_t m4, uint32_t k, uint32_t n);
int i8_gemm_fold4(const int8_t* planes, const int8_t* wq, const float* sx4, const float* sw, const float* bias,
                  float* y, uint32_t m4, uint32_t k, uint32_t n, hipStream_t s);

// Workspace bytes rumus_hip_i8_gemm takes for an m x k x n product (i32 partial sums where K is shared over
// workgroups); replays the dispatch, no device call.
size_t i8_gemm_workspace_need(uint32_t m, uint32_t k, uint32_t n);

// Decode kernel for m <= 4 on v_dot4_i32_i8 (i8_gemv.hip).
int i8_launch_gemv(const int8_t* xq, const int8_t* wq, const float* sx, const float* sw, const float* bias, int32_t* acc,
                   float* y, uint32_t m, uint32_t k, uint32_t n, hipStream_t s);

// 5 to 32 rows, K % 256 == 0: MFMA tiles fed straight from global memory (i8_gemv.hip).
// 5..64 rows with the activations resident in registers, where i8_resident_takes says so
bool i8_resident_takes(uint32_t m, uint32_t k, uint32_t n);
int i8_launch_resident(const int8_t* xq, const int8_t* wq, const float* sx, const float* sw, const float* bias, int32_t* acc,
                       float* y, uint32_t m, uint32_t k, uint32_t n, hipStream_t s);
int i8_launch_stream(const int8_t* xq, const int8_t* wq, const float* sx, const float* sw, const float* bias, int32_t* acc,
                     float* y, uint32_t m, uint32_t k, uint32_t n, hipStream_t s);

// chunk swizzle of an LDS row: bit0 = b1 ^ b3, bit1 = b2 of the row index
__device__ __forceinline__ uint32_t row_swizzle(uint32_t row) {
    return (((row >> 1) ^ (row >> 3)) & 1u) | ((row >> 1) & 2u);
}

// Epilogue shared by both kernels.  Accumulator register r of lane l is row
// 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 tile, so a store
// instruction writes two full 128-byte row segments.  Interior tiles take a
// branch-free path: the row scales of the lane are fetched up front as float4
// (four consecutive rows per register quad) and y is written with
// ordinary stores, which leave it in the last-level cache for its reader.
// FOLD4: the rows are the four digit planes of M / 4 activation rows, interleaved (row 4 r + p is plane p
// of activation row r, sx[4 r + p] its weight): the four registers of a quad are the four planes of one output,
// y[r, col] = sum over p, in order, of (f32(acc) * sx[4 r + p]) * sw[col] (+ bias), and y has M / 4 rows.
template <int TM, int TN, int BM, int BN, bool FOLD4 = false>
__device__ __forceinline__ void i8_epilogue(const v16i (&acc)[TM][TN], const float* __restrict__ sx,
                                            const float* __restrict__ sw,
                                            const float* __restrict__ bias,
                                            int32_t* __restrict__ acc_out, float* __restrict__ y,
                                            uint32_t M, uint32_t N, uint32_t m0, uint32_t n0,
                                            uint32_t wm, uint32_t wn, uint32_t lane) {
    const uint32_t col_l = lane & 31, row_l = (lane >> 5) * 4;
    if constexpr (FOLD4) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const uint32_t col = n0 + (wn * TN + j) * 32 + col_l;
            if (col >= N) continue;
            const float swc = sw[col];
            const float bc = bias ? bias[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * g + row_l;    // a multiple of 4, as is M
                    if (row >= M) continue;
                    const float4 s4 = *reinterpret_cast<const float4*>(sx + row);
                    float v = __fmul_rn(__fmul_rn((float)acc[i][j][4 * g], s4.x), swc);
                    v = __fadd_rn(v, __fmul_rn(__fmul_rn((float)acc[i][j][4 * g + 1], s4.y), swc));
                    v = __fadd_rn(v, __fmul_rn(__fmul_rn((float)acc[i][j][4 * g + 2], s4.z), swc));
                    v = __fadd_rn(v, __fmul_rn(__fmul_rn((float)acc[i][j][4 * g + 3], s4.w), swc));
                    if (bias) v = __fadd_rn(v, bc);
                    y[(uint64_t)(row / 4) * N + col] = v;
                }
            }
        }
        return;
    }
    // whole 32-column MFMA tiles are in or out when N % 32 == 0, so the fast path
    // only needs all rows of the block inside M
    const bool interior = m0 + BM <= M && N % 32 == 0 && ((reinterpret_cast<uintptr_t>(sx) & 15) == 0);
    if (interior && y && !acc_out) {
        float4 sxv[TM][4];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int q = 0; q < 4; q++)
                sxv[i][q] = *reinterpret_cast<const float4*>(sx + m0 + (wm * TM + i) * 32 + 8 * q + row_l);
        // A store's address is a base that is the same for the whole wave (row tile, row of the quad: scalar registers)
        // plus one 32-bit byte offset per lane and column tile (the lane's own row of four and its column), so that an
        // element costs the conversion and its two multiplications and nothing for its address; the bias is a
        // path of its own rather than a select per element.
        const bool narrow = N < (1u << 27);                // the lane offsets, (4 N + column) floats at most, fit 32 bits
        auto body = [&](auto bias_tag, auto narrow_tag) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const uint32_t col = n0 + (wn * TN + j) * 32 + col_l;
                if (n0 + (wn * TN + j) * 32 >= N) continue;    // uniform: this column tile lies past N
                const float swc = sw[col];
                const float bc = decltype(bias_tag)::value ? bias[col] : 0.0f;
                const uint32_t lane_off = (row_l * N + col) * (uint32_t)sizeof(float);
#pragma unroll
                for (int i = 0; i < TM; i++) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const uint32_t row_u = m0 + (wm * TM + i) * 32 + 8 * (r / 4) + (r % 4);      // uniform part of the row
                        const float4 s4 = sxv[i][r / 4];
                        const float sr = (r % 4) == 0 ? s4.x : (r % 4) == 1 ? s4.y : (r % 4) == 2 ? s4.z : s4.w;
                        float v = __fmul_rn(__fmul_rn((float)acc[i][j][r], sr), swc);
                        if (decltype(bias_tag)::value) v = __fadd_rn(v, bc);
                        // ordinary stores: the output stays in the Infinity Cache for whoever reads it next, and the
                        // launch ends 1.5 % sooner than with the non-temporal hint (102.9 -> 101.3 us at 2048 x 4096 x 11008)
                        if constexpr (decltype(narrow_tag)::value) {
                            uint8_t* const base = reinterpret_cast<uint8_t*>(y + (uint64_t)row_u * N);
                            *reinterpret_cast<float*>(base + lane_off) = v;
                        } else {
                            y[(uint64_t)(row_u + row_l) * N + col] = v;
                        }
                    }
                }
            }
        };
        if (bias) {
            if (narrow) body(std::true_type{}, std::true_type{});
            else body(std::true_type{}, std::false_type{});
        } else {
            if (narrow) body(std::false_type{}, std::true_type{});
            else body(std::false_type{}, std::false_type{});
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const uint32_t col = n0 + (wn * TN + j) * 32 + col_l;
        if (col >= N) continue;
        const float swc = y ? sw[col] : 0.0f;
        const float bc = (y && bias) ? bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * (r / 4) + row_l + (r % 4);
                if (row >= M) continue;
                const int32_t a = acc[i][j][r];
                const uint64_t o = (uint64_t)row * N + col;
                if (acc_out) acc_out[o] = a;
                if (y) {
                    float v = __fmul_rn(__fmul_rn((float)a, sx[row]), swc);
                    if (bias) v = __fadd_rn(v, bc);
                    y[o] = v;
                }
            }
        }
    }
}

}  // namespace rumus
