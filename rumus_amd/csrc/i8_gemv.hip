// W8A8 for up to 4 rows (decode): a bandwidth kernel on v_dot4_i32_i8.
//
//   acc[m, n] = sum_k xq[m, k] * wq[n, k]      (i32, exact)
//   y[m, n]   = (f32(acc) * sx[m]) * sw[n] (+ bias[n])
//
// Both operands are K-contiguous, so an output column is one contiguous row of wq.  A wave owns
// kCols output columns; its lanes split K in 16-byte pieces (lane l takes bytes 16 l .. 16 l + 15 of
// every 1 KB of a row), which makes every load of a wave one contiguous kilobyte, and the kCols rows of
// a wave one contiguous slab.  K is walked in chunks of 4 KB: the 4 x kCols weight loads of a chunk and
// the activations of the chunk (read by every wave, served by the caches) are issued together, then
// multiplied with four dot4 per 16 bytes and row.  The 64 partial sums of an output meet in a butterfly
// of shuffles.  Integer sums are exact in any order: the accumulators equal the MFMA kernels' bit for bit.
#include "i8_gemm.h"

namespace rumus {

constexpr int kGemvCols = 2;                                   // output columns per wave: 8 loads per lane and 4 KB of K (4: 11.2 us at 1 x 4096 x 11008 from HBM, 2: 9.3 us, 1: 9.3 us but 14.8 instead of 12.7 us at 4 rows)
constexpr int kGemvWaves = 4;                                  // waves per workgroup

template <int M>
__global__ __launch_bounds__(64 * kGemvWaves) void i8_gemv_kernel(
    const int8_t* __restrict__ xq, const int8_t* __restrict__ wq, const float* __restrict__ sx,
    const float* __restrict__ sw, const float* __restrict__ bias, int32_t* __restrict__ acc_out,
    float* __restrict__ y, uint32_t K, uint32_t N) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n0 = (blockIdx.x * kGemvWaves + wave) * kGemvCols;
    if (n0 >= N) return;                                       // whole waves leave; nothing is shared
    const int8_t* wrow[kGemvCols];
#pragma unroll
    for (int j = 0; j < kGemvCols; j++) wrow[j] = wq + (uint64_t)min(n0 + j, N - 1) * K;   // past N: the last row again, not stored

    int32_t acc[M][kGemvCols];
#pragma unroll
    for (int r = 0; r < M; r++)
#pragma unroll
        for (int j = 0; j < kGemvCols; j++) acc[r][j] = 0;

    for (uint32_t k0 = 0; k0 < K; k0 += 4096) {
        v4i wv[4][kGemvCols], xv[4][M];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t kk = k0 + 1024 * i + 16 * lane;
            const bool in = kk < K;                            // K % 16 == 0: a piece is all-in or all-out
            const uint32_t ka = in ? kk : 0;
#pragma unroll
            for (int j = 0; j < kGemvCols; j++) {
                wv[i][j] = *reinterpret_cast<const v4i*>(wrow[j] + ka);
                if (!in) wv[i][j] = v4i{0, 0, 0, 0};
            }
#pragma unroll
            for (int r = 0; r < M; r++) xv[i][r] = *reinterpret_cast<const v4i*>(xq + (uint64_t)r * K + ka);
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < kGemvCols; j++)
#pragma unroll
                for (int r = 0; r < M; r++)
#pragma unroll
                    for (int d = 0; d < 4; d++)
                        acc[r][j] = __builtin_amdgcn_sdot4(xv[i][r][d], wv[i][j][d], acc[r][j], false);
    }

#pragma unroll
    for (int r = 0; r < M; r++)
#pragma unroll
        for (int j = 0; j < kGemvCols; j++) {
            int32_t v = acc[r][j];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
            acc[r][j] = v;
        }
    // lane j of the first kCols lanes writes column n0 + j of every row
    if (lane < kGemvCols && n0 + lane < N) {
        const uint32_t col = n0 + lane;
        const float swc = y ? sw[col] : 0.0f, bc = (y && bias) ? bias[col] : 0.0f;
#pragma unroll
        for (int r = 0; r < M; r++) {
            int32_t a = acc[r][0];
#pragma unroll
            for (int j = 1; j < kGemvCols; j++) a = lane == (uint32_t)j ? acc[r][j] : a;
            const uint64_t o = (uint64_t)r * N + col;
            if (acc_out) acc_out[o] = a;
            if (y) {
                float v = __fmul_rn(__fmul_rn((float)a, sx[r]), swc);
                if (bias) v = __fadd_rn(v, bc);
                y[o] = v;
            }
        }
    }
}

template <int M>
static int launch_i8_gemv(const int8_t* xq, const int8_t* wq, const float* sx, const float* sw, const float* bias,
                          int32_t* acc, float* y, uint32_t k, uint32_t n, hipStream_t s) {
    hipLaunchKernelGGL(i8_gemv_kernel<M>, dim3(ceil_div(n, kGemvWaves * kGemvCols)), dim3(64 * kGemvWaves), 0, s, xq, wq,
                       sx, sw, bias, acc, y, k, n);
    return check_launch("i8_gemv_kernel");
}

// m <= 4, k % 16 == 0, 16-byte aligned operands (what rumus_hip_i8_gemm requires anyway)
int i8_launch_gemv(const int8_t* xq, const int8_t* wq, const float* sx, const float* sw, const float* bias, int32_t* acc,
                   float* y, uint32_t m, uint32_t k, uint32_t n, hipStream_t s) {
    switch (m) {
        case 1: return launch_i8_gemv<1>(xq, wq, sx, sw, bias, acc, y, k, n, s);
        case 2: return launch_i8_gemv<2>(xq, wq, sx, sw, bias, acc, y, k, n, s);
        case 3: return launch_i8_gemv<3>(xq, wq, sx, sw, bias, acc, y, k, n, s);
        case 4: return launch_i8_gemv<4>(xq, wq, sx, sw, bias, acc, y, k, n, s);
    }
    return set_error(RUMUS_HIP_EINVAL, "i8 gemv: m = %u out of range", m);
}

}  // namespace rumus
