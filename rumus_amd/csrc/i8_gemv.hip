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
                // read once, by this wave only: the non-temporal hint (1 x 4096 x 11008 from HBM: 9.9 -> 9.4 us)
                wv[i][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wrow[j] + ka));
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
            acc[r][j] = wave_sum(acc[r][j]);
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

// ---------------------------------------------------------------------------------------------------
// 5 to 32 rows: still a bandwidth problem, but too many dot products for the vector ALU.  A workgroup
// owns 16 output columns; its four waves take a quarter of K each and feed v_mfma_i32_16x16x64_i8
// straight from global memory: lane (c = lane % 16, q = lane / 16) loads bytes 16 q .. 16 q + 15 of every
// 64 of weight row c as the B operand and of activation row c as the A operand (the activations come
// out of the caches: every wave reads all of them).  No LDS on the way in, eight K steps of loads in
// flight per lane; the four partial 16 x 16 tiles meet in LDS at the end.  Exact i32 sums.
// TN: column tiles of 16 per workgroup.  Every workgroup reads all of the activations, so two column tiles halve
// that traffic per weight byte; it pays where the launch still has several workgroups per compute unit (from HBM,
// 4096 x 22016: 16 rows 31.7 -> 27.7 us, 8 rows 26.9 -> 25.8 us; 4096 x 11008, 688 -> 344 workgroups: 15.3 -> 18.1 us).
template <int RT, int TN>
__global__ __launch_bounds__(256) void i8_stream_kernel(
    const int8_t* __restrict__ xq, const int8_t* __restrict__ wq, const float* __restrict__ sx,
    const float* __restrict__ sw, const float* __restrict__ bias, int32_t* __restrict__ acc_out,
    float* __restrict__ y, uint32_t M, uint32_t K, uint32_t N) {
    __shared__ int32_t part[3][RT * TN][4][64];                // waves 1..3: [row tile, column tile][register][lane]
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t c = lane & 15, q = lane >> 4;
    const uint32_t n0 = blockIdx.x * 16 * TN;
    const uint32_t kq = K / 4;                                 // K % 256 == 0: a quarter is whole K steps of 64
    const int8_t* bp[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) bp[j] = wq + (uint64_t)min(n0 + 16 * j + c, N - 1) * K + wave * kq + 16 * q;
    const int8_t* ap[RT];
#pragma unroll
    for (int t = 0; t < RT; t++) ap[t] = xq + (uint64_t)min(16 * t + c, M - 1) * K + wave * kq + 16 * q;
    v4i acc[RT][TN];
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[t][j] = v4i{0, 0, 0, 0};
    for (uint32_t k0 = 0; k0 < kq; k0 += 512) {                // 8 K steps per round, the last round maybe shorter
        v4i b[8][TN], a[8][RT];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t kk = min(k0 + 64 * i, kq - 64);     // past the end: the last step again, not multiplied
#pragma unroll
            for (int j = 0; j < TN; j++) b[i][j] = *reinterpret_cast<const v4i*>(bp[j] + kk);
#pragma unroll
            for (int t = 0; t < RT; t++) a[i][t] = *reinterpret_cast<const v4i*>(ap[t] + kk);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (k0 + 64 * i < kq) {
#pragma unroll
                for (int t = 0; t < RT; t++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[t][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i][t], b[i][j], acc[t][j], 0, 0, 0);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) part[wave - 1][t * TN + j][r][lane] = acc[t][j][r];
    }
    __syncthreads();
    if (wave > 0) return;
    // register r of lane l: row 4 (l / 16) + r, column l % 16 of the 16 x 16 tile
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const uint32_t col = n0 + 16 * j + c;
        if (col >= N) continue;
        const float swc = y ? sw[col] : 0.0f, bc = (y && bias) ? bias[col] : 0.0f;
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t row = 16 * t + 4 * q + r;
                if (row >= M) continue;
                const int u = t * TN + j;
                const int32_t v = acc[t][j][r] + part[0][u][r][lane] + part[1][u][r][lane] + part[2][u][r][lane];
                const uint64_t o = (uint64_t)row * N + col;
                if (acc_out) acc_out[o] = v;
                if (y) {
                    float f = __fmul_rn(__fmul_rn((float)v, sx[row]), swc);
                    if (bias) f = __fadd_rn(f, bc);
                    y[o] = f;
                }
            }
    }
}

// 5 <= m <= 32, k % 256 == 0, 16-byte aligned operands
int i8_launch_stream(const int8_t* xq, const int8_t* wq, const float* sx, const float* sw, const float* bias, int32_t* acc,
                     float* y, uint32_t m, uint32_t k, uint32_t n, hipStream_t s) {
    const bool two = m >= 8 && m <= 16 && ceil_div(n, 16) >= 1280;    // five workgroups per compute unit or more
    if (two)
        hipLaunchKernelGGL((i8_stream_kernel<1, 2>), dim3(ceil_div(n, 32)), dim3(256), 0, s, xq, wq, sx, sw, bias, acc, y, m, k, n);
    else if (m <= 16)
        hipLaunchKernelGGL((i8_stream_kernel<1, 1>), dim3(ceil_div(n, 16)), dim3(256), 0, s, xq, wq, sx, sw, bias, acc, y, m, k, n);
    else
        hipLaunchKernelGGL((i8_stream_kernel<2, 1>), dim3(ceil_div(n, 16)), dim3(256), 0, s, xq, wq, sx, sw, bias, acc, y, m, k, n);
    return check_launch("i8_stream_kernel");
}

}  // namespace rumus
