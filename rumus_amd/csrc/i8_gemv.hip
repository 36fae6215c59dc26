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
#include <type_traits>

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

// 5 to 64 rows with the activations resident in registers.  Eight waves, each an eighth of the K steps of 64 (the
// last waves maybe fewer), load their part of the 16 RT activation rows once (8 CH steps at most: 32 RT CH registers)
// and then walk over the workgroup's column tiles of 16 (blockIdx.x, + gridDim.x, ...) in chunks of 8 K steps, the
// weights of the next chunk in flight while the matrix cores work on this one.  Against i8_stream_kernel the
// activations cross the caches once per workgroup instead of once per column tile, and the weight stream of a
// compute unit does not pause between tiles.  The eight partial tiles meet in LDS, one barrier per tile (two sets of
// partial sums in turn: a wave that writes set p again has passed the barrier of the tile in between, which every
// wave reaches only after it has read set p).  Exact i32 sums.
template <int RT, int CH>
__global__ __launch_bounds__(512) void i8_resident_kernel(
    const int8_t* __restrict__ xq, const int8_t* __restrict__ wq, const float* __restrict__ sx,
    const float* __restrict__ sw, const float* __restrict__ bias, int32_t* __restrict__ acc_out,
    float* __restrict__ y, uint32_t M, uint32_t K, uint32_t N) {
    __shared__ int32_t part[2][8][RT][4][64];                  // [set][wave][row tile][register][lane]
    // the wave index is made scalar: the K offsets of the loads below are then scalar work, one address register per tile
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t c = lane & 15, q = lane >> 4;
    const uint32_t tiles = (N + 15) / 16;
    const uint32_t steps = K / 64, ks = (steps + 7) / 8;       // ks <= 8 CH
    const uint32_t first = wave * ks;
    const uint32_t mine = first < steps ? min(ks, steps - first) : 0;   // K steps of this wave
    // byte offset of the wave's K step i; past the wave's last step some valid step, not multiplied
    auto koff = [&](uint32_t i) { return 64 * min(first + i, steps - 1); };
    // Buffer loads: the K offset rides in a scalar register, the lane's part (row and 16-byte piece, below 64 K) in one
    // vector register per operand, and rows past the end (of M, of N) read as zeros, by the range check on the lane's part.
    auto load = [](__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t k_off) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, k_off, 0));
    };
    v4i a[8 * CH][RT];
    {
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(xq), 0, (int)(M * K), 0x00020000);
#pragma unroll
        for (int i = 0; i < 8 * CH; i++)
#pragma unroll
            for (int t = 0; t < RT; t++) a[i][t] = load(rx, (16 * t + c) * K + 16 * q, koff(i));
    }
    v4i b[2][8];
    auto fetch = [&](auto buf, uint32_t tile, int ch) {
        const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<int8_t*>(wq) + (uint64_t)(16 * tile) * K, 0, (int)(min(16u, N - 16 * tile) * K), 0x00020000);
#pragma unroll
        for (int i = 0; i < 8; i++) b[decltype(buf)::value][i] = load(rw, c * K + 16 * q, koff(8 * ch + i));
    };
    // par: the buffer that holds the tile's first chunk; more: another tile follows (a path of its own for the last
    // tile, so that each path counts its loads in flight exactly)
    auto tile_of = [&](uint32_t tile, uint32_t set, auto par, auto more) {
        constexpr int P = decltype(par)::value;
        v4i acc[RT];
#pragma unroll
        for (int t = 0; t < RT; t++) acc[t] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int ch = 0; ch < CH; ch++) {
            // the loads of the next chunk start here, not earlier: the buffer they fill is free only now
            if (CH > 1) __builtin_amdgcn_sched_barrier(0);
            if (ch + 1 < CH) {
                if ((P + ch) & 1) fetch(std::integral_constant<int, 0>{}, tile, ch + 1);
                else fetch(std::integral_constant<int, 1>{}, tile, ch + 1);
            } else if constexpr (decltype(more)::value) {
                if ((P + ch) & 1) fetch(std::integral_constant<int, 0>{}, tile + gridDim.x, 0);
                else fetch(std::integral_constant<int, 1>{}, tile + gridDim.x, 0);
            }
#pragma unroll
            for (int i = 0; i < 8; i++)
                if ((uint32_t)(8 * ch + i) < mine) {
#pragma unroll
                    for (int t = 0; t < RT; t++)
                        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[8 * ch + i][t], b[(P + ch) & 1][i], acc[t], 0, 0, 0);
                }
        }
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) part[set][wave][t][r][lane] = acc[t][r];
        __syncthreads();
        // register r of lane l: row 4 (l / 16) + r, column l % 16 of the 16 x 16 tile; the waves take the 4 RT registers in turn
        const uint32_t col = 16 * tile + c;
        if (col < N) {
#pragma unroll
            for (uint32_t idx = wave; idx < 4 * RT; idx += 8) {
                const uint32_t t = idx >> 2, r = idx & 3, row = 16 * t + 4 * q + r;
                if (row >= M) continue;
                int32_t v = 0;
#pragma unroll
                for (int w = 0; w < 8; w++) v += part[set][w][t][r][lane];
                const uint64_t o = (uint64_t)row * N + col;
                if (acc_out) acc_out[o] = v;
                if (y) {
                    float f = __fmul_rn(__fmul_rn((float)v, sx[row]), sw[col]);
                    if (bias) f = __fadd_rn(f, bias[col]);
                    y[o] = f;
                }
            }
        }
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, CH & 1>;            // CH chunks later the first chunk sits in this buffer
    fetch(P0{}, blockIdx.x, 0);                                // blockIdx.x < tiles
    for (uint32_t tile = blockIdx.x;;) {
        if (tile + gridDim.x >= tiles) { tile_of(tile, 0, P0{}, std::false_type{}); break; }
        tile_of(tile, 0, P0{}, std::true_type{});
        tile += gridDim.x;
        if (tile + gridDim.x >= tiles) { tile_of(tile, 1, P1{}, std::false_type{}); break; }
        tile_of(tile, 1, P1{}, std::true_type{});
        tile += gridDim.x;
    }
}

// the fewest workgroups, one per compute unit at most, that keep the longest walk over column tiles as short
static uint32_t resident_grid(uint32_t n) {
    const uint32_t tiles = ceil_div(n, 16);
    return ceil_div(tiles, ceil_div(tiles, 256));
}

// which shapes i8_resident_kernel takes: K steps of 64, at least 6 of them per wave (fewer keep too little in flight) and
// at most 8 CH, with 32 RT CH <= 128 activation registers
bool i8_resident_takes(uint32_t m, uint32_t k, uint32_t n) {
    if (m < 5 || m > 64 || k % 64 != 0 || n == 0) return false;
    const uint32_t ks = ceil_div(k / 64, 8), ch = ceil_div(ks, 8), rt = ceil_div(m, 16);
    return ks >= 6 && (ch == 1 || (ch == 2 && rt <= 2) || (ch == 3 && rt == 1));
}

int i8_launch_resident(const int8_t* xq, const int8_t* wq, const float* sx, const float* sw, const float* bias, int32_t* acc,
                       float* y, uint32_t m, uint32_t k, uint32_t n, hipStream_t s) {
    const uint32_t ch = ceil_div(ceil_div(k / 64, 8), 8), rt = ceil_div(m, 16);
    const dim3 grid(resident_grid(n)), block(512);
#define RUMUS_RESIDENT(RT, CH) \
    hipLaunchKernelGGL((i8_resident_kernel<RT, CH>), grid, block, 0, s, xq, wq, sx, sw, bias, acc, y, m, k, n)
    if (ch == 1) {
        if (rt == 1) RUMUS_RESIDENT(1, 1);
        else if (rt == 2) RUMUS_RESIDENT(2, 1);
        else if (rt == 3) RUMUS_RESIDENT(3, 1);
        else RUMUS_RESIDENT(4, 1);
    } else if (ch == 2) {
        if (rt == 1) RUMUS_RESIDENT(1, 2);
        else RUMUS_RESIDENT(2, 2);
    } else {
        RUMUS_RESIDENT(1, 3);
    }
#undef RUMUS_RESIDENT
    return check_launch("i8_resident_kernel");
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
