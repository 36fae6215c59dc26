// f32 x Q8 batches on the gfx950 i8 matrix cores when a column holds several blocks
// (matmul_q8.wgsl:37-96 computes the same sums one output per thread).
//
//   c[m, n] = sum over the blocks kb of column n:  s[n, kb] * sum_{k in kb} x[m, k] * q[n, k]
//
// The activations arrive as four signed 7-bit digit planes (q8_split_rows_kernel in q8.hip):
// x f = d0 + 128 d1 + 128^2 d2 + 128^3 d3 with f a power of two per row, so every digit plane
// times the block's bytes is an exact i8 x i8 -> i32 MFMA sum.  A wave owns 32 rows x all four
// planes x TN*32 columns; at the end of a block (or earlier, every `period` K halves of 32, so
// that the integers below stay inside 32 bits) it folds the four i32 tiles into the f32 result:
//   lo = 128 acc1 + acc0,  hi = 128 acc3 + acc2            (integer, exact: |.| < 2^31 for 1024 k)
//   out += f32(hi) * (2^14 s) ;  out += f32(lo) * s        (two fused multiply-adds)
// which is 6 vector instructions per 4 accumulators.  With 32-element blocks that work, not the
// matrix cores, sets the pace (96 instructions per 4 MFMAs and column tile).
//
// The weights are read where they lie: a 16-byte chunk of a block sits 4 bytes past a 4-byte
// boundary because of the block header, which global loads take; the block scale of a lane's
// column comes out of the same cache lines one K step ahead of its use.
//
// Workgroup = WM x WN waves, block tile (32 WM) rows x (32 TN WN) columns, K step 64 bytes, two
// LDS stages (global -> registers -> LDS of step t+1 under the MFMAs of step t), rows of 64 bytes
// with the chunk swizzle of the W8A8 kernels.
#include <hip/hip_fp16.h>

#include "i8_gemm.h"

namespace rumus {

typedef int v4i_a4 __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kQ8GemmPlanes = 4;

template <int WM, int WN, int TN, bool EVERY>
__global__ __launch_bounds__(64 * WM * WN, 2) void q8_gemm_blocks_kernel(
    const int8_t* __restrict__ planes, const float* __restrict__ sx, const uint8_t* __restrict__ b,
    float* __restrict__ c, uint32_t M, uint32_t K, uint32_t N, uint32_t bs, uint32_t bs_magic,
    uint32_t stride_bytes, uint32_t bpc, uint32_t period, uint32_t tiles_m, uint32_t tiles_n) {
    constexpr int P = kQ8GemmPlanes;
    constexpr int T = 64 * WM * WN;
    constexpr int BM = 32 * WM, BN = 32 * TN * WN;
    constexpr int A_ROWS = P * BM;
    constexpr int A_BYTES = A_ROWS * kBK, B_BYTES = BN * kBK;
    constexpr int ROWS_PER_PASS = T / 4;                       // 4 chunks of 16 bytes per row
    constexpr int A_LOADS = A_ROWS / ROWS_PER_PASS, B_LOADS = BN / ROWS_PER_PASS;
    static_assert(A_ROWS % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile does not divide over the threads");
    __shared__ __attribute__((aligned(16))) int8_t lds[2][A_BYTES + B_BYTES];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
    const uint32_t m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;

    // ---- global -> LDS staging ----------------------------------------------------------------
    const uint32_t ld_row = tid >> 2, ld_c = tid & 3;
    const uint32_t ld_lds = ld_row * kBK + ((ld_c ^ row_swizzle(ld_row)) & 3) * 16;   // ROWS_PER_PASS % 16 == 0
    const int8_t* pa[A_LOADS];
    const uint8_t* pb[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
        const uint32_t lr = ld_row + ROWS_PER_PASS * i;        // plane-major rows of the A tile
        const uint32_t plane = lr / BM, r = lr % BM;
        pa[i] = planes + ((uint64_t)plane * M + min(m0 + r, M - 1)) * K + ld_c * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
        const uint32_t col = min(n0 + ld_row + ROWS_PER_PASS * i, N - 1);
        pb[i] = b + (uint64_t)col * bpc * stride_bytes + 4;
    }
    v4i ga[A_LOADS], gb[B_LOADS];
    auto load_global = [&](uint32_t k0) {
        const uint32_t kpos = k0 + ld_c * 16;
        const bool ok = kpos < K;                              // K % 32 == 0: a chunk is all-in or all-out
        const uint32_t blk = __umulhi(kpos, bs_magic);
        const uint32_t boff = blk * stride_bytes + (kpos - blk * bs);
#pragma unroll
        for (int i = 0; i < A_LOADS; i++)
            ga[i] = ok ? *reinterpret_cast<const v4i*>(pa[i] + k0) : v4i{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) {
            if (ok) {
                const v4i_a4 v = *reinterpret_cast<const v4i_a4*>(pb[i] + boff);
                gb[i] = v4i{v.x, v.y, v.z, v.w};
            } else {
                gb[i] = v4i{0, 0, 0, 0};
            }
        }
    };
    auto store_lds = [&](int stage) {
        int8_t* base = lds[stage];
#pragma unroll
        for (int i = 0; i < A_LOADS; i++)
            *reinterpret_cast<v4i*>(base + ld_lds + i * ROWS_PER_PASS * kBK) = ga[i];
#pragma unroll
        for (int i = 0; i < B_LOADS; i++)
            *reinterpret_cast<v4i*>(base + A_BYTES + ld_lds + i * ROWS_PER_PASS * kBK) = gb[i];
    };

    // ---- block scales of this lane's columns -----------------------------------------------------
    const uint32_t col_l = lane & 31;
    const uint8_t* ph[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const uint32_t col = min(n0 + (wn * TN + j) * 32 + col_l, N - 1);
        ph[j] = b + (uint64_t)col * bpc * stride_bytes;
    }
    float sc_cur[2][TN], sc_nxt[2][TN];
    auto load_scales = [&](uint32_t k0, float (&sc)[2][TN]) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t kpos = k0 + 32 * h;
            const uint32_t blk = min(__umulhi(kpos, bs_magic), bpc - 1);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const uint32_t header = *reinterpret_cast<const uint32_t*>(ph[j] + (uint64_t)blk * stride_bytes);
                const float s = __half2float(__ushort_as_half((unsigned short)(header & 0xFFFFu)));
                sc[h][j] = kpos < K ? s : 0.0f;
            }
        }
    };

    // ---- fragment read addressing ------------------------------------------------------------------
    const uint32_t fr = lane & 31, fh = lane >> 5, fsw = row_swizzle(fr);
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
        const uint32_t chunk = ((2 * s + fh) ^ fsw) & 3;
        a_off[s] = (wm * 32 + fr) * kBK + chunk * 16;
        b_off[s] = A_BYTES + (wn * 32 * TN + fr) * kBK + chunk * 16;
    }

    v16i acc[P][TN];
    float out[TN][16];
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int r = 0; r < 16; r++) out[j][r] = 0.0f;
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[p][j][r] = 0;
    }
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    const uint32_t ksteps = (K + kBK - 1) / kBK;
    uint32_t left = period;                                    // K halves until the next fold
    load_global(0);
    load_scales(0, sc_cur);
    store_lds(0);
    __syncthreads();

    for (uint32_t kt = 0; kt < ksteps; kt++) {
        const int cur = kt & 1;
        const bool more = kt + 1 < ksteps;
        if (more) {
            load_global((kt + 1) * kBK);
            load_scales((kt + 1) * kBK, sc_nxt);
        }
        const int8_t* base = lds[cur];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            v4i af[P], bf[TN];
#pragma unroll
            for (int p = 0; p < P; p++)
                af[p] = *reinterpret_cast<const v4i*>(base + a_off[s] + p * BM * kBK);
#pragma unroll
            for (int j = 0; j < TN; j++)
                bf[j] = *reinterpret_cast<const v4i*>(base + b_off[s] + j * 32 * kBK);
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int p = 0; p < P; p++)
                    acc[p][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[p], bf[j], EVERY ? zero : acc[p][j], 0, 0, 0);
            bool fold = EVERY;
            if (!EVERY) {
                left--;
                fold = left == 0;
            }
            if (fold) {
                left = period;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const float s_lo = sc_cur[s][j], s_hi = s_lo * 16384.0f;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int lo = acc[1][j][r] * 128 + acc[0][j][r];
                        const int hi = acc[3][j][r] * 128 + acc[2][j][r];
                        out[j][r] = fmaf((float)hi, s_hi, out[j][r]);
                        out[j][r] = fmaf((float)lo, s_lo, out[j][r]);
                        if (!EVERY) {
#pragma unroll
                            for (int p = 0; p < P; p++) acc[p][j][r] = 0;
                        }
                    }
                }
            }
        }
        if (more) store_lds(cur ^ 1);
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int j = 0; j < TN; j++) sc_cur[h][j] = sc_nxt[h][j];
    }

    // ---- rows back to their scale: register r of lane l is row 8 (r/4) + 4 (l/32) + r%4, column l%32 ----
    const uint32_t row_l = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const uint32_t col = n0 + (wn * TN + j) * 32 + col_l;
        if (col >= N) continue;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t row = m0 + wm * 32 + 8 * (r / 4) + row_l + (r % 4);
            if (row < M) c[(uint64_t)row * N + col] = out[j][r] * sx[row];
        }
    }
}

template <int WM, int WN, int TN, bool EVERY>
static int launch_q8_gemm_blocks(const int8_t* planes, const float* sx, const uint32_t* b, float* c, uint32_t m,
                                 uint32_t k, uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, uint32_t period,
                                 hipStream_t s) {
    const uint32_t tm = ceil_div(m, 32 * WM), tn = ceil_div(n, 32 * TN * WN);
    const uint32_t magic = (uint32_t)((0x100000000ull + bs - 1) / bs);
    hipLaunchKernelGGL((q8_gemm_blocks_kernel<WM, WN, TN, EVERY>), dim3(tm * tn), dim3(64 * WM * WN), 0, s, planes, sx,
                       reinterpret_cast<const uint8_t*>(b), c, m, k, n, bs, magic, stride * 4, bpc, period, tm, tn);
    return check_launch("q8_gemm_blocks_kernel");
}

// planes: [4][m][k] digit planes, sx: [m] the rows' 1 / f.  Needs bs % 32 == 0, k % bs == 0 and
// k * bs < 2^32 (the division by bs is a multiply).
int q8_gemm_blocks(const int8_t* planes, const float* sx, const uint32_t* b, float* c, uint32_t m, uint32_t k,
                   uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, hipStream_t s) {
    // fold period in K halves: the largest divisor of the block's halves that keeps 1024 k between folds
    uint32_t period = 1;
    for (uint32_t d = 32; d > 1; d--)
        if ((bs / 32) % d == 0) { period = d; break; }
    const bool small = m <= 32;
    if (period == 1) {
        // a fold per MFMA group: two column tiles per wave would not fit the registers next to the staging
        if (small) return launch_q8_gemm_blocks<1, 2, 1, true>(planes, sx, b, c, m, k, n, bs, stride, bpc, period, s);
        return launch_q8_gemm_blocks<2, 2, 1, true>(planes, sx, b, c, m, k, n, bs, stride, bpc, period, s);
    }
    if (small) return launch_q8_gemm_blocks<1, 2, 1, false>(planes, sx, b, c, m, k, n, bs, stride, bpc, period, s);
    if ((uint64_t)ceil_div(m, 64) * ceil_div(n, 128) >= 256)
        return launch_q8_gemm_blocks<2, 2, 2, false>(planes, sx, b, c, m, k, n, bs, stride, bpc, period, s);
    return launch_q8_gemm_blocks<2, 2, 1, false>(planes, sx, b, c, m, k, n, bs, stride, bpc, period, s);
}

}  // namespace rumus
