// f32 x Q8 batches on the gfx950 i8 matrix cores, block scales applied inside the K loop
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
// which is 6 vector instructions per 4 accumulators.  With a fold at every K half that work, not the
// matrix cores, sets the pace (29 vector instructions per MFMA, vector ALU 78 % busy); blocks of 32 and
// 64 elements and large batches therefore take the f16 variant further down.
//
// The weights are read where they lie: a 16-byte chunk of a block sits 4 bytes past a 16-byte
// boundary at best because of the block headers, which the loads take; the headers with the
// block scales of the tile's columns ride along as 4-byte loads.
//
// Workgroup = WM x WN waves, block tile (32 WM) rows x (32 TN WN) columns, K step 64 bytes, NS
// LDS stages filled by direct-to-LDS loads (NS - 1 steps in flight: with a single step in flight
// a step took as long as a trip to memory, 1.3 to 1.7 us), rows of 64 bytes with the chunk
// swizzle of the W8A8 kernels, one barrier per step.  Problems with few tiles share K out over
// blockIdx.y as well and add the partial results in a second kernel, in a fixed order.
#include <hip/hip_fp16.h>

#include "i8_gemm.h"

namespace rumus {

constexpr int kQ8GemmPlanes = 4;

template <int WM, int WN, int TN, int NS>
__global__ __launch_bounds__(64 * WM * WN, 2) void q8_gemm_blocks_kernel(
    const int8_t* __restrict__ planes, const float* __restrict__ sx, const uint8_t* __restrict__ b,
    float* __restrict__ c, uint32_t M, uint32_t K, uint32_t N, uint32_t bs, uint32_t bs_magic,
    uint32_t stride_bytes, uint32_t bpc, uint32_t period, uint32_t tiles_m, uint32_t tiles_n, uint32_t steps_per) {
    constexpr int P = kQ8GemmPlanes;
    constexpr int WAVES = WM * WN;
    constexpr int BM = 32 * WM, BN = 32 * TN * WN;
    constexpr int A_ROWS = P * BM;
    constexpr int A_BYTES = A_ROWS * kBK, B_BYTES = BN * kBK, S_BYTES = 2 * BN * 4;
    constexpr int STAGE = A_BYTES + B_BYTES + S_BYTES;
    // a wave-wide 16-byte LDS-DMA load fills 16 rows of 64 bytes, a 4-byte one 64 header words
    constexpr int A_BLOCKS = A_ROWS / 16, B_BLOCKS = BN / 16, S_BLOCKS = 2 * BN / 64;
    constexpr int A_LOADS = (A_BLOCKS + WAVES - 1) / WAVES, B_LOADS = (B_BLOCKS + WAVES - 1) / WAVES;
    constexpr int S_LOADS = (S_BLOCKS + WAVES - 1) / WAVES;
    constexpr int LOADS = A_LOADS + B_LOADS + S_LOADS;
    static_assert(BN % 64 == 0, "a header load must stay inside one K half");
    static_assert((NS - 2) * LOADS <= 63, "more loads in flight than the counter holds");
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];   // [NS][STAGE]

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: LDS-DMA destinations are
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
    const uint32_t m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;

    // ---- global side of the LDS-DMA loads -----------------------------------------------------------
    // lane l of a 16-row block fetches row l/4, logical chunk (l%4) ^ swizzle(row) and lands in
    // physical chunk l%4; the swizzle only looks at row bits 1..3, the same for every block
    const uint32_t lr = lane >> 2, lc = ((lane & 3) ^ row_swizzle(lr)) & 3;
    const int8_t* pa[A_LOADS];
    const uint8_t* pb[B_LOADS];
    const uint8_t* ps[S_LOADS];
    uint32_t blk_a[A_LOADS], blk_b[B_LOADS], blk_s[S_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
        blk_a[i] = min(i * WAVES + wave, (uint32_t)A_BLOCKS - 1);
        const uint32_t row = blk_a[i] * 16 + lr;               // plane-major rows of the A tile
        const uint32_t plane = row / BM, r = row % BM;
        pa[i] = planes + ((uint64_t)plane * M + min(m0 + r, M - 1)) * K;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
        blk_b[i] = min(i * WAVES + wave, (uint32_t)B_BLOCKS - 1);
        const uint32_t col = min(n0 + blk_b[i] * 16 + lr, N - 1);
        pb[i] = b + (uint64_t)col * bpc * stride_bytes + 4;
    }
#pragma unroll
    for (int i = 0; i < S_LOADS; i++) {
        blk_s[i] = min(i * WAVES + wave, (uint32_t)S_BLOCKS - 1);
        const uint32_t col = min(n0 + (blk_s[i] * 64 + lane) % BN, N - 1);
        ps[i] = b + (uint64_t)col * bpc * stride_bytes;
    }
    // A K half past the end of K (K % 64 == 32) is fetched from the half before it: what it adds to
    // the integer sums is never folded in, or folded in with scale 0.
    auto issue = [&](uint32_t kt, uint32_t stage) {
        int8_t* base = lds + stage * STAGE;
        const uint32_t k0 = kt * kBK;
        uint32_t kpos = k0 + lc * 16;
        if (kpos >= K) kpos -= 32;
        const uint32_t blk = __umulhi(kpos, bs_magic);
        const uint32_t boff = blk * stride_bytes + (kpos - blk * bs);
#pragma unroll
        for (int i = 0; i < A_LOADS; i++)
            __builtin_amdgcn_global_load_lds((gptr_t)(pa[i] + kpos), (lptr_t)(base + blk_a[i] * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < B_LOADS; i++)
            __builtin_amdgcn_global_load_lds((gptr_t)(pb[i] + boff), (lptr_t)(base + A_BYTES + blk_b[i] * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < S_LOADS; i++) {
            uint32_t kh = k0 + 32 * (blk_s[i] * 64 / BN);
            if (kh >= K) kh -= 32;
            const uint32_t hb = __umulhi(kh, bs_magic);
            __builtin_amdgcn_global_load_lds((gptr_t)(ps[i] + (uint64_t)hb * stride_bytes),
                                             (lptr_t)(base + A_BYTES + B_BYTES + blk_s[i] * 256), 4, 0, 0);
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
    const uint32_t s_off = A_BYTES + B_BYTES + (wn * TN * 32 + fr) * 4;

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
    // ---- pipeline: NS - 1 K steps in flight, one barrier per step -------------------------------------
    // Every step issues exactly LOADS loads per wave, also past the end of K (the last step is then
    // fetched again into a stage nobody reads any more), so the counter arithmetic has no tail cases.
    // blockIdx.y picks the share of the K steps (a multiple of the fold period) this workgroup sums
    const uint32_t kt0 = blockIdx.y * steps_per, ksteps = min((K + kBK - 1) / kBK, kt0 + steps_per);
    uint32_t left = period;                                    // K halves until the next fold
#pragma unroll
    for (int s = 0; s < NS - 1; s++) issue(min(kt0 + s, ksteps - 1), s);
    uint32_t cur = 0;
    for (uint32_t kt = kt0; kt < ksteps; kt++) {
        // step kt has landed once only the NS-2 younger steps are outstanding; past the barrier every
        // wave has also finished reading the stage of step kt-1, which is refilled at once
        RUMUS_WAIT_VMCNT((NS - 2) * LOADS);
        __builtin_amdgcn_s_barrier();
        issue(min(kt + (NS - 1), ksteps - 1), cur == 0 ? NS - 1 : cur - 1);
        const int8_t* base = lds + cur * STAGE;
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
                    acc[p][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[p], bf[j], acc[p][j], 0, 0, 0);
            if (--left == 0) {
                left = period;
                const bool live = kt * kBK + 32 * s < K;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const uint32_t header = *reinterpret_cast<const uint32_t*>(base + s_off + (s * BN + j * 32) * 4);
                    const float s_lo = live ? __half2float(__ushort_as_half((unsigned short)(header & 0xFFFFu))) : 0.0f;
                    const float s_hi = s_lo * 16384.0f;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int lo = acc[1][j][r] * 128 + acc[0][j][r];
                        const int hi = acc[3][j][r] * 128 + acc[2][j][r];
                        out[j][r] = fmaf((float)hi, s_hi, out[j][r]);
                        out[j][r] = fmaf((float)lo, s_lo, out[j][r]);
#pragma unroll
                        for (int p = 0; p < P; p++) acc[p][j][r] = 0;
                    }
                }
            }
        }
        cur = cur + 1 == NS ? 0 : cur + 1;
    }
    RUMUS_WAIT_VMCNT(0);         // no LDS-DMA write may outlive the workgroup

    // ---- rows back to their scale: register r of lane l is row 8 (r/4) + 4 (l/32) + r%4, column l%32 ----
    const uint32_t col_l = lane & 31, row_l = (lane >> 5) * 4;
    c += (uint64_t)blockIdx.y * M * N;                         // partial sums of K share y when K is split
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

// ---------------------------------------------------------------------------------------------------
// The same tiles on the f16 matrix cores, for small blocks.  With a fold at every 32 k the integer
// variant above spends its time in the vector ALU (29 instructions per MFMA).  Here the activations
// are two f16 planes, x f = hi + lo (22 bits of every element, f a power of two per row that puts the
// row maximum below 2^15), the block's bytes become f16 in registers (exact: u = q + 128 is spliced
// into the mantissa of 1024 + u, then 1152 is subtracted two at a time), v_mfma_f32_32x32x16_f16
// sums a block in f32 (every product is exact, the sum is rounded like any f32 sum), and the fold is
// one multiply-add per accumulator with the block's scale.  A K step is 64 elements: two "pairs" of
// 32, each a ds_read_b128 of B (lane half h holds k = 16 h .. 16 h + 15 of the pair: bytes 0..7 feed
// the first MFMA, 8..15 the second) against 16-byte pieces of the A rows in the same k order.
// LDS: A as [2 pairs][2 planes x BM rows][64 bytes], B and the headers as above.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

// 16 int8 (four words) -> two B operands of 8 f16
__device__ __forceinline__ void q8_bytes_to_f16(const v4i& w, v8h& first, v8h& second) {
    const v2h off = {(_Float16)1152.0f, (_Float16)1152.0f};
    v2h h[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t u = (uint32_t)w[i] ^ 0x80808080u;                  // q + 128 in every byte
        const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);   // (0x64, u1, 0x64, u0)
        const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);   // (0x64, u3, 0x64, u2)
        h[2 * i] = __builtin_bit_cast(v2h, lo) - off;
        h[2 * i + 1] = __builtin_bit_cast(v2h, hi) - off;
    }
    first = v8h{h[0][0], h[0][1], h[1][0], h[1][1], h[2][0], h[2][1], h[3][0], h[3][1]};
    second = v8h{h[4][0], h[4][1], h[5][0], h[5][1], h[6][0], h[6][1], h[7][0], h[7][1]};
}

template <int WM, int WN, int TN, int NS, bool EVERY>
__global__ __launch_bounds__(64 * WM * WN, 2) void q8_gemm_blocks_f16_kernel(
    const _Float16* __restrict__ planes, const float* __restrict__ sx, const uint8_t* __restrict__ b,
    float* __restrict__ c, uint32_t M, uint32_t K, uint32_t N, uint32_t bs, uint32_t bs_magic,
    uint32_t stride_bytes, uint32_t bpc, uint32_t period, uint32_t tiles_m, uint32_t tiles_n, uint32_t steps_per) {
    constexpr int P = 2;                                       // hi and lo
    constexpr int WAVES = WM * WN;
    constexpr int BM = 32 * WM, BN = 32 * TN * WN;
    constexpr int A_ROWS = P * BM;                             // per pair
    constexpr int A_PAIR = A_ROWS * kBK, A_BYTES = 2 * A_PAIR, B_BYTES = BN * kBK, S_BYTES = 2 * BN * 4;
    constexpr int STAGE = A_BYTES + B_BYTES + S_BYTES;
    constexpr int A_BLOCKS = 2 * A_ROWS / 16, B_BLOCKS = BN / 16, S_BLOCKS = 2 * BN / 64;
    constexpr int A_LOADS = (A_BLOCKS + WAVES - 1) / WAVES, B_LOADS = (B_BLOCKS + WAVES - 1) / WAVES;
    constexpr int S_LOADS = (S_BLOCKS + WAVES - 1) / WAVES;
    constexpr int LOADS = A_LOADS + B_LOADS + S_LOADS;
    static_assert(BN % 64 == 0, "a header load must stay inside one pair");
    static_assert((NS - 2) * LOADS <= 63, "more loads in flight than the counter holds");
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];   // [NS][STAGE]

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
    const uint32_t m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;

    // ---- global side of the LDS-DMA loads -----------------------------------------------------------
    const uint32_t lr = lane >> 2, lc = ((lane & 3) ^ row_swizzle(lr)) & 3;
    const int8_t* pa[A_LOADS];
    const uint8_t* pb[B_LOADS];
    const uint8_t* ps[S_LOADS];
    uint32_t blk_a[A_LOADS], pair_a[A_LOADS], blk_b[B_LOADS], blk_s[S_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
        blk_a[i] = min(i * WAVES + wave, (uint32_t)A_BLOCKS - 1);
        pair_a[i] = blk_a[i] / (A_ROWS / 16);
        const uint32_t row = (blk_a[i] % (A_ROWS / 16)) * 16 + lr;   // plane-major rows of the pair
        const uint32_t plane = row / BM, r = row % BM;
        // 16-byte piece lc of the pair's 32 elements
        pa[i] = reinterpret_cast<const int8_t*>(planes + ((uint64_t)plane * M + min(m0 + r, M - 1)) * K) + lc * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
        blk_b[i] = min(i * WAVES + wave, (uint32_t)B_BLOCKS - 1);
        const uint32_t col = min(n0 + blk_b[i] * 16 + lr, N - 1);
        pb[i] = b + (uint64_t)col * bpc * stride_bytes + 4;
    }
#pragma unroll
    for (int i = 0; i < S_LOADS; i++) {
        blk_s[i] = min(i * WAVES + wave, (uint32_t)S_BLOCKS - 1);
        const uint32_t col = min(n0 + (blk_s[i] * 64 + lane) % BN, N - 1);
        ps[i] = b + (uint64_t)col * bpc * stride_bytes;
    }
    // A pair past the end of K (K % 64 == 32) is fetched from the pair before it (finite values): what
    // it adds to the sums is never folded in, or folded in with scale 0.
    auto issue = [&](uint32_t kt, uint32_t stage) {
        int8_t* base = lds + stage * STAGE;
        const uint32_t k0 = kt * 64;
        uint32_t kpos = k0 + lc * 16;
        if (kpos >= K) kpos -= 32;
        const uint32_t blk = __umulhi(kpos, bs_magic);
        const uint32_t boff = blk * stride_bytes + (kpos - blk * bs);
#pragma unroll
        for (int i = 0; i < A_LOADS; i++) {
            uint32_t ka = k0 + 32 * pair_a[i];
            if (ka >= K) ka -= 32;
            __builtin_amdgcn_global_load_lds((gptr_t)(pa[i] + (uint64_t)ka * 2), (lptr_t)(base + blk_a[i] * 1024), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; i++)
            __builtin_amdgcn_global_load_lds((gptr_t)(pb[i] + boff), (lptr_t)(base + A_BYTES + blk_b[i] * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < S_LOADS; i++) {
            uint32_t kh = k0 + 32 * (blk_s[i] * 64 / BN);
            if (kh >= K) kh -= 32;
            const uint32_t hb = __umulhi(kh, bs_magic);
            __builtin_amdgcn_global_load_lds((gptr_t)(ps[i] + (uint64_t)hb * stride_bytes),
                                             (lptr_t)(base + A_BYTES + B_BYTES + blk_s[i] * 256), 4, 0, 0);
        }
    };

    // ---- fragment read addressing ------------------------------------------------------------------
    // lane (row or column fr, half fh); MFMA i of a pair takes k = 16 fh + 8 i .. + 7 of the pair
    const uint32_t fr = lane & 31, fh = lane >> 5, fsw = row_swizzle(fr);
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; i++) a_off[i] = (wm * 32 + fr) * kBK + (((2 * fh + i) ^ fsw) & 3) * 16;
#pragma unroll
    for (int s = 0; s < 2; s++) b_off[s] = A_BYTES + (wn * 32 * TN + fr) * kBK + (((2 * s + fh) ^ fsw) & 3) * 16;
    const uint32_t s_off = A_BYTES + B_BYTES + (wn * TN * 32 + fr) * 4;

    v16f acc[TN];
    float out[TN][16];
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            out[j][r] = 0.0f;
            acc[j][r] = 0.0f;
        }
    const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    const uint32_t kt0 = blockIdx.y * steps_per, ksteps = min((K + 63) / 64, kt0 + steps_per);
    uint32_t left = period;                                    // pairs until the next fold
#pragma unroll
    for (int s = 0; s < NS - 1; s++) issue(min(kt0 + s, ksteps - 1), s);
    uint32_t cur = 0;
    for (uint32_t kt = kt0; kt < ksteps; kt++) {
        RUMUS_WAIT_VMCNT((NS - 2) * LOADS);
        __builtin_amdgcn_s_barrier();
        issue(min(kt + (NS - 1), ksteps - 1), cur == 0 ? NS - 1 : cur - 1);
        const int8_t* base = lds + cur * STAGE;
        // The bytes of the step's second pair become f16 while the MFMAs of its first pair run (a wave issues nothing
        // while it waits to issue an MFMA, so conversion and MFMAs of the same pair one after the other leave the
        // vector ALU idle during the MFMAs and the matrix cores idle during the conversion).
        v8h bf[2][TN][2];
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const v4i w = *reinterpret_cast<const v4i*>(base + b_off[0] + j * 32 * kBK);
            q8_bytes_to_f16(w, bf[0][j][0], bf[0][j][1]);
        }
#pragma unroll
        for (int s = 0; s < 2; s++) {
            v8h af[P][2];
#pragma unroll
            for (int p = 0; p < P; p++)
#pragma unroll
                for (int i = 0; i < 2; i++)
                    af[p][i] = *reinterpret_cast<const v8h*>(base + s * A_PAIR + a_off[i] + p * BM * kBK);
            if (s == 0) {
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const v4i w = *reinterpret_cast<const v4i*>(base + b_off[1] + j * 32 * kBK);
                    q8_bytes_to_f16(w, bf[1][j][0], bf[1][j][1]);
                }
            }
            bool fold = EVERY;
            if (!EVERY) {
                left--;
                fold = left == 0;
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[0][0], bf[s][j][0], EVERY ? zero : acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[0][1], bf[s][j][1], acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[1][0], bf[s][j][0], acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[1][1], bf[s][j][1], acc[j], 0, 0, 0);
            }
            if (s == 0) {
#pragma unroll
                for (int i = 0; i < 4 * TN; i++) {             // an MFMA, then its share of the second pair's conversion
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
                }
            }
            if (fold) {
                left = period;
                const bool live = kt * 64 + 32 * s < K;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const uint32_t header = *reinterpret_cast<const uint32_t*>(base + s_off + (s * BN + j * 32) * 4);
                    const float sc = live ? __half2float(__ushort_as_half((unsigned short)(header & 0xFFFFu))) : 0.0f;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        out[j][r] = fmaf(acc[j][r], sc, out[j][r]);
                        if (!EVERY) acc[j][r] = 0.0f;
                    }
                }
            }
        }
        cur = cur + 1 == NS ? 0 : cur + 1;
    }
    RUMUS_WAIT_VMCNT(0);         // no LDS-DMA write may outlive the workgroup

    const uint32_t col_l = lane & 31, row_l = (lane >> 5) * 4;
    c += (uint64_t)blockIdx.y * M * N;                         // partial sums of K share y when K is split
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

// c = sum over the K shares of their partial results, in share order
__global__ __launch_bounds__(256) void q8_gemm_add_shares_kernel(const float* __restrict__ part, float* __restrict__ c,
                                                                 uint32_t count, uint32_t shares) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    float v = part[i];
    for (uint32_t z = 1; z < shares; z++) v += part[(uint64_t)z * count + i];
    c[i] = v;
}

template <int WM, int WN, int TN, int NS>
static int launch_q8_gemm_blocks(const int8_t* planes, const float* sx, const uint32_t* b, float* c, uint32_t m,
                                 uint32_t k, uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, uint32_t period,
                                 float* part, uint32_t max_shares, hipStream_t s) {
    constexpr size_t lds_bytes = (size_t)NS * ((kQ8GemmPlanes * 32 * WM + 32 * TN * WN) * kBK + 2 * 32 * TN * WN * 4);
    static_assert(lds_bytes <= 160 * 1024, "more LDS than a compute unit has");
    static bool attr_set = false;   // benign race: setting the attribute is idempotent
    if (!attr_set && lds_bytes > 64 * 1024) {
        if (int rc = check_hip(hipFuncSetAttribute(
                reinterpret_cast<const void*>(&q8_gemm_blocks_kernel<WM, WN, TN, NS>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes), "hipFuncSetAttribute"))
            return rc;
        attr_set = true;
    }
    const uint32_t tm = ceil_div(m, 32 * WM), tn = ceil_div(n, 32 * TN * WN);
    const uint32_t magic = (uint32_t)((0x100000000ull + bs - 1) / bs);
    // too few tiles for the chip: K is shared out as well, in whole fold periods of at least 8 steps
    const uint32_t ksteps = ceil_div(k, kBK);
    uint32_t shares = 1, steps_per = ksteps;
    if (part && tm * tn < 256) {
        const uint32_t unit = period * ceil_div(8, period);
        shares = min(min(max_shares, 512 / (tm * tn)), max(1u, ksteps / unit));
        steps_per = ceil_div(ceil_div(ksteps, shares), unit) * unit;
        shares = ceil_div(ksteps, steps_per);
    }
    hipLaunchKernelGGL((q8_gemm_blocks_kernel<WM, WN, TN, NS>), dim3(tm * tn, shares), dim3(64 * WM * WN),
                       lds_bytes, s, planes, sx, reinterpret_cast<const uint8_t*>(b), shares > 1 ? part : c, m, k, n, bs,
                       magic, stride * 4, bpc, period, tm, tn, steps_per);
    if (int rc = check_launch("q8_gemm_blocks_kernel")) return rc;
    if (shares == 1) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(q8_gemm_add_shares_kernel, dim3(ceil_div(m * n, 256)), dim3(256), 0, s, part, c, m * n, shares);
    return check_launch("q8_gemm_add_shares_kernel");
}

template <int WM, int WN, int TN, int NS, bool EVERY>
static int launch_q8_gemm_blocks_f16(const _Float16* planes, const float* sx, const uint32_t* b, float* c, uint32_t m,
                                     uint32_t k, uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, float* part,
                                     uint32_t max_shares, hipStream_t s) {
    constexpr size_t lds_bytes = (size_t)NS * ((4 * 32 * WM + 32 * TN * WN) * kBK + 2 * 32 * TN * WN * 4);
    static_assert(lds_bytes <= 160 * 1024, "more LDS than a compute unit has");
    static bool attr_set = false;   // benign race: setting the attribute is idempotent
    if (!attr_set && lds_bytes > 64 * 1024) {
        if (int rc = check_hip(hipFuncSetAttribute(
                reinterpret_cast<const void*>(&q8_gemm_blocks_f16_kernel<WM, WN, TN, NS, EVERY>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes), "hipFuncSetAttribute"))
            return rc;
        attr_set = true;
    }
    const uint32_t tm = ceil_div(m, 32 * WM), tn = ceil_div(n, 32 * TN * WN);
    const uint32_t magic = (uint32_t)((0x100000000ull + bs - 1) / bs);
    const uint32_t period = bs / 32;                           // pairs of 32 k per block: f32 sums need no earlier fold
    const uint32_t ksteps = ceil_div(k, 64);
    uint32_t shares = 1, steps_per = ksteps;
    if (part && tm * tn < 256) {
        const uint32_t unit = period * ceil_div(8, period);
        shares = min(min(max_shares, 512 / (tm * tn)), max(1u, ksteps / unit));
        steps_per = ceil_div(ceil_div(ksteps, shares), unit) * unit;
        shares = ceil_div(ksteps, steps_per);
    }
    hipLaunchKernelGGL((q8_gemm_blocks_f16_kernel<WM, WN, TN, NS, EVERY>), dim3(tm * tn, shares), dim3(64 * WM * WN),
                       lds_bytes, s, planes, sx, reinterpret_cast<const uint8_t*>(b), shares > 1 ? part : c, m, k, n, bs,
                       magic, stride * 4, bpc, period, tm, tn, steps_per);
    if (int rc = check_launch("q8_gemm_blocks_f16_kernel")) return rc;
    if (shares == 1) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(q8_gemm_add_shares_kernel, dim3(ceil_div(m * n, 256)), dim3(256), 0, s, part, c, m * n, shares);
    return check_launch("q8_gemm_add_shares_kernel");
}

#define RUMUS_Q8_LAUNCH_F16(WM, WN, TN, NS, EV) \
    launch_q8_gemm_blocks_f16<WM, WN, TN, NS, EV>(planes, sx, b, c, m, k, n, bs, stride, bpc, part, max_shares, s)

// planes: [2][m][k] f16 (hi, lo), sx: [m] the rows' 1 / f.  Same preconditions as q8_gemm_blocks.
// Measured at 4096 x 11008: up to 32 rows one 32-row tile per workgroup, beyond that 64 x 128 tiles,
// two workgroups per compute unit (2048 rows, 32-element blocks: 600-645 us; 32 x 128 and 64 x 64
// tiles with three workgroups per compute unit 720-865 us, 64 x 256 and 128 x 128 tiles with one
// workgroup of eight waves 627-650 us, and slower than the choice at 512 rows).
int q8_gemm_blocks_f16(const _Float16* planes, const float* sx, const uint32_t* b, float* c, uint32_t m, uint32_t k,
                       uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, float* part, uint32_t max_shares,
                       hipStream_t s) {
    if (bs == 32) return m <= 32 ? RUMUS_Q8_LAUNCH_F16(1, 4, 1, 4, true) : RUMUS_Q8_LAUNCH_F16(2, 2, 2, 3, true);
    return m <= 32 ? RUMUS_Q8_LAUNCH_F16(1, 4, 1, 4, false) : RUMUS_Q8_LAUNCH_F16(2, 2, 2, 3, false);
}

// planes: [4][m][k] digit planes, sx: [m] the rows' 1 / f.  Needs bs % 32 == 0, k % bs == 0 and
// k * bs < 2^32 (the division by bs is a multiply).  part: room for max_shares x m x n partial
// results (or null): small problems share K out over workgroups as well.  One 32-row tile per
// workgroup: the caller sends batches beyond 64 rows to the f16 variant.
int q8_gemm_blocks(const int8_t* planes, const float* sx, const uint32_t* b, float* c, uint32_t m, uint32_t k,
                   uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, float* part, uint32_t max_shares,
                   hipStream_t s) {
    // fold period in K halves: the largest divisor of the block's halves that keeps 1024 k between folds
    uint32_t period = 1;
    for (uint32_t d = 32; d > 1; d--)
        if ((bs / 32) % d == 0) { period = d; break; }
    return launch_q8_gemm_blocks<1, 4, 1, 4>(planes, sx, b, c, m, k, n, bs, stride, bpc, period, part, max_shares, s);
}

}  // namespace rumus
