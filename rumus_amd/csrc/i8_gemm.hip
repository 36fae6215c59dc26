// W8A8 INT8 GEMM on the gfx950 i8 matrix cores.
//
//   acc[m,n] = sum_k xq[m,k] * wq[n,k]        (i32, exact)
//   y[m,n]   = (f32(acc) * sx[m]) * sw[n] (+ bias[n])
//
// Both operands are K-contiguous, which is the layout the MFMA operands want:
// v_mfma_i32_32x32x32_i8 takes 16 consecutive K bytes of one row per lane
// (lane l: row l%32, K half l/32) for A and for B alike, so the same 128-bit
// LDS read feeds either operand and any K order is fine as long as A and B
// agree (integer sums are order-independent, hence bit-exact).
//
// Workgroup = 4 waves (2x2), block tile (64*TM) x (64*TN), K step 64 bytes,
// two LDS stages: global -> registers -> LDS for step t+1 overlaps the MFMAs of
// step t; one barrier per step.  LDS rows are 64 bytes with the 16-byte chunk
// index XOR-swizzled by a function of row bits 1..3, chosen so that the
// 128-bit fragment reads (consecutive lanes = consecutive rows, same chunk) hit
// distinct 16-byte bank groups whether the LDS serves them 8 lanes per 128
// bytes or 16 lanes per 256 bytes; the 128-bit writes cover whole rows and are
// conflict-free under any per-row permutation.
#include "i8_gemm.h"

namespace rumus {

template <int TM, int TN, int OCC>
__global__ __launch_bounds__(256, OCC) void i8_gemm_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ B, const float* __restrict__ sx,
    const float* __restrict__ sw, const float* __restrict__ bias, int32_t* __restrict__ acc_out,
    float* __restrict__ y, uint32_t M, uint32_t K, uint32_t N, uint32_t tiles_m, uint32_t tiles_n) {
    constexpr int BM = 64 * TM, BN = 64 * TN;
    constexpr int A_BYTES = BM * kBK, B_BYTES = BN * kBK;
    constexpr int A_LOADS = BM / 64, B_LOADS = BN / 64;  // 16-byte chunks per thread per stage
    __shared__ __attribute__((aligned(16))) int8_t lds[2][A_BYTES + B_BYTES];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;

    // XCD-contiguous tile order, M fastest: the tiles an XCD runs together
    // share their B panels and the (small) set of A panels in its L2.
    const uint32_t tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
    const uint32_t m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;

    // ---- global -> LDS staging assignment --------------------------------
    const uint32_t ld_row = tid >> 2, ld_c = tid & 3;
    const uint32_t ld_lds = ld_row * kBK + ((ld_c ^ row_swizzle(ld_row)) & 3) * 16;
    const int8_t* pa[A_LOADS];
    const int8_t* pb[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
        uint32_t r = min(m0 + ld_row + 64 * i, M - 1);
        pa[i] = A + (uint64_t)r * K + ld_c * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
        uint32_t r = min(n0 + ld_row + 64 * i, N - 1);
        pb[i] = B + (uint64_t)r * K + ld_c * 16;
    }
    v4i ga[A_LOADS], gb[B_LOADS];

    auto load_global = [&](uint32_t k0) {
        const bool ok = k0 + ld_c * 16 < K;  // K % 16 == 0: a chunk is all-in or all-out
#pragma unroll
        for (int i = 0; i < A_LOADS; i++)
            ga[i] = ok ? *reinterpret_cast<const v4i*>(pa[i] + k0) : v4i{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < B_LOADS; i++)
            gb[i] = ok ? *reinterpret_cast<const v4i*>(pb[i] + k0) : v4i{0, 0, 0, 0};
    };
    auto store_lds = [&](int stage) {
        int8_t* base = lds[stage];
#pragma unroll
        for (int i = 0; i < A_LOADS; i++)
            *reinterpret_cast<v4i*>(base + ld_lds + i * 64 * kBK) = ga[i];
#pragma unroll
        for (int i = 0; i < B_LOADS; i++)
            *reinterpret_cast<v4i*>(base + A_BYTES + ld_lds + i * 64 * kBK) = gb[i];
    };

    // ---- fragment read addressing ------------------------------------------
    const uint32_t fr = lane & 31, fh = lane >> 5, fsw = row_swizzle(fr);
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
        uint32_t chunk = ((2 * s + fh) ^ fsw) & 3;
        a_off[s] = (wm * 32 * TM + fr) * kBK + chunk * 16;
        b_off[s] = A_BYTES + (wn * 32 * TN + fr) * kBK + chunk * 16;
    }

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    const uint32_t ksteps = (K + kBK - 1) / kBK;
    load_global(0);
    store_lds(0);
    __syncthreads();

    for (uint32_t kt = 0; kt < ksteps; kt++) {
        const int cur = kt & 1;
        const bool more = kt + 1 < ksteps;
        if (more) load_global((kt + 1) * kBK);
        const int8_t* base = lds[cur];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            v4i af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                af[i] = *reinterpret_cast<const v4i*>(base + a_off[s] + i * 32 * kBK);
#pragma unroll
            for (int j = 0; j < TN; j++)
                bf[j] = *reinterpret_cast<const v4i*>(base + b_off[s] + j * 32 * kBK);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (more) store_lds(cur ^ 1);
        __syncthreads();
    }

    i8_epilogue<TM, TN, BM, BN>(acc, sx, sw, bias, acc_out, y, M, N, m0, n0, wm, wn, lane);
}

// ---------------------------------------------------------------------------
// Large shapes (K % 64 == 0): 8 waves (4 x 2) per workgroup, one workgroup per
// CU, block tile 256 x 128, five LDS stages fed by direct-to-LDS loads.
//
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight
// into LDS (lane l of a wave lands at base + 16*l), so a K step needs no
// staging registers and several steps can be in flight, which is what hides the
// L2/HBM latency (a step is only ~0.25 us of MFMA work).  The swizzled LDS
// layout is produced on the global side: lane l of a 16-row block fetches row
// l/4, logical chunk (l%4) ^ swizzle(row), and therefore lands in physical
// chunk l%4.  Synchronisation is explicit: s_waitcnt vmcnt(n) leaves the
// younger steps in flight, then one s_barrier per step.
//
// Measured on MI355X (2.2 GHz under MFMA load), per K step of one workgroup:
// 512 cycles of MFMA per SIMD; fragment reads cost nothing extra once they are
// interleaved with the MFMAs (571 cycles per step with the loads removed); the
// LDS *write* side is the scarce resource: ds_write_b128 saturates at ~80 B/clk
// per CU and the LDS-DMA path at less, so the 24 KB that a step brings in cost
// ~350 cycles that do not hide under the MFMAs (~910 cycles per step in all).
// ---------------------------------------------------------------------------
// WM x WN waves, each owning a (32*TM) x (32*TN) part of the block tile.
template <int TM, int TN, int WM, int WN, int NS, bool FOLD4 = false>
__global__ __launch_bounds__(64 * WM * WN) void i8_gemm_dma_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ B, const float* __restrict__ sx,
    const float* __restrict__ sw, const float* __restrict__ bias, int32_t* __restrict__ acc_out,
    float* __restrict__ y, uint32_t M, uint32_t K, uint32_t N, uint32_t tiles_m, uint32_t tiles_n, uint32_t steps_per) {
    constexpr int WAVES = WM * WN;
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr int A_BYTES = BM * kBK, B_BYTES = BN * kBK, STAGE = A_BYTES + B_BYTES;
    // 16-row blocks per wave and step; when the blocks do not divide evenly the
    // last block is fetched twice (same bytes to the same place), so that every
    // wave issues the same number of loads per step
    constexpr int A_BLOCKS = BM / 16, B_BLOCKS = BN / 16;
    constexpr int A_LOADS = (A_BLOCKS + WAVES - 1) / WAVES, B_LOADS = (B_BLOCKS + WAVES - 1) / WAVES;
    constexpr int LOADS = A_LOADS + B_LOADS;
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];   // [NS][STAGE]

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    // the wave index is made scalar: LDS-DMA destinations then cost SALU work only
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
    const uint32_t m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;

    // blockIdx.y picks a share of the K steps (small problems: more workgroups than tiles); the shares'
    // accumulators go to acc_out + share * M * N and are added by i8_splitk_finish_kernel
    const uint32_t kt_base = blockIdx.y * steps_per;
    const uint32_t ksteps = min(K / kBK - kt_base, steps_per);

    // ---- global side of the LDS-DMA loads ------------------------------------
    // block b = i*WAVES + wave holds rows 16b .. 16b+15 of the operand tile
    const uint32_t lr = lane >> 2, lp = lane & 3;
    const int8_t* pa[A_LOADS];
    const int8_t* pb[B_LOADS];
    uint32_t blk_a[A_LOADS], blk_b[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
        blk_a[i] = min(i * WAVES + wave, (uint32_t)A_BLOCKS - 1);
        const uint32_t row = blk_a[i] * 16 + lr;
        const uint32_t c = (lp ^ row_swizzle(row)) & 3;
        pa[i] = A + (uint64_t)min(m0 + row, M - 1) * K + c * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
        blk_b[i] = min(i * WAVES + wave, (uint32_t)B_BLOCKS - 1);
        const uint32_t row = blk_b[i] * 16 + lr;
        const uint32_t c = (lp ^ row_swizzle(row)) & 3;
        pb[i] = B + (uint64_t)min(n0 + row, N - 1) * K + c * 16;
    }
    // loads [first, first + count) of a step: A blocks, then B blocks
    auto issue_part = [&](uint32_t kt, uint32_t stage, int first, int count) {
        int8_t* base = lds + stage * STAGE;
        const uint32_t k0 = (kt_base + kt) * kBK;
#pragma unroll
        for (int q = 0; q < LOADS; q++) {
            if (q < first || q >= first + count) continue;
            if (q < A_LOADS)
                __builtin_amdgcn_global_load_lds((gptr_t)(pa[q] + k0), (lptr_t)(base + blk_a[q] * 1024), 16, 0, 0);
            else
                __builtin_amdgcn_global_load_lds((gptr_t)(pb[q - A_LOADS] + k0),
                                                 (lptr_t)(base + A_BYTES + blk_b[q - A_LOADS] * 1024), 16, 0, 0);
        }
    };
    auto issue = [&](uint32_t kt, uint32_t stage) { issue_part(kt, stage, 0, LOADS); };

    // ---- fragment read addressing ----------------------------------------------
    const uint32_t fr = lane & 31, fh = lane >> 5, fsw = row_swizzle(fr);
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
        uint32_t chunk = ((2 * s + fh) ^ fsw) & 3;
        a_off[s] = (wm * 32 * TM + fr) * kBK + chunk * 16;
        b_off[s] = A_BYTES + (wn * 32 * TN + fr) * kBK + chunk * 16;
    }

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // ---- software pipeline -----------------------------------------------------
    // A wave sustains only one 128-bit LDS read per ~28 cycles, so fragment reads
    // are never waited for in bulk: the reads of K half 1 of step kt are
    // interleaved one-for-one with the MFMAs of half 0, and the reads of half 0 of
    // step kt+1 with the MFMAs of half 1.  For that, the barrier of step kt
    // publishes step kt+1 (one step ahead of its use), which leaves NS-2 steps of
    // flight time to the LDS-DMA loads.
    // Every step issues exactly LOADS loads, also past the end of K (the last
    // step is then fetched again into a stage nobody reads any more): the memory
    // counter arithmetic below needs no tail cases and the loop stays branch-free.
#pragma unroll
    for (int s = 0; s < NS - 1; s++) issue(min((uint32_t)s, ksteps - 1), s);

    v4i af[2][TM], bf[2][TN];
    auto read_half = [&](int h, uint32_t stage) {
        const int8_t* base = lds + stage * STAGE;
#pragma unroll
        for (int j = 0; j < TN; j++)
            bf[h][j] = *reinterpret_cast<const v4i*>(base + b_off[h] + j * 32 * kBK);
#pragma unroll
        for (int i = 0; i < TM; i++)
            af[h][i] = *reinterpret_cast<const v4i*>(base + a_off[h] + i * 32 * kBK);
    };
    auto mfma_half = [&](int h) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[h][i], bf[h][j], acc[i][j], 0, 0, 0);
    };
    // (MFMA, read) pairs, then the MFMAs that are left; `dma` LDS-DMA loads are
    // spread over the first pairs, one each, and split evenly over the two halves
    // instead of being issued in a burst.
    constexpr int DMA0 = LOADS / 2, DMA1 = LOADS - DMA0;
    auto interleave = [&](int dma) {
#pragma unroll
        for (int q = 0; q < TM + TN; q++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (q < dma) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
    };

    // step 0 is visible once only the NS-2 younger steps are outstanding
    RUMUS_WAIT_VMCNT((NS - 2) * LOADS);
    __builtin_amdgcn_s_barrier();
    read_half(0, 0);

    uint32_t cur = 0;            // stage of step kt
    for (uint32_t kt = 0; kt + 1 < ksteps; kt++) {
        const uint32_t nxt = cur + 1 == NS ? 0 : cur + 1;        // stage of step kt+1
        const uint32_t prv = cur == 0 ? NS - 1 : cur - 1;        // stage of step kt-1 (free)
        // step kt+1 has landed once only the NS-3 younger steps are outstanding
        RUMUS_WAIT_VMCNT((NS - 3) * LOADS);
        __builtin_amdgcn_s_barrier();
        // the refill of the stage freed by the barrier rides along with the MFMAs
        const uint32_t kf = min(kt + (NS - 1), ksteps - 1);
        issue_part(kf, prv, 0, DMA0);
        read_half(1, cur);
        mfma_half(0);
        interleave(DMA0);
        issue_part(kf, prv, DMA0, DMA1);
        read_half(0, nxt);
        mfma_half(1);
        interleave(DMA1);
        cur = nxt;
    }
    read_half(1, cur);
    mfma_half(0);
    interleave(0);
    mfma_half(1);
    RUMUS_WAIT_VMCNT(0);         // no LDS-DMA write may outlive the workgroup

    if (gridDim.y > 1) acc_out += (uint64_t)blockIdx.y * M * N;
    i8_epilogue<TM, TN, BM, BN, FOLD4>(acc, sx, sw, bias, acc_out, y, M, N, m0, n0, wm, wn, lane);
}

// Sum of the K shares' i32 accumulators (exact, any order), then the rescale and bias of the epilogue.
__global__ __launch_bounds__(256) void i8_splitk_finish_kernel(const int32_t* __restrict__ part, uint32_t shares,
                                                               const float* __restrict__ sx, const float* __restrict__ sw,
                                                               const float* __restrict__ bias, int32_t* __restrict__ acc_out,
                                                               float* __restrict__ y, uint32_t M, uint32_t N) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;         // M * N fits 32 bits for the shapes that split K
    if (i >= M * N) return;
    int32_t a = part[i];
    for (uint32_t z = 1; z < shares; z++) a += part[(uint64_t)z * M * N + i];
    if (acc_out) acc_out[i] = a;
    if (y) {
        float v = __fmul_rn(__fmul_rn((float)a, sx[i / N]), sw[i % N]);
        if (bias) v = __fadd_rn(v, bias[i % N]);
        y[i] = v;
    }
}

template <int TM, int TN, int WM, int WN, int NS, bool FOLD4 = false>
static int launch_dma(const int8_t* A, const int8_t* B, const float* sx, const float* sw,
                      const float* bias, int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N,
                      hipStream_t s) {
    constexpr int BM = 32 * TM * WM, BN = 32 * TN * WN;
    constexpr size_t lds_bytes = (size_t)NS * (BM + BN) * kBK;
    static bool attr_set = false;   // benign race: setting the attribute is idempotent
    if (!attr_set && lds_bytes > 64 * 1024) {
        if (int rc = check_hip(hipFuncSetAttribute(
                reinterpret_cast<const void*>(&i8_gemm_dma_kernel<TM, TN, WM, WN, NS, FOLD4>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes), "hipFuncSetAttribute"))
            return rc;
        attr_set = true;
    }
    uint32_t tm = ceil_div(M, BM), tn = ceil_div(N, BN);
    hipLaunchKernelGGL((i8_gemm_dma_kernel<TM, TN, WM, WN, NS, FOLD4>), dim3(tm * tn), dim3(64 * WM * WN),
                       lds_bytes, s, A, B, sx, sw, bias, acc, y, M, K, N, tm, tn, K / kBK);
    return check_launch("i8_gemm_dma_kernel");
}

// K shares of launch_small: towards 512 one-wave tiles in flight; more shares cost more in partial sums than
// they gain (1024: 25.7 us against 20.8).
static uint32_t small_shares(uint32_t M, uint32_t K, uint32_t N, uint32_t* steps_per) {
    const uint32_t tm = ceil_div(M, 64), tn = ceil_div(N, 64), ksteps = K / kBK;
    uint32_t shares = 512 / (tm * tn);
    if (shares > 8) shares = 8;
    if (shares > ksteps / 8) shares = ksteps / 8;
    if (shares < 1) shares = 1;
    *steps_per = ceil_div(ksteps, shares);
    return ceil_div(ksteps, *steps_per);
}

// K shares of launch_mid: towards 256 workgroups, but the partial sums are paid per share: from 64 tiles on only
// a long K is shared (256 x 4096 x 4096, 64 tiles: 18.5 us whole, 20.1 in four shares; 256 x 11008 x 4096: 53.0
// and 28.4).
static uint32_t mid_shares(uint32_t M, uint32_t K, uint32_t N, uint32_t* steps_per) {
    const uint32_t tm = ceil_div(M, 128), tn = ceil_div(N, 128), ksteps = K / kBK;
    const uint32_t tiles = tm * tn, min_steps = tiles < 64 ? 16 : 32;
    uint32_t shares = 256 / tiles;
    if (shares > 8) shares = 8;
    if (shares > ksteps / min_steps) shares = ksteps / min_steps;
    if (shares < 1 || (tiles >= 64 && ksteps < 128)) shares = 1;
    *steps_per = ceil_div(ksteps, shares);
    return ceil_div(ksteps, *steps_per);
}

// Few tiles (K % 64 == 0): one wave per 64 x 64 tile, eight stages of direct-to-LDS loads deep, and K
// shared over up to 8 workgroups per tile so that the weights stream from all of the chip.  The
// register-staged kernel with one K step in flight spent a trip to memory per step on these shapes
// (32 x 4096 x 11008: 29 us for 45 MB of weights).
static int launch_small(const int8_t* A, const int8_t* B, const float* sx, const float* sw, const float* bias,
                        int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N, hipStream_t s) {
    constexpr int NS = 8;
    constexpr size_t lds_bytes = (size_t)NS * 128 * kBK;       // 64 KB
    const uint32_t tm = ceil_div(M, 64), tn = ceil_div(N, 64);
    uint32_t steps_per = 0;
    const uint32_t shares = small_shares(M, K, N, &steps_per);
    if (shares == 1) {
        hipLaunchKernelGGL((i8_gemm_dma_kernel<2, 2, 1, 1, NS>), dim3(tm * tn, 1), dim3(64), lds_bytes, s, A, B, sx, sw,
                           bias, acc, y, M, K, N, tm, tn, steps_per);
        return check_launch("i8_gemm_dma_kernel");
    }
    void* ws = nullptr;
    WorkspaceLease lease;                                    // until both kernels are queued
    if (int rc = workspace_get(s, (size_t)shares * M * N * sizeof(int32_t), &ws, lease)) return rc;
    int32_t* part = static_cast<int32_t*>(ws);
    hipLaunchKernelGGL((i8_gemm_dma_kernel<2, 2, 1, 1, NS>), dim3(tm * tn, shares), dim3(64), lds_bytes, s, A, B,
                       (const float*)nullptr, (const float*)nullptr, (const float*)nullptr, part, (float*)nullptr, M, K, N,
                       tm, tn, steps_per);
    if (int rc = check_launch("i8_gemm_dma_kernel")) return rc;
    hipLaunchKernelGGL(i8_splitk_finish_kernel, dim3(ceil_div(M * N, 256)), dim3(256), 0, s, part, shares, sx, sw, bias, acc,
                       y, M, N);
    return check_launch("i8_splitk_finish_kernel");
}

// Between the two (K % 64 == 0): 128 x 128 tiles of four waves, two workgroups per CU, K shared over workgroups
// while the tiles alone would leave CUs idle.
static int launch_mid(const int8_t* A, const int8_t* B, const float* sx, const float* sw, const float* bias,
                      int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N, hipStream_t s) {
    constexpr int NS = 4;
    constexpr size_t lds_bytes = (size_t)NS * 256 * kBK;       // 64 KB
    const uint32_t tm = ceil_div(M, 128), tn = ceil_div(N, 128);
    uint32_t steps_per = 0;
    const uint32_t shares = mid_shares(M, K, N, &steps_per);
    if (shares == 1) {
        hipLaunchKernelGGL((i8_gemm_dma_kernel<2, 2, 2, 2, NS>), dim3(tm * tn, 1), dim3(256), lds_bytes, s, A, B, sx, sw,
                           bias, acc, y, M, K, N, tm, tn, steps_per);
        return check_launch("i8_gemm_dma_kernel");
    }
    void* ws = nullptr;
    WorkspaceLease lease;                                    // until both kernels are queued
    if (int rc = workspace_get(s, (size_t)shares * M * N * sizeof(int32_t), &ws, lease)) return rc;
    int32_t* part = static_cast<int32_t*>(ws);
    hipLaunchKernelGGL((i8_gemm_dma_kernel<2, 2, 2, 2, NS>), dim3(tm * tn, shares), dim3(256), lds_bytes, s, A, B,
                       (const float*)nullptr, (const float*)nullptr, (const float*)nullptr, part, (float*)nullptr, M, K, N,
                       tm, tn, steps_per);
    if (int rc = check_launch("i8_gemm_dma_kernel")) return rc;
    hipLaunchKernelGGL(i8_splitk_finish_kernel, dim3(ceil_div(M * N, 256)), dim3(256), 0, s, part, shares, sx, sw, bias, acc,
                       y, M, N);
    return check_launch("i8_splitk_finish_kernel");
}

template <int TM, int TN, int OCC>
static int launch(const int8_t* A, const int8_t* B, const float* sx, const float* sw,
                  const float* bias, int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N,
                  hipStream_t s) {
    uint32_t tm = ceil_div(M, 64 * TM), tn = ceil_div(N, 64 * TN);
    hipLaunchKernelGGL((i8_gemm_kernel<TM, TN, OCC>), dim3(tm * tn), dim3(256), 0, s, A, B, sx, sw,
                       bias, acc, y, M, K, N, tm, tn);
    return check_launch("i8_gemm_kernel");
}

// Launch cost by rounds, in units of one round of 256 x 256 blocks (the wide kernel at width 8; 70 us at K = 4096,
// 161 us at K = 11008), from measurements on N = 4096 .. 22016: a round of 256 x 32w blocks costs w/8; a round of
// 256 x 128 tiles 0.63 (half the area: the wide blocks are the better kernel where they fill their rounds); below
// 256 of those tiles the 128 x 128 tiles run two per CU, a pair at 0.83 and a single one at 0.38.
struct I8Plan { double cost; int wide; };    // wide: block width in 32-column units, 0 = the narrower tiles
static double i8_round_cost(int w) { return w ? w / 8.0 : 0.63; }
static I8Plan i8_plan_single(uint32_t m, uint32_t n) {
    const uint64_t narrow = (uint64_t)ceil_div(m, 256) * ceil_div(n, 128);
    if (narrow < 256) {
        const uint64_t per_cu = ((uint64_t)ceil_div(m, 128) * ceil_div(n, 128) + 255) / 256;
        return {(per_cu / 2) * 0.83 + (per_cu % 2) * 0.38, 0};
    }
    I8Plan best{(double)((narrow + 255) / 256) * i8_round_cost(0), 0};
    for (int w = 8; w <= 12; w++) {
        const uint64_t blocks = (uint64_t)ceil_div(m, 256) * ceil_div(n, 32 * w);
        const double c = (double)((blocks + 255) / 256) * i8_round_cost(w);
        if (c < best.cost) best = {c, w};
    }
    return best;
}

// Which kernel takes an m x k x n product.  Pure host arithmetic: rumus_hip_i8_gemm launches what this returns,
// and rumus_hip_i8_gemm_workspace_size replays it to size the workspace.
enum class I8Route { Gemv, Resident, Stream, SplitRows, Wide, Dma256, Reg4x2, Mid, Small, Reg2x2, Reg1x1 };
struct I8Choice { I8Route route; uint32_t split_rows; int wide; };

static I8Choice i8_choose(uint32_t m, uint32_t k, uint32_t n) {
    // decode: up to 4 rows on v_dot4_i32_i8 (4096 x 11008 from a HIP graph over rotating weight copies: 9.3, 10.0,
    // 12.7 us for 1, 2, 4 rows against 18.3 us for 8 rows on the one-wave MFMA tiles)
    if (m <= 4) return {I8Route::Gemv, 0, 0};
    // 5 to 64 rows over K of 3072 to 4096 (to 8192 up to 32 rows, to 12288 up to 16): the activations stay in registers
    // and a workgroup walks over its column tiles (from HBM, 4096 x 11008 at 5, 16, 32, 64 rows: 13.0, 14.5, 16.2, 20.6 us
    // against 14.0, 17.6, 22.4, 26.7 for the routes below; 3072 x 8192: 8.5, 9.3, 11.4, 15.4 against 10.6, 12.9, 17.8, 20.1)
    if (i8_resident_takes(m, k, n)) return {I8Route::Resident, 0, 0};
    // other K, 5 to 16 rows (to 32 on smaller weights): MFMA tiles fed straight from global memory, a workgroup per 16
    // columns (from HBM, 8 rows: 4096 x 11008 14.5 us against 18.1 us for the LDS-staged tiles below, 4096 x 4096 7.4
    // against 12.8; 32 rows: 22.5 against 20.6 and 10.8 against 14.6)
    if (k % 256 == 0 && (m <= 16 || (m <= 32 && (uint64_t)n * k <= (32ull << 20)))) return {I8Route::Stream, 0, 0};
    // Largest tile that still gives every CU a workgroup.
    const uint64_t big = (uint64_t)ceil_div(m, 256) * ceil_div(n, 128);
    const uint64_t mid = (uint64_t)ceil_div(m, 128) * ceil_div(n, 128);
    if (big >= 256 && k % kBK == 0) {
        // Workgroups of the large tiles run one per CU, in rounds of 256 that last the same full or not, so the
        // kernel is chosen by rounds: see i8_plan_single.  Rows are independent, so when whole rounds of one
        // kernel plus a cheaper launch for the rest cost less than any single launch (6144 x 11008 x 4096: three
        // rounds of 256 x 128 tiles 357 us; 4096 rows in one round of 256 x 256 blocks + 2048 rows 263 us), the
        // two parts are launched apart; same results.
        const I8Plan one = i8_plan_single(m, n);
        uint32_t split_rows = 0;
        double split_cost = one.cost * 0.97;                     // a second launch has to pay for itself
        for (int w = 0; w <= 12; w = w ? w + 1 : 8) {            // 0: the 256 x 128 tiles
            const uint32_t cols = ceil_div(n, w ? 32 * w : 128);
            if (cols > 256) continue;
            const uint32_t rows_per_round = (256 / cols) * 256;
            if (m <= rows_per_round) continue;
            const uint32_t m1 = (m / rows_per_round) * rows_per_round;
            if (m1 == m) continue;
            const double c = (m1 / rows_per_round) * i8_round_cost(w) + i8_plan_single(m - m1, n).cost;
            if (c < split_cost) { split_cost = c; split_rows = m1; }
        }
        if (split_rows) return {I8Route::SplitRows, split_rows, 0};
        if (one.wide) return {I8Route::Wide, 0, one.wide};
        return {I8Route::Dma256, 0, 0};
    }
    if (big >= 256) return {I8Route::Reg4x2, 0, 0};
    // more than 128 rows, fewer than 256 of the big tiles: 128 x 128 tiles, two workgroups per CU
    // (1024 x 4096 x 4096: 39.6 -> 24.2 us, 1024 x 11008 x 4096: 97.5 -> 59.1 us, 256 x 4096 x 11008: 32.9 -> 22.9 us)
    if (k % kBK == 0 && m > 128 && (uint64_t)m * n < (1ull << 28)) return {I8Route::Mid, 0, 0};
    // up to 128 rows: the deep-pipelined one-wave tiles with K shared over workgroups
    // (4096 x 11008: 28 -> 17-21 us; 11008 x 4096: 66 -> 18-25 us)
    if (k % kBK == 0 && (uint64_t)m * n < (1ull << 28)) return {I8Route::Small, 0, 0};
    if (mid >= 256) return {I8Route::Reg2x2, 0, 0};
    return {I8Route::Reg1x1, 0, 0};
}

// Workspace bytes rumus_hip_i8_gemm takes for this shape: the i32 partial sums of the K shares of the 64 x 64
// and 128 x 128 tile kernels (at most 8 and 16 MiB), for the larger of the two parts when the rows are split.
size_t i8_gemm_workspace_need(uint32_t m, uint32_t k, uint32_t n) {
    if (m == 0 || n == 0 || k == 0 || k % 16 != 0) return 0;
    const I8Choice c = i8_choose(m, k, n);
    uint32_t steps_per = 0, shares = 1;
    switch (c.route) {
        case I8Route::SplitRows: {
            const size_t a = i8_gemm_workspace_need(c.split_rows, k, n), b = i8_gemm_workspace_need(m - c.split_rows, k, n);
            return a > b ? a : b;
        }
        case I8Route::Small: shares = small_shares(m, k, n, &steps_per); break;
        case I8Route::Mid: shares = mid_shares(m, k, n, &steps_per); break;
        default: break;
    }
    return shares > 1 ? (size_t)shares * m * n * sizeof(int32_t) : 0;
}

// Routes whose kernels have the plane-adding epilogue: the two kernels of large shapes, and row splits into them.
bool i8_gemm_fold4_supported(uint32_t m4, uint32_t k, uint32_t n) {
    if (m4 == 0 || m4 % 4 != 0 || n == 0 || k == 0 || k % 16 != 0) return false;
    const I8Choice c = i8_choose(m4, k, n);
    switch (c.route) {
        case I8Route::Wide:
        case I8Route::Dma256: return true;
        case I8Route::SplitRows:
            return c.split_rows % 4 == 0 && i8_gemm_fold4_supported(c.split_rows, k, n) &&
                   i8_gemm_fold4_supported(m4 - c.split_rows, k, n);
        default: return false;
    }
}

int i8_gemm_fold4(const int8_t* planes, const int8_t* wq, const float* sx4, const float* sw, const float* bias,
                  float* y, uint32_t m4, uint32_t k, uint32_t n, hipStream_t s) {
    RUMUS_REQUIRE(i8_gemm_fold4_supported(m4, k, n), "i8 gemm: no plane-adding kernel for %u x %u x %u", m4, k, n);
    RUMUS_REQUIRE((reinterpret_cast<uintptr_t>(sx4) & 15) == 0, "i8 gemm: plane weights must be 16-byte aligned");
    const I8Choice c = i8_choose(m4, k, n);
    switch (c.route) {
        case I8Route::SplitRows: {
            const uint32_t m1 = c.split_rows;
            if (int rc = i8_gemm_fold4(planes, wq, sx4, sw, bias, y, m1, k, n, s)) return rc;
            return i8_gemm_fold4(planes + (uint64_t)m1 * k, wq, sx4 + m1, sw, bias, y + (uint64_t)(m1 / 4) * n, m4 - m1, k, n, s);
        }
        case I8Route::Wide: return i8_gemm_launch_wide(c.wide, planes, wq, sx4, sw, bias, nullptr, y, m4, k, n, s, true);
        default: return launch_dma<2, 2, 4, 2, 5, true>(planes, wq, sx4, sw, bias, nullptr, y, m4, k, n, s);
    }
}

}  // namespace rumus

using namespace rumus;

extern "C" int rumus_hip_i8_gemm(const int8_t* xq, const int8_t* wq, const float* sx,
                                 const float* sw, const float* bias, int32_t* acc, float* y,
                                 uint32_t m, uint32_t k, uint32_t n, rumus_hip_stream_t stream) {
    if (m == 0 || n == 0) {                                  // nothing to read or write: null pointers are fine
        RUMUS_REQUIRE(k > 0 && k % 16 == 0, "i8_gemm: k must be a positive multiple of 16 (got %u)", k);
        return RUMUS_HIP_OK;
    }
    RUMUS_REQUIRE(xq && wq, "i8_gemm: null operand");
    RUMUS_REQUIRE(acc || y, "i8_gemm: both outputs are null");
    RUMUS_REQUIRE(!y || (sx && sw), "i8_gemm: y needs sx and sw");
    RUMUS_REQUIRE(k > 0 && k % 16 == 0, "i8_gemm: k must be a positive multiple of 16 (got %u)", k);
    RUMUS_REQUIRE(((reinterpret_cast<uintptr_t>(xq) | reinterpret_cast<uintptr_t>(wq)) & 15) == 0,
                  "i8_gemm: operands must be 16-byte aligned");
    hipStream_t s = as_stream(stream);
    const I8Choice c = i8_choose(m, k, n);
    switch (c.route) {
        case I8Route::Gemv: return i8_launch_gemv(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Resident: return i8_launch_resident(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Stream: return i8_launch_stream(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::SplitRows: {
            const uint32_t m1 = c.split_rows;
            if (int rc = rumus_hip_i8_gemm(xq, wq, sx, sw, bias, acc, y, m1, k, n, stream)) return rc;
            return rumus_hip_i8_gemm(xq + (uint64_t)m1 * k, wq, sx ? sx + m1 : nullptr, sw, bias,
                                     acc ? acc + (uint64_t)m1 * n : nullptr, y ? y + (uint64_t)m1 * n : nullptr,
                                     m - m1, k, n, stream);
        }
        case I8Route::Wide: return i8_gemm_launch_wide(c.wide, xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Dma256: return launch_dma<2, 2, 4, 2, 5>(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Reg4x2: return launch<4, 2, 2>(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Mid: return launch_mid(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Small: return launch_small(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Reg2x2: return launch<2, 2, 2>(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
        case I8Route::Reg1x1: return launch<1, 1, 2>(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
    }
    return set_error(RUMUS_HIP_EINVAL, "i8_gemm: no kernel for %u x %u x %u", m, k, n);
}

extern "C" uint64_t rumus_hip_i8_gemm_workspace_size(uint32_t m, uint32_t k, uint32_t n) {
    return i8_gemm_workspace_need(m, k, n);
}
