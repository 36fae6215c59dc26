// W8A8 INT8 GEMM, large shapes: one workgroup per 256 x (32*W) block of y, W
// chosen so that the blocks are dealt to the 256 CUs in whole rounds (for the
// prefill shape 2048 x 4096 x 11008: W = 11, 8 x 32 = 256 blocks of 256 x 352,
// 2 % padding) instead of 2.7 rounds of 256 x 128 tiles.  A wide block also
// halves the bytes that go through the texture path and into LDS per MFMA,
// which is what bounds the narrower kernel (LDS writes saturate near 80 B/clk
// per CU).
//
// Eight waves in a 4 (M) x 2 (N) grid; waves w and w+4 share a SIMD and split
// the block's W column tiles between them, ceil(W/2) and floor(W/2), so every
// SIMD carries the same 2 x W MFMA tiles (v_mfma_i32_32x32x32_i8) per K half.
// A wave owns 64 rows = 2 row tiles, i.e. up to 2 x 6 x 16 = 192 accumulator
// registers, which leaves no room for a full set of B fragments; fragments
// stream instead: the K step is walked as 2*TN "slots" (K half h, column tile
// j), a slot is two MFMAs (both row tiles against one B fragment), and the B
// fragment of slot s+3 is read from LDS while slot s multiplies (a ring of
// registers).  The two A fragments of the next K half are read during the
// current half.  Operands reach LDS through global_load_lds_dwordx4, four
// stages deep; the barrier of step t publishes step t+1, so reads run ahead
// across the step boundary and no MFMA waits for a bulk transfer.
#include <type_traits>

#include "i8_gemm.h"

namespace rumus {

constexpr int kWideBM = 256;
constexpr int kWideStages = 4;
constexpr int kWideLook = 3;   // B fragments are read this many slots ahead
constexpr int kWideWaves = 8, kWideWM = 4;

constexpr int ring_size(int slots, int at_least) {
    int r = at_least;
    while (slots % r) r++;
    return r;
}

// What a wave needs to issue its share of the LDS-DMA loads of one K step.
template <int LOADS>
struct WideLoads {
    const int8_t* src[LOADS];   // global address at K offset 0
    uint32_t dst[LOADS];        // byte offset inside a stage
    uint32_t ksteps;
};

// The K loop and the epilogue of one wave: rows [64*wm, 64*wm+64), column tiles
// [ct0, ct0+TN) of the block.  Both kinds of waves of a workgroup (TN differs)
// run the same number of barriers and issue the same number of loads per step.
template <int TN, int W, int LOADS, bool FOLD4>
__device__ __forceinline__ void wide_wave(const WideLoads<LOADS>& ld, int8_t* lds, const float* __restrict__ sx,
                                          const float* __restrict__ sw, const float* __restrict__ bias,
                                          int32_t* __restrict__ acc_out, float* __restrict__ y, uint32_t M,
                                          uint32_t N, uint32_t m0, uint32_t n0, uint32_t wm, uint32_t ct0,
                                          uint32_t lane) {
    constexpr int TM = kWideBM / (32 * kWideWM), NS = kWideStages, LOOK = kWideLook;
    constexpr int A_BYTES = kWideBM * kBK, STAGE = (kWideBM + 32 * W) * kBK;
    constexpr int SLOTS = 2 * TN;      // per K step
    static_assert(TN >= LOOK && TN >= TM && SLOTS >= LOADS, "slot schedule");
    // B fragments live in a ring indexed by slot % RING; the ring holds LOOK+1 fragments
    // and divides the slots of a step, so every step sees the same register for a slot
    constexpr int RING = ring_size(SLOTS, LOOK + 1);

    // Every step issues exactly LOADS loads, also past the end of K (the last step is
    // fetched again into a stage nobody reads any more): no tail cases in the counters.
    auto issue_one = [&](uint32_t kt, uint32_t stage, int q) {
        const uint32_t k0 = min(kt, ld.ksteps - 1) * kBK;
        __builtin_amdgcn_global_load_lds((gptr_t)(ld.src[q] + k0), (lptr_t)(lds + stage * STAGE + ld.dst[q]), 16, 0,
                                         0);
    };

    const uint32_t fr = lane & 31, fh = lane >> 5, fsw = row_swizzle(fr);
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const uint32_t chunk = ((2 * h + fh) ^ fsw) & 3;
        a_off[h] = (wm * 32 * TM + fr) * kBK + chunk * 16;
        b_off[h] = A_BYTES + (ct0 * 32 + fr) * kBK + chunk * 16;
    }

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    v4i af[2][TM];     // [K half]
    v4i bring[RING];

    // ---- prologue ------------------------------------------------------------------------
#pragma unroll
    for (int s = 0; s < NS - 1; s++)
#pragma unroll
        for (int q = 0; q < LOADS; q++) issue_one(s, s, q);
    RUMUS_WAIT_VMCNT((NS - 2) * LOADS);      // step 0 landed
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < TM; i++) af[0][i] = *reinterpret_cast<const v4i*>(lds + a_off[0] + i * 32 * kBK);
#pragma unroll
    for (int s = 0; s < LOOK; s++) bring[s % RING] = *reinterpret_cast<const v4i*>(lds + b_off[0] + s * 32 * kBK);

    // One K step.  LAST: nothing follows (no refill, no reads of the next step).
    auto step = [&](uint32_t kt, uint32_t cur, auto last_tag) {
        constexpr bool LAST = decltype(last_tag)::value;
        const uint32_t nxt = cur + 1 == NS ? 0 : cur + 1;
        const uint32_t prv = cur == 0 ? NS - 1 : cur - 1;
        if (!LAST) {
            // step kt+1 has landed once only the NS-3 younger steps are outstanding
            RUMUS_WAIT_VMCNT((NS - 3) * LOADS);
            __builtin_amdgcn_s_barrier();
        }
        const int8_t* base_c = lds + cur * STAGE;
        const int8_t* base_n = lds + nxt * STAGE;
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            const int h = s / TN, j = s % TN;
            const int s2 = s + LOOK;              // B fragment of slot s+LOOK (maybe next half / next step)
            if (s2 < SLOTS) {
                bring[s2 % RING] = *reinterpret_cast<const v4i*>(base_c + b_off[s2 / TN] + (s2 % TN) * 32 * kBK);
            } else if (!LAST) {
                bring[s2 % RING] = *reinterpret_cast<const v4i*>(base_n + b_off[0] + (s2 - SLOTS) * 32 * kBK);
            }
            if (j < TM) {                         // A fragments of the next K half
                if (h == 0) {
                    af[1][j] = *reinterpret_cast<const v4i*>(base_c + a_off[1] + j * 32 * kBK);
                } else if (!LAST) {
                    af[0][j] = *reinterpret_cast<const v4i*>(base_n + a_off[0] + j * 32 * kBK);
                }
            }
            // refill of the stage freed by the barrier, spread over the slots
            if (!LAST && s < LOADS) issue_one(kt + (NS - 1), prv, s);
#pragma unroll
            for (int i = 0; i < TM; i++)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[h][i], bring[s % RING], acc[i][j], 0, 0, 0);
        }
        // issue order, slot by slot: the reads and the load of a slot, then its MFMAs
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
            const int j = s % TN;
            const int reads = ((s + LOOK < SLOTS || !LAST) ? 1 : 0) + ((j < TM && (s / TN == 0 || !LAST)) ? 1 : 0);
            if (reads == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            if (reads == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (!LAST && s < LOADS) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, TM, 0);
        }
    };

    uint32_t cur = 0;
    for (uint32_t kt = 0; kt + 1 < ld.ksteps; kt++) {
        step(kt, cur, std::false_type{});
        cur = cur + 1 == NS ? 0 : cur + 1;
    }
    step(ld.ksteps - 1, cur, std::true_type{});
    RUMUS_WAIT_VMCNT(0);         // no LDS-DMA write may outlive the workgroup

    i8_epilogue<TM, TN, kWideBM, 32 * W, FOLD4>(acc, sx, sw, bias, acc_out, y, M, N, m0, n0 + ct0 * 32, wm, 0, lane);
}

template <int W, bool FOLD4>
__global__ __launch_bounds__(64 * kWideWaves, 1) void i8_gemm_wide_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ B, const float* __restrict__ sx,
    const float* __restrict__ sw, const float* __restrict__ bias, int32_t* __restrict__ acc_out,
    float* __restrict__ y, uint32_t M, uint32_t K, uint32_t N, uint32_t tiles_m, uint32_t tiles_n) {
    constexpr int WAVES = kWideWaves;
    constexpr int TN0 = (W + 1) / 2, TN1 = W / 2;
    constexpr int A_BYTES = kWideBM * kBK;
    constexpr int A_BLOCKS = kWideBM / 16, B_BLOCKS = 2 * W;      // 16-row blocks of 1 KB
    constexpr int A_LOADS = A_BLOCKS / WAVES, B_LOADS = (B_BLOCKS + WAVES - 1) / WAVES;
    constexpr int LOADS = A_LOADS + B_LOADS;
    static_assert((kWideStages - 1) * LOADS < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];   // [NS][STAGE]

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // scalar: LDS-DMA bases cost SALU only
    const uint32_t tile = xcd_contiguous(blockIdx.x, tiles_m * tiles_n);
    const uint32_t m0 = (tile % tiles_m) * kWideBM, n0 = (tile / tiles_m) * (32 * W);

    // lane l of a block fetches row l/4, logical chunk (l%4) ^ swizzle(row) and lands in
    // physical chunk l%4.  A block that does not exist for this wave (B blocks need not
    // divide by the waves) repeats the last one: same bytes to the same place.
    const uint32_t lr = lane >> 2, lp = lane & 3;
    WideLoads<LOADS> ld;
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
        const uint32_t b = i * WAVES + wave, row = b * 16 + lr;
        ld.src[i] = A + (uint64_t)min(m0 + row, M - 1) * K + ((lp ^ row_swizzle(row)) & 3) * 16;
        ld.dst[i] = b * 1024;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
        const uint32_t b = min(i * WAVES + wave, (uint32_t)B_BLOCKS - 1), row = b * 16 + lr;
        ld.src[A_LOADS + i] = B + (uint64_t)min(n0 + row, N - 1) * K + ((lp ^ row_swizzle(row)) & 3) * 16;
        ld.dst[A_LOADS + i] = A_BYTES + b * 1024;
    }
    ld.ksteps = K / kBK;

    const uint32_t wm = wave % kWideWM;
    if (wave < kWideWM) wide_wave<TN0, W, LOADS, FOLD4>(ld, lds, sx, sw, bias, acc_out, y, M, N, m0, n0, wm, 0, lane);
    else wide_wave<TN1, W, LOADS, FOLD4>(ld, lds, sx, sw, bias, acc_out, y, M, N, m0, n0, wm, TN0, lane);
}

template <int W, bool FOLD4>
static int launch_wide(const int8_t* A, const int8_t* B, const float* sx, const float* sw, const float* bias,
                       int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N, hipStream_t s) {
    constexpr size_t lds_bytes = (size_t)kWideStages * (kWideBM + 32 * W) * kBK;
    static_assert(lds_bytes <= 160 * 1024, "stages do not fit the 160 KB LDS");
    static bool attr_set = false;   // benign race: setting the attribute is idempotent
    if (!attr_set) {
        if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&i8_gemm_wide_kernel<W, FOLD4>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes),
                               "hipFuncSetAttribute"))
            return rc;
        attr_set = true;
    }
    const uint32_t tm = ceil_div(M, kWideBM), tn = ceil_div(N, 32 * W);
    hipLaunchKernelGGL((i8_gemm_wide_kernel<W, FOLD4>), dim3(tm * tn), dim3(64 * kWideWaves), lds_bytes, s, A, B, sx, sw,
                       bias, acc, y, M, K, N, tm, tn);
    return check_launch("i8_gemm_wide_kernel");
}

template <bool FOLD4>
static int launch_wide_w(int w, const int8_t* A, const int8_t* B, const float* sx, const float* sw,
                         const float* bias, int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N,
                         hipStream_t s) {
    switch (w) {
        case 8: return launch_wide<8, FOLD4>(A, B, sx, sw, bias, acc, y, M, K, N, s);
        case 9: return launch_wide<9, FOLD4>(A, B, sx, sw, bias, acc, y, M, K, N, s);
        case 10: return launch_wide<10, FOLD4>(A, B, sx, sw, bias, acc, y, M, K, N, s);
        case 11: return launch_wide<11, FOLD4>(A, B, sx, sw, bias, acc, y, M, K, N, s);
        case 12: return launch_wide<12, FOLD4>(A, B, sx, sw, bias, acc, y, M, K, N, s);
    }
    return set_error(RUMUS_HIP_EINVAL, "i8 gemm: no wide kernel for width %d", w);
}

int i8_gemm_launch_wide(int w, const int8_t* A, const int8_t* B, const float* sx, const float* sw,
                        const float* bias, int32_t* acc, float* y, uint32_t M, uint32_t K, uint32_t N,
                        hipStream_t s, bool fold4) {
    return fold4 ? launch_wide_w<true>(w, A, B, sx, sw, bias, acc, y, M, K, N, s)
                 : launch_wide_w<false>(w, A, B, sx, sw, bias, acc, y, M, K, N, s);
}

}  // namespace rumus
