// INT4 engine: dequant-fused GEMM on the f16 matrix cores, for m > 8.
//
//   y[m,n] = sum_g scales[g,n] * ( sum_{k in g} x[m,k] * q[k,n] - zp[g,n] * sum_{k in g} x[m,k] ) (+ bias[n])
//
// which equals sum_k x[m,k] * (q[k,n] - zp) * scale with the scale applied once
// per group in f32.  Inside a group only x and the raw nibbles meet in the MFMA:
//   - q is 0..15, exact in f16;
//   - x is split as hi + lo with hi = f16(x), lo = f16(x - hi) (gfx950 MFMAs keep
//     f16 subnormals), two MFMAs per tile, f32 accumulate.  x keeps ~21
//     significant bits, so the f32 tolerance of this path (rel 1e-3 / abs 1e-4)
//     holds; a single f16 x, or scale folded into f16 weights, would not hold it
//     for outputs near zero.
//
// One accumulator set serves all groups: it is kept in units of the current
// group's scale.  When a group ends, the zero-point term is subtracted
// (zp * sum of x over the group, the sums come with the staged activations) and
// the accumulator is multiplied by scale_cur / scale_next; the last unit is
// multiplied out in the epilogue.  That is ~2 extra f32 roundings per group,
// far inside the tolerance, and it halves the accumulator registers compared
// with a second "finished groups" set.  A zero scale is replaced by 1e-30 (its
// group then contributes ~0, as it should).
//
// Weights never pass through LDS.  v_mfma_f32_32x32x16_f16 wants, per lane, 8
// consecutive k of one column: exactly one packed u32 word
// (rumus-vision/src/quant.rs:98-100).  Lane l of a wave loads the two words of
// columns 2*(l%32), +1 at word row 2*step + l/32 with one 64-bit load (a wave
// covers 64 columns x 16 rows of K per step, 256-byte segments) and converts
// each word to a B fragment in registers (magic-number nibble -> f16, packed f16
// math).  The conversion yields k in the order 0,4,1,5,2,6,3,7; the A fragments
// are stored in the same order, and a dot product does not care.  MFMA j of a
// lane works on columns 2*(l%32)+j, so the two results of a row are adjacent
// and leave as one float2.  The eight loads of a stage sit in eight registers
// pairs that are refilled for the next stage as soon as they are consumed, so
// one stage of weights (4 KB per wave, 32 KB per workgroup) is always in flight.
//
// A workgroup covers 512 columns and 32 or 64 rows with 8 or 4 waves (see the kernel's
// comment for the wave grids).  Per
// stage of 128 rows of K the activations of the BM rows are converted once (hi/lo
// f16, fragment layout, sums per 16 k for the zero-point term) into one of two
// LDS buffers while the previous stage is multiplied; one barrier per stage.
// `perm` (act-order) gathers x columns at this point.
//
// The zero-point term of a group, -zp[n] * X[m] with X the sum of x over the
// group, is a rank-1 update: it is added by one v_mfma_f32_32x32x2_f32 per tile
// (f32 operands, so nothing is lost), not by the vector ALU.
//
// Few output tiles (small m): K is split over gridDim.z workgroups, each
// writes its partial tile to the workspace, and a second kernel adds the
// partials in a fixed order (deterministic, no atomics) and the bias.
#include <type_traits>

#include "w4.h"

namespace rumus {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kTileCols = 512;   // columns per workgroup of eight waves
constexpr int kStageK = 128;     // rows of K staged per barrier (8 MFMA steps of 16)
constexpr int kMaxSplits = 16;
constexpr uint32_t kZpFlagWords = 256;   // blocks of w4_zp_scan_kernel, one flag word each

// one packed word -> B fragment, k order 0,4,1,5,2,6,3,7, with the column's integer zero-point z taken off on the way:
// the magic-number conversion ends in a subtraction anyway (1024 + n - 1024, and (1024 + 16 n) / 16 - 64 for the nibbles
// that sit four bits higher), so 1024 + z and 64 + z in place of the constants cost nothing.  n - z is an exact f16.
// big = {1024 + z, 1024 + z}, small = {-(64 + z), -(64 + z)}.
__device__ __forceinline__ v8h nibbles_to_f16(uint32_t w, v2h big, v2h small) {
    const v2h k16th = {(_Float16)0.0625f, (_Float16)0.0625f};
    // (w & mask) | 0x64006400 in one instruction each: v_and_or_b32 may read one scalar register only, so the masks
    // live in vector registers (the compiler, left to itself, keeps both constants scalar and issues an AND and an OR)
    const uint32_t m_lo = 0x000F000Fu, m_hi = 0x00F000F0u, magic = 0x64006400u;
    const uint32_t w8 = w >> 8;
    uint32_t t0, t1, t2, t3;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t0) : "v"(w), "v"(m_lo), "s"(magic));    // 1024 + n0, 1024 + n4
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t1) : "v"(w), "v"(m_hi), "s"(magic));    // 1024 + 16 n1, 1024 + 16 n5
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t2) : "v"(w8), "v"(m_lo), "s"(magic));   // n2, n6
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t3) : "v"(w8), "v"(m_hi), "s"(magic));   // 16 n3, 16 n7
    const v2h h0 = __builtin_bit_cast(v2h, t0) - big;
    const v2h h1 = __builtin_elementwise_fma(__builtin_bit_cast(v2h, t1), k16th, small);   // exact: (1024+16n)/16 - 64 - z
    const v2h h2 = __builtin_bit_cast(v2h, t2) - big;
    const v2h h3 = __builtin_elementwise_fma(__builtin_bit_cast(v2h, t3), k16th, small);
    return v8h{h0[0], h0[1], h1[0], h1[1], h2[0], h2[1], h3[0], h3[1]};
}

// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() also waits
// for every global load in flight (vmcnt(0)), which would drain the weight prefetch at each
// stage; nothing here communicates through global memory inside a workgroup.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);          // lgkmcnt(0); vmcnt and expcnt untouched
    __builtin_amdgcn_s_barrier();
}

// Words and metadata of TN adjacent columns, TN = 2 or 4.
template <int TN> struct WVec;
template <> struct WVec<2> { typedef uint2 words; typedef float2 floats; };
template <> struct WVec<4> { typedef uint4 words; typedef float4 floats; };
__device__ __forceinline__ uint32_t word_of(const uint2& v, int j) { return j == 0 ? v.x : v.y; }
__device__ __forceinline__ uint32_t word_of(const uint4& v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }
__device__ __forceinline__ float flt_of(const float2& v, int j) { return j == 0 ? v.x : v.y; }
__device__ __forceinline__ float flt_of(const float4& v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }
__device__ __forceinline__ float2 nonzero(float2 s) { return make_float2(s.x == 0.0f ? 1e-30f : s.x, s.y == 0.0f ? 1e-30f : s.y); }
__device__ __forceinline__ float4 nonzero(float4 s) {
    return make_float4(s.x == 0.0f ? 1e-30f : s.x, s.y == 0.0f ? 1e-30f : s.y, s.z == 0.0f ? 1e-30f : s.z,
                       s.w == 0.0f ? 1e-30f : s.w);
}
__device__ __forceinline__ float2 splat_of(float v, float2) { return make_float2(v, v); }
__device__ __forceinline__ float4 splat_of(float v, float4) { return make_float4(v, v, v, v); }
__device__ __forceinline__ float2 zp4_load(const uint32_t* zp4, uint32_t g, uint32_t n, uint32_t col, float2) {
    return w4_zp4_load2(zp4, g, n, col);
}
__device__ __forceinline__ float4 zp4_load(const uint32_t* zp4, uint32_t g, uint32_t n, uint32_t col, float4) {
    return w4_zp4_load4(zp4, g, n, col);
}

// The WAVES (8 or 4) waves of a workgroup form a WM x (WAVES/WM) grid; a wave owns RT row tiles of 32 and TN
// column tiles (its lanes hold TN adjacent columns each), so the workgroup covers
// BM = 32*RT*WM rows and 32*TN*WAVES/WM columns (512 with eight waves side by side).  Wide wave tiles matter: every wave reads the A fragments
// of its rows from LDS at every step, and with 64-column waves (TN = 2) side by side those
// reads, not the MFMAs, bound the 128-row tile.
// DEPTH = stages of weights in flight; FOLD = MFMA steps between settlements of the zero-point
// term (group_size / 16, at most a stage); ZP4: zero-points come packed, eight integers per
// word along n.  out = y when gridDim.z == 1, else the partial tiles [split][m][n].
//
// The stage body is straight-line code: loads past the end of the work are clamped to valid
// addresses and their results never used, instead of being skipped, and nothing is consumed
// right after it was loaded, so that the memory counter never has to drain.
//
// PRE: the activations arrive already split into hi and lo f16 planes in A-fragment order, with
// the sums of every 16 of them beside (w4_convert_x_kernel), and a stage is copied into LDS as
// it is.  Without it every workgroup of a row tile converts the same activations again, once
// per 512 columns of the output.
template <int RT, int WM, int TN, int WAVES, int DEPTH, int FOLD, bool ZP4, bool PRE>
__global__ __launch_bounds__(64 * WAVES, 2) void w4_gemm_tile_kernel(W4Args a, float* __restrict__ out,
                                                                      uint32_t stages_per_split) {
    // a.x: rows of a.k floats, a.k % 4 == 0, 16-byte aligned, columns already in weight order
    // (the launcher copies x into that form when the caller's x is not)
    typedef typename WVec<TN>::words words_t;
    typedef typename WVec<TN>::floats floats_t;
    constexpr int WN = WAVES / WM;
    constexpr int RPP = 8 * WAVES;               // rows staged per pass: 8 threads per row
    constexpr int COLS = WN * 32 * TN;           // columns per workgroup
    constexpr int BM = 32 * RT * WM;
    // bytes of one k16 step of one plane: [row tile][k block][row] x 16, plus 128 bytes of skew so
    // that the eight staging lanes of a row (one step each) do not write to the same banks
    constexpr int STEP = (BM / 32) * 1024 + 128;
    constexpr int NI = BM > RPP ? BM / RPP : 1;  // (row, step) pairs staged per thread
    constexpr int PLANE = 8 * STEP;
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][2][PLANE];   // [buffer][hi, lo]
    __shared__ __attribute__((aligned(16))) float lds_xs[2][8][BM];       // [buffer][k16 step][row]: sum of x
    __shared__ float lds_rf[BM];                                          // the rows' factors for the results

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t l32 = lane & 31, kb = lane >> 5;
    const uint32_t m0 = blockIdx.y * BM;
    const uint32_t colbase = blockIdx.x * COLS + wn * (32 * TN) + TN * l32;   // this lane's TN columns
    const bool col_ok = colbase < a.n;                   // n % 4 == 0
    const uint32_t col_c = col_ok ? colbase : 0;
    const uint32_t nstages = (a.padded_k + kStageK - 1) / kStageK;
    const uint32_t st_begin = blockIdx.z * stages_per_split;
    const uint32_t st_end = min(nstages, st_begin + stages_per_split);
    const uint32_t word_rows = a.padded_k / 8;
    const uint32_t k_end = min(a.padded_k, st_end * kStageK);
    if (tid < BM) lds_rf[tid] = a.rfac[min(m0 + tid, a.m - 1)];          // read after the stages' barriers

    // Whether any zero-point of the table has a rest at all (found by w4_zp_scan_kernel before this launch):
    // checkpoints store integers (as f32 here, or packed), and then the rank-1 updates - an eighth of the
    // matrix-core time at groups of 128 - are left out.  Requested here, looked at before the first stage.
    // (No flags - small batches, where the look costs more than it saves: the updates run.)
    uint4 zflag = make_uint4(0, 0, 0, 0);
    if constexpr (!ZP4) zflag = a.zflags ? reinterpret_cast<const uint4*>(a.zflags)[lane] : make_uint4(1, 0, 0, 0);
    static_assert(kZpFlagWords == 256, "four flag words per lane");

    // ---- staging role: thread t converts 16 consecutive k (MFMA step t%8) of row t/8 -----
    const uint32_t s_row = tid >> 3, s_step = tid & 7;
    const bool s_active = s_row < BM;            // 32 rows, 8 waves: half of the threads stage
    // PRE: a stage is (BM/32) row tiles x 8 steps x 2 planes of 1 KB fragment blocks, NCH 16-byte
    // chunks per thread, and BM x 8 sums, NS per thread
    constexpr int T = 64 * WAVES;
    constexpr int NCH = PRE ? (BM / 32) * 8 * 2 * 64 / T : 1;
    constexpr int NS = PRE ? (BM * 8 + T - 1) / T : 1;
    static_assert(!PRE || (BM * 8) % T == 0, "the sums of a stage divide evenly over the threads");
    float4 xraw[DEPTH][NI][4];                   // DEPTH stages of activations in flight, too
    // PRE: this thread's chunks and sums of the stage in flight, as named registers (an array
    // indexed through the staging lambdas is left in scratch memory by the compiler)
    static_assert(!PRE || (DEPTH == 1 && (NCH == 4 || NCH == 8) && NS <= 2), "PRE staging shape");
    float4 xp0, xp1, xp2, xp3, xp4, xp5, xp6, xp7;
    float xsr0 = 0.0f, xsr1 = 0.0f;
    auto pre_src = [&](uint64_t tile0, int i) __attribute__((always_inline)) {
        const uint32_t c = tid + T * i, blk = c >> 6, ln = c & 63;
        const uint32_t plane = blk / ((BM / 32) * 8), rt = (blk / 8) % (BM / 32), step = blk % 8;
        const uint8_t* src = (plane ? a.xl : a.xh) + ((tile0 + (uint64_t)rt * a.xsteps + step) * 64 + ln) * 16;
        return *reinterpret_cast<const float4*>(src);
    };
    auto pre_dst = [&](uint32_t buf, int i) __attribute__((always_inline)) {
        const uint32_t c = tid + T * i, blk = c >> 6, ln = c & 63;
        const uint32_t plane = blk / ((BM / 32) * 8), rt = (blk / 8) % (BM / 32), step = blk % 8;
        return reinterpret_cast<float4*>(lds_a[buf][plane] + step * STEP + rt * 1024 + ln * 16);
    };
    auto pre_sum_src = [&](uint64_t tile0, int i) __attribute__((always_inline)) {
        const uint32_t e = tid + T * i, step = e / BM, row = e % BM;
        return a.xs[(tile0 + (uint64_t)(row / 32) * a.xsteps + step) * 32 + (row & 31)];
    };
    auto stage_load = [&](uint32_t st, int slot) __attribute__((always_inline)) {
        if constexpr (PRE) {
            const uint32_t gstage = min(st, nstages - 1);      // past the end: any valid stage, never used
            const uint64_t tile0 = (uint64_t)(m0 / 32) * a.xsteps + gstage * 8;
            xp0 = pre_src(tile0, 0); xp1 = pre_src(tile0, 1); xp2 = pre_src(tile0, 2); xp3 = pre_src(tile0, 3);
            if constexpr (NCH == 8) {
                xp4 = pre_src(tile0, 4); xp5 = pre_src(tile0, 5); xp6 = pre_src(tile0, 6); xp7 = pre_src(tile0, 7);
            }
            xsr0 = pre_sum_src(tile0, 0);
            if constexpr (NS == 2) xsr1 = pre_sum_src(tile0, 1);
        } else {
        if (!s_active) return;
        const uint32_t k0 = st * kStageK + s_step * 16;
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const float* xrow = a.x + (uint64_t)min(m0 + s_row + RPP * it, a.m - 1) * a.k;
#pragma unroll
            for (int i = 0; i < 4; i++)
                xraw[slot][it][i] = *reinterpret_cast<const float4*>(xrow + min(k0 + 4 * i, a.k - 4));
        }
        }
    };
    // Conversion of the values loaded for stage `st`, in 2*NI pieces of 8 values so that it can
    // be spread over the MFMA steps of the stage being multiplied.
    constexpr int PIECES = PRE ? 4 : 2 * NI;             // spread over the last steps of a stage: the
    static_assert(!PRE || NCH % 4 == 0, "chunks per piece"); // loads were issued at its first step
    float xsum[NI];
    float s_rinv[NI];                                    // non-PRE: the factor of each row this thread converts
#pragma unroll
    for (int it = 0; it < NI; it++) s_rinv[it] = PRE ? 1.0f : a.rinv[min(m0 + s_row + RPP * it, a.m - 1)];
    auto stage_store_piece = [&](uint32_t st, uint32_t buf, int piece, int slot) __attribute__((always_inline)) {
        if constexpr (PRE) {                               // NCH/4 chunks per piece, the sums with the last
            if constexpr (NCH == 4) {
                switch (piece) {
                    case 0: *pre_dst(buf, 0) = xp0; break;
                    case 1: *pre_dst(buf, 1) = xp1; break;
                    case 2: *pre_dst(buf, 2) = xp2; break;
                    default: *pre_dst(buf, 3) = xp3; break;
                }
            } else {
                switch (piece) {
                    case 0: *pre_dst(buf, 0) = xp0; *pre_dst(buf, 1) = xp1; break;
                    case 1: *pre_dst(buf, 2) = xp2; *pre_dst(buf, 3) = xp3; break;
                    case 2: *pre_dst(buf, 4) = xp4; *pre_dst(buf, 5) = xp5; break;
                    default: *pre_dst(buf, 6) = xp6; *pre_dst(buf, 7) = xp7; break;
                }
            }
            if (piece == PIECES - 1) {
                lds_xs[buf][tid / BM][tid % BM] = xsr0;
                if constexpr (NS == 2) lds_xs[buf][(tid + T) / BM][(tid + T) % BM] = xsr1;
            }
        } else {
        if (!s_active) return;
        const int it = piece >> 1, b = piece & 1;         // b: which 8-k block of this thread's step
        const uint32_t row = s_row + RPP * it;
        const uint32_t rt = row >> 5, r32 = row & 31;
        const uint32_t kk = st * kStageK + s_step * 16 + 8 * b;
        const bool row_ok = m0 + row < a.m;
        const float4 q0 = xraw[slot][it][2 * b], q1 = xraw[slot][it][2 * b + 1];
        const bool in0 = row_ok && kk < a.k, in1 = row_ok && kk + 4 < a.k;   // k % 4 == 0
        const float rv = s_rinv[it];                       // exact: a power of two
        const float xv[8] = {in0 ? q0.x * rv : 0.0f, in0 ? q0.y * rv : 0.0f, in0 ? q0.z * rv : 0.0f, in0 ? q0.w * rv : 0.0f,
                             in1 ? q1.x * rv : 0.0f, in1 ? q1.y * rv : 0.0f, in1 ? q1.z * rv : 0.0f, in1 ? q1.w * rv : 0.0f};
        v8h hi, lo;
        float sum = b ? xsum[it] : 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int j = (e >> 1) + 4 * (e & 1);         // fragment element e holds k offset j
            const float x = xv[j];
            const _Float16 h = (_Float16)x;
            hi[e] = h;
            lo[e] = (_Float16)(x - (float)h);
            sum += x;                                     // hi + lo equals x to 2^-22 |x|
        }
        const uint32_t off = s_step * STEP + (rt * 2 + b) * 512 + r32 * 16;
        *reinterpret_cast<v8h*>(lds_a[buf][0] + off) = hi;
        *reinterpret_cast<v8h*>(lds_a[buf][1] + off) = lo;
        xsum[it] = sum;
        if (b) lds_xs[buf][s_step][row] = sum;
        }
    };

    // ---- weights: one load of TN words per MFMA step; a register is refilled for DEPTH stages
    // later right after its step has been converted -----------------------------------------
    words_t wq[DEPTH][8];
    auto weight_load = [&](uint32_t st, int set, int s) __attribute__((always_inline)) {
        const uint32_t kr = min(st * 16 + s * 2 + kb, word_rows - 1);
        wq[set][s] = *reinterpret_cast<const words_t*>(a.packed + (uint64_t)kr * a.n + col_c);
    };

    v16f acc[RT][TN];
#pragma unroll
    for (int i = 0; i < RT; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // scale / zero-point: of the current group, and (requested DEPTH stages ahead, like the
    // weights) of the group that follows each settlement point of a stage
    constexpr int NF = 8 / FOLD;                 // settlements per stage
    auto meta_load = [&](uint32_t g, floats_t& sc, floats_t& zp) __attribute__((always_inline)) {
        g = min(g, a.num_groups - 1);
        sc = *reinterpret_cast<const floats_t*>(a.scales + (uint64_t)g * a.n + col_c);
        zp = ZP4 ? zp4_load(a.zp4, g, a.n, col_c, floats_t{})
                 : *reinterpret_cast<const floats_t*>(a.zp + (uint64_t)g * a.n + col_c);
    };
    uint32_t g_cur = st_begin * kStageK / a.group_size;
    floats_t sc_cur, zp_cur, sc_after[DEPTH][NF], zp_after[DEPTH][NF];
    meta_load(g_cur, sc_cur, zp_cur);
    sc_cur = nonzero(sc_cur);
    // The zero-point of the current group, split: its nearest integer z (kept within what 1024 + z holds exactly in
    // f16) leaves the weights in the conversion, so that the matrix cores sum x (q - z) - an element that towers over
    // its row then weighs in with its own small product where q is near the zero-point, not with two large sums that
    // cancel -, and the rest, zp - z, stays in the rank-1 update below.
    // The weights of a step are converted while the matrix cores work on the step before (b_next below), so the
    // conversion's constants change one step ahead of the group: z_rest belongs to the group being multiplied,
    // z_rest_next to the one being converted.
    v2h z_big[TN], z_small[TN];
    float z_rest[TN], z_rest_next[TN];
    auto split_zero = [&](const floats_t& zps) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const float zp = flt_of(zps, j);
            float z = fminf(fmaxf(rintf(zp), -1008.0f), 1008.0f);
            z = zp == zp ? z : 0.0f;                          // a NaN zero-point stays whole in the rank-1 term
            z_rest_next[j] = zp - z;
            const _Float16 b = (_Float16)(1024.0f + z), sm = (_Float16)(-64.0f - z);
            z_big[j] = v2h{b, b};
            z_small[j] = v2h{sm, sm};
        }
    };
    split_zero(zp_cur);
#pragma unroll
    for (int j = 0; j < TN; j++) z_rest[j] = z_rest_next[j];

    // metadata of the groups that follow the settlement points of stage `st`
    auto stage_meta_load = [&](uint32_t st, int set) __attribute__((always_inline)) {
#pragma unroll
        for (int f = 0; f < NF; f++)
            meta_load((st * kStageK + (f + 1) * FOLD * 16) / a.group_size, sc_after[set][f], zp_after[set][f]);
    };

    constexpr bool PIPE = WAVES == 8 && FOLD >= 4;      // groups of 32 change their constants every other step: 5 % slower pipelined
    // PIPE: the factor that takes the accumulators from one group's scale to the next one's is applied tile by tile
    // in front of the next step's first MFMAs (1 where no group ended), not in one block that has to wait for the
    // last MFMA of this step and keeps the matrix cores waiting in turn.
    floats_t rv_next = splat_of(1.0f, floats_t{});           // (a vector, not an array: arrays reached through the lambdas end up in scratch memory)
    auto fold = [&](uint32_t buf, int s_last, uint32_t kend, int set, int f, auto rest_tag) __attribute__((always_inline)) {
        // rank-1 update acc[i][j] += X[i] (x) (-(zp[j] - z[j])) on the f32 matrix core: operand slot k=0
        // carries the values (lanes 0..31), slot k=1 (lanes 32..63) is zero; compiled out of the loop that runs when
        // every zero-point is an integer
        if constexpr (decltype(rest_tag)::value) {
            float zb[TN];
#pragma unroll
            for (int j = 0; j < TN; j++) zb[j] = kb == 0 ? -z_rest[j] : 0.0f;
#pragma unroll
            for (int i = 0; i < RT; i++) {
                float xs = 0.0f;
#pragma unroll
                for (int cc = 0; cc < FOLD; cc++) xs += lds_xs[buf][s_last - cc][(wm * RT + i) * 32 + l32];
                xs = kb == 0 ? xs : 0.0f;
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(xs, zb[j], acc[i][j], 0, 0, 0);
            }
        }
        const uint32_t g_after = kend / a.group_size;
        if (kend < k_end && g_after != g_cur) {           // uniform: a new group starts
            const floats_t sn = nonzero(sc_after[set][f]);
            float rv[TN];
#pragma unroll
            for (int j = 0; j < TN; j++) rv[j] = flt_of(sc_cur, j) / flt_of(sn, j);
            if constexpr (PIPE) {
                rv_next = sc_cur / sn;                          // the same quotients, component by component
            } else {
#pragma unroll
                for (int i = 0; i < RT; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[i][j][r] *= rv[j];
            }
            g_cur = g_after;
            sc_cur = sn;
            zp_cur = zp_after[set][f];
#pragma unroll
            for (int j = 0; j < TN; j++) z_rest[j] = z_rest_next[j];      // split when the group's first step was converted
        } else if constexpr (PIPE) {
            rv_next = splat_of(1.0f, floats_t{});
        }
    };

    // A fragments of MFMA step s; with PREFETCH they are read one step ahead of their use, into
    // the slot of the step's parity (not for the largest tile: it has no registers to spare and
    // sixteen MFMAs per step to hide the read behind).
    constexpr bool PREFETCH = RT * TN <= 4;
    v8h ah[PREFETCH ? 2 : 1][RT], al[PREFETCH ? 2 : 1][RT];
    auto read_frags = [&](uint32_t buf, int s, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RT; i++) {
            const uint32_t off = s * STEP + (wm * RT + i) * 1024 + lane * 16;
            ah[slot][i] = *reinterpret_cast<const v8h*>(lds_a[buf][0] + off);
            al[slot][i] = *reinterpret_cast<const v8h*>(lds_a[buf][1] + off);
        }
    };

    // Multiply stage `st` from LDS buffer `buf`; refill the weight registers for stage
    // st+DEPTH and convert the activations of stage st+1 into the other buffer.
    // B fragments of the step that comes next, converted while the matrix cores are busy with the current one: a wave
    // cannot issue anything while it waits to issue an MFMA, so conversion and MFMAs of the same step one after
    // the other leave the vector ALU idle during the MFMAs and the matrix cores idle during the conversion.
    // (Not the four-wave shape: it has no registers for a second set of fragments and converts in place.)
    v8h b_next[TN];
    auto convert_words = [&](const words_t& wv) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; j++) b_next[j] = nibbles_to_f16(word_of(wv, j), z_big[j], z_small[j]);
    };
    auto compute = [&](uint32_t st, uint32_t buf, auto set_tag, auto rest_tag) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_tag)::value;
        constexpr int SETN = (SET + 1) % DEPTH;              // the set of the stage after this one
        if (PREFETCH) read_frags(buf, 0, 0);
#pragma unroll
        for (int s = 0; s < 8; s++) {
            constexpr int kOne = 1;
            const int cur = PREFETCH ? (s & kOne) : 0;
            if (PREFETCH) {
                if (s + 1 < 8) read_frags(buf, s + 1, (s + 1) & 1);
                __builtin_amdgcn_sched_barrier(0);    // keep the reads above this step's arithmetic
            } else {
                read_frags(buf, s, 0);
            }
            v8h bfr[TN];
            const uint32_t kend = st * kStageK + (s + 1) * 16;
            const bool group_ends = (s + 1) % FOLD == 0 && kend < k_end && kend / a.group_size != g_cur;
            if constexpr (PIPE) {
#pragma unroll
                for (int j = 0; j < TN; j++) bfr[j] = b_next[j];
                // the next step: of this stage, or the first of the next one (its words were requested a stage ago;
                // past the end of K they are some valid words and the result is never used).  Where a group ends
                // with this step, the next one is converted with the constants of the group that follows.
                if (group_ends) split_zero(zp_after[SET][s / FOLD]);
                if (s + 1 < 8) {
                    convert_words(wq[SET][s + 1]);
                    weight_load(st + DEPTH, SET, s + 1);
                } else {
                    convert_words(wq[SETN][0]);
                    weight_load(st + 1 + DEPTH, SETN, 0);
                }
            } else {
                convert_words(wq[SET][s]);
                weight_load(st + DEPTH, SET, s);
#pragma unroll
                for (int j = 0; j < TN; j++) bfr[j] = b_next[j];
            }
            // all hi products, then all lo products: dependent MFMAs are TN*RT apart
            constexpr bool RESCALE = PIPE && true;
            const bool after_fold = s % FOLD == 0;            // the step before settled a group (or the kernel starts: factor 1)
#pragma unroll
            for (int i = 0; i < RT; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    if (RESCALE && after_fold) {
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[i][j][r] *= flt_of(rv_next, j);
                    }
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[cur][i], bfr[j], acc[i][j], 0, 0, 0);
                }
#pragma unroll
            for (int i = 0; i < RT; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[cur][i], bfr[j], acc[i][j], 0, 0, 0);
            if constexpr (PIPE) {                     // one MFMA, then its share of the conversion's vector instructions in its shadow
                constexpr int kConv = (9 * TN + 6 + 2 * RT * TN - 1) / (2 * RT * TN);
                if (after_fold) {                     // (a tile's 16 multiplications stand in front of its first MFMA)
                    __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
                    for (int i = 1; i < RT * TN; i++) {
                        __builtin_amdgcn_sched_group_barrier(0x002, 16 + kConv, 0);
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x002, 2 * kConv, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
                    for (int i = 1; i < RT * TN; i++) {
                        __builtin_amdgcn_sched_group_barrier(0x002, kConv, 0);
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 2 * RT * TN; i++) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, kConv, 0);
                    }
                }
            }
            if (!PIPE && group_ends) split_zero(zp_after[SET][s / FOLD]);     // this step's words are converted: the next group's constants
            if ((s + 1) % FOLD == 0) fold(buf, s, kend, SET, s / FOLD, rest_tag);
            if (s >= 8 - PIECES) stage_store_piece(st + 1, buf ^ 1, s - (8 - PIECES), DEPTH - 1 - SET);
        }
        stage_meta_load(st + DEPTH, SET);
    };

    // Stage st_begin + i lives in weight set and activation slot i % DEPTH.  While stage st is
    // multiplied, the activations of st+1 (loaded a stage earlier when DEPTH is 2) are converted
    // and those of st+DEPTH are requested.
    stage_load(st_begin, 0);
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
#pragma unroll
        for (int s = 0; s < 8; s++) weight_load(st_begin + d, d, s);
#pragma unroll
    for (int d = 0; d < DEPTH; d++) stage_meta_load(st_begin + d, d);
    if (DEPTH == 2) stage_load(st_begin + 1, DEPTH - 1);
#pragma unroll
    for (int piece = 0; piece < PIECES; piece++) stage_store_piece(st_begin, 0, piece, 0);
    if constexpr (PIPE) {
        convert_words(wq[0][0]);
        weight_load(st_begin + DEPTH, 0, 0);
    }
    // The loop exists twice, with and without the rank-1 updates.
    auto stages = [&](auto rest_tag) __attribute__((always_inline)) {
        uint32_t buf = 0;
        for (uint32_t st = st_begin; st < st_end; st += DEPTH) {
            lds_barrier();                                // buffer `buf` staged; the other one is free
            stage_load(st + DEPTH, 0);
            compute(st, buf, std::integral_constant<int, 0>{}, rest_tag);
            buf ^= 1;
            if (DEPTH == 2 && st + 1 < st_end) {
                lds_barrier();
                stage_load(st + 1 + DEPTH, DEPTH - 1);
                compute(st + 1, buf, std::integral_constant<int, DEPTH - 1>{}, rest_tag);
                buf ^= 1;
            }
        }
    };
    if constexpr (ZP4) {
        stages(std::false_type{});
    } else {
        if (__builtin_amdgcn_ballot_w64((zflag.x | zflag.y | zflag.z | zflag.w) != 0) != 0) stages(std::true_type{});
        else stages(std::false_type{});
    }

    // ---- store: for each row a lane holds TN adjacent columns ----------------------------
    if (!col_ok) return;
    const bool final_out = gridDim.z == 1;
    float* dst = out + (final_out ? 0 : (uint64_t)blockIdx.z * a.m * a.n);
    float bv[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) bv[j] = 0.0f;
    if (final_out && a.bias) {
        const floats_t b = *reinterpret_cast<const floats_t*>(a.bias + colbase);
#pragma unroll
        for (int j = 0; j < TN; j++) bv[j] = flt_of(b, j);
    }
#pragma unroll
    for (int i = 0; i < RT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t row = m0 + (wm * RT + i) * 32 + 8 * (r / 4) + 4 * kb + (r % 4);
            if (row >= a.m) continue;
            const float rf = lds_rf[row - m0];             // back to the row's own scale: exact, a power of two
            float o[TN];
#pragma unroll
            for (int j = 0; j < TN; j++) o[j] = fmaf(acc[i][j][r] * rf, flt_of(sc_cur, j), bv[j]);
            float* p = dst + (uint64_t)row * a.n + colbase;
            if (TN == 4) *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[TN - 1]);
            else *reinterpret_cast<float2*>(p) = make_float2(o[0], o[1]);
        }
}

// y = part[0] + part[1] + ... (in that order) + bias; count4 = m*n/4.  All partials are requested
// before the first is added (a split beyond the last re-reads the last one and is not added), so
// the kernel costs one round trip to memory instead of one per split.
__global__ __launch_bounds__(256) void w4_gemm_reduce_kernel(const float4* __restrict__ part,
                                                             const float* __restrict__ bias,
                                                             float4* __restrict__ y, uint32_t count4,
                                                             uint32_t n4, uint32_t splits) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= count4) return;
    float4 v[kMaxSplits];
#pragma unroll
    for (uint32_t p = 0; p < kMaxSplits; p++) v[p] = part[(uint64_t)min(p, splits - 1) * count4 + idx];
    float4 b = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (bias) b = *reinterpret_cast<const float4*>(bias + 4 * (idx % n4));
    float4 s = v[0];
#pragma unroll
    for (uint32_t p = 1; p < kMaxSplits; p++) {
        if (p < splits) { s.x += v[p].x; s.y += v[p].y; s.z += v[p].z; s.w += v[p].w; }
    }
    if (bias) { s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w; }
    y[idx] = s;
}

bool w4_gemm_supported(const W4Args& a) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a.packed) | reinterpret_cast<uintptr_t>(a.scales) |
                           reinterpret_cast<uintptr_t>(a.zp) | reinterpret_cast<uintptr_t>(a.y) |
                           (a.bias ? reinterpret_cast<uintptr_t>(a.bias) : 0);
    // zero-point terms are settled every 32, 64 or 128 rows of K: groups must end there
    const bool group_ok = a.group_size == 32 || a.group_size == 64 || a.group_size % kStageK == 0;
    return a.m >= 1 && a.n % 4 == 0 && (bits & 15) == 0 && !a.g_idx && group_ok;
}

// K splits for `tiles` output tiles on a 256-CU device: enough workgroups to cover the
// chip while every split keeps at least one stage; capped, since partial tiles cost traffic.
static uint32_t pick_splits(uint32_t tiles, uint32_t nstages, uint32_t* stages_per_split) {
    uint32_t want = tiles >= 192 ? 1 : min(min((uint32_t)kMaxSplits, nstages), max(1u, 256 / tiles));
    const uint32_t sps = ceil_div(nstages, want);
    *stages_per_split = sps;
    return ceil_div(nstages, sps);                       // no empty split
}

// flags[block] = 1 when the block's share of the zero-point table (count4 float4) holds a value that is no integer
// within the range that the tile kernel takes off inside its f16 conversion, else 0.  Every word is written by every
// launch: nothing to clear.
__global__ __launch_bounds__(256) void w4_zp_scan_kernel(const float4* __restrict__ zp, uint32_t count4,
                                                         uint32_t* __restrict__ flags) {
    bool mine = false;
    const uint32_t step = kZpFlagWords * 256;
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < count4; i += 4 * step) {
        float4 z[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; u++) z[u] = zp[min(i + u * step, count4 - 1)];
#pragma unroll
        for (uint32_t u = 0; u < 4; u++) {
            const float v[4] = {z[u].x, z[u].y, z[u].z, z[u].w};
#pragma unroll
            for (int j = 0; j < 4; j++) mine = mine || !(v[j] == rintf(v[j]) && fabsf(v[j]) <= 1008.0f);   // a NaN counts
        }
    }
    const int any = __syncthreads_or(mine);
    if (threadIdx.x == 0) flags[blockIdx.x] = any ? 1u : 0u;
}

// xp[r][j] = x[r][perm[j]] (perm null: j) for j < k, 0 for k <= j < k4: the act-order column
// gather done once per call instead of once per workgroup column, and the padding / alignment
// of rows that the tile kernel's 128-bit loads need.
// One workgroup per row of x: rinv[row] = 2^(141 - E) for a largest magnitude a * 2^(E - 127), 1 <= a < 2, so that
// the scaled row lies in [2^14, 2^15) -- inside the range of f16 whatever the row's own size, and with its small
// elements' low halves clear of f16's subnormals -- and rfac[row] = 1 / rinv[row].  Both are powers of two: scaling
// by them is exact, so rows that needed none give the bits they gave without.  A row of zeros, or one that holds
// an infinity or a NaN (which poisons the row's results, as it should), keeps the factor 1.
// amax: bits of the row's largest magnitude.  2^(141 - E) has the biased exponent 268 - e; kept within [14, 240] so
// that both factors are normal numbers (rows below 2^-99 are scaled by 2^113 only: they stay far inside f16's
// range all the same).  Returns the bits of rinv; rfac has the biased exponent 254 minus that one.
__device__ __forceinline__ uint32_t w4_row_factor_exponent(uint32_t amax) {
    const uint32_t e = amax >> 23;                           // biased exponent of the largest magnitude
    return e == 0 || e == 255 ? 127u : min(268u - e, 240u);
}

__global__ __launch_bounds__(256) void w4_row_factor_kernel(const float* __restrict__ x, uint32_t k,
                                                            float* __restrict__ rinv, float* __restrict__ rfac) {
    __shared__ uint32_t part[4];
    const uint32_t tid = threadIdx.x, row = blockIdx.x;
    const float* xr = x + (uint64_t)row * k;
    uint32_t amax = 0;                                       // bit patterns of |x| order like the values; NaN sorts last
    if (k % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        for (uint32_t i = tid; i < k / 4; i += 256) {
            const float4 v = reinterpret_cast<const float4*>(xr)[i];
            amax = max(max(amax, __float_as_uint(v.x) & 0x7FFFFFFFu), __float_as_uint(v.y) & 0x7FFFFFFFu);
            amax = max(max(amax, __float_as_uint(v.z) & 0x7FFFFFFFu), __float_as_uint(v.w) & 0x7FFFFFFFu);
        }
    } else {
        for (uint32_t i = tid; i < k; i += 256) amax = max(amax, __float_as_uint(xr[i]) & 0x7FFFFFFFu);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) amax = max(amax, (uint32_t)__shfl_xor((int)amax, o));
    if ((tid & 63) == 0) part[tid >> 6] = amax;
    __syncthreads();
    if (tid == 0) {
        amax = max(max(part[0], part[1]), max(part[2], part[3]));
        const uint32_t b = w4_row_factor_exponent(amax);
        rinv[row] = __uint_as_float(b << 23);
        rfac[row] = __uint_as_float((254u - b) << 23);
    }
}

__global__ __launch_bounds__(256) void w4_prepare_x_kernel(const float* __restrict__ x,
                                                           const int32_t* __restrict__ perm,
                                                           float* __restrict__ xp, uint32_t k, uint32_t k4) {
    const uint32_t j = blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (j >= k4) return;
    float v = 0.0f;
    if (j < k) v = x[(uint64_t)row * k + (perm ? (uint32_t)perm[j] : j)];
    xp[(uint64_t)row * k4 + j] = v;
}

// Activations -> the form the PRE tile kernel copies into LDS.  Workgroup = one row tile of 32
// and four steps of 16 k; thread t holds 8 consecutive k (t % 8) of row t / 8, as the staging
// role of the tile kernel does.  Per (row tile, step) it writes two 1 KB fragment blocks (hi, lo:
// lane = 32 * (k block of 8) + row, 8 halves in the k order 0,4,1,5,2,6,3,7 of the weight
// fragment) and 32 sums.  Rows beyond m and columns beyond k are written as zeros, so that the
// tile kernel needs no mask.  perm: act-order gather (x[row][perm[j]]).
template <bool VEC>
__global__ __launch_bounds__(256) void w4_convert_x_kernel(const float* __restrict__ x,
                                                           const int32_t* __restrict__ perm,
                                                           uint8_t* __restrict__ xh, uint8_t* __restrict__ xl,
                                                           float* __restrict__ xs, uint32_t m, uint32_t k,
                                                           uint32_t xsteps, const float* __restrict__ rinv) {
    const uint32_t tid = threadIdx.x, row = tid >> 3, kblk = tid & 7;
    const uint32_t tile = blockIdx.y, step = blockIdx.x * 4 + (kblk >> 1), kb = kblk & 1;
    const uint32_t grow = tile * 32 + row, k0 = step * 16 + kb * 8;
    float xv[8];
    if (VEC) {                                               // no perm, k % 8 == 0, 16-byte aligned x
        const bool in = grow < m && k0 < k;
        const float* src = x + (uint64_t)(in ? grow : 0) * k + (in ? k0 : 0);
        const float4 lo4 = *reinterpret_cast<const float4*>(src), hi4 = *reinterpret_cast<const float4*>(src + 4);
        xv[0] = in ? lo4.x : 0.0f; xv[1] = in ? lo4.y : 0.0f; xv[2] = in ? lo4.z : 0.0f; xv[3] = in ? lo4.w : 0.0f;
        xv[4] = in ? hi4.x : 0.0f; xv[5] = in ? hi4.y : 0.0f; xv[6] = in ? hi4.z : 0.0f; xv[7] = in ? hi4.w : 0.0f;
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const bool in = grow < m && k0 + j < k;
            const uint32_t kk = in ? k0 + j : 0;
            const float v = x[(uint64_t)(in ? grow : 0) * k + (perm ? (uint32_t)perm[kk] : kk)];
            xv[j] = in ? v : 0.0f;
        }
    }
    v8h hi, lo;
    float sum = 0.0f;
    const float rv = rinv[min(grow, m - 1)];                 // exact: a power of two
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int j = (e >> 1) + 4 * (e & 1);                // fragment element e holds k offset j
        const float v = xv[j] * rv;
        const _Float16 h = (_Float16)v;
        hi[e] = h;
        lo[e] = (_Float16)(v - (float)h);                    // hi + lo equals v to 2^-22 |v|
        sum += v;
    }
    sum += __shfl_xor(sum, 1);                               // the other 8 of this row's step
    const uint64_t blk = (uint64_t)tile * xsteps + step;
    *reinterpret_cast<v8h*>(xh + (blk * 64 + kb * 32 + row) * 16) = hi;
    *reinterpret_cast<v8h*>(xl + (blk * 64 + kb * 32 + row) * 16) = lo;
    if (kb == 0) xs[blk * 32 + row] = sum;
}

// The same planes from whole rows: a workgroup copies `rows` rows of x into LDS with contiguous reads, finds each
// row's factor there (no pass of its own over x, no launch of its own) and converts from LDS.  With act-order
// weights (x[row][perm[j]]) the gather happens in LDS too: from global memory a wave instruction would touch 64
// cache lines for 256 bytes.  Thread = (row, MFMA step): 16 values, both k blocks of the step.
// Dynamic LDS: rows * kpad floats, kpad = k rounded up to 4.
__global__ __launch_bounds__(256) void w4_convert_x_rows_kernel(const float* __restrict__ x,
                                                                const int32_t* __restrict__ perm,
                                                                uint8_t* __restrict__ xh, uint8_t* __restrict__ xl,
                                                                float* __restrict__ xs, uint32_t m, uint32_t k,
                                                                uint32_t xsteps, uint32_t rows, uint32_t kpad,
                                                                float* __restrict__ rfac) {
    extern __shared__ __attribute__((aligned(16))) float lds_rows[];
    __shared__ uint32_t rowmax[8];
    const uint32_t tid = threadIdx.x;
    if (tid < 8) rowmax[tid] = 0;
    const uint32_t row0 = blockIdx.x * rows;                  // rows divides 32: a workgroup stays inside a row tile
    const uint32_t live = row0 < m ? min(rows, m - row0) : 0;
    const float* src = x + (uint64_t)row0 * k;
    if ((k % 4 == 0) && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        const uint32_t vec = live * (k / 4);                  // the live rows are one contiguous run, and kpad == k
        for (uint32_t i = tid; i < vec; i += 256)
            reinterpret_cast<float4*>(lds_rows)[i] = reinterpret_cast<const float4*>(src)[i];
    } else {
        for (uint32_t r = 0; r < live; r++)
            for (uint32_t i = tid; i < k; i += 256) lds_rows[r * kpad + i] = src[(uint64_t)r * k + i];
    }
    __syncthreads();
    const uint32_t r = tid % rows, grow = row0 + r, tile = grow / 32, row = grow % 32;
    const float* lr = lds_rows + r * kpad;
    // the row's factor (w4_row_factor_kernel's), from the copy in LDS
    {
        uint32_t am = 0;
        if (grow < m)
            for (uint32_t i = tid / rows; i < k; i += 256 / rows) am = max(am, __float_as_uint(lr[i]) & 0x7FFFFFFFu);
        atomicMax(&rowmax[r], am);
    }
    __syncthreads();
    const uint32_t fb = w4_row_factor_exponent(rowmax[r]);
    const float rv = __uint_as_float(fb << 23);               // exact: a power of two
    if (tid < rows && grow < m) rfac[grow] = __uint_as_float((254u - fb) << 23);
    for (uint32_t step = tid / rows; step < xsteps; step += 256 / rows) {
        const uint32_t k0 = step * 16;
        float xv[16];
        if (!perm && grow < m && k0 + 16 <= k) {             // plain order: kpad % 4 == 0, so the row is aligned
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 v = *reinterpret_cast<const float4*>(lr + k0 + 4 * q);
                xv[4 * q] = v.x; xv[4 * q + 1] = v.y; xv[4 * q + 2] = v.z; xv[4 * q + 3] = v.w;
            }
        } else if (perm && grow < m && k0 + 16 <= k && (reinterpret_cast<uintptr_t>(perm) & 15) == 0) {
            int4 pj[4];
#pragma unroll
            for (int q = 0; q < 4; q++) pj[q] = *reinterpret_cast<const int4*>(perm + k0 + 4 * q);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                xv[4 * q] = lr[(uint32_t)pj[q].x]; xv[4 * q + 1] = lr[(uint32_t)pj[q].y];
                xv[4 * q + 2] = lr[(uint32_t)pj[q].z]; xv[4 * q + 3] = lr[(uint32_t)pj[q].w];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const bool in = grow < m && k0 + j < k;
                const float v = lr[in ? (perm ? (uint32_t)perm[k0 + j] : k0 + j) : 0];
                xv[j] = in ? v : 0.0f;
            }
        }
        const uint64_t blk = (uint64_t)tile * xsteps + step;
        float sum[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            v8h hi, lo;
            sum[kb] = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int j = (e >> 1) + 4 * (e & 1);            // fragment element e holds k offset j
                const float v = xv[8 * kb + j] * rv;
                const _Float16 h = (_Float16)v;
                hi[e] = h;
                lo[e] = (_Float16)(v - (float)h);
                sum[kb] += v;
            }
            *reinterpret_cast<v8h*>(xh + (blk * 64 + kb * 32 + row) * 16) = hi;
            *reinterpret_cast<v8h*>(xl + (blk * 64 + kb * 32 + row) * 16) = lo;
        }
        xs[blk * 32 + row] = sum[0] + sum[1];                 // the order of w4_convert_x_kernel: eight and eight
    }
}

// The same planes for plain x (no gather, k % 8 == 0, 16-byte aligned rows) in one pass over x and no launch for the
// factors: a workgroup takes four rows, thread (row t % 4, step t / 4 + 64 i) keeps its ITER steps of 16 values in
// registers between finding the row's largest magnitude and writing the planes.  ITER = ceil(xsteps / 64) up to 16
// (K up to 16384).
template <int ITER>
__global__ __launch_bounds__(256) void w4_convert_x_regs_kernel(const float* __restrict__ x, uint8_t* __restrict__ xh,
                                                                uint8_t* __restrict__ xl, float* __restrict__ xs,
                                                                float* __restrict__ rfac, uint32_t m, uint32_t k,
                                                                uint32_t xsteps) {
    __shared__ uint32_t rowmax[4];
    const uint32_t tid = threadIdx.x, r = tid & 3, s0 = tid >> 2;
    const uint32_t grow = blockIdx.x * 4 + r, tile = grow >> 5, row = grow & 31;
    const bool live = grow < m;
    const float* xr = x + (uint64_t)(live ? grow : 0) * k;
    if (tid < 4) rowmax[tid] = 0;
    float4 v[ITER][4];
    uint32_t am = 0;
#pragma unroll
    for (int i = 0; i < ITER; i++) {
        const uint32_t k0 = (s0 + 64 * i) * 16;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t kk = k0 + 4 * q;
            const bool in = live && kk < k;                  // k % 4 == 0: a float4 is all in or all out
            const float4 f = *reinterpret_cast<const float4*>(xr + (in ? kk : 0));
            v[i][q] = in ? f : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            am = max(max(am, __float_as_uint(v[i][q].x) & 0x7FFFFFFFu), __float_as_uint(v[i][q].y) & 0x7FFFFFFFu);
            am = max(max(am, __float_as_uint(v[i][q].z) & 0x7FFFFFFFu), __float_as_uint(v[i][q].w) & 0x7FFFFFFFu);
        }
    }
#pragma unroll
    for (int o = 4; o <= 32; o <<= 1) am = max(am, (uint32_t)__shfl_xor((int)am, o));   // the lanes of this row
    __syncthreads();                                         // rowmax is zeroed
    if ((tid & 63) < 4) atomicMax(&rowmax[r], am);
    __syncthreads();
    const uint32_t fb = w4_row_factor_exponent(rowmax[r]);
    const float rv = __uint_as_float(fb << 23);              // exact: a power of two
    if (tid < 4 && live) rfac[grow] = __uint_as_float((254u - fb) << 23);
#pragma unroll
    for (int i = 0; i < ITER; i++) {
        const uint32_t step = s0 + 64 * i;
        if (step >= xsteps) break;
        const uint64_t blk = (uint64_t)tile * xsteps + step;
        const float xv[16] = {v[i][0].x, v[i][0].y, v[i][0].z, v[i][0].w, v[i][1].x, v[i][1].y, v[i][1].z, v[i][1].w,
                              v[i][2].x, v[i][2].y, v[i][2].z, v[i][2].w, v[i][3].x, v[i][3].y, v[i][3].z, v[i][3].w};
        float sum[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            v8h hi, lo;
            sum[kb] = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int j = (e >> 1) + 4 * (e & 1);        // fragment element e holds k offset j
                const float t = xv[8 * kb + j] * rv;
                const _Float16 h = (_Float16)t;
                hi[e] = h;
                lo[e] = (_Float16)(t - (float)h);
                sum[kb] += t;
            }
            *reinterpret_cast<v8h*>(xh + (blk * 64 + kb * 32 + row) * 16) = hi;
            *reinterpret_cast<v8h*>(xl + (blk * 64 + kb * 32 + row) * 16) = lo;
        }
        xs[blk * 32 + row] = sum[0] + sum[1];                // the order of w4_convert_x_kernel: eight and eight
    }
}

// rows of x per workgroup of w4_convert_x_rows_kernel (a power of two up to 8), 0: k too long for LDS
static uint32_t convert_perm_rows(uint32_t kpad) {
    const uint32_t fit = (64u * 1024) / (kpad * 4);
    return fit >= 8 ? 8 : fit >= 4 ? 4 : fit >= 2 ? 2 : fit;
}

template <int RT, int WM, int TN, int WAVES, int DEPTH, int FOLD>
static int launch_tile(const W4Args& a_in, hipStream_t s) {
    W4Args a = a_in;
    const uint32_t tn = ceil_div(a.n, (WAVES / WM) * 32 * TN), tm = ceil_div(a.m, 32 * RT * WM);
    const uint32_t nstages = ceil_div(a.padded_k, kStageK);
    uint32_t sps = nstages;
    const uint32_t splits = pick_splits(tn * tm, nstages, &sps);
    // 64-row tiles of eight waves: activations converted once, up front (10 % at m = 512).  The
    // four-wave shape has no registers to spare for the staged chunks and converts in place.
    constexpr bool PRE = RT * WM >= 2 && (WAVES == 8 || (WAVES == 4 && TN == 2));
    constexpr uint32_t BM = 32 * RT * WM;
    // workspace: [activations in the form the kernel reads][partial tiles]
    const bool prepare = !PRE && (a.perm || a.k % 4 != 0 || (reinterpret_cast<uintptr_t>(a.x) & 15) != 0);
    const uint32_t k4 = (a.k + 3) & ~3u;
    const uint32_t xtiles = tm * (BM / 32), xsteps = nstages * 8;   // whole workgroup tiles, whole stages
    RUMUS_REQUIRE(!(prepare || PRE) || max(a.m, xtiles) <= 65535,
                  "qmatmul_int4: m %u is beyond the grid limit of the activation copy", a.m);
    const size_t plane_bytes = (size_t)xtiles * xsteps * 1024, sums_bytes = (size_t)xtiles * xsteps * 128;
    const size_t x_bytes = PRE ? 2 * plane_bytes + sums_bytes
                               : prepare ? (((size_t)a.m * k4 * sizeof(float) + 255) & ~size_t(255)) : 0;
    const size_t part_bytes = splits > 1 ? (size_t)splits * a.m * a.n * sizeof(float) : 0;
    const size_t flag_bytes = kZpFlagWords * sizeof(uint32_t);
    const size_t fac_bytes = flag_bytes + (((size_t)2 * a.m * sizeof(float) + 255) & ~size_t(255));   // flags, rinv[m], rfac[m]
    float* out = a.y;
    WorkspaceLease lease;                                    // until the last kernel of this call is queued
    {
        void* ws = nullptr;
        if (int rc = workspace_get(s, fac_bytes + x_bytes + part_bytes, &ws, lease)) return rc;
        uint32_t* zflags = static_cast<uint32_t*>(ws);
        float* fac = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + flag_bytes);
        ws = static_cast<uint8_t*>(ws) + fac_bytes;
        // the look at the zero-points takes 2.5 to 3 us: from 128 rows on the updates it may save cost more
        if (!a.zp4 && a.m >= 128) {
            hipLaunchKernelGGL(w4_zp_scan_kernel, dim3(kZpFlagWords), dim3(256), 0, s, reinterpret_cast<const float4*>(a.zp),
                               (uint32_t)((uint64_t)a.num_groups * a.n / 4), zflags);
            if (int rc = check_launch("w4_zp_scan_kernel")) return rc;
            a.zflags = zflags;
        }
        a.rinv = fac;
        a.rfac = fac + a.m;
        // the pre-converting kernels that hold whole rows (in LDS for the gather, in registers for plain x) find
        // the factors themselves
        const bool vec8 = !a.perm && a.k % 8 == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15) == 0;
        const uint32_t regs_iter = PRE && vec8 ? ceil_div(xsteps, 64u) : 0;   // steps of 16 k per thread
        const bool in_regs = regs_iter >= 1 && regs_iter <= 16;
        if (!(PRE && ((a.perm && convert_perm_rows(k4)) || in_regs))) {
            hipLaunchKernelGGL(w4_row_factor_kernel, dim3(a.m), dim3(256), 0, s, a.x, a.k, fac, fac + a.m);
            if (int rc = check_launch("w4_row_factor_kernel")) return rc;
        }
        if (PRE) {
            uint8_t* base = static_cast<uint8_t*>(ws);
            const bool vec = !a.perm && a.k % 8 == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15) == 0;
            const dim3 grid(xsteps / 4, xtiles);
            float* sums = reinterpret_cast<float*>(base + 2 * plane_bytes);
            const uint32_t perm_rows = a.perm ? convert_perm_rows(k4) : 0;   // 0: a row does not fit LDS
            if (in_regs) {
                const dim3 g4(xtiles * 8);                   // four rows each
#define RUMUS_W4_REGS(N) hipLaunchKernelGGL(w4_convert_x_regs_kernel<N>, g4, dim3(256), 0, s, a.x, base, base + plane_bytes, \
                                            sums, fac + a.m, a.m, a.k, xsteps)
                if (regs_iter <= 4) RUMUS_W4_REGS(4);
                else if (regs_iter <= 8) RUMUS_W4_REGS(8);
                else if (regs_iter <= 11) RUMUS_W4_REGS(11);
                else RUMUS_W4_REGS(16);
#undef RUMUS_W4_REGS
            } else if (perm_rows)
                hipLaunchKernelGGL(w4_convert_x_rows_kernel, dim3(xtiles * 32 / perm_rows), dim3(256),
                                   (size_t)perm_rows * k4 * sizeof(float), s, a.x, a.perm, base, base + plane_bytes, sums,
                                   a.m, a.k, xsteps, perm_rows, k4, fac + a.m);
            else if (vec) hipLaunchKernelGGL(w4_convert_x_kernel<true>, grid, dim3(256), 0, s, a.x, a.perm, base,
                                             base + plane_bytes, sums, a.m, a.k, xsteps, a.rinv);
            else hipLaunchKernelGGL(w4_convert_x_kernel<false>, grid, dim3(256), 0, s, a.x, a.perm, base,
                                    base + plane_bytes, sums, a.m, a.k, xsteps, a.rinv);
            if (int rc = check_launch("w4_convert_x_kernel")) return rc;
            a.xh = base;
            a.xl = base + plane_bytes;
            a.xs = sums;
            a.xsteps = xsteps;
        } else if (prepare) {
            float* xp = static_cast<float*>(ws);
            hipLaunchKernelGGL(w4_prepare_x_kernel, dim3(ceil_div(k4, 256), a.m), dim3(256), 0, s, a.x, a.perm, xp,
                               a.k, k4);
            if (int rc = check_launch("w4_prepare_x_kernel")) return rc;
            a.x = xp;
            a.perm = nullptr;
            a.k = k4;                                     // the added columns are zero
        }
        if (splits > 1) out = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + x_bytes);
    }
    if (a.zp4)
        hipLaunchKernelGGL((w4_gemm_tile_kernel<RT, WM, TN, WAVES, DEPTH, FOLD, true, PRE>), dim3(tn, tm, splits),
                           dim3(64 * WAVES), 0, s, a, out, sps);
    else
        hipLaunchKernelGGL((w4_gemm_tile_kernel<RT, WM, TN, WAVES, DEPTH, FOLD, false, PRE>), dim3(tn, tm, splits),
                           dim3(64 * WAVES), 0, s, a, out, sps);
    if (int rc = check_launch("w4_gemm_tile_kernel")) return rc;
    if (splits > 1) {
        const uint32_t count4 = (uint32_t)((uint64_t)a.m * a.n / 4);
        hipLaunchKernelGGL(w4_gemm_reduce_kernel, dim3(ceil_div(count4, 256)), dim3(256), 0, s,
                           reinterpret_cast<const float4*>(out), a.bias, reinterpret_cast<float4*>(a.y), count4,
                           a.n / 4, splits);
        return check_launch("w4_gemm_reduce_kernel");
    }
    return RUMUS_HIP_OK;
}

template <int RT, int WM, int TN, int WAVES, int DEPTH>
static int launch_fold(const W4Args& a, hipStream_t s) {
    switch (a.group_size) {                              // MFMA steps of 16 per zero-point settlement
        case 32: return launch_tile<RT, WM, TN, WAVES, DEPTH, 2>(a, s);
        case 64: return launch_tile<RT, WM, TN, WAVES, DEPTH, 4>(a, s);
        default: return launch_tile<RT, WM, TN, WAVES, DEPTH, 8>(a, s);  // a multiple of 128: once per stage
    }
}

int w4_launch_gemm(const W4Args& a, hipStream_t s) {
    RUMUS_REQUIRE((uint64_t)a.m * a.n < (1ull << 32), "qmatmul_int4: m * n must fit 32 bits");
    RUMUS_REQUIRE(a.m <= 65535 * 32, "qmatmul_int4: m %u is beyond the grid limit", a.m);
    // Two shapes of workgroup, eight waves side by side over 512 columns, chosen by how many
    // tiles the problem makes (measured on n = 4096 and n = 11008, m = 16 .. 8192):
    //   up to 72 tiles of 32 rows: 32 rows x 64 columns per wave; the small tile keeps more
    //       workgroups in flight when there are fewer tiles than CUs, and converts its few
    //       activations itself;
    //   beyond: 64 rows x 64 columns per wave, so that a converted weight fragment serves two row
    //       tiles, on activations converted once by w4_convert_x_kernel.
    // (Four waves of 64 x 128 each, two workgroups per CU, halve the LDS fragment reads but have
    // no registers left for pre-converted activations: 3-20 % slower from m = 1024 to 4096.)
    const uint64_t col_tiles = ceil_div(a.n, kTileCols);
    if (ceil_div(a.m, 32) * col_tiles <= 72) return launch_fold<1, 1, 2, 8, 1>(a, s);
    // The 64-row workgroups run one per CU, in rounds of 256 that last the same full or not (4096 x 11008, 1024 rows:
    // 352 workgroups take as long as 512).  When the last round would be poorly filled, the same tile with four
    // waves over 256 columns runs two per CU and a CU's last one alone at 3/4 of the time, while a pair costs 5 %
    // more than one eight-wave workgroup (1024 rows: 255 -> 220 us, 768: 251 -> 210, but 2048: 405 -> 425).  Same
    // order of the sums over K, same bits.
    const uint64_t row_tiles = ceil_div(a.m, 64);
    const uint64_t full_rounds = ceil_div(row_tiles * col_tiles, 256);
    const uint64_t halves = ceil_div(row_tiles * ceil_div(a.n, kTileCols / 2), 256);       // on the busiest CU
    if (row_tiles * col_tiles >= 192 && (halves / 2) * 105 + (halves % 2) * 75 < full_rounds * 97)
        return launch_fold<2, 1, 2, 4, 1>(a, s);
    return launch_fold<2, 1, 2, 8, 1>(a, s);
}

}  // namespace rumus
