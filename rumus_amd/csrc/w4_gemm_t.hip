// grad_x of the INT4 Linear for batches, on the f16 matrix cores:
//   out[m, k] = sum_n gy[m, n] * (q[k, n] - zp[g, n]) * s[g, n],   g = k / group_size
// (custom_forward(&QMatMulINT4TransposeOp, ..) quant.rs:262-317; qmatmul_int4_transpose.wgsl:37-74
// computes the same sums one output per thread with n as the serial loop).
//
// The sum runs over n, and scale and zero-point change with n, so they cannot be taken out of the
// sum the way the forward kernel takes them out per group.  They can be moved to the other operand:
//   out[m, k] = sum_n A_g[m, n] * (q[k, n] - z0[g, n])  -  c[m, g],
//   A_g[m, n] = gy[m, n] s[g, n],   z0 = rint(zp),   c[m, g] = sum_n A_g[m, n] (zp[g, n] - z0[g, n])
// so the matrix cores multiply small integers (exact in f16) with activations that are re-scaled once
// per group of output columns.  (Taking the whole zero-point out, q against c = sum A zp, costs
// accuracy: the 2^-23 the f16 planes lose of A is then multiplied by q instead of by q - zp, which
// near-zero weights make many times larger than the term itself.)  A workgroup owns 64 rows x 128 consecutive k of one
// group (group_size % 128 == 0; 64 or 32 k for groups of 64 or 32) and walks n in steps of 32:
//   * conversion (all 256 threads, 8 values each): a = (gy f_row) (s / S) with f_row and S powers of two
//     that put |a| below 2^14 (w4t_prepare_kernel: row maxima of gy, maximum of the scales), split into
//     hi + lo f16 (22 bits), written to LDS in A-fragment rows of 64 bytes; c accumulates in f32;
//   * every wave owns 32 of the 128 k: lane (k = lane % 32, half = lane / 32) reads the 8 consecutive
//     words of word row k / 8 that hold its 8 values of n, takes nibble k % 8 of each, and splices them
//     under the mantissa of 1024 (minus 1024, two at a time): 20 instructions per B fragment, which
//     serves 4 MFMAs (two row tiles x hi, lo);
//   * v_mfma_f32_32x32x16_f16 accumulates in f32; the epilogue subtracts c and undoes f_row and S.
// Few tiles: n is shared out over blockIdx.z as well and the partial results are added in a fixed order.
#include "common.h"
#include "i8_gemm.h"

namespace rumus {

typedef _Float16 t8h __attribute__((ext_vector_type(8)));
typedef _Float16 t2h __attribute__((ext_vector_type(2)));
typedef float t16f __attribute__((ext_vector_type(16)));

constexpr int kTMaxSplits = 16;

// Per call, before the GEMM:
//   blocks [0, m): f_row = 2^(140 - e) for a row maximum a 2^(e - 127), 1 <= a < 2, so |gy f| < 2^14
//       (0 for an all-zero or tiny row, NaN marker for a row with inf / nan);
//   blocks [m, m + groups): for group g, S_g = the power of two at or above its largest scale, and per
//       column the three things the GEMM needs of scale and zero-point: s / S_g (f32, at most 1),
//       zp - z0 (f32) and 1024 + z0 (f16), z0 = rint(zp) held within +-1000, so that no workgroup works
//       them out again.
//       sgrp[g] = S_g; 0 when every scale of the group is zero or denormal, NaN when one is not finite
//       or S_g or 1 / S_g would leave the normal range: the GEMM then writes zeros / NaNs for the group.
__global__ __launch_bounds__(256) void w4t_prepare_kernel(const float* __restrict__ gy, const float* __restrict__ scales,
                                                          const float* __restrict__ zp, float* __restrict__ rowf,
                                                          float* __restrict__ sgrp, float* __restrict__ sp,
                                                          float* __restrict__ zf, _Float16* __restrict__ zo,
                                                          uint32_t m, uint32_t n) {
    __shared__ uint32_t red[4];
    const uint32_t tid = threadIdx.x;
    const bool is_row = blockIdx.x < m;
    const float* r = is_row ? gy + (uint64_t)blockIdx.x * n : scales + (uint64_t)(blockIdx.x - m) * n;   // n % 4 == 0, aligned
    // The first kPrepCache steps of a thread (n up to 12288) stay in registers between the pass that finds the maximum
    // and the pass that writes the tables, and the zero-points are asked for together with them: one trip to memory
    // instead of one per four steps and pass.
    constexpr int kPrepCache = 12;
    const uint32_t g = is_row ? 0 : blockIdx.x - m;
    const float* zr = zp + (uint64_t)g * n;
    float4 cs[kPrepCache], cz[kPrepCache];
#pragma unroll
    for (int i = 0; i < kPrepCache; i++) {
        const uint32_t j = min(4 * tid + 1024 * i, n - 4);      // clamped: no load under a branch
        cs[i] = *reinterpret_cast<const float4*>(r + j);
        cz[i] = *reinterpret_cast<const float4*>(zr + j);       // a row's workgroup reads group 0's and drops them
    }
    auto max4 = [](uint32_t a, const float4& t) {
        return max(max(a, max(__float_as_uint(t.x) & 0x7FFFFFFFu, __float_as_uint(t.y) & 0x7FFFFFFFu)),
                   max(__float_as_uint(t.z) & 0x7FFFFFFFu, __float_as_uint(t.w) & 0x7FFFFFFFu));
    };
    uint32_t amax = 0;
#pragma unroll
    for (int i = 0; i < kPrepCache; i++)
        if (4 * tid + 1024 * i < n) amax = max4(amax, cs[i]);
#pragma unroll 4
    for (uint32_t j = 4 * tid + 1024 * kPrepCache; j < n; j += 1024) amax = max4(amax, *reinterpret_cast<const float4*>(r + j));
    amax = wave_max(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = max(max(red[0], red[1]), max(red[2], red[3]));
    if (is_row) {
        const uint32_t e = amax >> 23;
        if (tid == 0)
            rowf[blockIdx.x] = e >= 255 ? __uint_as_float(0x7FC00000u) : e < 14 ? 0.0f : __uint_as_float((267u - e) << 23);
        return;
    }
    const uint32_t se = (amax >> 23) + ((amax & 0x7FFFFFu) ? 1u : 0u);      // S_g = 2^(se - 127)
    const bool ok = se >= 1 && se <= 253;                      // S_g and 1 / S_g are normal floats
    const float s_inv = ok ? __uint_as_float((254u - se) << 23) : 0.0f;
    if (tid == 0) sgrp[g] = ok ? __uint_as_float(se << 23) : (amax >= 0x7F000000u ? __uint_as_float(0x7FC00000u) : 0.0f);
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    auto emit = [&](uint32_t j, const float4& sv, const float4& z) {
        // zero-points are 0 .. 15 unless a group's weights sit far from zero (zp = -min / scale); beyond
        // +-1000 the integer part stops growing and the rest goes into the f32 correction with the fraction
        auto whole = [](float v) { return fminf(fmaxf(rintf(v), -1000.0f), 1000.0f); };
        const float4 z0 = make_float4(whole(z.x), whole(z.y), whole(z.z), whole(z.w));
        // s / S_g is exact (a power of two); 1024 + z0 is exact in f16 for |z0| <= 1024
        *reinterpret_cast<float4*>(sp + (uint64_t)g * n + j) = make_float4(sv.x * s_inv, sv.y * s_inv, sv.z * s_inv, sv.w * s_inv);
        *reinterpret_cast<float4*>(zf + (uint64_t)g * n + j) = make_float4(z.x - z0.x, z.y - z0.y, z.z - z0.z, z.w - z0.w);
        *reinterpret_cast<v4h*>(zo + (uint64_t)g * n + j) =
            v4h{(_Float16)(1024.0f + z0.x), (_Float16)(1024.0f + z0.y), (_Float16)(1024.0f + z0.z), (_Float16)(1024.0f + z0.w)};
    };
#pragma unroll
    for (int i = 0; i < kPrepCache; i++)
        if (4 * tid + 1024 * i < n) emit(4 * tid + 1024 * i, cs[i], cz[i]);
#pragma unroll 4
    for (uint32_t j = 4 * tid + 1024 * kPrepCache; j < n; j += 1024)   // independent iterations: their loads overlap
        emit(j, *reinterpret_cast<const float4*>(r + j), *reinterpret_cast<const float4*>(zr + j));
}

// One workgroup: rows [64 y, 64 y + 64), k [128 x, 128 x + 128), n steps [z steps_per, ..).
//
// Operands travel global -> LDS by direct-to-LDS loads, kTStages steps deep: per step the raw tile of
// grad_y (64 rows x 32 floats), the 16 word rows x 32 words of the weights and the group's 32 scaled
// scales, 32 zero-point fractions and 32 f16 zero-point integers, 10.5 KB.  The raw tile of step t+1
// is converted into the A-fragment buffer (double-buffered) while the MFMAs of step t run; one barrier
// per step.
constexpr int kTRawGy = 64 * 128, kTRawW = 16 * 128, kTRawSz = 256, kTRawZo = 256;   // 64 bytes of zero-point integers used
constexpr int kTRawWt = kTRawW + kTRawSz + kTRawZo;           // weights and tables of one step
constexpr int kTAbuf = 2 * 64 * 64;                           // hi, lo planes
constexpr int kTSlots = 12;                                   // wave-wide loads per step: 8 grad_y, 1-2 weights, 2 tables
// The raw tile of grad_y of step t is dead once it has been converted (during step t - 1), the weights and tables of
// step t are read during step t: one slot fewer for grad_y than for the rest, at the same depth of loads in flight.
constexpr size_t w4t_lds_bytes(int stages) {
    return (size_t)(stages - 1) * kTRawGy + (size_t)stages * kTRawWt + 2 * kTAbuf + 64 * sizeof(float);
}

// KW = waves per workgroup = 32-column slices of k per tile: 4 when groups are multiples of 128, 2 for
// groups of 64, 1 for groups of 32 (a tile must lie inside one group, since the activations are re-scaled
// per group; the smaller workgroups convert the same 64 x 32 activations for fewer output columns).
// HALF: at most 32 rows (one row tile, half full): the loads, the conversion and the MFMAs of rows 32..63 are
// left out (4096 x 11008 at 16 rows: the call 44.6 -> 40.7 us; groups of 64 at 24 rows 56.1 -> 47.4 us).
template <int kTStages, int KW, bool HALF = false>
__global__ __launch_bounds__(64 * KW, 2) void w4t_gemm_kernel(
    const float* __restrict__ gy, const uint32_t* __restrict__ packed, const float* __restrict__ sp,
    const float* __restrict__ zf, const _Float16* __restrict__ zo, const float* __restrict__ rowf,
    const float* __restrict__ sgrp, float* __restrict__ out, uint32_t m, uint32_t k, uint32_t n, uint32_t gs,
    uint32_t steps_per) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t* const raw_gy = lds;                               // [kTStages - 1][kTRawGy]
    uint8_t* const raw_wt = lds + (kTStages - 1) * kTRawGy;    // [kTStages][kTRawWt]
    uint8_t* const abuf = raw_wt + kTStages * kTRawWt;         // [2][kTAbuf]
    float* const lds_c = reinterpret_cast<float*>(abuf + 2 * kTAbuf);
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int kTLoads = (HALF ? kTSlots - 4 : kTSlots) / KW;   // per wave and step
    constexpr int RTILES = HALF ? 1 : 2;                       // 32-row tiles of the accumulators
    constexpr int WS = KW == 4 ? 2 : 1;                        // slots of weight words (8 word rows each)
    const uint32_t k0 = blockIdx.x * (32 * KW), m0 = blockIdx.y * 64;
    const uint32_t g = k0 / gs;
    const uint32_t nsteps = (n + 31) / 32;
    const uint32_t st0 = blockIdx.z * steps_per, st1 = min(nsteps, st0 + steps_per);   // st0 < st1 by the launch

    // ---- global side of the direct-to-LDS loads: load q = 4 i + wave of a step --------------------------
    //   q 0..7: rows 8 q .. 8 q + 7 of grad_y (lane: row lane / 8, floats 4 (lane % 8) .. + 3)
    //   q 8 (and 9 when KW = 4): word rows 8 (q - 8) .. + 7 of the weights (lane: row lane / 8, words
    //         4 (lane % 8) .. + 3)
    //   next: lanes 0..31 scaled scale, 32..63 zero-point fraction of column lane % 32
    //   last (and any slot left over): lanes 0..15 two f16 zero-point integers each (columns 2 lane,
    //         2 lane + 1); the other lanes fetch the same words again, into the unused tail of the stage
    const uint32_t l8 = lane >> 3, p8 = lane & 7;
    // Address of a load = a base that is the same for the whole wave (array, tile, and the step's columns: scalar
    // registers, advanced by scalar arithmetic) + a 32-bit offset per lane that never changes (row, column inside the
    // step): no vector instruction per load and step.  Only a step that reaches past n (the last one when n % 32 != 0)
    // works its addresses out lane by lane, to send the columns past n to column 0.
    const uint8_t* ubase[kTLoads];                             // wave-uniform
    uint32_t voff[kTLoads], colw[kTLoads];                     // per lane; colw: the lane's first column inside a step
    uint32_t dst[kTLoads], esz[kTLoads];                       // dst: offset inside the slot of its kind
    bool wide[kTLoads], is_gy[kTLoads];
    const uint32_t zf_off = (uint32_t)(reinterpret_cast<const uint8_t*>(zf) - reinterpret_cast<const uint8_t*>(sp));   // one workspace: < 2^32
#pragma unroll
    for (int i = 0; i < kTLoads; i++) {
        uint32_t q = KW * i + wave;
        if (HALF && q >= 4) q += 4;                            // no loads of rows 32..63 of grad_y
        is_gy[i] = q < 8;
        if (q < 8) {
            const uint32_t row = min(m0 + 8 * q + l8, m - 1) - m0;
            ubase[i] = reinterpret_cast<const uint8_t*>(gy + (uint64_t)m0 * n);
            // rows two apart would put the conversion's 128-bit reads two to a bank: every other pair of rows
            // holds its 16-byte pieces swapped in twos (LDS piece p of row r = piece p ^ (r / 2 % 2) of the tile)
            dst[i] = q * 1024; colw[i] = 4 * (p8 ^ ((l8 >> 1) & 1)); wide[i] = true; esz[i] = 4;
            voff[i] = (row * n + colw[i]) * 4;                 // < 64 n 4
        } else if (q < 8 + WS) {
            // the tile's 4 KW word rows (< padded_k / 8: whole groups exist in the arrays); lanes past them
            // fetch its last row again, into room the stage keeps for that
            const uint32_t wr = min(8 * (q - 8) + l8, 4u * KW - 1);
            ubase[i] = reinterpret_cast<const uint8_t*>(packed + (uint64_t)(k0 / 8) * n);
            dst[i] = (q - 8) * 1024; colw[i] = 4 * p8; wide[i] = true; esz[i] = 4;
            voff[i] = (wr * n + colw[i]) * 4;
        } else if (q == 8 + WS) {
            ubase[i] = reinterpret_cast<const uint8_t*>(sp + (uint64_t)g * n);   // zf lies zf_off behind sp
            dst[i] = kTRawW; colw[i] = lane & 31; wide[i] = false; esz[i] = 4;
            voff[i] = colw[i] * 4 + (lane < 32 ? 0 : zf_off);
        } else {
            ubase[i] = reinterpret_cast<const uint8_t*>(zo + (uint64_t)g * n);
            dst[i] = kTRawW + kTRawSz; colw[i] = 2 * (lane & 15); wide[i] = false; esz[i] = 2;
            voff[i] = colw[i] * 2;
        }
    }
    auto issue = [&](uint32_t st, uint32_t gslot, uint32_t wslot) {
        uint8_t* const gbase = raw_gy + gslot * kTRawGy;
        uint8_t* const wbase = raw_wt + wslot * kTRawWt;
        const uint32_t c0 = min(st, st1 - 1) * 32;
        if (c0 + 32 <= n) {
#pragma unroll
            for (int i = 0; i < kTLoads; i++) {
                uint8_t* const base = is_gy[i] ? gbase : wbase;
                const uint8_t* const sb = ubase[i] + (uint64_t)c0 * esz[i];
                if (wide[i]) __builtin_amdgcn_global_load_lds((gptr_t)(sb + voff[i]), (lptr_t)(base + dst[i]), 16, 0, 0);
                else __builtin_amdgcn_global_load_lds((gptr_t)(sb + voff[i]), (lptr_t)(base + dst[i]), 4, 0, 0);
            }
        } else {
            // columns past n are fetched from column 0: the conversion turns them into zeros
#pragma unroll
            for (int i = 0; i < kTLoads; i++) {
                uint8_t* const base = is_gy[i] ? gbase : wbase;
                const uint32_t col = c0 + colw[i] < n ? c0 + colw[i] : 0;
                const uint8_t* const p = ubase[i] + (voff[i] - colw[i] * esz[i]) + (uint64_t)col * esz[i];
                if (wide[i]) __builtin_amdgcn_global_load_lds((gptr_t)p, (lptr_t)(base + dst[i]), 16, 0, 0);
                else __builtin_amdgcn_global_load_lds((gptr_t)p, (lptr_t)(base + dst[i]), 4, 0, 0);
            }
        }
    };

    // ---- conversion role: row tid / KW, its chunks of 8 consecutive n: 4 / KW of them from (tid % KW) 4 / KW ----
    constexpr int CPT = 4 / KW;
    const uint32_t s_row = tid / KW, s_ch0 = (tid % KW) * CPT;
    const float frow_raw = rowf[min(m0 + s_row, m - 1)];
    const float frow = frow_raw != frow_raw ? 0.0f : frow_raw; // inf / nan in the row: NaN times 0 poisons it below
    float csum = 0.0f;
    auto convert_chunk = [&](uint32_t st, uint32_t gslot, uint32_t wslot, int buf, uint32_t s_ch) {
        const uint32_t s_lds = s_row * 64 + ((s_ch ^ row_swizzle(s_row)) & 3) * 16;
        const uint8_t* gbase = raw_gy + gslot * kTRawGy;
        const uint8_t* tbase = raw_wt + wslot * kTRawWt + kTRawW;
        const uint32_t sw = (s_row >> 1) & 1;                  // see the loads: pieces swapped in twos
        const float4 g0 = *reinterpret_cast<const float4*>(gbase + s_row * 128 + ((2 * s_ch) ^ sw) * 16);
        const float4 g1 = *reinterpret_cast<const float4*>(gbase + s_row * 128 + ((2 * s_ch + 1) ^ sw) * 16);
        const float4 s0 = *reinterpret_cast<const float4*>(tbase + s_ch * 32);
        const float4 s1 = *reinterpret_cast<const float4*>(tbase + s_ch * 32 + 16);
        const float4 z0 = *reinterpret_cast<const float4*>(tbase + 128 + s_ch * 32);
        const float4 z1 = *reinterpret_cast<const float4*>(tbase + 128 + s_ch * 32 + 16);
        const uint32_t c0 = st * 32 + s_ch * 8;
        // n % 4 == 0: four columns are all-in or all-out; the columns past n hold values of column 0
        const float f0 = c0 < n ? frow : 0.0f, f1 = c0 + 4 < n ? frow : 0.0f;
        // powers of two first: gy f is exact, the product with s / S is rounded once
        const float a[8] = {(g0.x * f0) * s0.x, (g0.y * f0) * s0.y, (g0.z * f0) * s0.z, (g0.w * f0) * s0.w,
                            (g1.x * f1) * s1.x, (g1.y * f1) * s1.y, (g1.z * f1) * s1.z, (g1.w * f1) * s1.w};
        const float zv[8] = {z0.x, z0.y, z0.z, z0.w, z1.x, z1.y, z1.z, z1.w};
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            csum = fmaf(a[e], zv[e], csum);
            csum = fmaf(a[e + 1], zv[e + 1], csum);
            // hi = a cut to 11 bits (one instruction for two values), lo = the rest cut to 11 bits: 2^-21 of a
            // is lost at most.  The explicit conversion also keeps the compiler from rounding a product
            // to f16 in two different ways (v_fma_mixlo_f16 of the exact product here, a conversion of the
            // rounded f32 there), which on a tie differ by a whole f16 step that hi + lo then misses.
            const auto h2 = __builtin_amdgcn_cvt_pkrtz(a[e], a[e + 1]);
            // a - hi is exact (the low bits of a): one mixed-precision fma each (the f16 half read in place) instead of
            // a conversion and a subtraction, which is what the compiler makes of the plain expression
            const uint32_t h2b = __builtin_bit_cast(uint32_t, h2);
            float r0, r1;
            asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r0) : "v"(h2b), "v"(a[e]));
            asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r1) : "v"(h2b), "v"(a[e + 1]));
            const auto l2 = __builtin_amdgcn_cvt_pkrtz(r0, r1);
            hi[e / 2] = __builtin_bit_cast(uint32_t, h2);
            lo[e / 2] = __builtin_bit_cast(uint32_t, l2);
        }
        uint8_t* ab = abuf + buf * kTAbuf;
        *reinterpret_cast<uint4*>(ab + s_lds) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        *reinterpret_cast<uint4*>(ab + 64 * 64 + s_lds) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    };
    auto convert = [&](uint32_t st, uint32_t gslot, uint32_t wslot, int buf) {
        if (HALF && s_row >= 32) return;                       // whole waves when KW >= 2
#pragma unroll
        for (int cc = 0; cc < CPT; cc++) convert_chunk(st, gslot, wslot, buf, s_ch0 + cc);
    };

    // ---- B role: lane (k = 32 wave + lane % 32, half = lane / 32): 8 words of word row 4 wave + k / 8 ----
    const uint32_t bc = lane & 31, bh = lane >> 5;
    const uint32_t shift = 4 * (bc & 7);
    const uint32_t b_off = (4 * wave + (bc >> 3)) * 128 + bh * 32;
    auto b_frag = [&](int t, uint32_t wslot) {
        const uint8_t* sb = raw_wt + wslot * kTRawWt;
        const uint4 w0 = *reinterpret_cast<const uint4*>(sb + b_off + t * 64), w1 = *reinterpret_cast<const uint4*>(sb + b_off + t * 64 + 16);
        const uint32_t w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        const t8h off = *reinterpret_cast<const t8h*>(sb + kTRawW + kTRawSz + 32 * t + 16 * bh);   // 1024 + z0
        t2h h[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q0 = (w[2 * i] >> shift) & 0xFu, q1 = (w[2 * i + 1] >> shift) & 0xFu;
            h[i] = __builtin_bit_cast(t2h, (q1 << 16) | q0 | 0x64006400u) - t2h{off[2 * i], off[2 * i + 1]};   // (1024 + q) - (1024 + z0): exact
        }
        return t8h{h[0][0], h[0][1], h[1][0], h[1][1], h[2][0], h[2][1], h[3][0], h[3][1]};
    };

    // ---- A fragment reads: lane (row fr, half fh), MFMA step t: logical chunk 2 t + fh -----------------
    const uint32_t fr = lane & 31, fh = lane >> 5, fsw = row_swizzle(fr);
    uint32_t a_off[2];
#pragma unroll
    for (int t = 0; t < 2; t++) a_off[t] = fr * 64 + (((2 * t + fh) ^ fsw) & 3) * 16;

    t16f acc[RTILES];
#pragma unroll
    for (int i = 0; i < RTILES; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;

    // ---- pipeline -----------------------------------------------------------------------------------------
    // Every step issues exactly kTLoads loads per wave, also past the end (the last step again, into a
    // stage nobody reads any more), so the counter arithmetic has no tail cases.
#pragma unroll
    for (int s = 0; s < kTStages - 1; s++) issue(st0 + s, s, s);
    RUMUS_WAIT_VMCNT((kTStages - 2) * kTLoads);               // step st0 has landed
    __builtin_amdgcn_s_barrier();
    convert(st0, 0, 0, 0);
    // The B fragments of a step are cut out of its words while the MFMAs of the step before run (a wave issues
    // nothing while it waits to issue an MFMA: fragments and MFMAs of the same step one after the other leave the
    // vector ALU idle during the MFMAs and the matrix cores idle during the cutting).
    t8h b0 = b_frag(0, 0), b1 = b_frag(1, 0);
    uint32_t cur = 0, gcur = 0;                                // slots of step st: weights and tables, grad_y
    for (uint32_t st = st0; st < st1; st++) {
        const int ab = (st - st0) & 1;
        const uint32_t nxt = cur + 1 == kTStages ? 0 : cur + 1, prv = cur == 0 ? kTStages - 1 : cur - 1;
        const uint32_t gnxt = gcur + 1 == kTStages - 1 ? 0 : gcur + 1;
        // step st+1 has landed once only the kTStages-3 younger steps are outstanding; past the barrier
        // the A fragments of step st are visible, the weight slot of step st-1 is free and so is the grad_y
        // slot of step st itself (converted during step st-1)
        RUMUS_WAIT_VMCNT((kTStages - 3) * kTLoads);
        __builtin_amdgcn_s_barrier();
        issue(st + (kTStages - 1), gcur, prv);
        const t8h nb0 = b_frag(0, nxt), nb1 = b_frag(1, nxt);   // step st+1 has landed (after the last step: that step's words again, unused)
        const uint8_t* abp = abuf + ab * kTAbuf;
#pragma unroll
        for (int i = 0; i < RTILES; i++) {
            const uint8_t* hi = abp + i * 32 * 64;
            const uint8_t* lo = abp + 64 * 64 + i * 32 * 64;
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(hi + a_off[0]), b0, acc[i], 0, 0, 0);
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(lo + a_off[0]), b0, acc[i], 0, 0, 0);
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(hi + a_off[1]), b1, acc[i], 0, 0, 0);
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(lo + a_off[1]), b1, acc[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4 * RTILES; i++) {                 // an MFMA, then its share of the 40 instructions of the next fragments
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 40 / (4 * RTILES), 0);
        }
        if (st + 1 < st1) convert(st + 1, gnxt, nxt, ab ^ 1);
        b0 = nb0;
        b1 = nb1;
        cur = nxt;
        gcur = gnxt;
    }
    RUMUS_WAIT_VMCNT(0);         // no direct-to-LDS write may outlive the workgroup

    // ---- c[row]: the KW conversion threads of a row are neighbours in a wave ---------------------------
    if (KW >= 2) csum += __shfl_xor(csum, 1);
    if (KW == 4) csum += __shfl_xor(csum, 2);
    if (tid % KW == 0) lds_c[s_row] = csum;
    __syncthreads();

    // ---- register r of lane l is row 8 (r/4) + 4 (l/32) + r%4, column l%32 of its 32 x 32 tile -------
    float* dst_out = out + (uint64_t)blockIdx.z * m * k;
    const uint32_t col = k0 + 32 * wave + bc;
    const float s_big = sgrp[g];
    if (col < k) {
#pragma unroll
        for (int i = 0; i < RTILES; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t lr = 32 * i + 8 * (r / 4) + 4 * fh + (r % 4), row = m0 + lr;
                if (row >= m) continue;
                const float f = rowf[row];
                // 1 / f_row = 2^(e - 140): from the bits of f (f = 2^(140 - e), biased exponent 267 - e)
                const float finv = f != f ? f : f == 0.0f ? 0.0f : __uint_as_float((254u - (__float_as_uint(f) >> 23)) << 23);
                dst_out[(uint64_t)row * k + col] = ((acc[i][r] - lds_c[lr]) * finv) * s_big;
            }
    }
}

// out = sum over the shares of n of their partial results, in share order
__global__ __launch_bounds__(256) void w4t_add_shares_kernel(const float4* __restrict__ part, float4* __restrict__ out,
                                                             uint32_t count4, uint32_t shares) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count4) return;
    float4 v = part[i];
    for (uint32_t z = 1; z < shares; z++) {
        const float4 t = part[(uint64_t)z * count4 + i];
        v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
    }
    out[i] = v;
}

bool w4_gemm_t_supported(uint32_t m, uint32_t k, uint32_t n, uint32_t group_size, const void* gy, const void* packed,
                         const void* scales, const void* zp, const void* out) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(packed) |
                           reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(zp) |
                           reinterpret_cast<uintptr_t>(out);
    return (group_size % 128 == 0 || group_size == 64 || group_size == 32) && n % 4 == 0 && k % 4 == 0 && (bits & 15) == 0 &&
           (uint64_t)m * k < (1ull << 32) && (uint64_t)m * n < (1ull << 40);
}

template <int NS, int KW, bool HALF = false>
static int launch_w4t(uint32_t ktiles, uint32_t mtiles, uint32_t shares, hipStream_t s, const float* gy,
                      const uint32_t* packed, const float* sp, const float* zf, const _Float16* zo, const float* rowf,
                      const float* sgrp, float* out, uint32_t m, uint32_t k, uint32_t n, uint32_t gs, uint32_t steps_per) {
    constexpr size_t lds_bytes = w4t_lds_bytes(NS);
    static bool attr_set = false;   // benign race: setting the attribute is idempotent
    if (!attr_set && lds_bytes > 64 * 1024) {
        if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&w4t_gemm_kernel<NS, KW, HALF>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes),
                               "hipFuncSetAttribute"))
            return rc;
        attr_set = true;
    }
    hipLaunchKernelGGL((w4t_gemm_kernel<NS, KW, HALF>), dim3(ktiles, mtiles, shares), dim3(64 * KW), lds_bytes, s, gy, packed, sp, zf, zo,
                       rowf, sgrp, out, m, k, n, gs, steps_per);
    return check_launch("w4t_gemm_kernel");
}

#define RUMUS_W4T_LAUNCH(NS, KW)                                                                                  \
    (m <= 32 ? launch_w4t<NS, KW, true>(ktiles, mtiles, shares, s, gy, packed, sp, zf, zo, rowf, sgrp,              \
                                        shares > 1 ? part : out, m, k, n, group_size, steps_per)                   \
             : launch_w4t<NS, KW>(ktiles, mtiles, shares, s, gy, packed, sp, zf, zo, rowf, sgrp,                    \
                                  shares > 1 ? part : out, m, k, n, group_size, steps_per))

int w4_launch_gemm_t(const float* gy, const uint32_t* packed, const float* scales, const float* zp, float* out,
                     uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k, uint32_t group_size, uint32_t num_groups,
                     hipStream_t s) {
    const int kw = group_size % 128 == 0 ? 4 : group_size / 32;   // waves per workgroup: 32-column slices of one group
    const uint32_t ktiles = padded_k / (32 * kw), mtiles = ceil_div(m, 64), nsteps = ceil_div(n, 32);
    RUMUS_REQUIRE(mtiles <= 65535, "qmatmul_int4_t: m %u is beyond the grid limit", m);
    // fewer tiles than two per compute unit: n is shared out too, in shares of at least 16 steps
    uint32_t shares = 1, steps_per = nsteps;
    const uint64_t tiles = (uint64_t)ktiles * mtiles;
    if (tiles < 512) {
        shares = (uint32_t)(1024 / tiles);
        // one row tile: up to 16 shares (46 us instead of 60 for up to 64 rows); beyond, the partial results
        // of more than 8 shares cost more than the shares gain (128 rows: 84 us against 72)
        const uint32_t cap = mtiles == 1 ? kTMaxSplits : kTMaxSplits / 2;
        if (shares > cap) shares = cap;
        if (shares > nsteps / 16) shares = nsteps / 16;
        if (shares < 1) shares = 1;
        steps_per = ceil_div(nsteps, shares);
        shares = ceil_div(nsteps, steps_per);
    }
    auto up = [](size_t v) { return (v + 255) & ~size_t(255); };
    const size_t gn = (size_t)num_groups * n;
    const size_t rowf_bytes = up((size_t)m * sizeof(float)), sgrp_bytes = up((size_t)num_groups * sizeof(float));
    const size_t sp_bytes = up(gn * sizeof(float)), zo_bytes = up(gn * sizeof(_Float16) + 64);
    const size_t part_bytes = shares > 1 ? (size_t)shares * m * k * sizeof(float) : 0;
    void* ws = nullptr;
    WorkspaceLease lease;                                    // until the last kernel of this call is queued
    if (int rc = workspace_get(s, rowf_bytes + sgrp_bytes + 2 * sp_bytes + zo_bytes + part_bytes, &ws, lease)) return rc;
    uint8_t* b = static_cast<uint8_t*>(ws);
    float* rowf = reinterpret_cast<float*>(b);
    float* sgrp = reinterpret_cast<float*>(b + rowf_bytes);
    float* sp = reinterpret_cast<float*>(b + rowf_bytes + sgrp_bytes);
    float* zf = reinterpret_cast<float*>(b + rowf_bytes + sgrp_bytes + sp_bytes);
    _Float16* zo = reinterpret_cast<_Float16*>(b + rowf_bytes + sgrp_bytes + 2 * sp_bytes);
    float* part = reinterpret_cast<float*>(b + rowf_bytes + sgrp_bytes + 2 * sp_bytes + zo_bytes);
    hipLaunchKernelGGL(w4t_prepare_kernel, dim3(m + num_groups), dim3(256), 0, s, gy, scales, zp, rowf, sgrp, sp, zf, zo, m,
                       n);
    if (int rc = check_launch("w4t_prepare_kernel")) return rc;
    // Three weight slots and two grad_y slots: 39.75 KB of LDS, four workgroups per compute unit.  Workgroups run in
    // rounds of that many per CU and a round lasts almost the same whether it is full or not, so what matters is how
    // many fit: with four stages (three per CU) 2048 rows x 4096 took 0.70 ms for 1024 workgroups on 768 places, with
    // three stages 0.57 ms on 1024 places, and the four-stage form was faster for no batch from 256 to 4096 rows.
    const int rc = kw == 4 ? RUMUS_W4T_LAUNCH(3, 4) : kw == 2 ? RUMUS_W4T_LAUNCH(3, 2) : RUMUS_W4T_LAUNCH(3, 1);
    if (rc) return rc;
    if (shares == 1) return RUMUS_HIP_OK;
    const uint32_t count4 = (uint32_t)((uint64_t)m * k / 4);
    hipLaunchKernelGGL(w4t_add_shares_kernel, dim3(ceil_div(count4, 256)), dim3(256), 0, s,
                       reinterpret_cast<const float4*>(part), reinterpret_cast<float4*>(out), count4, shares);
    return check_launch("w4t_add_shares_kernel");
}

}  // namespace rumus
