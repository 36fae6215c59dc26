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
// Weights never pass through LDS.  v_mfma_f32_16x16x32_f16 wants, per lane, 8
// consecutive k of one column: that is exactly one packed u32 word
// (rumus-vision/src/quant.rs:98-100).  Lane l of a wave loads the four words of
// columns 4*(l%16) .. +3 at word row 4*step + l/16 with one 128-bit load (a wave
// covers 64 columns x 32 rows, 256-byte segments) and converts each word to a
// B fragment in registers (magic-number nibble -> f16, packed f16 math).  The
// conversion yields k in the order 0,4,1,5,2,6,3,7; the A fragments are stored in
// the same order, and a dot product does not care.
//
// Activations: a workgroup (4 waves = 4 column strips = 256 columns) shares the
// A fragments of its BM rows.  Per stage of 128 rows of K they are converted
// once (hi/lo f16, fragment layout, per-step sums for the zero-point term) into
// one of two LDS buffers while the previous stage is being multiplied; one
// barrier per stage.  `perm` (act-order) gathers x columns at this point.
#include <type_traits>

#include "w4.h"

namespace rumus {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kGemmCols = 256;   // columns per workgroup (4 strips of 64)
constexpr int kGemmStageK = 128; // rows of K staged per barrier (4 MFMA steps of 32)

// one packed word -> B fragment, k order 0,4,1,5,2,6,3,7
__device__ __forceinline__ v8h nibbles_to_f16(uint32_t w) {
    const v2h k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    const v2h k64 = {(_Float16)64.0f, (_Float16)64.0f};
    const v2h k16th = {(_Float16)0.0625f, (_Float16)0.0625f};
    const uint32_t t0 = (w & 0x000F000Fu) | 0x64006400u;          // 1024 + n0, 1024 + n4
    const uint32_t t1 = (w & 0x00F000F0u) | 0x64006400u;          // 1024 + 16 n1, 1024 + 16 n5
    const uint32_t w8 = w >> 8;
    const uint32_t t2 = (w8 & 0x000F000Fu) | 0x64006400u;         // n2, n6
    const uint32_t t3 = (w8 & 0x00F000F0u) | 0x64006400u;         // 16 n3, 16 n7
    const v2h h0 = __builtin_bit_cast(v2h, t0) - k1024;
    const v2h h1 = __builtin_bit_cast(v2h, t1) * k16th - k64;     // exact: (1024+16n)/16 = 64+n
    const v2h h2 = __builtin_bit_cast(v2h, t2) - k1024;
    const v2h h3 = __builtin_bit_cast(v2h, t3) * k16th - k64;
    return v8h{h0[0], h0[1], h1[0], h1[1], h2[0], h2[1], h3[0], h3[1]};
}

// RT = 16-row tiles per workgroup (BM = 16 * RT rows, RT <= 4).
//
// SPLITK = false: the four waves own four adjacent 64-column strips and share
// the staged activations (two LDS buffers, one barrier per stage).
// SPLITK = true (small m): the workgroup owns one strip and the four waves take
// the stages of K round-robin, each staging its own activations in a private
// LDS region (no barrier in the loop); the four partial results are added in a
// fixed order at the end.  This keeps the grid at n/64 workgroups when there
// are only one or two row tiles, without atomics.
template <int RT, bool SPLITK>
__global__ __launch_bounds__(256) void w4_gemm_kernel(W4Args a) {
    constexpr int BM = 16 * RT;
    // A fragment planes of one stage: [step][k block][row] x 16 bytes, with 64
    // bytes of skew per step so that the four lanes that stage one row (one step
    // each) write to different banks
    constexpr int STEP_BYTES = 4 * BM * 16 + 64;
    constexpr int PLANE = 4 * STEP_BYTES;
    constexpr int NBUF = SPLITK ? 4 : 2;                 // per wave, or double buffer
    constexpr int NI = SPLITK ? RT : 1;                  // rows staged per thread
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[NBUF][2][PLANE];   // [buffer][hi, lo]
    __shared__ __attribute__((aligned(16))) float lds_xs[NBUF][4][BM];        // [buffer][step][row]: sum of x

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t lr = lane & 15, lb = lane >> 4;
    const uint32_t m0 = blockIdx.y * BM;
    const uint32_t colbase = SPLITK ? blockIdx.x * 64 + 4 * lr
                                    : blockIdx.x * kGemmCols + wave * 64 + 4 * lr;   // this lane's 4 columns
    const bool col_ok = colbase < a.n;                   // n % 4 == 0
    const uint32_t col_c = col_ok ? colbase : 0;
    const uint32_t nstages = (a.padded_k + kGemmStageK - 1) / kGemmStageK;
    const uint32_t nsteps = a.padded_k / 32;             // group_size % 32 == 0
    const uint32_t word_rows = a.padded_k / 8;

    // ---- staging role: MFMA step = t%4 (32 consecutive k), row = t/4 (+16 per pass) --
    const uint32_t s_t = SPLITK ? lane : tid;
    const uint32_t s_row = s_t >> 2, s_step = s_t & 3;
    const bool s_active = s_row < BM;
    const bool x_vec = !a.perm && (a.k % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.x) & 15) == 0);
    float xv[NI][32];
    auto stage_load = [&](uint32_t st) {
        const uint32_t k0 = st * kGemmStageK + s_step * 32;
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const uint32_t row = m0 + s_row + 16 * it;
            const bool row_ok = s_active && row < a.m;
            const float* xrow = a.x + (uint64_t)min(row, a.m - 1) * a.k;
            if (x_vec) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const uint32_t kk = k0 + 4 * i;
                    const bool in = row_ok && kk < a.k;   // k % 4 == 0: all four in or out
                    const float4 v = *reinterpret_cast<const float4*>(xrow + (in ? kk : 0));
                    xv[it][4 * i] = in ? v.x : 0.0f; xv[it][4 * i + 1] = in ? v.y : 0.0f;
                    xv[it][4 * i + 2] = in ? v.z : 0.0f; xv[it][4 * i + 3] = in ? v.w : 0.0f;
                }
            } else {
                // act-order: the 32 source columns first (contiguous), then the gather
                uint32_t src[32];
#pragma unroll
                for (int i = 0; i < 32; i++) {
                    const uint32_t kk = min(k0 + i, a.k - 1);
                    src[i] = a.perm ? (uint32_t)a.perm[kk] : kk;
                }
#pragma unroll
                for (int i = 0; i < 32; i++) {
                    const float v = xrow[src[i]];
                    xv[it][i] = (row_ok && k0 + i < a.k) ? v : 0.0f;
                }
            }
        }
    };
    auto stage_store = [&](uint32_t buf) {
        if (!s_active) return;
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const uint32_t row = s_row + 16 * it;
            float sum = 0.0f;
            uint8_t* hi_base = lds_a[buf][0] + s_step * STEP_BYTES + row * 16;
            uint8_t* lo_base = lds_a[buf][1] + s_step * STEP_BYTES + row * 16;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                v8h hi, lo;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int j = (e >> 1) + 4 * (e & 1);  // fragment element e holds k offset j
                    const float x = xv[it][8 * b + j];
                    const _Float16 h = (_Float16)x;
                    const float back = (float)h;
                    const _Float16 l = (_Float16)(x - back);
                    hi[e] = h;
                    lo[e] = l;
                    sum += back + (float)l;
                }
                *reinterpret_cast<v8h*>(hi_base + b * BM * 16) = hi;
                *reinterpret_cast<v8h*>(lo_base + b * BM * 16) = lo;
            }
            lds_xs[buf][s_step][row] = sum;                // the value the MFMAs see, summed
        }
    };

    // ---- weights: one 128-bit load per MFMA step, a whole stage in flight -------
    uint4 wq[2][4];
    auto weight_load = [&](uint32_t st, int set) {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const uint32_t kr = min(st * 16 + s * 4 + lb, word_rows - 1);
            wq[set][s] = *reinterpret_cast<const uint4*>(a.packed + (uint64_t)kr * a.n + col_c);
        }
    };

    v4f acc[RT][4], fin[RT][4];
    float xsg[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc[rt][j] = v4f{0, 0, 0, 0};
            fin[rt][j] = v4f{0, 0, 0, 0};
            xsg[rt][j] = 0.0f;
        }

    // stages of this wave: first, first + stride, ...
    const uint32_t first = SPLITK ? wave : 0, stride = SPLITK ? 4 : 1;
    // scale / zero-point of the group that the next fold needs, fetched ahead
    auto meta_load = [&](uint32_t step, float4& sc, float4& zp) {
        const uint32_t g = min(step * 32 / a.group_size, a.num_groups - 1);
        sc = *reinterpret_cast<const float4*>(a.scales + (uint64_t)g * a.n + col_c);
        zp = *reinterpret_cast<const float4*>(a.zp + (uint64_t)g * a.n + col_c);
    };
    float4 sc_next, zp_next;
    meta_load(first * 4, sc_next, zp_next);

    // Multiply one stage from LDS buffer `buf` and weight set SET.  The partial
    // sums are folded into the result whenever a group of K ends; a wave that
    // owns only part of a group (SPLITK, group_size > 128) also folds at the end
    // of its stage, which is exact because the fold is linear in (acc, xsum).
    auto compute = [&](uint32_t st, uint32_t buf, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const uint32_t step = st * 4 + s;
            if (step >= nsteps) break;                    // padded_k % 128 != 0: short last stage
            const uint32_t wv[4] = {wq[SET][s].x, wq[SET][s].y, wq[SET][s].z, wq[SET][s].w};
            v8h bfr[4];
#pragma unroll
            for (int j = 0; j < 4; j++) bfr[j] = nibbles_to_f16(wv[j]);
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                const uint32_t off = s * STEP_BYTES + (lb * BM + rt * 16 + lr) * 16;
                const v8h ah = *reinterpret_cast<const v8h*>(lds_a[buf][0] + off);
                const v8h al = *reinterpret_cast<const v8h*>(lds_a[buf][1] + off);
                const float4 xs4 = *reinterpret_cast<const float4*>(&lds_xs[buf][s][rt * 16 + lb * 4]);
                xsg[rt][0] += xs4.x; xsg[rt][1] += xs4.y; xsg[rt][2] += xs4.z; xsg[rt][3] += xs4.w;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    acc[rt][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bfr[j], acc[rt][j], 0, 0, 0);
                    acc[rt][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, bfr[j], acc[rt][j], 0, 0, 0);
                }
            }
            const bool group_end = ((step + 1) * 32) % a.group_size == 0;
            const bool run_end = SPLITK && (s == 3 || step + 1 == nsteps);
            if (group_end || run_end) {
                const float4 sc = sc_next, zp = zp_next;
                // the step this wave multiplies next decides the next group
                const uint32_t next_step = (s == 3 || step + 1 == nsteps) ? (st + stride) * 4 : step + 1;
                meta_load(next_step, sc_next, zp_next);
                const float scv[4] = {sc.x, sc.y, sc.z, sc.w}, zv[4] = {zp.x, zp.y, zp.z, zp.w};
#pragma unroll
                for (int rt = 0; rt < RT; rt++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
#pragma unroll
                        for (int i = 0; i < 4; i++)
                            fin[rt][j][i] = fmaf(scv[j], fmaf(-zv[j], xsg[rt][i], acc[rt][j][i]), fin[rt][j][i]);
                        acc[rt][j] = v4f{0, 0, 0, 0};
                    }
#pragma unroll
                for (int rt = 0; rt < RT; rt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) xsg[rt][i] = 0.0f;
            }
        }
    };
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, 1>;

    if (SPLITK) {
        // wave-private pipeline: LDS accesses of one wave execute in order, so the
        // staged fragments need no barrier before the same wave reads them
        if (first < nstages) {
            stage_load(first);
            weight_load(first, 0);
        }
        for (uint32_t st = first; st < nstages; st += 2 * stride) {
            stage_store(wave);
            if (st + stride < nstages) { stage_load(st + stride); weight_load(st + stride, 1); }
            compute(st, wave, Set0{});
            if (st + stride >= nstages) break;
            stage_store(wave);
            if (st + 2 * stride < nstages) { stage_load(st + 2 * stride); weight_load(st + 2 * stride, 0); }
            compute(st + stride, wave, Set1{});
        }
        // fixed-order sum of the four partial results, through LDS (reusing the planes)
        __syncthreads();
        float* red = reinterpret_cast<float*>(&lds_a[0][0][0]);   // [wave][RT*16 values][64 lanes]
        static_assert(sizeof(lds_a) >= 4 * RT * 16 * 64 * sizeof(float), "reduction buffer too small");
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    red[(wave * RT * 16 + (rt * 16 + j * 4 + i)) * 64 + lane] = fin[rt][j][i];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int v = rt * 16 + j * 4 + i;
                    fin[rt][j][i] = (red[(0 * RT * 16 + v) * 64 + lane] + red[(1 * RT * 16 + v) * 64 + lane]) +
                                    (red[(2 * RT * 16 + v) * 64 + lane] + red[(3 * RT * 16 + v) * 64 + lane]);
                }
    } else {
        stage_load(0);
        weight_load(0, 0);
        stage_store(0);
        for (uint32_t st = 0; st < nstages; st += 2) {
            // even stage: LDS buffer 0, weight set 0
            __syncthreads();                              // buffer 0 staged; buffer 1 free
            if (st + 1 < nstages) { stage_load(st + 1); weight_load(st + 1, 1); }
            compute(st, 0, Set0{});
            if (st + 1 < nstages) stage_store(1);
            if (st + 1 >= nstages) break;
            // odd stage: LDS buffer 1, weight set 1
            __syncthreads();
            if (st + 2 < nstages) { stage_load(st + 2); weight_load(st + 2, 0); }
            compute(st + 1, 1, Set1{});
            if (st + 2 < nstages) stage_store(0);
        }
    }

    // ---- store: a lane holds 4 consecutive columns of 4 rows per tile ------------
    if (!col_ok) return;
    float4 bv = make_float4(0, 0, 0, 0);
    if (a.bias) bv = *reinterpret_cast<const float4*>(a.bias + colbase);
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t row = m0 + rt * 16 + lb * 4 + i;
            if (row >= a.m) continue;
            float4 o = make_float4(fin[rt][0][i] + bv.x, fin[rt][1][i] + bv.y, fin[rt][2][i] + bv.z,
                                   fin[rt][3][i] + bv.w);
            *reinterpret_cast<float4*>(a.y + (uint64_t)row * a.n + colbase) = o;
        }
}

bool w4_gemm_supported(const W4Args& a) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a.packed) | reinterpret_cast<uintptr_t>(a.scales) |
                           reinterpret_cast<uintptr_t>(a.zp) | reinterpret_cast<uintptr_t>(a.y) |
                           (a.bias ? reinterpret_cast<uintptr_t>(a.bias) : 0);
    return a.m >= 1 && a.n % 4 == 0 && (bits & 15) == 0 && !a.g_idx && a.group_size % 32 == 0;
}

template <int RT, bool SPLITK>
static int launch_rt(const W4Args& a, hipStream_t s) {
    dim3 grid(ceil_div(a.n, SPLITK ? 64 : kGemmCols), ceil_div(a.m, 16 * RT));
    hipLaunchKernelGGL((w4_gemm_kernel<RT, SPLITK>), grid, dim3(256), 0, s, a);
    return check_launch("w4_gemm_kernel");
}

int w4_launch_gemm(const W4Args& a, hipStream_t s) {
    // Few rows: one strip per workgroup with K split over its waves, so that the
    // grid still covers the chip.  Many rows: 64-row tiles, which reuse each
    // converted weight fragment four times.
    if (a.m <= 16) return launch_rt<1, true>(a, s);
    if (a.m <= 32) return launch_rt<2, true>(a, s);
    return launch_rt<4, false>(a, s);
}

}  // namespace rumus
