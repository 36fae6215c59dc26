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
// group (group_size % 128 == 0) and walks n in steps of 32:
//   * staging (all 256 threads, 8 values each): a = (gy f_row) (s / S) with f_row and S powers of two
//     that put |a| below 2^14 (w4t_prepare_kernel: row maxima of gy, maximum of the scales), split into
//     hi + lo f16 (22 bits), written to LDS in A-fragment rows of 64 bytes; c accumulates in f32;
//   * every wave owns 32 of the 128 k: lane (k = lane % 32, half = lane / 32) loads the 8 consecutive
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

constexpr int kTScaleParts = 64;                               // partial maxima of the scales
constexpr int kTMaxSplits = 8;

// blocks [0, m): f_row = 2^(140 - e) for a row maximum a 2^(e - 127), 1 <= a < 2, so |gy f| < 2^14
// (0 for an all-zero or tiny row, NaN marker for a row with inf / nan); blocks [m, m + 64): partial
// maxima of the scales as bits.
__global__ __launch_bounds__(256) void w4t_prepare_kernel(const float* __restrict__ gy, const float* __restrict__ scales,
                                                          float* __restrict__ rowf, uint32_t* __restrict__ smax_part,
                                                          uint32_t m, uint32_t n, uint64_t nscales) {
    __shared__ uint32_t red[4];
    const uint32_t tid = threadIdx.x;
    uint32_t amax = 0;
    if (blockIdx.x < m) {
        const float* r = gy + (uint64_t)blockIdx.x * n;        // n % 4 == 0, 16-byte aligned
        for (uint32_t j = 4 * tid; j < n; j += 1024) {
            const float4 t = *reinterpret_cast<const float4*>(r + j);
            amax = max(max(amax, max(__float_as_uint(t.x) & 0x7FFFFFFFu, __float_as_uint(t.y) & 0x7FFFFFFFu)),
                       max(__float_as_uint(t.z) & 0x7FFFFFFFu, __float_as_uint(t.w) & 0x7FFFFFFFu));
        }
    } else {
        const uint32_t part = blockIdx.x - m;
        const uint64_t per = (nscales + kTScaleParts - 1) / kTScaleParts;
        const uint64_t lo = part * per, hi = min(nscales, lo + per);
        for (uint64_t j = lo + tid; j < hi; j += 256) amax = max(amax, __float_as_uint(scales[j]) & 0x7FFFFFFFu);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = max(amax, (uint32_t)__shfl_xor((int)amax, off));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    if (tid != 0) return;
    amax = max(max(red[0], red[1]), max(red[2], red[3]));
    if (blockIdx.x >= m) {
        smax_part[blockIdx.x - m] = amax;
        return;
    }
    const uint32_t e = amax >> 23;
    float f = e >= 255 ? __uint_as_float(0x7FC00000u) : e < 14 ? 0.0f : __uint_as_float((267u - e) << 23);
    rowf[blockIdx.x] = f;
}

// One workgroup: rows [64 y, 64 y + 64), k [128 x, 128 x + 128), n steps [z steps_per, ..).
__global__ __launch_bounds__(256, 2) void w4t_gemm_kernel(
    const float* __restrict__ gy, const uint32_t* __restrict__ packed, const float* __restrict__ scales,
    const float* __restrict__ zp, const float* __restrict__ rowf, const uint32_t* __restrict__ smax_part,
    float* __restrict__ out, uint32_t m, uint32_t k, uint32_t n, uint32_t gs, uint32_t steps_per) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][2][64 * 64];   // [buffer][hi, lo][row][32 n] f16
    __shared__ __attribute__((aligned(16))) _Float16 lds_z[2][32];          // [buffer][n]: 1024 + z0
    __shared__ float lds_c[64];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t k0 = blockIdx.x * 128, m0 = blockIdx.y * 64;
    const uint32_t g = k0 / gs;
    const uint32_t nsteps = (n + 31) / 32;
    const uint32_t st0 = blockIdx.z * steps_per, st1 = min(nsteps, st0 + steps_per);

    // ---- S: the power of two at or above the largest scale -------------------------------------------
    uint32_t smax = smax_part[lane];                           // kTScaleParts == 64
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) smax = max(smax, (uint32_t)__shfl_xor((int)smax, off));
    const uint32_t se = (smax >> 23) + ((smax & 0x7FFFFFu) ? 1u : 0u);      // S = 2^(se - 127)
    // se in 1 .. 253: both S and 1 / S are normal floats; otherwise (all scales zero or denormal,
    // or huge / inf / nan) the workgroup writes what the plain product would: zeros or NaNs
    const bool s_ok = se >= 1 && se <= 253;
    const float s_inv = s_ok ? __uint_as_float((254u - se) << 23) : 0.0f;
    const float s_big = s_ok ? __uint_as_float(se << 23) : (smax >= 0x7F000000u ? __uint_as_float(0x7FC00000u) : 0.0f);

    // ---- staging role: 8 consecutive n (chunk tid % 4) of row tid / 4 --------------------------------
    const uint32_t s_row = tid >> 2, s_ch = tid & 3;
    const uint32_t grow = min(m0 + s_row, m - 1);
    const float frow_raw = rowf[grow];
    const bool row_bad = frow_raw != frow_raw;                 // inf / nan in the row of gy
    const float frow = row_bad ? 0.0f : frow_raw;
    const float* gy_r = gy + (uint64_t)grow * n;
    const float* sc_g = scales + (uint64_t)g * n;
    const float* zp_g = zp + (uint64_t)g * n;
    const uint32_t s_lds = s_row * 64 + ((s_ch ^ row_swizzle(s_row)) & 3) * 16;
    float4 gv0, gv1, sv0, sv1, zv0, zv1;
    auto load_stage = [&](uint32_t st) {
        const uint32_t c0 = st * 32 + s_ch * 8;
        const bool in0 = c0 < n, in1 = c0 + 4 < n;             // n % 4 == 0: a float4 is all-in or all-out
        const uint32_t a0 = in0 ? c0 : 0, a1 = in1 ? c0 + 4 : 0;
        gv0 = *reinterpret_cast<const float4*>(gy_r + a0);
        gv1 = *reinterpret_cast<const float4*>(gy_r + a1);
        sv0 = *reinterpret_cast<const float4*>(sc_g + a0);
        sv1 = *reinterpret_cast<const float4*>(sc_g + a1);
        zv0 = *reinterpret_cast<const float4*>(zp_g + a0);
        zv1 = *reinterpret_cast<const float4*>(zp_g + a1);
        if (!in0) gv0 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (!in1) gv1 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    };
    float csum = 0.0f;
    auto store_stage = [&](int buf) {
        const float gvv[8] = {gv0.x, gv0.y, gv0.z, gv0.w, gv1.x, gv1.y, gv1.z, gv1.w};
        const float svv[8] = {sv0.x, sv0.y, sv0.z, sv0.w, sv1.x, sv1.y, sv1.z, sv1.w};
        const float zvv[8] = {zv0.x, zv0.y, zv0.z, zv0.w, zv1.x, zv1.y, zv1.z, zv1.w};
        t8h hi, lo, zoff;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            // powers of two first: (gy f) and (s / S) are exact, their product is rounded once
            const float a = (gvv[e] * frow) * (svv[e] * s_inv);
            const float z0 = rintf(zvv[e]);
            csum = fmaf(a, zvv[e] - z0, csum);
            zoff[e] = (_Float16)(1024.0f + z0);                // exact for |z0| <= 1024; zero-points are 0 .. 15
            // hi = a rounded to 11 bits by integer arithmetic, so that it converts to f16 exactly: left to
            // the compiler, (_Float16)a of a product becomes v_fma_mixlo_f16 (one rounding of the exact
            // product) in one place and a conversion of the rounded f32 in another, and on a tie the two
            // differ by a whole f16 step, which hi + lo then misses
            const float a_hi = __uint_as_float((__float_as_uint(a) + 0x1000u) & 0xFFFFE000u);
            const _Float16 h = (_Float16)a_hi;                 // exact above 2^-14; below, any rounding does
            hi[e] = h;
            lo[e] = (_Float16)(a - (float)h);
        }
        *reinterpret_cast<t8h*>(&lds_a[buf][0][s_lds]) = hi;
        *reinterpret_cast<t8h*>(&lds_a[buf][1][s_lds]) = lo;
        if (s_row == 0) *reinterpret_cast<t8h*>(&lds_z[buf][8 * s_ch]) = zoff;
    };

    // ---- B role: lane (k = 32 wave + lane % 32, half = lane / 32) -----------------------------------
    const uint32_t bc = lane & 31, bh = lane >> 5;
    const uint32_t kk = k0 + 32 * wave + bc;                   // < padded_k: whole groups exist in the arrays
    const uint32_t shift = 4 * (kk & 7);
    const uint32_t* wrow = packed + (uint64_t)(kk >> 3) * n;
    uint4 bw[2][2];                                            // [MFMA step t][low, high four words]
    auto load_b = [&](uint32_t st) {
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const uint32_t c0 = st * 32 + 16 * t + 8 * bh;
            const uint32_t a0 = c0 < n ? c0 : 0, a1 = c0 + 4 < n ? c0 + 4 : 0;   // past n: any words, times a = 0
            bw[t][0] = *reinterpret_cast<const uint4*>(wrow + a0);
            bw[t][1] = *reinterpret_cast<const uint4*>(wrow + a1);
        }
    };
    auto b_frag = [&](int t, int buf) {
        const uint32_t w[8] = {bw[t][0].x, bw[t][0].y, bw[t][0].z, bw[t][0].w, bw[t][1].x, bw[t][1].y, bw[t][1].z, bw[t][1].w};
        const t8h off = *reinterpret_cast<const t8h*>(&lds_z[buf][16 * t + 8 * bh]);   // 1024 + z0 of this lane's 8 n
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

    t16f acc[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;

    if (st0 < st1) {
        load_stage(st0);
        load_b(st0);
        store_stage(0);
    }
    __syncthreads();
    for (uint32_t st = st0; st < st1; st++) {
        const int cur = (st - st0) & 1;
        const bool more = st + 1 < st1;
        const t8h b0 = b_frag(0, cur), b1 = b_frag(1, cur);    // the words of this step, loaded a step ago
        if (more) {
            load_stage(st + 1);
            load_b(st + 1);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint8_t* hi = &lds_a[cur][0][i * 32 * 64];
            const uint8_t* lo = &lds_a[cur][1][i * 32 * 64];
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(hi + a_off[0]), b0, acc[i], 0, 0, 0);
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(lo + a_off[0]), b0, acc[i], 0, 0, 0);
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(hi + a_off[1]), b1, acc[i], 0, 0, 0);
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const t8h*>(lo + a_off[1]), b1, acc[i], 0, 0, 0);
        }
        if (more) store_stage(cur ^ 1);
        __syncthreads();
    }

    // ---- c[row]: the four staging threads of a row are neighbours in a wave ----------------------------
    csum += __shfl_xor(csum, 1);
    csum += __shfl_xor(csum, 2);
    if (s_ch == 0) lds_c[s_row] = csum;
    __syncthreads();

    // ---- register r of lane l is row 8 (r/4) + 4 (l/32) + r%4, column l%32 of its 32 x 32 tile -------
    float* dst = out + (uint64_t)blockIdx.z * m * k;
    const uint32_t col = k0 + 32 * wave + bc;
    if (col < k) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t lr = 32 * i + 8 * (r / 4) + 4 * fh + (r % 4), row = m0 + lr;
                if (row >= m) continue;
                const float f = rowf[row];
                // 1 / f_row = 2^(e - 140): from the bits of f (f = 2^(140 - e), biased exponent 267 - e)
                const float finv = f != f ? f : f == 0.0f ? 0.0f : __uint_as_float((254u - (__float_as_uint(f) >> 23)) << 23);
                dst[(uint64_t)row * k + col] = ((acc[i][r] - lds_c[lr]) * finv) * s_big;
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
    return group_size % 128 == 0 && n % 4 == 0 && k % 4 == 0 && (bits & 15) == 0 &&
           (uint64_t)m * k < (1ull << 32) && (uint64_t)m * n < (1ull << 40);
}

int w4_launch_gemm_t(const float* gy, const uint32_t* packed, const float* scales, const float* zp, float* out,
                     uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k, uint32_t group_size, uint32_t num_groups,
                     hipStream_t s) {
    const uint32_t ktiles = padded_k / 128, mtiles = ceil_div(m, 64), nsteps = ceil_div(n, 32);
    RUMUS_REQUIRE(mtiles <= 65535, "qmatmul_int4_t: m %u is beyond the grid limit", m);
    // few tiles: n is shared out too, in shares of at least 16 steps
    uint32_t shares = 1, steps_per = nsteps;
    const uint64_t tiles = (uint64_t)ktiles * mtiles;
    if (tiles < 256) {
        shares = (uint32_t)(512 / tiles);
        if (shares > (uint32_t)kTMaxSplits) shares = kTMaxSplits;
        if (shares > nsteps / 16) shares = nsteps / 16;
        if (shares < 1) shares = 1;
        steps_per = ceil_div(nsteps, shares);
        shares = ceil_div(nsteps, steps_per);
    }
    const size_t rowf_bytes = ((size_t)m * sizeof(float) + 255) & ~size_t(255);
    const size_t part_bytes = shares > 1 ? (size_t)shares * m * k * sizeof(float) : 0;
    void* ws = nullptr;
    if (int rc = workspace_get(s, rowf_bytes + 256 + part_bytes, &ws)) return rc;
    float* rowf = static_cast<float*>(ws);
    uint32_t* smax_part = reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(ws) + rowf_bytes);
    float* part = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + rowf_bytes + 256);
    hipLaunchKernelGGL(w4t_prepare_kernel, dim3(m + kTScaleParts), dim3(256), 0, s, gy, scales, rowf, smax_part, m, n,
                       (uint64_t)num_groups * n);
    if (int rc = check_launch("w4t_prepare_kernel")) return rc;
    hipLaunchKernelGGL(w4t_gemm_kernel, dim3(ktiles, mtiles, shares), dim3(256), 0, s, gy, packed, scales, zp, rowf,
                       smax_part, shares > 1 ? part : out, m, k, n, group_size, steps_per);
    if (int rc = check_launch("w4t_gemm_kernel")) return rc;
    if (shares == 1) return RUMUS_HIP_OK;
    const uint32_t count4 = (uint32_t)((uint64_t)m * k / 4);
    hipLaunchKernelGGL(w4t_add_shares_kernel, dim3(ceil_div(count4, 256)), dim3(256), 0, s,
                       reinterpret_cast<const float4*>(part), reinterpret_cast<float4*>(out), count4, shares);
    return check_launch("w4t_add_shares_kernel");
}

}  // namespace rumus
