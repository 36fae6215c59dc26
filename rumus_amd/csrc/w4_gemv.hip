// INT4 engine: fused dequant-matmul kernels that are bound by HBM bandwidth
// (decode shapes, m <= 8), the reference-order kernel for every other case the
// MFMA kernel does not take, the transpose kernel for grad_x, and the entry
// points that pick between them.
//
// Packed layout (rumus-vision/src/quant.rs:98-100): word (k/8)*N + col holds
// rows 8*(k/8)..+7 of column col; scales / zero_points are f32 [groups, N].
#include <mutex>

#include "w4.h"

namespace rumus {

// ---------------------------------------------------------------------------
// Reference-order kernel.  One thread per column, MR rows per thread, strictly
// ascending k, w = (f32(q) - zp) * scale then sum += x * w with every
// operation rounded separately (qmatmul_int4.wgsl:50-84): the result is
// bit-identical to a scalar CPU loop in the same order.
// ---------------------------------------------------------------------------
template <int MR>
__global__ __launch_bounds__(64) void w4_generic_kernel(W4Args a) {
    const uint32_t col = blockIdx.x * 64 + threadIdx.x;
    const uint32_t row0 = blockIdx.y * MR;
    if (col >= a.n) return;
    float sum[MR];
#pragma unroll
    for (int r = 0; r < MR; r++) sum[r] = 0.0f;
    const uint32_t wpg = a.group_size / 8;
    for (uint32_t g = 0; g < a.num_groups; g++) {
        float scale = a.scales[(uint64_t)g * a.n + col];
        float z = a.zp4 ? w4_zp4_load1(a.zp4, g, a.n, col) : a.zp[(uint64_t)g * a.n + col];
        for (uint32_t w = 0; w < wpg; w++) {
            const uint32_t k_base = g * a.group_size + w * 8;
            if (k_base >= a.k) break;
            const uint32_t word = a.packed[(uint64_t)(k_base / 8) * a.n + col];
            for (uint32_t j = 0; j < 8; j++) {
                const uint32_t kk = k_base + j;
                if (kk >= a.k) break;  // padding rows (qmatmul_int4.wgsl:71)
                const float q = (float)((word >> (4 * j)) & 0xFu);
                if (a.g_idx) {
                    const uint64_t gi = (uint64_t)a.g_idx[kk], mi = gi * a.n + col;
                    scale = a.scales[mi];
                    z = a.zp4 ? w4_zp4_load1(a.zp4, gi, a.n, col) : a.zp[mi];
                }
                const float wv = __fmul_rn(__fsub_rn(q, z), scale);
                const uint32_t xk = a.perm ? (uint32_t)a.perm[kk] : kk;
#pragma unroll
                for (int r = 0; r < MR; r++) {
                    if (row0 + r < a.m) {
                        const float xv = a.x[(uint64_t)(row0 + r) * a.k + xk];
                        sum[r] = __fadd_rn(sum[r], __fmul_rn(xv, wv));
                    }
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < MR; r++) {
        if (row0 + r < a.m) {
            float v = sum[r];
            if (a.bias) v = __fadd_rn(v, a.bias[col]);
            a.y[(uint64_t)(row0 + r) * a.n + col] = v;
        }
    }
}

int w4_launch_generic(const W4Args& a, hipStream_t s) {
    constexpr int MR = 4;
    hipLaunchKernelGGL((w4_generic_kernel<MR>), dim3(ceil_div(a.n, 64), ceil_div(a.m, MR)), dim3(64),
                       0, s, a);
    return check_launch("w4_generic_kernel");
}

// ---------------------------------------------------------------------------
// Bandwidth kernel, m <= 8.
//
// A workgroup owns 16 adjacent columns over the whole of K, so no partial
// sums cross workgroups (no atomics, no zero-fill, deterministic).  Four lanes
// cover the 16 columns with one 128-bit load each (4 words = 4 columns x 8
// rows); the other lane bits and the four waves walk the K/8 word rows 64 at
// a time.  A word row is then a 64-byte segment per workgroup: the XCD-
// contiguous workgroup order puts the workgroup that reads the other half of
// each 128-byte line on the same L2.  All loads of a pass are issued before
// any arithmetic.  Per (word, column) the kernel forms d = sum_j x_j * q_j in
// f32 straight from the nibbles (v_cvt_f32_ubyte on masked words) and applies
// scale * (d - zp * sum_j x_j), which equals sum_j x_j * (q_j - zp) * scale.
// Rows of x live in LDS (zero beyond k, so padded nibbles contribute nothing).
// ---------------------------------------------------------------------------
constexpr int kGemvCols = 16;   // columns per workgroup
constexpr int kGemvRows = 64;   // word rows per pass (256 threads / 4 column lanes)
constexpr int kGemvUnroll = 8;  // passes whose loads are in flight together

__device__ __forceinline__ float ubyte(uint32_t v, int i) { return (float)((v >> (8 * i)) & 0xFFu); }

template <int M>
__global__ __launch_bounds__(256) void w4_gemv_kernel(W4Args a, uint32_t nchunks) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* xs = smem;                            // [M][padded_k]
    float* red = smem + (size_t)M * a.padded_k;  // [4 waves][M][16]

    const uint32_t tid = threadIdx.x;
    const uint32_t chunk = xcd_contiguous(blockIdx.x, nchunks);
    const uint32_t c0 = chunk * kGemvCols;

    for (uint32_t i = tid; i < M * a.padded_k; i += 256) {
        const uint32_t r = i / a.padded_k, j = i - r * a.padded_k;
        float v = 0.0f;
        if (j < a.k) v = a.x[(uint64_t)r * a.k + (a.perm ? (uint32_t)a.perm[j] : j)];
        xs[i] = v;
    }
    __syncthreads();

    const uint32_t cq = tid & 3, rsub = tid >> 2;
    const uint32_t col = c0 + 4 * cq;
    const bool col_ok = col < a.n;  // n % 4 == 0: all four columns in or out
    const uint32_t R = a.padded_k / 8;

    float acc[M][4];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[m][c] = 0.0f;

    for (uint32_t r0 = 0; r0 < R; r0 += kGemvRows * kGemvUnroll) {
        uint4 w[kGemvUnroll];
        float4 sc[kGemvUnroll], z[kGemvUnroll];
#pragma unroll
        for (int u = 0; u < kGemvUnroll; u++) {
            const uint32_t r = r0 + u * kGemvRows + rsub;
            if (col_ok && r < R) {
                const uint32_t g = (r * 8) / a.group_size;
                w[u] = *reinterpret_cast<const uint4*>(a.packed + (uint64_t)r * a.n + col);
                sc[u] = *reinterpret_cast<const float4*>(a.scales + (uint64_t)g * a.n + col);
                z[u] = *reinterpret_cast<const float4*>(a.zp + (uint64_t)g * a.n + col);
            } else {
                w[u] = make_uint4(0, 0, 0, 0);
                sc[u] = make_float4(0, 0, 0, 0);
                z[u] = make_float4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < kGemvUnroll; u++) {
            const uint32_t r = min(r0 + u * kGemvRows + rsub, R - 1);
            const uint32_t wv[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
            const float scv[4] = {sc[u].x, sc[u].y, sc[u].z, sc[u].w};
            const float zv[4] = {z[u].x, z[u].y, z[u].z, z[u].w};
            float q[4][8];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t lo = wv[c] & 0x0F0F0F0Fu, hi = (wv[c] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    q[c][2 * b] = ubyte(lo, b);
                    q[c][2 * b + 1] = ubyte(hi, b);
                }
            }
#pragma unroll
            for (int m = 0; m < M; m++) {
                const float4 xa = *reinterpret_cast<const float4*>(xs + (size_t)m * a.padded_k + r * 8);
                const float4 xb = *reinterpret_cast<const float4*>(xs + (size_t)m * a.padded_k + r * 8 + 4);
                const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
                const float xsum = ((xa.x + xa.y) + (xa.z + xa.w)) + ((xb.x + xb.y) + (xb.z + xb.w));
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    float d = 0.0f;
#pragma unroll
                    for (int j = 0; j < 8; j++) d = fmaf(xv[j], q[c][j], d);
                    acc[m][c] = fmaf(scv[c], fmaf(-zv[c], xsum, d), acc[m][c]);
                }
            }
        }
    }

    // lanes that share cq hold partial sums of the same columns: fold lane bits 2..5
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float v = acc[m][c];
            v += __shfl_xor(v, 4);
            v += __shfl_xor(v, 8);
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            acc[m][c] = v;
        }
    const uint32_t lane = tid & 63, wave = tid >> 6;
    if (lane < 4) {
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int c = 0; c < 4; c++) red[(wave * M + m) * kGemvCols + lane * 4 + c] = acc[m][c];
    }
    __syncthreads();
    if (tid < M * kGemvCols) {
        const uint32_t m = tid / kGemvCols, c = tid % kGemvCols;
        if (c0 + c < a.n) {
            float v = (red[(0 * M + m) * kGemvCols + c] + red[(1 * M + m) * kGemvCols + c]) +
                      (red[(2 * M + m) * kGemvCols + c] + red[(3 * M + m) * kGemvCols + c]);
            if (a.bias) v += a.bias[c0 + c];
            a.y[(uint64_t)m * a.n + c0 + c] = v;
        }
    }
}

static size_t gemv_lds_bytes(const W4Args& a) {
    return ((size_t)a.m * a.padded_k + 4 * (size_t)a.m * kGemvCols) * sizeof(float);
}

bool w4_gemv_supported(const W4Args& a) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a.packed) | reinterpret_cast<uintptr_t>(a.scales) |
                           reinterpret_cast<uintptr_t>(a.zp);
    return a.m >= 1 && a.m <= 8 && a.n % 4 == 0 && (bits & 15) == 0 && !a.g_idx && !a.zp4 &&
           gemv_lds_bytes(a) <= 64 * 1024;
}

template <int M>
static int launch_gemv_m(const W4Args& a, hipStream_t s) {
    const uint32_t nchunks = ceil_div(a.n, kGemvCols);
    hipLaunchKernelGGL((w4_gemv_kernel<M>), dim3(nchunks), dim3(256), gemv_lds_bytes(a), s, a, nchunks);
    return check_launch("w4_gemv_kernel");
}

int w4_launch_gemv(const W4Args& a, hipStream_t s) {
    switch (a.m) {
        case 1: return launch_gemv_m<1>(a, s);
        case 2: return launch_gemv_m<2>(a, s);
        case 3: return launch_gemv_m<3>(a, s);
        case 4: return launch_gemv_m<4>(a, s);
        case 5: return launch_gemv_m<5>(a, s);
        case 6: return launch_gemv_m<6>(a, s);
        case 7: return launch_gemv_m<7>(a, s);
        case 8: return launch_gemv_m<8>(a, s);
    }
    return set_error(RUMUS_HIP_EINVAL, "w4 gemv: m = %u out of range", a.m);
}

// ---------------------------------------------------------------------------
// Transpose kernel (grad_x): out[m,k] = sum_n a[m,n] * dequant(W)[k,n]
// (qmatmul_int4_transpose.wgsl:37-74).  A workgroup owns KR word rows (8 KR
// output columns k) and MR rows of a; threads stride over n, so packed words,
// scales and zero-points are read coalesced, once per block of MR rows, and
// every value of a once per 8 KR outputs.
// ---------------------------------------------------------------------------
template <int MR, int KR>
__global__ __launch_bounds__(256) void w4_transpose_kernel(
    const float* __restrict__ a, const uint32_t* __restrict__ packed,
    const float* __restrict__ scales, const float* __restrict__ zp, float* __restrict__ out,
    uint32_t m, uint32_t k, uint32_t n, uint32_t gs, uint32_t word_rows) {
    __shared__ float red[4][KR][MR][8];
    const uint32_t kr0 = blockIdx.x * KR, row0 = blockIdx.y * MR, tid = threadIdx.x;
    float acc[KR][MR][8];
#pragma unroll
    for (int q = 0; q < KR; q++)
#pragma unroll
        for (int r = 0; r < MR; r++)
#pragma unroll
            for (int j = 0; j < 8; j++) acc[q][r][j] = 0.0f;
#pragma unroll(MR * KR == 1 ? 4 : 1)
    for (uint32_t c = tid; c < n; c += 256) {
        float av[MR];
#pragma unroll
        for (int r = 0; r < MR; r++) av[r] = row0 + r < m ? a[(uint64_t)(row0 + r) * n + c] : 0.0f;
#pragma unroll
        for (int q = 0; q < KR; q++) {
            const uint32_t kr = min(kr0 + q, word_rows - 1);        // past the end: recomputes the last row, not stored
            const uint32_t g = (kr * 8) / gs;
            const uint32_t word = packed[(uint64_t)kr * n + c];
            const float sc = scales[(uint64_t)g * n + c], z = zp[(uint64_t)g * n + c];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float wv = ((float)((word >> (4 * j)) & 0xFu) - z) * sc;
#pragma unroll
                for (int r = 0; r < MR; r++) acc[q][r][j] = fmaf(av[r], wv, acc[q][r][j]);
            }
        }
    }
#pragma unroll
    for (int q = 0; q < KR; q++)
#pragma unroll
        for (int r = 0; r < MR; r++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float v = wave_sum(acc[q][r][j]);
                if ((tid & 63) == 0) red[tid >> 6][q][r][j] = v;
            }
    __syncthreads();
    for (uint32_t e = tid; e < KR * MR * 8; e += 256) {
        const uint32_t q = e / (MR * 8), r = (e / 8) % MR, j = e % 8;
        const uint32_t kk = (kr0 + q) * 8 + j;
        if (row0 + r < m && kk < k)
            out[(uint64_t)(row0 + r) * k + kk] = (red[0][q][r][j] + red[1][q][r][j]) + (red[2][q][r][j] + red[3][q][r][j]);
    }
}

// The same product for a few rows on vector loads (n % 4 == 0, 16-byte aligned arrays, KR word rows inside one
// group): out[m, k] = sum_n t[m, n] q[k, n] - sum_n t[m, n] zp[g, n] with t = a * scale[g], so the scale and the
// zero-point are applied once per column and row of a instead of once per nibble, a nibble costs one byte-to-float
// conversion and one multiply-add, and every thread reads four columns per load.  4096 x 11008 from HBM: one row
// 17.3 -> 11.2 us, four rows 57 -> 16.7 us against the scalar-load kernel above, which remains for other shapes.
template <int MR, int KR>
__global__ __launch_bounds__(256) void w4_transpose_vec_kernel(
    const float* __restrict__ a, const uint32_t* __restrict__ packed,
    const float* __restrict__ scales, const float* __restrict__ zp, float* __restrict__ out,
    uint32_t m, uint32_t k, uint32_t n, uint32_t gs, uint32_t word_rows) {
    __shared__ float red[4][MR][KR * 8 + 1];
    const uint32_t kr0 = blockIdx.x * KR, row0 = blockIdx.y * MR, tid = threadIdx.x;
    const uint32_t nv = n / 4, g = (kr0 * 8) / gs;
    const float4* a4 = reinterpret_cast<const float4*>(a);
    const float4* sc4 = reinterpret_cast<const float4*>(scales) + (uint64_t)g * nv;
    const float4* zp4 = reinterpret_cast<const float4*>(zp) + (uint64_t)g * nv;
    const uint4* w4[KR];
#pragma unroll
    for (int q = 0; q < KR; q++)            // past the end: the last row again, not stored
        w4[q] = reinterpret_cast<const uint4*>(packed) + (uint64_t)min(kr0 + q, word_rows - 1) * nv;
    float acc[MR][KR][8], u[MR];
#pragma unroll
    for (int r = 0; r < MR; r++) {
        u[r] = 0.0f;
#pragma unroll
        for (int q = 0; q < KR; q++)
#pragma unroll
            for (int j = 0; j < 8; j++) acc[r][q][j] = 0.0f;
    }
#pragma unroll 2
    for (uint32_t v = tid; v < nv; v += 256) {
        const float4 s4 = sc4[v], z4 = zp4[v];
        uint4 w[KR];
#pragma unroll
        for (int q = 0; q < KR; q++) w[q] = w4[q][v];
        float4 av[MR];
#pragma unroll
        for (int r = 0; r < MR; r++) {
            av[r] = a4[(uint64_t)min(row0 + r, m - 1) * nv + v];
            if (row0 + r >= m) av[r] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
        const float sc[4] = {s4.x, s4.y, s4.z, s4.w}, z[4] = {z4.x, z4.y, z4.z, z4.w};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            float t[MR];
#pragma unroll
            for (int r = 0; r < MR; r++) {
                const float ar = c == 0 ? av[r].x : c == 1 ? av[r].y : c == 2 ? av[r].z : av[r].w;
                t[r] = ar * sc[c];
                u[r] = fmaf(t[r], z[c], u[r]);
            }
#pragma unroll
            for (int q = 0; q < KR; q++) {
                const uint32_t word = c == 0 ? w[q].x : c == 1 ? w[q].y : c == 2 ? w[q].z : w[q].w;
                const uint32_t lo = word & 0x0f0f0f0fu, hi = (word >> 4) & 0x0f0f0f0fu;   // nibbles 0,2,4,6 | 1,3,5,7
                // (float)((x >> 8 i) & 0xff) is one v_cvt_f32_ubyte<i>
                const float f[8] = {(float)(lo & 0xffu), (float)(hi & 0xffu),
                                    (float)((lo >> 8) & 0xffu), (float)((hi >> 8) & 0xffu),
                                    (float)((lo >> 16) & 0xffu), (float)((hi >> 16) & 0xffu),
                                    (float)(lo >> 24), (float)(hi >> 24)};
#pragma unroll
                for (int j = 0; j < 8; j++)
#pragma unroll
                    for (int r = 0; r < MR; r++) acc[r][q][j] = fmaf(t[r], f[j], acc[r][q][j]);
            }
        }
    }
    const uint32_t wave = tid >> 6;
#pragma unroll
    for (int r = 0; r < MR; r++) {
#pragma unroll
        for (int q = 0; q < KR; q++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float s = wave_sum(acc[r][q][j]);
                if ((tid & 63) == 0) red[wave][r][q * 8 + j] = s;
            }
        const float su = wave_sum(u[r]);
        if ((tid & 63) == 0) red[wave][r][KR * 8] = su;
    }
    __syncthreads();
    for (uint32_t e = tid; e < MR * KR * 8; e += 256) {
        const uint32_t r = e / (KR * 8), i = e % (KR * 8);
        const uint32_t kk = kr0 * 8 + i;
        if (row0 + r < m && kk < k && kr0 + i / 8 < word_rows) {
            const float dot = (red[0][r][i] + red[1][r][i]) + (red[2][r][i] + red[3][r][i]);
            const float zs = (red[0][r][KR * 8] + red[1][r][KR * 8]) + (red[2][r][KR * 8] + red[3][r][KR * 8]);
            out[(uint64_t)(row0 + r) * k + kk] = dot - zs;
        }
    }
}

static int validate(const W4Args& a, const char* who) {
    RUMUS_REQUIRE(a.group_size > 0 && a.group_size % 8 == 0,
                  "%s: group_size must be a multiple of 8 (got %u)", who, a.group_size);
    RUMUS_REQUIRE(a.padded_k == a.num_groups * a.group_size,
                  "%s: padded_k %u != num_groups %u * group_size %u", who, a.padded_k, a.num_groups,
                  a.group_size);
    RUMUS_REQUIRE(a.k <= a.padded_k && a.padded_k < a.k + a.group_size,
                  "%s: padded_k %u does not pad k %u to group_size %u", who, a.padded_k, a.k,
                  a.group_size);
    // a call without rows, columns or depth touches no array: null pointers are fine there (an empty tensor has none)
    RUMUS_REQUIRE(a.m == 0 || a.n == 0 || a.k == 0 || (a.x && a.packed && a.scales && (a.zp || a.zp4) && a.y),
                  "%s: null buffer", who);
    RUMUS_REQUIRE(!a.zp4 || a.n % 8 == 0, "%s: packed zero-points need n %% 8 == 0 (got %u)", who, a.n);
    return RUMUS_HIP_OK;
}

// Rows of x up to which the decode kernels beat the matrix-core kernel.  Measured on 4096 x 4096
// and 4096 x 11008 (g128): a decode launch costs 2.5 + 0.82 W us for one row and 0.45 W us per
// further row, W = millions of packed words; the matrix-core kernel 8.8 + 0.94 W us for any m up
// to 32.  The crossing is at 7 rows for 4096 x 4096 and 3 rows for 4096 x 11008; the decode
// kernels take at most 8.
uint32_t w4_decode_max_rows(uint32_t padded_k, uint32_t n) {
    const double mw = (double)(padded_k / 8) * n * 1e-6;
    if (mw <= 0.0) return 8;
    const double rows = 1.27 + 14.0 / mw;
    return rows >= 8.0 ? 8u : rows < 1.0 ? 1u : (uint32_t)rows;
}

static int dispatch(const W4Args& a, hipStream_t s) {
    if (a.m == 0 || a.n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(a.k > 0, "qmatmul_int4: k must be > 0");
    const bool few_rows = a.m <= w4_decode_max_rows(a.padded_k, a.n) || !w4_gemm_supported(a);
    if (few_rows && w4_gemv_dot8_supported(a)) return w4_launch_gemv_dot8(a, s);
    if (few_rows && w4_gemv_supported(a)) return w4_launch_gemv(a, s);
    if (w4_gemm_i8_supported(a)) return w4_launch_gemm_i8(a, s);
    if (w4_gemm_supported(a)) return w4_launch_gemm(a, s);
    // Batches the matrix-core kernel does not take (group sizes that are no multiple of 32): the
    // decode kernel, a few rows at a time, is far ahead of the reference-order kernel
    // (16 x 4096 x 11008, group 8: 1.2 ms there).
    {
        W4Args part = a;
        uint32_t rows = min(8u, a.m);                    // as many rows per launch as fit its LDS staging of x
        for (part.m = rows; rows > 1 && !w4_gemv_supported(part); part.m = --rows) {}
        if (w4_gemv_supported(part)) {
            for (uint32_t r0 = 0; r0 < a.m; r0 += rows) {
                part.m = min(rows, a.m - r0);
                part.x = a.x + (uint64_t)r0 * a.k;
                part.y = a.y + (uint64_t)r0 * a.n;
                if (int rc = w4_launch_gemv(part, s)) return rc;
            }
            return RUMUS_HIP_OK;
        }
    }
    return w4_launch_generic(a, s);
}

// ---- scratch memory of the entry point that allocates nothing -----------------------------------
// rumus_hip_qmatmul_int4_perm_static keeps what the matrix-core path parks in memory between its
// kernels (activations in matrix-core order, partial tiles of the K shares) in this array instead of
// the stream's workspace.  Every GPU the library runs on holds its own copy, at its own address, until
// the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress: the
// address the kernels get is the one looked up below, once per device.
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device.
static int static_scratch(void** out) {
    int device = 0;
    if (int rc = check_hip(hipGetDevice(&device), "hipGetDevice")) return rc;
    RUMUS_REQUIRE(device >= 0 && device < kMaxDevices, "static scratch: device %d beyond the %d supported", device,
                  kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void* ptr = nullptr;
        if (int rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
        RUMUS_REQUIRE(ptr != nullptr, "static scratch: no device address");
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return RUMUS_HIP_OK;
}

}  // namespace rumus

using namespace rumus;

extern "C" {

int rumus_hip_qmatmul_int4(const float* x, const uint32_t* packed, const float* scales,
                           const float* zero_points, const float* bias, const int32_t* g_idx,
                           float* y, uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                           uint32_t group_size, uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args a{x, packed, scales, zero_points, bias, g_idx, nullptr, y, m, k, n, padded_k, group_size, num_groups};
    if (int rc = validate(a, "qmatmul_int4")) return rc;
    return dispatch(a, as_stream(stream));
}

int rumus_hip_qmatmul_int4_perm(const float* x, const uint32_t* packed_sorted, const float* scales,
                                const float* zero_points, const float* bias, const int32_t* perm,
                                float* y, uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                                uint32_t group_size, uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args a{x, packed_sorted, scales, zero_points, bias, nullptr, perm, y, m, k, n, padded_k, group_size, num_groups};
    if (int rc = validate(a, "qmatmul_int4_perm")) return rc;
    RUMUS_REQUIRE(!perm || k == padded_k, "qmatmul_int4_perm: perm needs k == padded_k (%u vs %u)", k,
                  padded_k);
    return dispatch(a, as_stream(stream));
}

int rumus_hip_qmatmul_int4_decode(const float* x, const uint32_t* packed_t, const float* scales_t,
                                  const float* zero_points_t, const float* bias, const int32_t* perm, float* y,
                                  uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k, uint32_t group_size,
                                  uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args a{x, packed_t, scales_t, zero_points_t, bias, nullptr, perm, y, m, k, n, padded_k, group_size, num_groups,
             nullptr, true};
    if (int rc = validate(a, "qmatmul_int4_decode")) return rc;
    RUMUS_REQUIRE(!perm || k == padded_k, "qmatmul_int4_decode: perm needs k == padded_k (%u vs %u)", k, padded_k);
    RUMUS_REQUIRE(n % 16 == 0, "qmatmul_int4_decode: n must be a multiple of 16 (got %u)", n);
    RUMUS_REQUIRE(m <= 8, "qmatmul_int4_decode: at most 8 rows (got %u); larger batches take qmatmul_int4", m);
    if (m == 0 || n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(k > 0, "qmatmul_int4_decode: k must be > 0");
    RUMUS_REQUIRE(w4_gemv_dot8_supported(a),
                  "qmatmul_int4_decode: needs group_size %% 32 == 0 and 16-byte aligned buffers");
    return w4_launch_gemv_dot8(a, as_stream(stream));
}

uint32_t rumus_hip_qmatmul_int4_decode_max_rows(uint32_t padded_k, uint32_t n) {
    return w4_decode_max_rows(padded_k, n);
}

int rumus_hip_qmatmul_int4_decode_zp4(const float* x, const uint32_t* packed_t, const float* scales_t,
                                      const uint32_t* qzeros_t, const float* bias, const int32_t* perm, float* y,
                                      uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k, uint32_t group_size,
                                      uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args a{x, packed_t, scales_t, nullptr, bias, nullptr, perm, y, m, k, n, padded_k, group_size, num_groups,
             qzeros_t, true};
    if (int rc = validate(a, "qmatmul_int4_decode_zp4")) return rc;
    RUMUS_REQUIRE(!perm || k == padded_k, "qmatmul_int4_decode_zp4: perm needs k == padded_k (%u vs %u)", k, padded_k);
    RUMUS_REQUIRE(n % 16 == 0, "qmatmul_int4_decode_zp4: n must be a multiple of 16 (got %u)", n);
    RUMUS_REQUIRE(m <= 8, "qmatmul_int4_decode_zp4: at most 8 rows (got %u); larger batches take qmatmul_int4_zp4", m);
    if (m == 0 || n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(k > 0, "qmatmul_int4_decode_zp4: k must be > 0");
    RUMUS_REQUIRE(w4_gemv_dot8_supported(a),
                  "qmatmul_int4_decode_zp4: needs group_size %% 32 == 0 and 16-byte aligned buffers");
    return w4_launch_gemv_dot8(a, as_stream(stream));
}

int rumus_hip_qmatmul_int4_decode_swiglu(const float* gate_up, const uint32_t* packed_t, const float* scales_t,
                                         const float* zero_points_t, const float* bias, float* y, uint32_t m,
                                         uint32_t k, uint32_t n, uint32_t padded_k, uint32_t group_size,
                                         uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args a{gate_up, packed_t, scales_t, zero_points_t, bias, nullptr, nullptr, y, m, k, n, padded_k, group_size,
             num_groups, nullptr, true, true};
    if (int rc = validate(a, "qmatmul_int4_decode_swiglu")) return rc;
    RUMUS_REQUIRE(n % 16 == 0, "qmatmul_int4_decode_swiglu: n must be a multiple of 16 (got %u)", n);
    RUMUS_REQUIRE(m <= 8, "qmatmul_int4_decode_swiglu: at most 8 rows (got %u)", m);
    if (m == 0 || n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(k > 0 && k % 8 == 0, "qmatmul_int4_decode_swiglu: k must be a positive multiple of 8 (got %u)", k);
    RUMUS_REQUIRE(w4_gemv_dot8_supported(a),
                  "qmatmul_int4_decode_swiglu: needs group_size %% 32 == 0 and 16-byte aligned buffers");
    return w4_launch_gemv_dot8(a, as_stream(stream));
}

int rumus_hip_qmatmul_int4_decode_block(const float* x, const float* norm_weight, float eps, int swiglu,
                                        const uint32_t* packed_t, const float* scales_t, const float* zero_points_t,
                                        const float* bias, const float* residual, float* y, uint32_t m, uint32_t k,
                                        uint32_t n, uint32_t padded_k, uint32_t group_size, uint32_t num_groups,
                                        rumus_hip_stream_t stream) {
    W4Args a{x, packed_t, scales_t, zero_points_t, bias, nullptr, nullptr, y, m, k, n, padded_k, group_size,
             num_groups, nullptr, true, swiglu != 0};
    if (int rc = validate(a, "qmatmul_int4_decode_block")) return rc;
    RUMUS_REQUIRE(!(swiglu && norm_weight), "qmatmul_int4_decode_block: RMSNorm and SwiGLU inputs exclude each other");
    RUMUS_REQUIRE(n % 16 == 0, "qmatmul_int4_decode_block: n must be a multiple of 16 (got %u)", n);
    RUMUS_REQUIRE(m <= 8, "qmatmul_int4_decode_block: at most 8 rows (got %u)", m);
    if (m == 0 || n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(k > 0 && k % 8 == 0, "qmatmul_int4_decode_block: k must be a positive multiple of 8 (got %u)", k);
    RUMUS_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(norm_weight)) & 15) == 0,
                  "qmatmul_int4_decode_block: x and norm_weight must be 16-byte aligned");
    RUMUS_REQUIRE(y != x, "qmatmul_int4_decode_block: y must not be x (residual may be y)");
    RUMUS_REQUIRE(w4_gemv_dot8_supported(a),
                  "qmatmul_int4_decode_block: needs group_size %% 32 == 0 and 16-byte aligned buffers");
    return w4_launch_gemv_dot8_block(a, norm_weight, eps, residual, as_stream(stream));
}

int rumus_hip_qmatmul_int4_zp4(const float* x, const uint32_t* packed, const float* scales,
                               const uint32_t* qzeros, const float* bias, const int32_t* perm, float* y,
                               uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k, uint32_t group_size,
                               uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args a{x, packed, scales, nullptr, bias, nullptr, perm, y, m, k, n, padded_k, group_size, num_groups, qzeros};
    if (int rc = validate(a, "qmatmul_int4_zp4")) return rc;
    RUMUS_REQUIRE(!perm || k == padded_k, "qmatmul_int4_zp4: perm needs k == padded_k (%u vs %u)", k, padded_k);
    return dispatch(a, as_stream(stream));
}

int rumus_hip_qmatmul_int4_perm_static(const float* x, const uint32_t* packed_sorted, const float* scales,
                                       const float* zero_points, const float* bias, const int32_t* perm,
                                       float* y, uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                                       uint32_t group_size, uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args a{x, packed_sorted, scales, zero_points, bias, nullptr, perm, y, m, k, n, padded_k, group_size, num_groups};
    if (int rc = validate(a, "qmatmul_int4_perm_static")) return rc;
    RUMUS_REQUIRE(!perm || k == padded_k, "qmatmul_int4_perm_static: perm needs k == padded_k (%u vs %u)", k,
                  padded_k);
    void* ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    // every workspace request below is served from the array (or refused): same kernels, same order of
    // the sums, and every byte a kernel reads from the array has been written earlier in this call
    WorkspaceFixed fixed(ptr, kStaticScratchBytes);
    return dispatch(a, as_stream(stream));
}

uint64_t rumus_hip_static_scratch_bytes(void) { return kStaticScratchBytes; }

int rumus_hip_qmatmul_int4_t(const float* a, const uint32_t* packed, const float* scales,
                             const float* zero_points, float* out, uint32_t m, uint32_t k,
                             uint32_t n, uint32_t padded_k, uint32_t group_size,
                             uint32_t num_groups, rumus_hip_stream_t stream) {
    W4Args v{a, packed, scales, zero_points, nullptr, nullptr, nullptr, out, m, k, n, padded_k, group_size, num_groups};
    if (int rc = validate(v, "qmatmul_int4_t")) return rc;
    if (m == 0 || k == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(n > 0, "qmatmul_int4_t: n must be > 0");
    hipStream_t s = as_stream(stream);
    // where the matrix-core kernel is ahead of the vector kernel below, which takes four rows per pass (from HBM,
    // us, vector at 8 / 12 / 16 / 24 / 32 / 48 rows against the matrix cores at any of them: 4096 x 11008 g128
    // 30 / 31 / 40 / 53 / 65 / 97 against 49-51, g64 against 59-61, g32 against 105-110; 11008 x 4096 32 / 39 / 46 / 65 /
    // 83 / 120 against 37-42, 56-60, 139-143; 4096 x 4096 17 / 15 / 20 / 26 / 33 / 46 against 31-34, 38-41, 45-50)
    const uint32_t mfma_from = group_size % 128 == 0 ? 13 : group_size == 64 ? 21 : 49;
    if (m >= mfma_from && w4_gemm_t_supported(m, k, n, group_size, a, packed, scales, zero_points, out))
        return w4_launch_gemm_t(a, packed, scales, zero_points, out, m, k, n, padded_k, group_size, num_groups, s);
    const uint32_t word_rows = padded_k / 8;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(packed) |
                           reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(zero_points);
    if (n % 4 == 0 && (bits & 15) == 0 && group_size % 16 == 0) {
        const uint32_t mr = m <= 2 ? m : 4;           // rows per pass (eight at once: 34 us against 26 in two passes)
        // two word rows per workgroup (they share scale and zero-point) once the passes over the rows multiply the
        // workgroups; a single pass wants the workgroups (4096 x 11008: 4 rows 19.9 -> 16.7 us with one word row
        // each, 8 rows 22.7 -> 25.4 us)
        const bool two = m > 4 && word_rows >= 512;
        const dim3 grid(two ? ceil_div(word_rows, 2) : word_rows, ceil_div(m, mr));
#define RUMUS_W4T_VEC(MR)                                                                                              \
        do {                                                                                                           \
            if (two) hipLaunchKernelGGL((w4_transpose_vec_kernel<MR, 2>), grid, dim3(256), 0, s, a, packed, scales,    \
                                        zero_points, out, m, k, n, group_size, word_rows);                             \
            else hipLaunchKernelGGL((w4_transpose_vec_kernel<MR, 1>), grid, dim3(256), 0, s, a, packed, scales,        \
                                    zero_points, out, m, k, n, group_size, word_rows);                                 \
        } while (0)
        if (mr == 1) RUMUS_W4T_VEC(1);
        else if (mr == 2) RUMUS_W4T_VEC(2);
        else RUMUS_W4T_VEC(4);
#undef RUMUS_W4T_VEC
        return check_launch("w4_transpose_vec_kernel");
    }
    // other shapes (n % 4 != 0, unaligned arrays, odd group sizes): 4 rows x 32 outputs per workgroup from 3 rows on
    // (each value of a is then read once per 32 outputs, each word once per 4 rows); single rows keep one word
    // row per workgroup for the sake of parallelism
    if (m >= 3)
        hipLaunchKernelGGL((w4_transpose_kernel<4, 4>), dim3(ceil_div(word_rows, 4), ceil_div(m, 4)), dim3(256), 0, s, a,
                           packed, scales, zero_points, out, m, k, n, group_size, word_rows);
    else
        hipLaunchKernelGGL((w4_transpose_kernel<1, 1>), dim3(word_rows, m), dim3(256), 0, s, a, packed, scales,
                           zero_points, out, m, k, n, group_size, word_rows);
    return check_launch("w4_transpose_kernel");
}

}  // extern "C"
