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
// index XOR-swizzled by (row>>1)&3 so that both the 128-bit writes and the
// 128-bit fragment reads are bank-conflict free.
#include "common.h"

namespace rumus {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;  // K bytes per LDS stage

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
    const uint32_t ld_lds = ld_row * kBK + ((ld_c ^ (ld_row >> 1)) & 3) * 16;
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
    const uint32_t fr = lane & 31, fh = lane >> 5, fsw = (fr >> 1) & 3;
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

    // ---- epilogue -----------------------------------------------------------
    // Accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column
    // l%32 of its 32x32 tile: a store instruction writes two 128-byte row
    // segments.
    const uint32_t col_l = lane & 31, row_l = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const uint32_t col = n0 + (wn * TN + j) * 32 + col_l;
        if (col >= N) continue;
        const float swc = y ? sw[col] : 0.0f;
        const float bc = (y && bias) ? bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t row = m0 + (wm * TM + i) * 32 + 8 * (r / 4) + row_l + (r % 4);
                if (row >= M) continue;
                const int32_t a = acc[i][j][r];
                const uint64_t o = (uint64_t)row * N + col;
                if (acc_out) acc_out[o] = a;
                if (y) {
                    float v = __fmul_rn(__fmul_rn((float)a, sx[row]), swc);
                    if (bias) v = __fadd_rn(v, bc);
                    y[o] = v;
                }
            }
        }
    }
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

}  // namespace rumus

using namespace rumus;

extern "C" int rumus_hip_i8_gemm(const int8_t* xq, const int8_t* wq, const float* sx,
                                 const float* sw, const float* bias, int32_t* acc, float* y,
                                 uint32_t m, uint32_t k, uint32_t n, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(xq && wq, "i8_gemm: null operand");
    RUMUS_REQUIRE(acc || y, "i8_gemm: both outputs are null");
    RUMUS_REQUIRE(!y || (sx && sw), "i8_gemm: y needs sx and sw");
    RUMUS_REQUIRE(k > 0 && k % 16 == 0, "i8_gemm: k must be a positive multiple of 16 (got %u)", k);
    RUMUS_REQUIRE(((reinterpret_cast<uintptr_t>(xq) | reinterpret_cast<uintptr_t>(wq)) & 15) == 0,
                  "i8_gemm: operands must be 16-byte aligned");
    if (m == 0 || n == 0) return RUMUS_HIP_OK;
    hipStream_t s = as_stream(stream);
    // Largest tile that still gives every CU a workgroup.
    const uint64_t big = (uint64_t)ceil_div(m, 256) * ceil_div(n, 128);
    const uint64_t mid = (uint64_t)ceil_div(m, 128) * ceil_div(n, 128);
    if (big >= 256) return launch<4, 2, 2>(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
    if (mid >= 256) return launch<2, 2, 2>(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
    return launch<1, 1, 2>(xq, wq, sx, sw, bias, acc, y, m, k, n, s);
}
