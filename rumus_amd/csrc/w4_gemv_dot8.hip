// INT4 engine: the decode-shape kernel (m <= 8, group_size % (8*OCT) == 0).
//
// At 1 x 4096 x 4096 the whole problem is 9.4 MB: the launch lasts a few
// microseconds and is bound by latencies (dispatch, first byte from HBM) as
// much as by bandwidth.  Everything below is arranged to put all weight loads
// in flight at once, as early as possible, and to keep the dependent chain
// that follows their arrival short: no LDS staging and no barrier before the
// arithmetic.
//
// Data movement.  A workgroup owns 16 adjacent columns over the whole of K (no
// partial sums cross workgroups: no atomics, no zero-fill, deterministic).
// The four lanes of a quad cover the 16 columns with one 128-bit load each
// (4 words = 4 columns x 8 rows); each quad is one "row lane" and owns OCT
// consecutive packed word rows (a chunk of 8*OCT rows) per sweep.  A word row
// is a 64-byte segment per workgroup; the XCD-contiguous workgroup order puts
// the reader of the other half of each 128-byte line on the same L2.
//
// Arithmetic.  A packed word is 8 unsigned nibbles: exactly one operand of
// v_dot8_u32_u4.  The activations of a chunk are turned into 20-bit fixed
// point, X' = rint(x * f) + 2^19 (f a power of two from the chunk's abs-max),
// and split into five nibble planes laid out like the weights, so that
//   sum_j X'_j q_j = sum_i 16^i * dot8(word, plane_i)
// is exact integer arithmetic with no unpacking at all; the 2^19 offset is
// removed with dot8(word, 0x11111111) = sum_j q_j.  One conversion to f32 per
// (chunk, column) follows, then  y += scale * (part - zp * sum_j x_j).
// The planes never touch memory: the four lanes of a quad each build the
// planes of OCT/4 word rows of their own chunk and exchange them with DPP
// quad broadcasts.  Quantizing x to 20 bits relative to the abs-max of its
// chunk costs < 2^-19 relative error per activation, two orders below the f32
// tolerance of this path (rel 1e-3 / abs 1e-4).
#include "w4.h"

namespace rumus {

constexpr int kD8Cols = 16;  // columns per workgroup

__device__ __forceinline__ uint32_t udot8(uint32_t a, uint32_t b, uint32_t c) {
    return __builtin_amdgcn_udot8(a, b, c, false);
}

// DPP lane exchanges (one VALU op each, no LDS round trip).
#define RUMUS_DPP_F(v, ctrl) \
    __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xF, 0xF, true))
#define RUMUS_DPP_I(v, ctrl) __builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), 0xF, 0xF, true)
constexpr int kDppXor1 = 0xB1;   // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;   // quad_perm [2,3,0,1]
constexpr int kDppRowShr4 = 0x114, kDppRowShr8 = 0x118;

// silu(g) * u, the expression of swiglu_kernel (block_glue.hip), so that the fused and the
// separate path give the same bits
__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.0f + expf(-g)) * u; }

// value of quad lane Q in all four lanes of the quad
template <int Q> __device__ __forceinline__ uint32_t quad_bcast(uint32_t v) {
    return (uint32_t)RUMUS_DPP_I(v, Q * 0x55);
}

// Sum across the 16 quads of a wave (lanes that share lane & 3).
// Valid in lanes 12..15 afterwards.
__device__ __forceinline__ float reduce_row_lanes(float v) {
    v += RUMUS_DPP_F(v, kDppRowShr4);   // out-of-row reads give 0
    v += RUMUS_DPP_F(v, kDppRowShr8);
    // rows 0 + 1 and 2 + 3, then the halves: register swaps between lanes (v_permlane16_swap, v_permlane32_swap)
    // instead of two trips through the LDS crossbar; the same sums as v += shfl_xor(v, 16); v += shfl_xor(v, 32)
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    const auto h = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(h[0]) + __uint_as_float(h[1]);
    return v;
}


// Kernel arguments are passed flat.  This file is built with the first two
// arguments (the pointers to the packed words and the scales) preloaded into
// SGPRs at wave launch and the rest fetched by the wave: preloading more
// slows the launch of each of the 2048 waves by more than the fetch costs
// (the numbers are with the build flags).
//
// T threads = T/4 quads; a quad owns OCT consecutive word rows per sweep and
// each of its lanes prepares OPL = OCT/4 of them.  FASTX: activations are
// read with 128-bit loads (no perm, k % 8 == 0, 16-byte aligned x).
// ZP4: `zps` points at packed integer zero-points (eight per word along n) instead of floats.
// TILED: packed / scales / zps are tile-major copies (a tile = this workgroup's 16 columns, all
// rows), so the workgroup reads one contiguous 32 KB slab and each load instruction of a wave
// a contiguous 1 KB, instead of 64-byte segments 4*n bytes apart (10 % faster at 4096 x 4096).
// GLU (with FASTX): `xin` holds rows of 2k floats, gate | up, and the activations are
// silu(gate) * up computed on the way in: the SwiGLU between a fused gate|up projection and the
// down projection costs no launch and no round trip of its own.
// LDS of the fused norm: the waves' sums of squares per row (only the kernels with the norm allocate it)
template <int WAVES, int M>
__device__ __forceinline__ float* d8_sq_lds() {
    __shared__ float sq[WAVES * M];
    return sq;
}

// NORM (with FASTX): the activations are RMSNorm(x) = x * rsqrt(mean(x^2) + eps) * norm_w, the norm folded into the
// kernel that consumes it: the planes are built from x * norm_w, every lane adds the squares of the x it loads anyway
// (a workgroup's lanes load each element of the row exactly once), the sums of squares travel with the wave sums
// through LDS, and rsqrt(...) multiplies the result.  `resid` (or null): y = ... + resid[m][n], the residual add of
// the decoder block, in the epilogue.
// `resid` may be the output itself (each element is read by the thread that then stores it), so neither of the
// two pointers is declared restrict.
// BLOCK: the kernel looks at norm_w / eps / resid at all; the plain kernels are launched with nulls there and
// compile to what they were without these arguments.
template <int M, int T, int OCT, bool FASTX, bool ZP4, bool TILED, bool GLU = false, bool NORM = false, bool BLOCK = false>
__global__ __launch_bounds__(T) void w4_gemv_dot8_kernel(
    const uint32_t* __restrict__ packed, const float* __restrict__ scales,
    const float* __restrict__ zps, const float* __restrict__ xin, float* yout,
    uint32_t n, uint32_t k, uint32_t padded_k, uint32_t group_size,
    const float* __restrict__ bias, const int32_t* __restrict__ perm,
    const float* __restrict__ norm_w, float eps, const float* resid) {
    static_assert(!NORM || BLOCK, "the norm is one of the block's forms");
    static_assert(OCT == 4 || OCT == 8, "a quad shares 4 or 8 word rows");
    static_assert(!NORM || (FASTX && !GLU), "the fused norm reads plain rows with 128-bit loads");
    constexpr int RL = T / 4;      // quads per workgroup
    constexpr int WAVES = T / 64;
    constexpr int OPL = OCT / 4;   // word rows prepared per lane
    __shared__ float red[WAVES][M][kD8Cols];
    const uint32_t tid = threadIdx.x;
    const uint32_t nchunks = padded_k / (8 * OCT);

    // the grid size is recomputed from n: reading gridDim would cost a kernel-argument fetch
    const uint32_t cchunk = xcd_contiguous(blockIdx.x, (n + kD8Cols - 1) / kD8Cols);
    const uint32_t cq = tid & 3, rs = tid >> 2;
    const uint32_t col = cchunk * kD8Cols + 4 * cq;
    const bool col_ok = col < n;  // n % 4 == 0: a lane's four columns are all in or all out
    const uint32_t col_c = col_ok ? col : 0;

    float acc[M][4];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[m][c] = 0.0f;
    float ssq[NORM ? M : 1];                     // NORM: this lane's sum of squares per row
    if constexpr (NORM) {
#pragma unroll
        for (int m = 0; m < M; m++) ssq[m] = 0.0f;
    }

    // every quad runs the same number of sweeps; a dead quad carries scale 0
    for (uint32_t base = 0; base < nchunks; base += RL) {
        const uint32_t chunk = base + rs;
        const bool live = chunk < nchunks;
        const uint32_t ch = live ? chunk : 0;

        // ---- 1. loads, in the order their data is needed -----------------------
        // The memory counter retires in order, so the activation loads go first:
        // the nibble planes are then built while the weight loads are in flight.
        // Branch-free (clamped addresses, values zeroed by select) so that the
        // wait before the plane build covers x only.
        // The eight waves of a workgroup start together and the memory pipeline of the compute unit
        // takes their requests, and returns their data, in order: without help the oldest wave issues
        // all of its loads first and the activations of the other waves come back behind its weights
        // (measured: planes built 0.7 us after the start in wave 0, 1.3 us in waves 1-3, 1.9 us in
        // waves 4-7).  Raised priority while a wave asks for its activations puts the x requests of
        // the waves that start together ahead of their weight requests (planes at 0.8 us in waves
        // 0-3, 1.5 us in 4-7, which start 40 ns later; 0.03 to 0.2 us per launch by the machine).
        // With packed zero-points the same change costs 0.3 to 0.5 us, so it stays off there.
        constexpr bool kPrioX = !ZP4;
        float xv[M][OPL][8];
        if (kPrioX && base == 0) __builtin_amdgcn_s_setprio(3);
        const uint32_t k0 = (ch * OCT + cq * OPL) * 8;   // first row this lane prepares
#pragma unroll
        for (int m = 0; m < M; m++) {
#pragma unroll
            for (int t = 0; t < OPL; t++) {
                const uint32_t kt = k0 + 8 * t;
                if (FASTX) {
                    const bool in = kt < k;              // k % 8 == 0: all 8 in or out
                    const uint32_t kc = in ? kt : 0;
                    const float* xrow = xin + (uint64_t)m * (GLU ? 2 * k : k) + kc;
                    float4 lo = *reinterpret_cast<const float4*>(xrow);
                    float4 hi = *reinterpret_cast<const float4*>(xrow + 4);
                    if (GLU) {
                        const float4 ul = *reinterpret_cast<const float4*>(xrow + k);
                        const float4 uh = *reinterpret_cast<const float4*>(xrow + k + 4);
                        lo = make_float4(silu_mul(lo.x, ul.x), silu_mul(lo.y, ul.y), silu_mul(lo.z, ul.z),
                                         silu_mul(lo.w, ul.w));
                        hi = make_float4(silu_mul(hi.x, uh.x), silu_mul(hi.y, uh.y), silu_mul(hi.z, uh.z),
                                         silu_mul(hi.w, uh.w));
                    }
                    xv[m][t][0] = in ? lo.x : 0.0f; xv[m][t][1] = in ? lo.y : 0.0f;
                    xv[m][t][2] = in ? lo.z : 0.0f; xv[m][t][3] = in ? lo.w : 0.0f;
                    xv[m][t][4] = in ? hi.x : 0.0f; xv[m][t][5] = in ? hi.y : 0.0f;
                    xv[m][t][6] = in ? hi.z : 0.0f; xv[m][t][7] = in ? hi.w : 0.0f;
                    if constexpr (NORM) {
                        const float4 wl = *reinterpret_cast<const float4*>(norm_w + kc);
                        const float4 wh = *reinterpret_cast<const float4*>(norm_w + kc + 4);
                        const float nw[8] = {wl.x, wl.y, wl.z, wl.w, wh.x, wh.y, wh.z, wh.w};
#pragma unroll
                        for (int j = 0; j < 8; j++) {
                            // a quad past the end of K multiplies chunk 0 again, with scale 0: its x is not the row's
                            ssq[m] = live ? fmaf(xv[m][t][j], xv[m][t][j], ssq[m]) : ssq[m];
                            xv[m][t][j] *= nw[j];
                        }
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const bool in = kt + j < k;
                        const uint32_t kk = in ? kt + j : 0;
                        const uint32_t src = perm ? (uint32_t)perm[kk] : kk;
                        const float v = xin[(uint64_t)m * k + src];
                        xv[m][t][j] = in ? v : 0.0f;
                    }
                }
            }
        }
        if (kPrioX && base == 0) {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
        }
        const uint32_t g = (ch * 8 * OCT) / group_size;
        const uint64_t mo = TILED ? ((uint64_t)cchunk * (padded_k / group_size) + g) * kD8Cols + 4 * cq
                                  : (uint64_t)g * n + col_c;
        uint4 w[OCT];
        const uint32_t* p = TILED ? packed + ((uint64_t)cchunk * (padded_k / 8) + (uint64_t)ch * OCT) * kD8Cols + 4 * cq
                                  : packed + (uint64_t)ch * OCT * n + col_c;
        const uint64_t wstride = TILED ? kD8Cols : n;
        float4 sc, zp;          // zp: the four zero-points, or with ZP4 their packed word in .x (unpacked where it is used)
        auto load_meta = [&]() __attribute__((always_inline)) {
            sc = *reinterpret_cast<const float4*>(scales + mo);
            // ZP4 + TILED: the two zero-point words of a tile's 16 columns sit side by side per group
            if (!ZP4) zp = *reinterpret_cast<const float4*>(zps + mo);
            else zp.x = __uint_as_float(TILED ? reinterpret_cast<const uint32_t*>(zps)[
                                                    ((uint64_t)cchunk * (padded_k / group_size) + g) * 2 + (cq >> 1)] >> ((cq & 1) * 16)
                                              : reinterpret_cast<const uint32_t*>(zps)[(uint64_t)g * (n / 8) + col_c / 8] >> ((col_c & 4u) * 4u));
        };
#pragma unroll
        for (int u = 0; u < OCT; u++) w[u] = *reinterpret_cast<const uint4*>(p + (uint64_t)u * wstride);
        load_meta();
        if (!(live && col_ok)) sc = make_float4(0, 0, 0, 0);

        uint32_t wv[OCT][4];
#pragma unroll
        for (int u = 0; u < OCT; u++) { wv[u][0] = w[u].x; wv[u][1] = w[u].y; wv[u][2] = w[u].z; wv[u][3] = w[u].w; }
        const float scv[4] = {sc.x, sc.y, sc.z, sc.w};
        // the zero-points in f32, computed where they are used (after the dot products): unpacked here, the wait for
        // their word - the last load - would come ahead of every dot product
        auto zero_points = [&](float (&zv)[4]) __attribute__((always_inline)) {
            const float4 z = ZP4 ? w4_zp4_unpack4(__float_as_uint(zp.x)) : zp;
            zv[0] = z.x; zv[1] = z.y; zv[2] = z.z; zv[3] = z.w;
        };

#pragma unroll
        for (int m = 0; m < M; m++) {
            // ---- 2. activations of the chunk -> nibble planes (registers) -----
            // largest magnitude of the chunk, compared as integers: the bits of non-negative floats
            // order like the floats and a NaN sorts above infinity (a float max would skip it)
            uint32_t amax = 0;
#pragma unroll
            for (int t = 0; t < OPL; t++)
#pragma unroll
                for (int j = 0; j < 8; j++) amax = max(amax, __float_as_uint(xv[m][t][j]) & 0x7FFFFFFFu);
            const uint32_t lane_max = amax;                // of this lane's OPL octets
            amax = max(amax, (uint32_t)RUMUS_DPP_I(amax, kDppXor1));
            amax = max(amax, (uint32_t)RUMUS_DPP_I(amax, kDppXor2));
            // A chunk whose largest element towers over one of its four octets of 8 consecutive k (that octet's
            // largest more than 2^8 below it) would cost that octet its low bits in the fixed point below.  Such a
            // chunk is multiplied in f32 instead, element by element, at the end of this round (`wild`).  The
            // octets' maxima are the lanes' own (OPL == 1) on the way to amax; ordinary data never has such a chunk.
            uint32_t omin = lane_max;
            omin = min(omin, (uint32_t)RUMUS_DPP_I(omin, kDppXor1));
            omin = min(omin, (uint32_t)RUMUS_DPP_I(omin, kDppXor2));
            // (not with packed zero-points: there the same code costs 0.3 us per launch at 1 x 4096 x 4096, as the raised
            // priority above does, for reasons not found; that format keeps the plain fixed point)
            const bool wild = !ZP4 && omin + (8u << 23) < amax && amax < 0x7F800000u;
            // amax = a * 2^E (1 <= a < 2): scale by just under 2^(18-E) so that |x * f| < 2^19 - 1/2
            const uint32_t ebits = amax >> 23;             // biased exponent
            // the factor 1 - 2^-20 keeps rint(amax * f) at 2^19 - 1 or below
            float f = __uint_as_float((272u - ebits) << 23) * 0.99999905f;
            float finv = __uint_as_float((ebits - 18u) << 23) * 1.00000095f;
            if (ebits < 19) {              // zero or below 2^-108: contributes nothing
                f = 0.0f;
                finv = 0.0f;
            }
            if (ebits == 255) {            // inf / nan in the chunk: poison the result
                f = 0.0f;
                finv = __uint_as_float(0x7FC00000u);
            }
            finv = wild ? 0.0f : finv;     // a wild chunk's fixed point adds nothing; it is multiplied in f32 below
            uint32_t own[OPL][5];
            int xsum = 0;
#pragma unroll
            for (int t = 0; t < OPL; t++) {
                // adding 1.5*2^23 + 2^19 leaves rint(x*f) + 2^19 in the low 20 mantissa bits
                uint32_t X[8];
#pragma unroll
                for (int j = 0; j < 8; j++) X[j] = __float_as_uint(fmaf(xv[m][t][j], f, 13107200.0f));
                // plane i, nibble j = digit i of X[j]
                uint32_t ze[4], zo[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t A = X[2 * q], B = X[2 * q + 1];
                    ze[q] = (A & 0x0F0F0Fu) | ((B & 0x0F0F0Fu) << 4);   // bytes: digits 0,2,4 of (B,A)
                    zo[q] = ((A >> 4) & 0x0F0Fu) | (B & 0xF0F0u);       // bytes: digits 1,3 of (B,A)
                }
#pragma unroll
                for (int i = 0; i < 5; i++) {
                    const uint32_t* z = (i & 1) ? zo : ze;
                    const int sh = 8 * (i >> 1);
                    own[t][i] = ((z[0] >> sh) & 0xFFu) | (((z[1] >> sh) & 0xFFu) << 8) |
                                (((z[2] >> sh) & 0xFFu) << 16) | (((z[3] >> sh) & 0xFFu) << 24);
                }
                // sum_j X'_j from the planes, offsets removed: exact integer
                uint32_t s = 0;
#pragma unroll
                for (int i = 4; i >= 0; i--) s = s * 16u + udot8(own[t][i], 0x11111111u, 0u);
                xsum += (int)s - 8 * (1 << 19);
            }
            xsum += RUMUS_DPP_I(xsum, kDppXor1);
            xsum += RUMUS_DPP_I(xsum, kDppXor2);
            const float xs = (float)xsum * finv;
            // planes of the whole chunk: word row u was prepared by quad lane u / OPL
            uint32_t pl[OCT][5];
#pragma unroll
            for (int t = 0; t < OPL; t++)
#pragma unroll
                for (int i = 0; i < 5; i++) {
                    pl[0 * OPL + t][i] = quad_bcast<0>(own[t][i]);
                    pl[1 * OPL + t][i] = quad_bcast<1>(own[t][i]);
                    pl[2 * OPL + t][i] = quad_bcast<2>(own[t][i]);
                    pl[3 * OPL + t][i] = quad_bcast<3>(own[t][i]);
                }

            // ---- 3. dot products -------------------------------------------------
            // word row by word row, in the order the loads were issued and retire: the rows that have
            // arrived are multiplied while the later ones are still on their way, and only the last
            // row's 24 instructions follow the last byte
            uint32_t d[4][5], qsum[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                qsum[c] = 0;
#pragma unroll
                for (int i = 0; i < 5; i++) d[c][i] = 0;
            }
#pragma unroll
            for (int u = 0; u < OCT; u++)
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    qsum[c] = udot8(wv[u][c], 0x11111111u, qsum[c]);
#pragma unroll
                    for (int i = 0; i < 5; i++) d[c][i] = udot8(wv[u][c], pl[u][i], d[c][i]);
                }
            float zv[4];
            zero_points(zv);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                // D < 2^31: 8*OCT*225 * (16^5 - 1) / 15
                const uint32_t D = d[c][0] + 16u * (d[c][1] + 16u * (d[c][2] + 16u * (d[c][3] + 16u * d[c][4])));
                const int I = (int)D - (int)(qsum[c] << 19);
                const float part = (float)I * finv;
                acc[m][c] = fmaf(scv[c], fmaf(-zv[c], xs, part), acc[m][c]);
            }
            if (__builtin_expect(wild, 0)) {
                // (the fixed point added nothing: finv was zeroed)  The reference's loop over this chunk:
                // sum += x * ((q - zp) * scale), ascending k.  The activations are read again (the lanes of a quad
                // ask for the same address) rather than kept in registers for a case that ordinary data never has.
                float exact[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int u = 0; u < OCT; u++)
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const uint32_t kk = (ch * OCT + u) * 8 + j;
                        const bool in = kk < k;
                        const uint32_t kc = in ? kk : 0;
                        float xe;
                        if (FASTX) {
                            const float* xrow = xin + (uint64_t)m * (GLU ? 2 * k : k) + kc;
                            xe = xrow[0];
                            if (GLU) xe = silu_mul(xe, xrow[k]);
                            if constexpr (NORM) xe *= norm_w[kc];
                        } else {
                            xe = xin[(uint64_t)m * k + (perm ? (uint32_t)perm[kc] : kc)];
                        }
                        xe = in ? xe : 0.0f;
#pragma unroll
                        for (int c = 0; c < 4; c++)
                            exact[c] = fmaf(xe, ((float)((wv[u][c] >> (4 * j)) & 15u) - zv[c]) * scv[c], exact[c]);
                    }
#pragma unroll
                for (int c = 0; c < 4; c++) acc[m][c] += exact[c];
            }
        }
    }

    // ---- 4. reduce over the quads of a wave, then over the waves -----------------
    const uint32_t lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[m][c] = reduce_row_lanes(acc[m][c]);
    if (lane >= 12 && lane < 16) {
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int c = 0; c < 4; c++) red[wave][m][(lane - 12) * 4 + c] = acc[m][c];
    }
    if constexpr (NORM) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            // over the quad, then over the sixteen quads like the column sums: DPP and lane swaps, no LDS crossbar
            float q = ssq[m];
            q += RUMUS_DPP_F(q, kDppXor1);
            q += RUMUS_DPP_F(q, kDppXor2);
            q = reduce_row_lanes(q);
            if (lane == 15) d8_sq_lds<WAVES, M>()[wave * M + m] = q;
        }
    }
    __syncthreads();
    if (tid < M * kD8Cols) {
        const uint32_t m = tid / kD8Cols, c = tid % kD8Cols;
        const uint32_t oc = cchunk * kD8Cols + c;
        if (oc < n) {
            float v = 0.0f;
#pragma unroll
            for (int wi = 0; wi < WAVES; wi++) v += red[wi][m][c];
            if constexpr (NORM) {
                float q = 0.0f;
#pragma unroll
                for (int wi = 0; wi < WAVES; wi++) q += d8_sq_lds<WAVES, M>()[wi * M + m];
                v *= rsqrtf(q / (float)k + eps);
            }
            if (bias) v += bias[oc];
            if constexpr (BLOCK) {
                if (resid) v += resid[(uint64_t)m * n + oc];
            }
            yout[(uint64_t)m * n + oc] = v;
        }
    }
}

// Launch geometry: threads per workgroup and word rows per quad.
constexpr int kD8Threads = 512, kD8Oct = 4;

bool w4_gemv_dot8_supported(const W4Args& a) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a.packed) | reinterpret_cast<uintptr_t>(a.scales) |
                           reinterpret_cast<uintptr_t>(a.zp);
    return a.m >= 1 && a.m <= 8 && a.n % 4 == 0 && (bits & 15) == 0 && !a.g_idx &&
           a.group_size % (8 * kD8Oct) == 0;
}

template <int M, bool FASTX, bool ZP4, bool TILED, bool GLU = false>
static void launch_variant(const W4Args& a, hipStream_t s) {
    const float* zps = ZP4 ? reinterpret_cast<const float*>(a.zp4) : a.zp;
    // one row on packed zero-points: half as many waves with twice the word rows each start sooner than they
    // compute longer (1 x 4096 x 4096: 4.08 -> 3.98 us; with f32 zero-points the same change costs 0.1 us)
    if constexpr (M == 1 && FASTX && ZP4 && TILED && !GLU) {
        if (a.group_size % 64 == 0) {
            hipLaunchKernelGGL((w4_gemv_dot8_kernel<1, 256, 8, true, true, true, false>), dim3(ceil_div(a.n, kD8Cols)),
                               dim3(256), 0, s, a.packed, a.scales, zps, a.x, a.y, a.n, a.k, a.padded_k, a.group_size,
                               a.bias, a.perm, nullptr, 0.0f, nullptr);
            return;
        }
    }
    hipLaunchKernelGGL((w4_gemv_dot8_kernel<M, kD8Threads, kD8Oct, FASTX, ZP4, TILED, GLU>), dim3(ceil_div(a.n, kD8Cols)),
                       dim3(kD8Threads), 0, s, a.packed, a.scales, zps, a.x, a.y, a.n, a.k, a.padded_k,
                       a.group_size, a.bias, a.perm, nullptr, 0.0f, nullptr);
}

template <int M>
static int launch_m(const W4Args& a, hipStream_t s) {
    const bool fast_x = !a.perm && (a.k % 8 == 0) && ((reinterpret_cast<uintptr_t>(a.x) & 15) == 0);
    if (a.glu) {
        if (!(fast_x && a.tiled && !a.zp4))
            return set_error(RUMUS_HIP_EINVAL, "w4 gemv: the SwiGLU input needs the decode layout, f32 zero-points, "
                                               "k %% 8 == 0 and 16-byte aligned rows");
        launch_variant<M, true, false, true, true>(a, s);
    } else if (a.tiled && a.zp4) {
        if (fast_x) launch_variant<M, true, true, true>(a, s);
        else launch_variant<M, false, true, true>(a, s);
    } else if (a.tiled) {
        if (fast_x) launch_variant<M, true, false, true>(a, s);
        else launch_variant<M, false, false, true>(a, s);
    } else if (a.zp4) {
        if (fast_x) launch_variant<M, true, true, false>(a, s);
        else launch_variant<M, false, true, false>(a, s);
    } else {
        if (fast_x) launch_variant<M, true, false, false>(a, s);
        else launch_variant<M, false, false, false>(a, s);
    }
    return check_launch("w4_gemv_dot8_kernel");
}

int w4_launch_gemv_dot8(const W4Args& a, hipStream_t s) {
    switch (a.m) {
        case 1: return launch_m<1>(a, s);
        case 2: return launch_m<2>(a, s);
        case 3: return launch_m<3>(a, s);
        case 4: return launch_m<4>(a, s);
        case 5: return launch_m<5>(a, s);
        case 6: return launch_m<6>(a, s);
        case 7: return launch_m<7>(a, s);
        case 8: return launch_m<8>(a, s);
    }
    return set_error(RUMUS_HIP_EINVAL, "w4 gemv: m = %u out of range", a.m);
}

template <int M>
static int launch_block_m(const W4Args& a, const float* norm_w, float eps, const float* resid, hipStream_t s) {
    const dim3 grid(ceil_div(a.n, kD8Cols)), block(kD8Threads);
#define RUMUS_D8_BLOCK(GLU, NORM)                                                                                      \
    hipLaunchKernelGGL((w4_gemv_dot8_kernel<M, kD8Threads, kD8Oct, true, false, true, GLU, NORM, true>), grid, block, 0, \
                       s, a.packed, a.scales, a.zp, a.x, a.y, a.n, a.k, a.padded_k, a.group_size, a.bias,              \
                       static_cast<const int32_t*>(nullptr), norm_w, eps, resid)
    if (a.glu) RUMUS_D8_BLOCK(true, false);
    else if (norm_w) RUMUS_D8_BLOCK(false, true);
    else RUMUS_D8_BLOCK(false, false);
#undef RUMUS_D8_BLOCK
    return check_launch("w4_gemv_dot8_kernel");
}

// y = f(x) . dequant(W) + bias + resid on the decode layout with f32 zero-points: f = RMSNorm with `norm_w`
// (a.glu false, norm_w non-null), SwiGLU of gate | up rows (a.glu), or nothing.  The caller has checked the
// shapes (w4_gemv_dot8_supported, a.tiled, no packed zero-points, no perm, k % 8 == 0, 16-byte aligned x).
int w4_launch_gemv_dot8_block(const W4Args& a, const float* norm_w, float eps, const float* resid, hipStream_t s) {
    switch (a.m) {
        case 1: return launch_block_m<1>(a, norm_w, eps, resid, s);
        case 2: return launch_block_m<2>(a, norm_w, eps, resid, s);
        case 3: return launch_block_m<3>(a, norm_w, eps, resid, s);
        case 4: return launch_block_m<4>(a, norm_w, eps, resid, s);
        case 5: return launch_block_m<5>(a, norm_w, eps, resid, s);
        case 6: return launch_block_m<6>(a, norm_w, eps, resid, s);
        case 7: return launch_block_m<7>(a, norm_w, eps, resid, s);
        case 8: return launch_block_m<8>(a, norm_w, eps, resid, s);
    }
    return set_error(RUMUS_HIP_EINVAL, "w4 gemv: m = %u out of range", a.m);
}

}  // namespace rumus
