// INT8 engine, reference Q8 block format: quantize, dequantize, W8A32 matmul,
// plus the bias add and the transpose that surround them in the reference.
//
// Buffer format (rumus/src/tensor/core.rs:61-98): per block one header word
// (f16 scale in the low half) followed by block_size signed bytes.
#include <hip/hip_fp16.h>

#include "common.h"
#include "i8_gemm.h"

namespace rumus {

__device__ __forceinline__ int quant_i8(float v, float inv) {
    // quantize.wgsl:93: clamp(i32(round(v*inv)), -128, 127), round = half-even.
    float t = rintf(__fmul_rn(v, inv));
    t = fminf(fmaxf(t, -128.0f), 127.0f);
    return (int)t;
}

__device__ __forceinline__ uint32_t quant_word(const float4& v, float inv) {
    return ((uint32_t)quant_i8(v.x, inv) & 0xFFu) | (((uint32_t)quant_i8(v.y, inv) & 0xFFu) << 8) |
           (((uint32_t)quant_i8(v.z, inv) & 0xFFu) << 16) | (((uint32_t)quant_i8(v.w, inv) & 0xFFu) << 24);
}

// One wave per block: abs-max by wave reduction, then quantize and pack.  quantize.wgsl:29-100.
// A block of up to 4096 elements stays in registers between the two passes (16 float4 per lane, all
// loads in flight at once); longer blocks are read twice.
constexpr int kBlockCache = 16;

__global__ __launch_bounds__(256) void q8_quantize_kernel(const float* __restrict__ in,
                                                          uint32_t* __restrict__ out,
                                                          uint32_t numel, uint32_t bs,
                                                          uint32_t num_blocks, uint32_t stride) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t block = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (block >= num_blocks) return;
    const uint64_t start = (uint64_t)block * bs;
    const uint32_t words = bs / 4;
    const bool full = start + bs <= numel && ((reinterpret_cast<uintptr_t>(in) & 15) == 0);
    const bool cached = full && words <= 64u * kBlockCache;
    const float4* p = reinterpret_cast<const float4*>(in + start);
    float4 cache[kBlockCache];

    float amax = 0.0f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < kBlockCache; i++) {
            const uint32_t w = lane + 64 * i;
            cache[i] = w < words ? p[w] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int i = 0; i < kBlockCache; i++)
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(cache[i].x), fabsf(cache[i].y)), fmaxf(fabsf(cache[i].z), fabsf(cache[i].w))));
    } else if (full) {
        for (uint32_t w = lane; w < words; w += 64) {
            float4 v = p[w];
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    } else {
        for (uint32_t i = lane; i < bs; i += 64)
            if (start + i < numel) amax = fmaxf(amax, fabsf(in[start + i]));
    }
    amax = wave_max(amax);

    const float scale = amax == 0.0f ? 1.0f : __fdiv_rn(amax, 127.0f);  // :66
    const float inv = amax == 0.0f ? 0.0f : __fdiv_rn(127.0f, amax);    // :67
    uint32_t* ob = out + (uint64_t)block * stride;
    if (lane == 0) ob[0] = (uint32_t)__half_as_ushort(__float2half_rn(scale));  // :71-74

    if (cached) {
#pragma unroll
        for (int i = 0; i < kBlockCache; i++) {
            const uint32_t w = lane + 64 * i;
            if (w < words) ob[1 + w] = quant_word(cache[i], inv);
        }
    } else if (full) {
        for (uint32_t w = lane; w < words; w += 64) ob[1 + w] = quant_word(p[w], inv);
    } else {
        for (uint32_t w = lane; w < words; w += 64) {
            uint32_t word = 0;
            for (uint32_t b = 0; b < 4; b++) {
                uint64_t gi = start + w * 4 + b;
                int q = gi < numel ? quant_i8(in[gi], inv) : 0;
                word |= ((uint32_t)q & 0xFFu) << (8 * b);
            }
            ob[1 + w] = word;
        }
    }
}

// Blocks of up to 256 elements: LPB lanes per block (one float4 each), 256 / LPB blocks per
// workgroup, so that a 32-element block does not leave 56 lanes of a wave idle.
template <int LPB>
__global__ __launch_bounds__(256) void q8_quantize_small_kernel(const float* __restrict__ in, uint32_t* __restrict__ out,
                                                                uint32_t numel, uint32_t bs, uint32_t num_blocks,
                                                                uint32_t stride) {
    const uint32_t sub = threadIdx.x % LPB;
    const uint32_t block = blockIdx.x * (256 / LPB) + threadIdx.x / LPB;
    if (block >= num_blocks) return;                           // whole groups of LPB lanes leave together
    const uint64_t start = (uint64_t)block * bs;
    const uint32_t words = bs / 4;                             // <= LPB
    const bool full = start + bs <= numel && ((reinterpret_cast<uintptr_t>(in) & 15) == 0);
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (sub < words) {
        if (full) {
            v = reinterpret_cast<const float4*>(in + start)[sub];
        } else {
            const uint64_t g = start + 4 * sub;
            v.x = g < numel ? in[g] : 0.0f;
            v.y = g + 1 < numel ? in[g + 1] : 0.0f;
            v.z = g + 2 < numel ? in[g + 2] : 0.0f;
            v.w = g + 3 < numel ? in[g + 3] : 0.0f;
        }
    }
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
#pragma unroll
    for (int off = LPB / 2; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const float scale = amax == 0.0f ? 1.0f : __fdiv_rn(amax, 127.0f);  // :66
    const float inv = amax == 0.0f ? 0.0f : __fdiv_rn(127.0f, amax);    // :67
    uint32_t* ob = out + (uint64_t)block * stride;
    if (sub == 0) ob[0] = (uint32_t)__half_as_ushort(__float2half_rn(scale));  // :71-74
    if (sub < words) ob[1 + sub] = quant_word(v, inv);         // elements past numel quantize to 0
}

__device__ __forceinline__ float header_scale(uint32_t header) {
    return __half2float(__ushort_as_half((unsigned short)(header & 0xFFFFu)));
}

// One thread per data word (4 elements).  dequantize.wgsl:32-52.
__global__ __launch_bounds__(256) void q8_dequantize_kernel(const uint32_t* __restrict__ in,
                                                            float* __restrict__ out,
                                                            uint32_t numel, uint32_t bs,
                                                            uint32_t stride) {
    const uint32_t w = blockIdx.x * 256 + threadIdx.x;         // data-word index; numel fits 32 bits
    if (w >= numel / 4 + (numel % 4 != 0)) return;
    const uint32_t e0 = w * 4;                                 // < numel <= 2^32 - 1: the last word starts below 2^32 - 3
    const uint32_t block = e0 / bs;
    const uint32_t pos = e0 - block * bs;
    const uint32_t* ib = in + (uint64_t)block * stride;
    const float scale = header_scale(ib[0]);
    const uint32_t word = ib[1 + pos / 4];
    float v[4];
#pragma unroll
    for (int b = 0; b < 4; b++) v[b] = __fmul_rn((float)(int)(int8_t)((word >> (8 * b)) & 0xFFu), scale);
    if (numel - e0 >= 4 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        *reinterpret_cast<float4*>(out + e0) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
        for (int b = 0; b < 4; b++)
            if (b < (int)(numel - e0)) out[e0 + b] = v[b];
    }
}

// W8A32 matmul, 64x64 tile per workgroup, 4x4 outputs per thread, K in steps
// of 16.  Arithmetic follows matmul_q8.wgsl:77-80 per element:
// sum += (a * f32(q)) * scale.  Requires block_size % 16 == 0 so that a run of
// 16 bytes never straddles a block.
constexpr int kQ8Tile = 64;
constexpr int kQ8K = 16;

__global__ __launch_bounds__(256) void matmul_q8_tiled_kernel(
    const float* __restrict__ a, const uint32_t* __restrict__ b, float* __restrict__ c,
    uint32_t m, uint32_t k, uint32_t n, uint32_t bs, uint32_t stride, uint32_t blocks_per_col) {
    __shared__ float as[kQ8K][kQ8Tile + 4];
    __shared__ float ws[kQ8K][kQ8Tile + 4];   // f32(q)
    __shared__ float ss[kQ8Tile];             // block scale per column for this K step
    const uint32_t tid = threadIdx.x;
    const uint32_t row0 = blockIdx.y * kQ8Tile, col0 = blockIdx.x * kQ8Tile;
    const uint32_t tx = tid % 16, ty = tid / 16;
    float acc[4][4] = {};

    for (uint32_t k0 = 0; k0 < k; k0 += kQ8K) {
        // A tile: 64 rows x 16 k; thread loads 4 consecutive k of one row.
        {
            uint32_t r = tid / 4, kq = (tid % 4) * 4;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t kk = k0 + kq + i;
                float v = 0.0f;
                if (row0 + r < m && kk < k) v = a[(uint64_t)(row0 + r) * k + kk];
                as[kq + i][r] = v;
            }
        }
        // B tile: 64 columns x 16 k = one word per (column, k-quad).
        {
            uint32_t cidx = tid / 4, kq = (tid % 4) * 4;
            uint32_t col = col0 + cidx;
            uint32_t kk = k0 + kq;
            uint32_t word = 0;
            float sc = 0.0f;
            if (col < n && kk < k) {
                uint32_t blk = kk / bs, pos = kk % bs;
                const uint32_t* bb = b + ((uint64_t)col * blocks_per_col + blk) * stride;
                word = bb[1 + pos / 4];
                sc = header_scale(bb[0]);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float q = (float)(int)(int8_t)((word >> (8 * i)) & 0xFFu);
                ws[kq + i][cidx] = (k0 + kq + i < k) ? q : 0.0f;
            }
            if (kq == 0) ss[cidx] = sc;
        }
        __syncthreads();
        float sc[4];
#pragma unroll
        for (int j = 0; j < 4; j++) sc[j] = ss[tx * 4 + j];
#pragma unroll
        for (int kk = 0; kk < kQ8K; kk++) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; i++) av[i] = as[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; j++) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __fadd_rn(acc[i][j], __fmul_rn(__fmul_rn(av[i], wv[j]), sc[j]));
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t r = row0 + ty * 4 + i;
        if (r >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t cc = col0 + tx * 4 + j;
            if (cc < n) c[(uint64_t)r * n + cc] = acc[i][j];
        }
    }
}

// block_size % 16 == 0, up to 8 rows per launch: bound by reading the weights once per launch
// (more rows run as several launches, still well ahead of the LDS-tiled kernel below).  The rows of x are
// staged in LDS (zero-padded to a multiple of 16 k).  A workgroup owns 32 columns, each of its
// eight waves four of them; lane i takes the 16 bytes k = 16 i .. 16 i + 15 of each of the four
// (one 128-bit load per column, all four in flight together; a run of 16 never straddles a block)
// and multiplies them with one read of x.  The 64 partial sums of a column meet in a butterfly.
// A column's bytes are contiguous in the Q8 layout, so a wave reads 1 KB runs.
// Arithmetic: sum_k (a * f32(q)) per run of 16, times the block scale once per run
// (matmul_q8.wgsl:77-80 multiplies by the scale per element).
// run_magic = ceil(2^32 / runs_per_block): run / runs_per_block as a multiply (exact below 2^16);
// 0 stands for one run per block.
struct __attribute__((packed, aligned(4))) Q8Words4 { uint32_t x, y, z, w; };

// ONCE: one block per column.  The bytes of a column are then one unbroken run behind a single header and the
// loads carry the non-temporal hint (1 x 4096 x 11008 from HBM: 14.5 -> 13.2 us; with smaller blocks the same
// hint costs 0.4 to 1.2 us).
template <int M, bool ONCE>
__global__ __launch_bounds__(512) void matmul_q8_rows_kernel(
    const float* __restrict__ a, const uint32_t* __restrict__ b, float* __restrict__ c, uint32_t k,
    uint32_t n, uint32_t stride, uint32_t blocks_per_col, uint32_t kpad, uint32_t runs_per_block,
    uint32_t run_magic) {
    constexpr int CW = 4;                                     // columns per wave
    // x in LDS as [row][quarter of a run][run][4]: the lanes of a wave, one run each, then read
    // consecutive 16-byte pieces (run-major order would put them 64 bytes apart, 16 to a bank)
    extern __shared__ float xs[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t nruns = kpad / 16;
    const uint32_t col0 = blockIdx.x * 32 + wave * CW;
    const uint32_t* colbase[CW];
#pragma unroll
    for (int cc = 0; cc < CW; cc++)
        colbase[cc] = b + (uint64_t)min(col0 + cc, n - 1) * blocks_per_col * stride;   // past n: re-reads the last column
    // Weights of one run (16 k) of the wave's four columns.  Branch-free: a run past the end reads the last one
    // again (and is not multiplied), so that no wait for memory sits at the end of a branch.
    auto fetch = [&](uint32_t run, Q8Words4 (&w4)[CW], uint32_t (&hdr)[CW]) {
        const uint32_t rc = min(run, nruns - 1);
        const uint32_t blk = run_magic ? __umulhi(rc, run_magic) : rc;   // magic 0: one run per block
        const uint32_t in_blk = rc - blk * runs_per_block;
        const uint32_t off = blk * stride;                   // header word of the block; data follows
#pragma unroll
        for (int cc = 0; cc < CW; cc++) {
            hdr[cc] = colbase[cc][off];
            if constexpr (ONCE) {
                typedef uint32_t q8_u4 __attribute__((ext_vector_type(4), aligned(4)));
                const q8_u4 t = __builtin_nontemporal_load(reinterpret_cast<const q8_u4*>(colbase[cc] + off + 1 + in_blk * 4));
                w4[cc] = Q8Words4{t.x, t.y, t.z, t.w};
            } else {
                w4[cc] = *reinterpret_cast<const Q8Words4*>(colbase[cc] + off + 1 + in_blk * 4);
            }
        }
    };
    // Blocks smaller than a column: the first two runs of every lane are on their way while the activations are
    // staged, and two stay in flight (1 x 4096 x 11008 from HBM, blocks of 32: 16.8 -> 16.0 us, of 128: 16.1 -> 15.4).
    // One block per column streams with the non-temporal hint and is faster in the plain loop (13.3 against 14.9 us).
    Q8Words4 wa[CW], wb[CW];
    uint32_t ha[CW], hb[CW];
    if constexpr (!ONCE) {
        fetch(lane, wa, ha);
        fetch(lane + 64, wb, hb);
        __builtin_amdgcn_sched_barrier(0);
    }
    for (uint32_t r = 0; r < M; r++)
        for (uint32_t kk = tid; kk < kpad; kk += 512)
            xs[((r * 4 + (kk % 16) / 4) * nruns + kk / 16) * 4 + kk % 4] = kk < k ? a[(uint64_t)r * k + kk] : 0.0f;
    __syncthreads();
    float acc[CW][M];
#pragma unroll
    for (int cc = 0; cc < CW; cc++)
#pragma unroll
        for (int r = 0; r < M; r++) acc[cc][r] = 0.0f;
    auto multiply = [&](uint32_t run, const Q8Words4 (&w4)[CW], const uint32_t (&hdr)[CW]) {
        float part[CW][M];
#pragma unroll
        for (int cc = 0; cc < CW; cc++)
#pragma unroll
            for (int r = 0; r < M; r++) part[cc][r] = 0.0f;
#pragma unroll
        for (int wi = 0; wi < 4; wi++) {
            float4 xv[M];
#pragma unroll
            for (int r = 0; r < M; r++) xv[r] = *reinterpret_cast<const float4*>(xs + ((r * 4 + wi) * nruns + run) * 4);
#pragma unroll
            for (int cc = 0; cc < CW; cc++) {
                const uint32_t word = wi == 0 ? w4[cc].x : wi == 1 ? w4[cc].y : wi == 2 ? w4[cc].z : w4[cc].w;
                float q[4];
#pragma unroll
                for (int j = 0; j < 4; j++) q[j] = (float)(int)(int8_t)((word >> (8 * j)) & 0xFFu);
#pragma unroll
                for (int r = 0; r < M; r++) {
                    part[cc][r] = fmaf(xv[r].x, q[0], part[cc][r]);
                    part[cc][r] = fmaf(xv[r].y, q[1], part[cc][r]);
                    part[cc][r] = fmaf(xv[r].z, q[2], part[cc][r]);
                    part[cc][r] = fmaf(xv[r].w, q[3], part[cc][r]);
                }
            }
        }
#pragma unroll
        for (int cc = 0; cc < CW; cc++) {
            const float sc = header_scale(hdr[cc]);
#pragma unroll
            for (int r = 0; r < M; r++) acc[cc][r] = fmaf(part[cc][r], sc, acc[cc][r]);
        }
    };
    if constexpr (ONCE) {
        for (uint32_t run = lane; run < nruns; run += 64) {
            fetch(run, wa, ha);
            multiply(run, wa, ha);
        }
    }
    // two runs per lane in flight: the slot just multiplied is refilled two runs ahead
    for (uint32_t run = lane; !ONCE && run < nruns; run += 128) {
        Q8Words4 w0[CW];
        uint32_t h0[CW];
#pragma unroll
        for (int cc = 0; cc < CW; cc++) { w0[cc] = wa[cc]; h0[cc] = ha[cc]; }
        fetch(run + 128, wa, ha);
        __builtin_amdgcn_sched_barrier(0);
        multiply(run, w0, h0);
        Q8Words4 w1[CW];
        uint32_t h1[CW];
#pragma unroll
        for (int cc = 0; cc < CW; cc++) { w1[cc] = wb[cc]; h1[cc] = hb[cc]; }
        fetch(run + 192, wb, hb);                            // outside the branch: a load under one is waited for at its end
        __builtin_amdgcn_sched_barrier(0);
        if (run + 64 < nruns) multiply(run + 64, w1, h1);
    }
#pragma unroll
    for (int cc = 0; cc < CW; cc++)
#pragma unroll
        for (int r = 0; r < M; r++) {
            const float v = wave_sum(acc[cc][r]);
            if (lane == 0 && col0 + cc < n) c[(uint64_t)r * n + col0 + cc] = v;
        }
}

template <int M>
static int launch_q8_rows(const float* a, const uint32_t* b, float* c, uint32_t k, uint32_t n, uint32_t bs,
                          uint32_t stride, uint32_t blocks_per_col, uint32_t kpad, hipStream_t s) {
    const uint32_t runs_per_block = bs / 16;
    const uint32_t run_magic = runs_per_block == 1 ? 0u : (uint32_t)((0x100000000ull + runs_per_block - 1) / runs_per_block);
    if (blocks_per_col == 1)
        hipLaunchKernelGGL((matmul_q8_rows_kernel<M, true>), dim3(ceil_div(n, 32)), dim3(512), (size_t)M * kpad * sizeof(float), s,
                           a, b, c, k, n, stride, blocks_per_col, kpad, runs_per_block, run_magic);
    else
        hipLaunchKernelGGL((matmul_q8_rows_kernel<M, false>), dim3(ceil_div(n, 32)), dim3(512), (size_t)M * kpad * sizeof(float), s,
                           a, b, c, k, n, stride, blocks_per_col, kpad, runs_per_block, run_magic);
    return check_launch("matmul_q8_rows_kernel");
}

// Dequantize into the tensor's own [K, N] order: the buffer holds the transposed tensor ([N, K]
// flattened, blocks of bs consecutive elements), so out[kk, col] = value at flat index col * k + kk.
// 128 k x 32 columns per workgroup through LDS: words are read along k, rows written along n.
__global__ __launch_bounds__(256) void q8_dequantize_kn_kernel(const uint32_t* __restrict__ in, float* __restrict__ out,
                                                               uint32_t k, uint32_t n, uint32_t bs, uint32_t stride) {
    __shared__ float t[32][129];
    const uint32_t tx = threadIdx.x % 32, ty = threadIdx.x / 32;
    const uint32_t k0 = blockIdx.x * 128, c0 = blockIdx.y * 32;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t cc = ty + 8 * i, col = c0 + cc;
#pragma unroll
        for (int e = 0; e < 4; e++) {                         // element by element: col * k + kk need not be a multiple of 4
            const uint32_t kk = k0 + 4 * tx + e;
            float v = 0.0f;
            if (col < n && kk < k) {
                const uint64_t idx = (uint64_t)col * k + kk;
                const uint32_t block = (uint32_t)(idx / bs), pos = (uint32_t)(idx % bs);
                const uint32_t* ib = in + (uint64_t)block * stride;
                const int q = (int)(int8_t)((ib[1 + pos / 4] >> (8 * (pos % 4))) & 0xFFu);
                v = __fmul_rn((float)q, header_scale(ib[0]));
            }
            t[cc][4 * tx + e] = v;
        }
    }
    __syncthreads();
    for (uint32_t r = ty; r < 128; r += 8) {
        const uint32_t kk = k0 + r, col = c0 + tx;
        if (kk < k && col < n) out[(uint64_t)kk * n + col] = t[tx][r];
    }
}

// ---- batches on the matrix cores (one block per column, i.e. per-output-channel scales) ------
// f32 activations cannot go into the int8 MFMA directly, but signed 7-bit digits can:
//   x = (p0 + 128 p1 + 128^2 p2 + 128^3 p3) / f,  f a power of two with |x f| < 2^27 for the row,
// so x . q = sum_p (p_p . q) 128^p / f, each p_p . q an exact i8 x i8 -> i32 product.  The four
// digit planes are stacked as 4 m rows with row scales 128^p / f, the weights are copied out of
// the block format once per call (dense int8 [n, k] + the header scales), the W8A8 kernel does
// the rest and the four row blocks are added.  The activations keep 28 bits below the largest
// magnitude of their row: with three planes (21 bits) a row with one entry 3e4 times the others
// missed the tolerance tenfold, with four the error stays below that of an f32 accumulation.
constexpr int kQ8Planes = 4;

// largest magnitude of a row as bits (orders like the floats, and a NaN sorts above infinity).  Rows of
// up to 8192 elements stay in registers between the two passes: all loads of a thread are in flight at
// once instead of one trip to memory per 256 elements, and the row is read once.
constexpr int kSplitCache = 8;                                 // float4 per thread: 256 x 8 x 4 = 8192 elements

__device__ __forceinline__ uint32_t q8_row_amax(const float* __restrict__ ar, uint32_t k, uint32_t tid, bool cached,
                                                float4 (&v)[kSplitCache], uint32_t* red) {
    uint32_t amax = 0;
    if (cached) {
#pragma unroll
        for (int i = 0; i < kSplitCache; i++) {
            const uint32_t j = 4 * tid + 1024 * i;
            v[i] = j < k ? *reinterpret_cast<const float4*>(ar + j) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int i = 0; i < kSplitCache; i++)
            amax = max(max(amax, max(__float_as_uint(v[i].x) & 0x7FFFFFFFu, __float_as_uint(v[i].y) & 0x7FFFFFFFu)),
                       max(__float_as_uint(v[i].z) & 0x7FFFFFFFu, __float_as_uint(v[i].w) & 0x7FFFFFFFu));
    } else {
        for (uint32_t j = 4 * tid; j < k; j += 1024) {
            const float4 t = *reinterpret_cast<const float4*>(ar + j);
            amax = max(max(amax, max(__float_as_uint(t.x) & 0x7FFFFFFFu, __float_as_uint(t.y) & 0x7FFFFFFFu)),
                       max(__float_as_uint(t.z) & 0x7FFFFFFFu, __float_as_uint(t.w) & 0x7FFFFFFFu));
        }
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    return max(max(red[0], red[1]), max(red[2], red[3]));
}

// INTERLEAVED: plane p of row r is row 4 r + p of `planes` and sxp[4 r + p] its weight (the order the plane-adding
// epilogue of the int8 GEMM wants); otherwise the planes are stacked, row p m + r and sxp[p m + r].
template <bool INTERLEAVED>
__global__ __launch_bounds__(256) void q8_split_rows_kernel(const float* __restrict__ a, int8_t* __restrict__ planes,
                                                            float* __restrict__ sxp, uint32_t m, uint32_t k) {
    __shared__ uint32_t red[4];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const float* ar = a + (uint64_t)row * k;                   // k % 4 == 0
    const bool cached = k <= 1024u * kSplitCache;
    float4 cache[kSplitCache];
    const uint32_t amax = q8_row_amax(ar, k, tid, cached, cache, red);
    const uint32_t ebits = amax >> 23;                         // amax = a 2^(ebits-127), 1 <= a < 2
    float f = __uint_as_float((280u - ebits) << 23);           // 2^(153 - ebits): |x f| < 2^27
    uint32_t inv_bits = ebits - 26u;                           // 1 / f = 2^(ebits - 153), biased
    if (ebits < 27) { f = 0.0f; inv_bits = 0; }                // zero or below 2^-100: contributes nothing
    if (tid < kQ8Planes) {
        float s = inv_bits ? __uint_as_float((inv_bits + 7u * tid) << 23) : 0.0f;
        if (ebits == 255) s = __uint_as_float(0x7FC00000u);    // inf / nan in the row: poison it
        sxp[INTERLEAVED ? kQ8Planes * row + tid : tid * m + row] = s;
    }
    const bool poisoned = ebits == 255;
    auto emit = [&](uint32_t j, const float4& v) {
        const float xv[4] = {v.x, v.y, v.z, v.w};
        uint32_t word[kQ8Planes] = {};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int rest = poisoned ? 0 : (int)rintf(xv[e] * f);   // exact: f is a power of two, |x f| < 2^27
#pragma unroll
            for (int p = 0; p < kQ8Planes; p++) {
                const int digit = p + 1 < kQ8Planes ? ((rest + 64) & 127) - 64 : rest;   // the last one: -64 .. 64
                rest = (rest - digit) >> 7;
                word[p] |= (uint32_t)(digit & 0xFF) << (8 * e);
            }
        }
#pragma unroll
        for (int p = 0; p < kQ8Planes; p++)
            *reinterpret_cast<uint32_t*>(planes + (INTERLEAVED ? (uint64_t)kQ8Planes * row + p : (uint64_t)p * m + row) * k + j) =
                word[p];
    };
    if (cached) {
#pragma unroll
        for (int i = 0; i < kSplitCache; i++) {
            const uint32_t j = 4 * tid + 1024 * i;
            if (j < k) emit(j, cache[i]);
        }
    } else {
        for (uint32_t j = 4 * tid; j < k; j += 1024) emit(j, *reinterpret_cast<const float4*>(ar + j));
    }
}

// Q8 buffer with one block per column -> dense int8 [n, k] and the n header scales
__global__ __launch_bounds__(256) void q8_unpack_channels_kernel(const uint32_t* __restrict__ b,
                                                                 uint32_t* __restrict__ wq, float* __restrict__ sw,
                                                                 uint32_t kwords, uint32_t stride) {
    const uint32_t w = blockIdx.x * 256 + threadIdx.x, col = blockIdx.y;
    if (w >= kwords) return;
    const uint32_t* bb = b + (uint64_t)col * stride;
    wq[(uint64_t)col * kwords + w] = bb[1 + w];
    if (w == 0) sw[col] = header_scale(bb[0]);
}

// c[r, :] = sum over the planes of yp[p m + r, :], smallest plane first
__global__ __launch_bounds__(256) void q8_add_planes_kernel(const float* __restrict__ yp, float* __restrict__ c,
                                                            uint64_t count) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    float v = yp[i];
#pragma unroll
    for (int p = 1; p < kQ8Planes; p++) v += yp[p * count + i];
    c[i] = v;
}

static size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

// c = a x (wq, sw): wq dense int8 [n, k], sw [n].  The planes are added in the GEMM's epilogue where the shape
// has such a kernel (large ones), by a pass over the four partial outputs otherwise; both give the same bits.
// `ws` holds q8_dense_workspace(m, k, n) bytes, the int8 GEMM's own partial sums behind `own` of them.
struct Q8DenseWs { size_t planes, sx, y, own, total; bool fold; };

static Q8DenseWs q8_dense_workspace(uint32_t m, uint32_t k, uint32_t n) {
    Q8DenseWs w;
    w.fold = i8_gemm_fold4_supported(kQ8Planes * m, k, n);
    w.planes = align256((size_t)kQ8Planes * m * k);
    w.sx = align256((size_t)kQ8Planes * m * sizeof(float));
    w.y = w.fold ? 0 : align256((size_t)kQ8Planes * m * n * sizeof(float));
    w.own = w.planes + w.sx + w.y;
    w.total = w.own + (w.fold ? 0 : i8_gemm_workspace_need(kQ8Planes * m, k, n));
    return w;
}

static int matmul_q8_planes(const float* a, const int8_t* wq, const float* sw, float* c, uint32_t m, uint32_t k,
                            uint32_t n, const Q8DenseWs& w, uint8_t* base, hipStream_t s) {
    int8_t* planes = reinterpret_cast<int8_t*>(base);
    float* sxp = reinterpret_cast<float*>(base + w.planes);
    if (w.fold) {
        hipLaunchKernelGGL(q8_split_rows_kernel<true>, dim3(m), dim3(256), 0, s, a, planes, sxp, m, k);
        if (int rc = check_launch("q8_split_rows_kernel")) return rc;
        return i8_gemm_fold4(planes, wq, sxp, sw, nullptr, c, kQ8Planes * m, k, n, s);
    }
    float* yp = reinterpret_cast<float*>(base + w.planes + w.sx);
    hipLaunchKernelGGL(q8_split_rows_kernel<false>, dim3(m), dim3(256), 0, s, a, planes, sxp, m, k);
    if (int rc = check_launch("q8_split_rows_kernel")) return rc;
    if (int rc = rumus_hip_i8_gemm(planes, wq, sxp, sw, nullptr, nullptr, yp, kQ8Planes * m, k, n, s)) return rc;
    const uint64_t count = (uint64_t)m * n;
    hipLaunchKernelGGL(q8_add_planes_kernel, dim3((uint32_t)((count + 255) / 256)), dim3(256), 0, s, yp, c, count);
    return check_launch("q8_add_planes_kernel");
}

static int matmul_q8_mfma(const float* a, const uint32_t* b, float* c, uint32_t m, uint32_t k, uint32_t n,
                          uint32_t stride, hipStream_t s) {
    RUMUS_REQUIRE((uint64_t)kQ8Planes * m < (1ull << 31), "matmul_q8: m %u is beyond the grid limit", m);
    const Q8DenseWs w = q8_dense_workspace(m, k, n);
    const size_t wq_bytes = align256((size_t)n * k), sw_bytes = align256((size_t)n * sizeof(float));
    void* ws = nullptr;
    WorkspaceLease lease;                                    // until the last kernel of this call is queued
    if (int rc = workspace_get(s, wq_bytes + sw_bytes + w.total, &ws, lease)) return rc;
    WorkspaceNest nest(wq_bytes + sw_bytes + w.own);
    uint8_t* base = static_cast<uint8_t*>(ws);
    int8_t* wq = reinterpret_cast<int8_t*>(base);
    float* sw = reinterpret_cast<float*>(base + wq_bytes);
    hipLaunchKernelGGL(q8_unpack_channels_kernel, dim3(ceil_div(k / 4, 256), n), dim3(256), 0, s, b,
                       reinterpret_cast<uint32_t*>(wq), sw, k / 4, stride);
    if (int rc = check_launch("q8_unpack_channels_kernel")) return rc;
    return matmul_q8_planes(a, wq, sw, c, m, k, n, w, base + wq_bytes + sw_bytes, s);
}

// Activations for the f16 variant of the block-scale kernel: x f = hi + lo, two f16 planes [2][m][k]
// (22 bits of every element), f a power of two per row with |x f| < 2^15; sx[row] = 1 / f.
__global__ __launch_bounds__(256) void q8_split_rows_f16_kernel(const float* __restrict__ a, _Float16* __restrict__ planes,
                                                                float* __restrict__ sx, uint32_t m, uint32_t k) {
    __shared__ uint32_t red[4];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const float* ar = a + (uint64_t)row * k;                   // k % 4 == 0
    const bool cached = k <= 1024u * kSplitCache;
    float4 cache[kSplitCache];
    const uint32_t amax = q8_row_amax(ar, k, tid, cached, cache, red);
    const uint32_t ebits = amax >> 23;                         // amax = a 2^(ebits-127), 1 <= a < 2
    const bool poisoned = ebits == 255;                        // inf / nan in the row
    const bool nothing = ebits < 15;                           // zero or below 2^-112: contributes nothing
    const float f = (poisoned || nothing) ? 0.0f : __uint_as_float((268u - ebits) << 23);   // 2^(141 - ebits)
    if (tid == 0)
        sx[row] = poisoned ? __uint_as_float(0x7FC00000u) : nothing ? 0.0f : __uint_as_float((ebits - 14u) << 23);
    _Float16* hi = planes + (uint64_t)row * k;
    _Float16* lo = planes + ((uint64_t)m + row) * k;
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    auto emit = [&](uint32_t j, const float4& v) {
        const float xv[4] = {v.x, v.y, v.z, v.w};
        _Float16 h[4], l[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float t = poisoned ? 0.0f : xv[e] * f;       // exact: f is a power of two
            h[e] = (_Float16)t;
            l[e] = (_Float16)(t - (float)h[e]);
        }
        *reinterpret_cast<v4h*>(hi + j) = v4h{h[0], h[1], h[2], h[3]};
        *reinterpret_cast<v4h*>(lo + j) = v4h{l[0], l[1], l[2], l[3]};
    };
    if (cached) {
#pragma unroll
        for (int i = 0; i < kSplitCache; i++) {
            const uint32_t j = 4 * tid + 1024 * i;
            if (j < k) emit(j, cache[i]);
        }
    } else {
        for (uint32_t j = 4 * tid; j < k; j += 1024) emit(j, *reinterpret_cast<const float4*>(ar + j));
    }
}

// q8_gemm.hip: the same digit planes against blocks smaller than a column
int q8_gemm_blocks(const int8_t* planes, const float* sx, const uint32_t* b, float* c, uint32_t m, uint32_t k,
                   uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, float* part, uint32_t max_shares,
                   hipStream_t s);

int q8_gemm_blocks_f16(const _Float16* planes, const float* sx, const uint32_t* b, float* c, uint32_t m, uint32_t k,
                       uint32_t n, uint32_t bs, uint32_t stride, uint32_t bpc, float* part, uint32_t max_shares,
                       hipStream_t s);

static int matmul_q8_mfma_blocks(const float* a, const uint32_t* b, float* c, uint32_t m, uint32_t k, uint32_t n,
                                 uint32_t bs, uint32_t stride, uint32_t bpc, hipStream_t s) {
    const size_t planes_bytes = align256((size_t)kQ8Planes * m * k), sx_bytes = align256((size_t)kQ8Planes * m * sizeof(float));
    // few rows: room for the partial results of up to 8 shares of K
    const uint32_t max_shares = (uint64_t)m * n <= (1u << 22) ? 8 : 0;
    void* ws = nullptr;
    WorkspaceLease lease;                                    // until the last kernel of this call is queued
    if (int rc = workspace_get(s, planes_bytes + sx_bytes + (size_t)max_shares * m * n * sizeof(float), &ws, lease)) return rc;
    int8_t* planes = static_cast<int8_t*>(ws);
    float* sxp = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + planes_bytes);
    float* part = max_shares ? reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + planes_bytes + sx_bytes) : nullptr;
    // small blocks (a fold at every or every other 32 k) and larger batches: two f16 planes; otherwise four
    // exact digit planes on the int8 matrix cores
    if (bs <= 64 || m > 64) {
        _Float16* halves = reinterpret_cast<_Float16*>(ws);    // the same 4 m k bytes
        hipLaunchKernelGGL(q8_split_rows_f16_kernel, dim3(m), dim3(256), 0, s, a, halves, sxp, m, k);
        if (int rc = check_launch("q8_split_rows_f16_kernel")) return rc;
        return q8_gemm_blocks_f16(halves, sxp, b, c, m, k, n, bs, stride, bpc, part, max_shares, s);
    }
    hipLaunchKernelGGL(q8_split_rows_kernel<false>, dim3(m), dim3(256), 0, s, a, planes, sxp, m, k);
    if (int rc = check_launch("q8_split_rows_kernel")) return rc;
    return q8_gemm_blocks(planes, sxp, b, c, m, k, n, bs, stride, bpc, part, max_shares, s);   // sxp[0 .. m): the rows' 1 / f
}

// Any block_size % 4 == 0: one thread per output, the reference's own loop.
__global__ __launch_bounds__(256) void matmul_q8_naive_kernel(
    const float* __restrict__ a, const uint32_t* __restrict__ b, float* __restrict__ c,
    uint32_t m, uint32_t k, uint32_t n, uint32_t bs, uint32_t stride, uint32_t blocks_per_col) {
    const uint32_t col = blockIdx.x * 64 + threadIdx.x % 64;
    const uint32_t row = blockIdx.y * 4 + threadIdx.x / 64;
    if (row >= m || col >= n) return;
    float sum = 0.0f;
    uint32_t k_off = 0;
    for (uint32_t blk = 0; blk < blocks_per_col; blk++) {
        const uint32_t* bb = b + ((uint64_t)col * blocks_per_col + blk) * stride;
        const float sc = header_scale(bb[0]);
        const uint32_t len = min(bs, k - k_off);
        for (uint32_t r = 0; r < len; r++) {
            int q = (int)(int8_t)((bb[1 + r / 4] >> (8 * (r % 4))) & 0xFFu);
            sum = __fadd_rn(sum, __fmul_rn(__fmul_rn(a[(uint64_t)row * k + k_off + r], (float)q), sc));
        }
        k_off += bs;
    }
    c[(uint64_t)row * n + col] = sum;
}

// bias.wgsl:18-25, four columns per thread when n % 4 == 0.
__global__ __launch_bounds__(256) void add_bias_kernel(const float* __restrict__ mat,
                                                       const float* __restrict__ bias,
                                                       float* __restrict__ out, uint64_t total,
                                                       uint32_t n) {
    uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    out[i] = __fadd_rn(mat[i], bias[i % n]);
}

// 32x32 tile transpose through LDS.
__global__ __launch_bounds__(256) void transpose_kernel(const float* __restrict__ in,
                                                        float* __restrict__ out, uint32_t rows,
                                                        uint32_t cols) {
    __shared__ float t[32][33];
    const uint32_t tx = threadIdx.x % 32, ty = threadIdx.x / 32;  // 32 x 8
    const uint32_t r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        uint32_t r = r0 + ty + i, cc = c0 + tx;
        if (r < rows && cc < cols) t[ty + i][tx] = in[(uint64_t)r * cols + cc];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        uint32_t cc = c0 + ty + i, r = r0 + tx;
        if (r < rows && cc < cols) out[(uint64_t)cc * rows + r] = t[tx][ty + i];
    }
}

// 64x64 tile, 128-bit accesses on both sides (rows % 4 == 0, cols % 4 == 0, 16-byte aligned buffers).
// Thread (q = tid % 16, p = tid / 16): reads float4 at row p + 16 i, columns 4 q .. 4 q + 3; writes the
// float4 of output row (= input column) p + 16 i, output columns (= input rows) 4 q .. 4 q + 3, which it
// gathers from LDS rows of 65 floats: bank 4 q + e + p + 16 i (mod 64), distinct across a wave.
__global__ __launch_bounds__(256) void transpose64_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                          uint32_t rows, uint32_t cols) {
    __shared__ float t[64][65];
    const uint32_t q = threadIdx.x % 16, p = threadIdx.x / 16;
    const uint32_t r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t r = r0 + p + 16 * i, cc = c0 + 4 * q;
        float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (r < rows && cc < cols) v = *reinterpret_cast<const float4*>(in + (uint64_t)r * cols + cc);
        float* d = &t[p + 16 * i][4 * q];
        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t cc = c0 + p + 16 * i, r = r0 + 4 * q;
        if (cc < cols && r < rows)
            *reinterpret_cast<float4*>(out + (uint64_t)cc * rows + r) =
                make_float4(t[4 * q][p + 16 * i], t[4 * q + 1][p + 16 * i], t[4 * q + 2][p + 16 * i], t[4 * q + 3][p + 16 * i]);
    }
}

}  // namespace rumus

using namespace rumus;

extern "C" {

uint64_t rumus_hip_q8_buf_size(uint64_t numel, uint32_t block_size) {
    if (block_size == 0) return 0;
    uint64_t num_blocks = (numel + block_size - 1) / block_size;
    return (num_blocks * (4 + (uint64_t)block_size) + 3) & ~(uint64_t)3;
}

int rumus_hip_q8_quantize(const float* in, uint32_t* out, uint32_t numel, uint32_t block_size,
                          rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(block_size > 0 && block_size % 4 == 0,
                  "quantize: block_size must be > 0 and divisible by 4 (got %u)", block_size);
    RUMUS_REQUIRE(numel == 0 || (in && out), "quantize: null buffer");
    if (numel == 0) return RUMUS_HIP_OK;
    uint32_t num_blocks = ceil_div(numel, block_size);
    uint32_t stride = (4 + block_size + 3) / 4;
    hipStream_t s = as_stream(stream);
    if (block_size <= 32)
        hipLaunchKernelGGL(q8_quantize_small_kernel<8>, dim3(ceil_div(num_blocks, 32)), dim3(256), 0, s, in, out, numel,
                           block_size, num_blocks, stride);
    else if (block_size <= 64)
        hipLaunchKernelGGL(q8_quantize_small_kernel<16>, dim3(ceil_div(num_blocks, 16)), dim3(256), 0, s, in, out, numel,
                           block_size, num_blocks, stride);
    else if (block_size <= 128)
        hipLaunchKernelGGL(q8_quantize_small_kernel<32>, dim3(ceil_div(num_blocks, 8)), dim3(256), 0, s, in, out, numel,
                           block_size, num_blocks, stride);
    else if (block_size <= 256)
        hipLaunchKernelGGL(q8_quantize_small_kernel<64>, dim3(ceil_div(num_blocks, 4)), dim3(256), 0, s, in, out, numel,
                           block_size, num_blocks, stride);
    else
        hipLaunchKernelGGL(q8_quantize_kernel, dim3(ceil_div(num_blocks, 4)), dim3(256), 0, s, in, out, numel,
                           block_size, num_blocks, stride);
    return check_launch("q8_quantize_kernel");
}

int rumus_hip_q8_dequantize(const uint32_t* in, float* out, uint32_t numel, uint32_t block_size,
                            rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(block_size > 0 && block_size % 4 == 0,
                  "dequantize: block_size must be > 0 and divisible by 4 (got %u)", block_size);
    RUMUS_REQUIRE(numel == 0 || (in && out), "dequantize: null buffer");
    if (numel == 0) return RUMUS_HIP_OK;
    uint32_t stride = (4 + block_size + 3) / 4;
    uint32_t words = numel / 4 + (numel % 4 != 0);
    hipLaunchKernelGGL(q8_dequantize_kernel, dim3(ceil_div(words, 256)), dim3(256), 0,
                       as_stream(stream), in, out, numel, block_size, stride);
    return check_launch("q8_dequantize_kernel");
}

int rumus_hip_q8_dequantize_kn(const uint32_t* in, float* out, uint32_t k, uint32_t n, uint32_t block_size,
                               rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(block_size > 0 && block_size % 4 == 0,
                  "dequantize: block_size must be > 0 and divisible by 4 (got %u)", block_size);
    RUMUS_REQUIRE(k == 0 || n == 0 || (in && out), "dequantize: null buffer");
    if (k == 0 || n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(n <= 65535u * 32u, "dequantize: n %u is beyond the grid limit", n);
    const uint32_t stride = (4 + block_size + 3) / 4;
    hipLaunchKernelGGL(q8_dequantize_kn_kernel, dim3(ceil_div(k, 128), ceil_div(n, 32)), dim3(256), 0, as_stream(stream),
                       in, out, k, n, block_size, stride);
    return check_launch("q8_dequantize_kn_kernel");
}

int rumus_hip_matmul_q8(const float* a, const uint32_t* b, float* c, uint32_t m, uint32_t k,
                        uint32_t n, uint32_t block_size, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(block_size > 0 && block_size % 4 == 0,
                  "matmul_q8: block_size must be > 0 and divisible by 4 (got %u)", block_size);
    RUMUS_REQUIRE(m == 0 || n == 0 || (a && b && c), "matmul_q8: null buffer");
    if (m == 0 || n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(k > 0, "matmul_q8: k must be > 0");
    uint32_t blocks_per_col = ceil_div(k, block_size);
    uint32_t stride = (4 + block_size + 3) / 4;
    // Batches go to the matrix cores.  Measured at 4096 x 11008 (us, whole call):
    //                                                 rows    5..32    128    512    2048
    //   block-scale kernels, 32-element blocks (f16)          34..35     66    174     604   (few-rows kernel: 7.7 per row,
    //   block-scale kernels, 128-element blocks               33..36     60    151     545    LDS-tiled kernel: 15 ms at 2048)
    //   block-scale kernels, one block per column             29..33     60    151
    //   W8A8 kernel on a dense copy of the weights                62     83    148     526   (one block per column only)
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(c)) & 15) == 0;
    const bool block_kernel = block_size % 32 == 0 && k % block_size == 0 && m >= 5 && aligned &&
                              (uint64_t)k * block_size < (1ull << 32) && (uint64_t)kQ8Planes * m * k < (1ull << 40);
    if (blocks_per_col == 1 && k % 16 == 0 && m >= (block_kernel ? 384u : 8u) && n <= 65535 && aligned)
        return matmul_q8_mfma(a, b, c, m, k, n, stride, as_stream(stream));
    if (block_kernel)
        return matmul_q8_mfma_blocks(a, b, c, m, k, n, block_size, stride, blocks_per_col, as_stream(stream));
    const uint32_t kpad = (k + 15) & ~15u;
    if (block_size % 16 == 0 && kpad <= 16384) {
        // rows in groups whose x fits 64 KB of LDS: 4 rows at k = 4096, 1 at k = 11008, all 8 up to k = 2048
        const uint32_t group = min(8u, 16384u / kpad);
        hipStream_t s = as_stream(stream);
        for (uint32_t r0 = 0; r0 < m; r0 += group) {
            const uint32_t rows = min(group, m - r0);
            const float* ar = a + (uint64_t)r0 * k;
            float* cr = c + (uint64_t)r0 * n;
            int rc;
            switch (rows) {
                case 1: rc = launch_q8_rows<1>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
                case 2: rc = launch_q8_rows<2>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
                case 3: rc = launch_q8_rows<3>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
                case 4: rc = launch_q8_rows<4>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
                case 5: rc = launch_q8_rows<5>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
                case 6: rc = launch_q8_rows<6>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
                case 7: rc = launch_q8_rows<7>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
                default: rc = launch_q8_rows<8>(ar, b, cr, k, n, block_size, stride, blocks_per_col, kpad, s); break;
            }
            if (rc) return rc;
        }
        return RUMUS_HIP_OK;
    }
    if (block_size % 16 == 0) {
        dim3 grid(ceil_div(n, kQ8Tile), ceil_div(m, kQ8Tile));
        hipLaunchKernelGGL(matmul_q8_tiled_kernel, grid, dim3(256), 0, as_stream(stream), a, b, c,
                           m, k, n, block_size, stride, blocks_per_col);
        return check_launch("matmul_q8_tiled_kernel");
    }
    dim3 grid(ceil_div(n, 64), ceil_div(m, 4));
    hipLaunchKernelGGL(matmul_q8_naive_kernel, grid, dim3(256), 0, as_stream(stream), a, b, c, m,
                       k, n, block_size, stride, blocks_per_col);
    return check_launch("matmul_q8_naive_kernel");
}

int rumus_hip_q8_dense_layout(const uint32_t* b_q8, uint32_t k, uint32_t n, uint32_t block_size, int8_t* wq,
                              float* sw, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(n == 0 || (b_q8 && wq && sw), "q8_dense_layout: null buffer");
    RUMUS_REQUIRE(block_size > 0 && block_size % 4 == 0,
                  "q8_dense_layout: block_size must be > 0 and divisible by 4 (got %u)", block_size);
    RUMUS_REQUIRE(k > 0 && k % 4 == 0 && block_size >= k,
                  "q8_dense_layout: one block per column wanted (k %u, a multiple of 4, block_size %u >= k)", k, block_size);
    RUMUS_REQUIRE((reinterpret_cast<uintptr_t>(wq) & 3) == 0, "q8_dense_layout: wq must be 4-byte aligned");
    if (n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(n <= 65535, "q8_dense_layout: n %u is beyond the grid limit", n);
    hipLaunchKernelGGL(q8_unpack_channels_kernel, dim3(ceil_div(k / 4, 256), n), dim3(256), 0, as_stream(stream), b_q8,
                       reinterpret_cast<uint32_t*>(wq), sw, k / 4, (4 + block_size + 3) / 4);
    return check_launch("q8_unpack_channels_kernel");
}

int rumus_hip_matmul_q8_dense(const float* a, const int8_t* wq, const float* sw, float* c, uint32_t m, uint32_t k,
                              uint32_t n, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(m == 0 || n == 0 || (a && wq && sw && c), "matmul_q8_dense: null buffer");
    if (m == 0 || n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(k > 0 && k % 16 == 0, "matmul_q8_dense: k must be a positive multiple of 16 (got %u)", k);
    RUMUS_REQUIRE(((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(c) | reinterpret_cast<uintptr_t>(wq)) & 15) == 0,
                  "matmul_q8_dense: a, wq and c must be 16-byte aligned");
    RUMUS_REQUIRE((uint64_t)kQ8Planes * m < (1ull << 31), "matmul_q8_dense: m %u is beyond the grid limit", m);
    hipStream_t s = as_stream(stream);
    const Q8DenseWs w = q8_dense_workspace(m, k, n);
    void* ws = nullptr;
    WorkspaceLease lease;                                    // until the last kernel of this call is queued
    if (int rc = workspace_get(s, w.total, &ws, lease)) return rc;
    WorkspaceNest nest(w.own);
    return matmul_q8_planes(a, wq, sw, c, m, k, n, w, static_cast<uint8_t*>(ws), s);
}

int rumus_hip_add_bias(const float* mat, const float* bias, float* out, uint32_t m, uint32_t n,
                       rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(m == 0 || n == 0 || (mat && bias && out), "add_bias: null buffer");
    uint64_t total = (uint64_t)m * n;
    if (total == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(add_bias_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0,
                       as_stream(stream), mat, bias, out, total, n);
    return check_launch("add_bias_kernel");
}

int rumus_hip_transpose_f32(const float* in, float* out, uint32_t rows, uint32_t cols,
                            rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(rows == 0 || cols == 0 || (in && out), "transpose: null buffer");
    if (rows == 0 || cols == 0) return RUMUS_HIP_OK;
    if (rows % 4 == 0 && cols % 4 == 0 &&
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        RUMUS_REQUIRE(ceil_div(rows, 64) <= 65535, "transpose: rows %u beyond the grid limit", rows);
        hipLaunchKernelGGL(transpose64_kernel, dim3(ceil_div(cols, 64), ceil_div(rows, 64)), dim3(256), 0,
                           as_stream(stream), in, out, rows, cols);
        return check_launch("transpose64_kernel");
    }
    dim3 grid(ceil_div(cols, 32), ceil_div(rows, 32));
    hipLaunchKernelGGL(transpose_kernel, grid, dim3(256), 0, as_stream(stream), in, out, rows, cols);
    return check_launch("transpose_kernel");
}

}  // extern "C"
