// The f32 operators that sit between the quantized projections of a decoder
// block: RMSNorm, SwiGLU, residual add and scaled-dot-product attention
// (reference analogue for attention: flash_attention, rumus/src/tensor/ops.rs:
// 2685-2743 with shaders/flash_attn.wgsl; the others have no counterpart in the
// reference).  All of them are bandwidth- or latency-bound helpers around the
// INT4 / INT8 matmuls, written so that no permute or copy is needed between a
// projection's [tokens, heads*dim] output and the attention operands: every
// attention operand carries its own (batch, head, row) strides.
#include "common.h"

namespace rumus {

// ---- RMSNorm: y[r,:] = x[r,:] * rsqrt(mean(x[r,:]^2) + eps) * weight ---------------------
// One workgroup per row.  VEC: dim % 4 == 0, dim <= 8192 and 16-byte aligned rows: the row is
// read once with up to eight 128-bit loads per thread, all issued before the first use (a
// single decode row is pure latency otherwise: sixteen dependent 4-byte loads per thread).
// ADD: the row normalised is x + delta (the residual stream after a projection); the sum is
// written to `sum` as well, so that the separate addition and its launch disappear.
template <bool VEC, bool ADD>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* x, const float* delta,
                                                      const float* __restrict__ w, float* sum,
                                                      float* __restrict__ y, uint32_t dim, float eps) {
    // `sum` may be x or delta (the residual stream updated in place): every thread reads its own
    // elements before it writes them
    __shared__ float red[4];
    const uint64_t base = (uint64_t)blockIdx.x * dim;
    const float* xr = x + base;
    const float* dr = ADD ? delta + base : nullptr;
    float* sr = ADD ? sum + base : nullptr;
    float* yr = y + base;
    float4 v[8], wv[8];
    float ss = 0.0f;
    if (VEC) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t i = (j * 256 + threadIdx.x) * 4;
            const bool in = i < dim;
            v[j] = *reinterpret_cast<const float4*>(xr + (in ? i : 0));
            wv[j] = *reinterpret_cast<const float4*>(w + (in ? i : 0));
            if (ADD) {
                const float4 d = *reinterpret_cast<const float4*>(dr + (in ? i : 0));
                v[j] = make_float4(v[j].x + d.x, v[j].y + d.y, v[j].z + d.z, v[j].w + d.w);
            }
            if (!in) v[j] = make_float4(0, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            ss = fmaf(v[j].x, v[j].x, fmaf(v[j].y, v[j].y, fmaf(v[j].z, v[j].z, fmaf(v[j].w, v[j].w, ss))));
            const uint32_t i = (j * 256 + threadIdx.x) * 4;
            if (ADD && i < dim) *reinterpret_cast<float4*>(sr + i) = v[j];
        }
    } else {
        for (uint32_t i = threadIdx.x; i < dim; i += 256) {
            float t = xr[i];
            if (ADD) { t += dr[i]; sr[i] = t; }
            ss = fmaf(t, t, ss);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = 1.0f / sqrtf(total / (float)dim + eps);
    if (VEC) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t i = (j * 256 + threadIdx.x) * 4;
            if (i < dim)
                *reinterpret_cast<float4*>(yr + i) = make_float4(v[j].x * inv * wv[j].x, v[j].y * inv * wv[j].y,
                                                                 v[j].z * inv * wv[j].z, v[j].w * inv * wv[j].w);
        }
    } else {
        const float* src = ADD ? sr : xr;  // each thread re-reads the elements it wrote itself
        for (uint32_t i = threadIdx.x; i < dim; i += 256) yr[i] = src[i] * inv * w[i];
    }
}

// ---- SwiGLU: out = silu(gate) * up, silu(t) = t / (1 + exp(-t)) ----------------------------
__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                     float* __restrict__ out, uint64_t numel) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= numel) return;
    const float g = gate[i];
    out[i] = g / (1.0f + expf(-g)) * up[i];
}

// gate and up as the two halves of one [rows, 2n] matrix (the output of a fused gate|up projection)
__global__ __launch_bounds__(256) void swiglu_rows_kernel(const float* __restrict__ gate_up, float* __restrict__ out,
                                                          uint32_t n) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= n) return;
    const float* row = gate_up + (uint64_t)blockIdx.y * 2 * n;
    const float g = row[c];
    out[(uint64_t)blockIdx.y * n + c] = g / (1.0f + expf(-g)) * row[n + c];
}

__global__ __launch_bounds__(256) void add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                  float* __restrict__ out, uint64_t numel) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < numel) out[i] = a[i] + b[i];
}

// ---- attention -------------------------------------------------------------------------
// Operand (b, h, row, :) lives at base + b*sb + h*sh + row*sr, head_dim contiguous.
struct AttnArgs {
    const float *q, *k, *v;
    float* o;
    uint64_t q_sb, q_sh, q_sr, k_sb, k_sh, k_sr, v_sb, v_sh, v_sr, o_sb, o_sh, o_sr;
    uint32_t batch, heads, q_len, kv_len;
    float scale;
    int causal;
    // decode with append (attention_decode_kernel only; null otherwise): the newest key / value, position kv_len - 1,
    // are read from the projection output instead of the cache, and the workgroup of the last slice writes them
    // into the cache (k, v above, which are writable then)
    const float* k_new = nullptr;
    const float* v_new = nullptr;
    uint64_t kn_sb = 0, kn_sh = 0, vn_sb = 0, vn_sh = 0;
};

constexpr int kHeadDim = 128;

// Prefill / general case.  Workgroup = 64 query rows of one (batch, head); 4 lanes per row,
// each holding 32 of the 128 dims of q and of the output.  K/V tiles of 32 keys go through
// LDS (every lane reads the same key, so the reads are broadcasts); online softmax per row.
// Causal: query row i sits at position kv_len - q_len + i and sees keys up to its position.
__global__ __launch_bounds__(256) void attention_rows_kernel(AttnArgs a) {
    constexpr int BC = 32;
    __shared__ __attribute__((aligned(16))) float ks[BC][kHeadDim];
    __shared__ __attribute__((aligned(16))) float vs[BC][kHeadDim];
    const uint32_t tid = threadIdx.x, part = tid & 3, r = tid >> 2;
    const uint32_t bh = blockIdx.y, b = bh / a.heads, h = bh % a.heads;
    const uint32_t row = blockIdx.x * 64 + r;
    const bool row_ok = row < a.q_len;
    const uint32_t shift = a.kv_len - a.q_len;                 // causal offset of the query rows
    const float* qp = a.q + b * a.q_sb + h * a.q_sh + (uint64_t)min(row, a.q_len - 1) * a.q_sr + part * 32;
    float q[32], acc[32];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float4 t = *reinterpret_cast<const float4*>(qp + 4 * i);
        q[4 * i] = t.x * a.scale; q[4 * i + 1] = t.y * a.scale; q[4 * i + 2] = t.z * a.scale; q[4 * i + 3] = t.w * a.scale;
    }
#pragma unroll
    for (int i = 0; i < 32; i++) acc[i] = 0.0f;
    float mrun = -INFINITY, lrun = 0.0f;
    // keys this workgroup needs: all of them, or up to the position of its last row
    const uint32_t last_row = min(blockIdx.x * 64 + 63, a.q_len - 1);
    const uint32_t kv_end = a.causal ? min(a.kv_len, last_row + shift + 1) : a.kv_len;
    const uint32_t my_end = a.causal ? min(a.kv_len, row + shift + 1) : a.kv_len;   // exclusive
    const float* kb = a.k + b * a.k_sb + h * a.k_sh;
    const float* vb = a.v + b * a.v_sb + h * a.v_sh;
    for (uint32_t j0 = 0; j0 < kv_end; j0 += BC) {
        __syncthreads();
        // 32 keys x 128 floats = 1024 float4 per tile and operand: 4 per thread
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint32_t e = tid + 256 * t, kr = e >> 5, c4 = e & 31;
            const uint32_t key = min(j0 + kr, a.kv_len - 1);
            *reinterpret_cast<float4*>(&ks[kr][4 * c4]) = *reinterpret_cast<const float4*>(kb + (uint64_t)key * a.k_sr + 4 * c4);
            *reinterpret_cast<float4*>(&vs[kr][4 * c4]) = *reinterpret_cast<const float4*>(vb + (uint64_t)key * a.v_sr + 4 * c4);
        }
        __syncthreads();
        float s[BC];
        float mtile = -INFINITY;
#pragma unroll
        for (int j = 0; j < BC; j++) {
            float d = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float4 kk = *reinterpret_cast<const float4*>(&ks[j][part * 32 + 4 * i]);
                d = fmaf(q[4 * i], kk.x, d); d = fmaf(q[4 * i + 1], kk.y, d);
                d = fmaf(q[4 * i + 2], kk.z, d); d = fmaf(q[4 * i + 3], kk.w, d);
            }
            d += __shfl_xor(d, 1);
            d += __shfl_xor(d, 2);
            s[j] = (j0 + j < my_end) ? d : -INFINITY;
            mtile = fmaxf(mtile, s[j]);
        }
        const float mnew = fmaxf(mrun, mtile);
        if (mnew == -INFINITY) continue;                       // nothing visible yet (uniform per quad)
        const float corr = expf(mrun - mnew);                  // exp(-inf) = 0 on the first visible tile
        lrun *= corr;
#pragma unroll
        for (int i = 0; i < 32; i++) acc[i] *= corr;
#pragma unroll
        for (int j = 0; j < BC; j++) {
            const float p = expf(s[j] - mnew);                 // masked keys: exp(-inf) = 0
            lrun += p;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float4 vv = *reinterpret_cast<const float4*>(&vs[j][part * 32 + 4 * i]);
                acc[4 * i] = fmaf(p, vv.x, acc[4 * i]); acc[4 * i + 1] = fmaf(p, vv.y, acc[4 * i + 1]);
                acc[4 * i + 2] = fmaf(p, vv.z, acc[4 * i + 2]); acc[4 * i + 3] = fmaf(p, vv.w, acc[4 * i + 3]);
            }
        }
        mrun = mnew;
    }
    if (!row_ok) return;
    const float inv = lrun > 0.0f ? 1.0f / lrun : 0.0f;
    float* op = a.o + b * a.o_sb + h * a.o_sh + (uint64_t)row * a.o_sr + part * 32;
#pragma unroll
    for (int i = 0; i < 8; i++)
        *reinterpret_cast<float4*>(op + 4 * i) =
            make_float4(acc[4 * i] * inv, acc[4 * i + 1] * inv, acc[4 * i + 2] * inv, acc[4 * i + 3] * inv);
}

// Prefill on the matrix cores (v_mfma_f32_32x32x2_f32, f32 in and out).  Workgroup = 128 query
// rows of one (batch, head), 32 per wave; K/V tiles of 32 keys go through LDS.  Everything is
// computed transposed so that no fragment ever has to be re-laid out:
//   S^T = K Q^T   rows = keys (A operand, from LDS), columns = queries (B operand: the wave's Q
//                 rows, kept in 64 registers per lane for the whole kernel).  In the result a
//                 lane holds one query column and 16 of the tile's 32 keys, lane ^ 32 the other
//                 16: the softmax statistics of a query need one exchange between the halves.
//   O^T += V^T P^T  rows = dims (A operand, from LDS), columns = queries.  Result register r of
//                 S^T is exactly the B operand of step r (k index = the keys that lane holds).
// The 128 dims of the S^T product are walked as d = 64 * (lane / 32) + step, so that a lane's Q
// and K fragments are contiguous floats.  LDS tiles are [32 rows][33 chunks of 16 bytes]: the
// odd row stride spreads a column of chunks (the K fragment read, one row per lane) over all
// banks, a row (the V fragment read) stays contiguous, and every address is one per-lane base
// plus a compile-time offset.
typedef float attn_v16f __attribute__((ext_vector_type(16)));

constexpr uint32_t kAttnRowChunks = 33;
__device__ __forceinline__ uint32_t attn_tile_pos(uint32_t row, uint32_t chunk) {
    return row * kAttnRowChunks + chunk;
}

__global__ __launch_bounds__(256, 2) void attention_mfma_kernel(AttnArgs a) {
    constexpr uint32_t BC = 32, BQ = 128;
    __shared__ float4 ks[BC * kAttnRowChunks];
    __shared__ float4 vs[BC * kAttnRowChunks];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t l32 = lane & 31, kb = lane >> 5;
    // grid: x = (batch, head), y = block of 128 query rows, last block first: under a causal mask
    // the late rows see the most keys, and the long workgroups should not be the last to start
    const uint32_t bh = blockIdx.x, b = bh / a.heads, h = bh % a.heads;
    const uint32_t qblock = gridDim.y - 1 - blockIdx.y;
    const uint32_t shift = a.kv_len - a.q_len;                 // causal offset of the query rows
    const uint32_t q0 = qblock * BQ + wave * 32;               // first query row of this wave
    const uint32_t qrow = q0 + l32;                            // this lane's query
    const bool wave_live = q0 < a.q_len;

    // Q fragment, scaled by scale * log2(e) (the softmax runs on exp2): qf[s] = Q[qrow][64*kb + s]
    float qf[64];
    {
        const float* qp = a.q + b * a.q_sb + h * a.q_sh + (uint64_t)min(qrow, a.q_len - 1) * a.q_sr + 64 * kb;
        const float qs = a.scale * 1.44269504088896f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float4 t = *reinterpret_cast<const float4*>(qp + 4 * i);
            qf[4 * i] = t.x * qs; qf[4 * i + 1] = t.y * qs; qf[4 * i + 2] = t.z * qs; qf[4 * i + 3] = t.w * qs;
        }
    }
    attn_v16f oacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[dt][r] = 0.0f;
    constexpr float kMasked = -1e30f;                          // finite: exp2 of differences stays defined
    float mrun = kMasked, lrun = 0.0f;

    // keys the workgroup, this wave and this lane's query need (exclusive ends)
    const uint32_t wg_last = min(qblock * BQ + BQ - 1, a.q_len - 1);
    const uint32_t kv_end = a.causal ? min(a.kv_len, wg_last + shift + 1) : a.kv_len;
    const uint32_t wave_end = a.causal ? min(a.kv_len, min(q0 + 31, a.q_len - 1) + shift + 1) : a.kv_len;
    const uint32_t my_end = a.causal ? min(a.kv_len, qrow + shift + 1) : a.kv_len;

    // staging: a tile is 1024 chunks of K and of V, 4 of each per thread, fetched one tile ahead
    const float* kbase = a.k + b * a.k_sb + h * a.k_sh;
    const float* vbase = a.v + b * a.v_sb + h * a.v_sh;
    // (this thread's chunks: rows tid/32 + 8t, chunk tid%32; loads past the last tile re-read it)
    const uint32_t s_row = tid >> 5, s_chunk = tid & 31;
    const float* kstage = kbase + 4 * s_chunk;
    const float* vstage = vbase + 4 * s_chunk;
    float4 kreg0, kreg1, kreg2, kreg3, vreg0, vreg1, vreg2, vreg3;
#define RUMUS_ATTN_TILE_LOAD(J0)                                                                     \
    {                                                                                               \
        const uint32_t r0_ = min((J0) + s_row, a.kv_len - 1), r1_ = min((J0) + s_row + 8, a.kv_len - 1); \
        const uint32_t r2_ = min((J0) + s_row + 16, a.kv_len - 1), r3_ = min((J0) + s_row + 24, a.kv_len - 1); \
        kreg0 = *reinterpret_cast<const float4*>(kstage + (uint64_t)r0_ * a.k_sr);                  \
        kreg1 = *reinterpret_cast<const float4*>(kstage + (uint64_t)r1_ * a.k_sr);                  \
        kreg2 = *reinterpret_cast<const float4*>(kstage + (uint64_t)r2_ * a.k_sr);                  \
        kreg3 = *reinterpret_cast<const float4*>(kstage + (uint64_t)r3_ * a.k_sr);                  \
        vreg0 = *reinterpret_cast<const float4*>(vstage + (uint64_t)r0_ * a.v_sr);                  \
        vreg1 = *reinterpret_cast<const float4*>(vstage + (uint64_t)r1_ * a.v_sr);                  \
        vreg2 = *reinterpret_cast<const float4*>(vstage + (uint64_t)r2_ * a.v_sr);                  \
        vreg3 = *reinterpret_cast<const float4*>(vstage + (uint64_t)r3_ * a.v_sr);                  \
    }
    RUMUS_ATTN_TILE_LOAD(0u)
    for (uint32_t j0 = 0; j0 < kv_end; j0 += BC) {
        __syncthreads();                                       // the previous tile has been consumed
        {
            const uint32_t pos = attn_tile_pos(s_row, s_chunk);
            ks[pos] = kreg0; ks[pos + 8 * kAttnRowChunks] = kreg1;
            ks[pos + 16 * kAttnRowChunks] = kreg2; ks[pos + 24 * kAttnRowChunks] = kreg3;
            vs[pos] = vreg0; vs[pos + 8 * kAttnRowChunks] = vreg1;
            vs[pos + 16 * kAttnRowChunks] = vreg2; vs[pos + 24 * kAttnRowChunks] = vreg3;
        }
        __syncthreads();
        RUMUS_ATTN_TILE_LOAD(j0 + BC)                          // consumed at the top of the next round
        if (!wave_live || j0 >= wave_end) continue;            // wave-uniform: nothing visible in this tile

        // ---- S^T = K Q^T -----------------------------------------------------------------
        attn_v16f sacc;
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
        const float4* kfrag = ks + attn_tile_pos(l32, 16 * kb);
#pragma unroll
        for (int s4 = 0; s4 < 16; s4++) {
            const float4 kf = kfrag[s4];                       // K[key l32][64*kb + 4*s4 ..]
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.x, qf[4 * s4], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.y, qf[4 * s4 + 1], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.z, qf[4 * s4 + 2], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.w, qf[4 * s4 + 3], sacc, 0, 0, 0);
        }
        // ---- online softmax of this lane's query over its 16 keys + the other half's 16 ----
        // register r holds key j0 + (r/4)*8 + kb*4 + r%4
        float p[16];
        float mloc = kMasked;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = j0 + (r >> 2) * 8 + kb * 4 + (r & 3);
            p[r] = key < my_end ? sacc[r] : kMasked;
            mloc = fmaxf(mloc, p[r]);
        }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
        const float mnew = fmaxf(mrun, mloc);
        const float corr = exp2f(mrun - mnew);
        float lloc = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = j0 + (r >> 2) * 8 + kb * 4 + (r & 3);
            p[r] = key < my_end ? exp2f(p[r] - mnew) : 0.0f;
            lloc += p[r];
        }
        lloc += __shfl_xor(lloc, 32);
        lrun = lrun * corr + lloc;
        mrun = mnew;
        if (__any(corr != 1.0f)) {                             // the running maxima settle after a few tiles
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[dt][r] *= corr;
        }
        // ---- O^T += V^T P^T: step s multiplies keys (s/4)*8 + kb*4 + s%4, i.e. p[s] ----------
        const float* vfrag = reinterpret_cast<const float*>(vs + attn_tile_pos(kb * 4, 0)) + l32;
#pragma unroll
        for (int s = 0; s < 16; s++) {
            constexpr uint32_t kRowFloats = kAttnRowChunks * 4;
            const uint32_t krow = (s >> 2) * 8 + (s & 3);      // + kb * 4, already in vfrag
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const float vv = vfrag[krow * kRowFloats + dt * 32];   // V[krow + 4*kb][dt*32 + l32]
                oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv, p[s], oacc[dt], 0, 0, 0);
            }
        }
    }
#undef RUMUS_ATTN_TILE_LOAD
    if (qrow >= a.q_len) return;
    // oacc[dt][r] = O[qrow][dt*32 + (r/4)*8 + kb*4 + r%4]: four consecutive dims per r/4
    const float inv = lrun > 0.0f ? 1.0f / lrun : 0.0f;
    float* op = a.o + b * a.o_sb + h * a.o_sh + (uint64_t)qrow * a.o_sr;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            *reinterpret_cast<float4*>(op + dt * 32 + g * 8 + kb * 4) =
                make_float4(oacc[dt][4 * g] * inv, oacc[dt][4 * g + 1] * inv, oacc[dt][4 * g + 2] * inv,
                            oacc[dt][4 * g + 3] * inv);
}

// Decode case (q_len == 1): the keys of one (batch, head) are split over gridDim.x workgroups
// so that the chip is covered; each writes (max, sum, unnormalised output) of its slice and
// attention_merge_kernel combines the slices.  Within a workgroup: 8 lanes per key for the
// scores (32 keys per sweep), then one thread per 4 output dims and key group for p.V.
constexpr int kDecodeSlice = 256;   // most keys per workgroup

// lane exchanges inside 8 lanes without the LDS crossbar: quad_perm [1,0,3,2], [2,3,0,1], row_half_mirror
__device__ __forceinline__ float dpp8_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    return v;
}

// SLICE keys per workgroup (64, 128 or 256: the launcher takes the largest that still makes two workgroups per CU).
// Scores: 8 lanes per key, lane l of them holding dims 32 i + 4 l .. + 3, so that a load instruction of a wave reads
// whole 128-byte lines (8 keys x 128 bytes; with 4 lanes on 32 consecutive dims each it touched 64 lines for 16
// bytes apiece and the lines did not survive in the L1 until their other pieces were asked for).
template <int SLICE>
__global__ __launch_bounds__(256) void attention_decode_kernel(AttnArgs a, float* __restrict__ part) {
    __shared__ float sc[SLICE];
    __shared__ float red[4], lsum[8];
    __shared__ __attribute__((aligned(16))) float osum[8][kHeadDim];
    const uint32_t tid = threadIdx.x, lane8 = tid & 7, kq = tid >> 3;
    const uint32_t bh = blockIdx.y, b = bh / a.heads, h = bh % a.heads;
    const uint32_t j0 = blockIdx.x * SLICE, j1 = min(a.kv_len, j0 + SLICE);
    const float* qp = a.q + b * a.q_sb + h * a.q_sh + lane8 * 4;
    const float* kb = a.k + b * a.k_sb + h * a.k_sh;
    const float* vb = a.v + b * a.v_sb + h * a.v_sh;
    float q[16];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float4 t = *reinterpret_cast<const float4*>(qp + 32 * i);
        q[4 * i] = t.x * a.scale; q[4 * i + 1] = t.y * a.scale; q[4 * i + 2] = t.z * a.scale; q[4 * i + 3] = t.w * a.scale;
    }
    // p.V below: thread = (4 output dims, 1 of 8 key groups), eight 128-bit loads of V in flight
    const uint32_t c4 = tid & 31, kg = tid >> 5;
    auto load_v = [&](uint32_t jj, float4 (&vv)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const uint32_t vc = min(j0 + jj + 8 * u, a.kv_len - 1);
            const float* vp = (a.v_new && vc == a.kv_len - 1) ? a.v_new + b * a.vn_sb + h * a.vn_sh
                                                             : vb + (uint64_t)vc * a.v_sr;
            vv[u] = *reinterpret_cast<const float4*>(vp + 4 * c4);
        }
    };
    // All of the slice.s key loads are issued before the first is used; behind the last
    // group's loads goes the first batch of V (memory returns in order: asked for ahead of the keys it would hold
    // up the scores), so that its trip to memory overlaps the scores, the reduction and the barrier.
    constexpr int SWEEPS = SLICE / 32, GROUP = SWEEPS;
    float mloc = -INFINITY;
    float4 vfirst[8];
#pragma unroll
    for (int g0 = 0; g0 < SWEEPS; g0 += GROUP) {
        float4 kk[GROUP][4];
#pragma unroll
        for (int s = 0; s < GROUP; s++) {
            const uint32_t kc = min(j0 + (g0 + s) * 32 + kq, a.kv_len - 1);
            const float* kp = ((a.k_new && kc == a.kv_len - 1) ? a.k_new + b * a.kn_sb + h * a.kn_sh
                                                              : kb + (uint64_t)kc * a.k_sr) + lane8 * 4;
#pragma unroll
            for (int i = 0; i < 4; i++) kk[s][i] = *reinterpret_cast<const float4*>(kp + 32 * i);
        }
        if (g0 + GROUP >= SWEEPS) load_v(kg, vfirst);
        __builtin_amdgcn_sched_barrier(0);                 // the loads stay ahead of the arithmetic
#pragma unroll
        for (int s = 0; s < GROUP; s++) {
            const uint32_t jj = (g0 + s) * 32 + kq, key = j0 + jj;
            float d = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                d = fmaf(q[4 * i], kk[s][i].x, d); d = fmaf(q[4 * i + 1], kk[s][i].y, d);
                d = fmaf(q[4 * i + 2], kk[s][i].z, d); d = fmaf(q[4 * i + 3], kk[s][i].w, d);
            }
            d = dpp8_sum(d);
            d = key < j1 ? d : -INFINITY;
            if (lane8 == 0) sc[jj] = d;
            mloc = fmaxf(mloc, d);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mloc = fmaxf(mloc, __shfl_xor(mloc, o));
    if ((tid & 63) == 0) red[tid >> 6] = mloc;
    __syncthreads();
    const float m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));   // finite: the slice is not empty
    float4 o = make_float4(0, 0, 0, 0);
    float l = 0.0f;
#pragma unroll
    for (int it = 0; it < SLICE / 64; it++) {
        const uint32_t jj = kg + 64 * it;
        float p[8];
        float4 vv[8];
        if (it == 0) {
#pragma unroll
            for (int u = 0; u < 8; u++) vv[u] = vfirst[u];
        } else {
            load_v(jj, vv);
        }
#pragma unroll
        for (int u = 0; u < 8; u++) p[u] = j0 + jj + 8 * u < j1 ? expf(sc[jj + 8 * u] - m) : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            l += p[u];
            o.x = fmaf(p[u], vv[u].x, o.x); o.y = fmaf(p[u], vv[u].y, o.y);
            o.z = fmaf(p[u], vv[u].z, o.z); o.w = fmaf(p[u], vv[u].w, o.w);
        }
    }
    *reinterpret_cast<float4*>(&osum[kg][4 * c4]) = o;
    if (c4 == 0) lsum[kg] = l;
    // the append: no workgroup reads position kv_len - 1 of the cache in this launch
    if (a.k_new && blockIdx.x == gridDim.x - 1 && tid < 64) {
        const bool is_v = tid >= 32;
        const float* src = is_v ? a.v_new + b * a.vn_sb + h * a.vn_sh : a.k_new + b * a.kn_sb + h * a.kn_sh;
        float* dstc = const_cast<float*>(is_v ? vb + (uint64_t)(a.kv_len - 1) * a.v_sr : kb + (uint64_t)(a.kv_len - 1) * a.k_sr);
        reinterpret_cast<float4*>(dstc)[tid & 31] = reinterpret_cast<const float4*>(src)[tid & 31];
    }
    __syncthreads();
    if (tid < kHeadDim) {
        float* dst = part + ((uint64_t)bh * gridDim.x + blockIdx.x) * (kHeadDim + 2);
        float t = 0.0f;
#pragma unroll
        for (int g = 0; g < 8; g++) t += osum[g][tid];
        dst[2 + tid] = t;
        if (tid == 0) {
            float ls = 0.0f;
#pragma unroll
            for (int g = 0; g < 8; g++) ls += lsum[g];
            dst[0] = m;
            dst[1] = ls;
        }
    }
}

__global__ __launch_bounds__(kHeadDim) void attention_merge_kernel(AttnArgs a, const float* __restrict__ part,
                                                                   uint32_t slices) {
    const uint32_t bh = blockIdx.x, b = bh / a.heads, h = bh % a.heads, dim = threadIdx.x;
    const float* src = part + (uint64_t)bh * slices * (kHeadDim + 2);
    // slices is small (kv_len / 64 at most); the loads of a pass do not depend on each other
    float m = -INFINITY;
#pragma unroll 8
    for (uint32_t s = 0; s < slices; s++) m = fmaxf(m, src[s * (kHeadDim + 2)]);
    float l = 0.0f, o = 0.0f;
#pragma unroll 8
    for (uint32_t s = 0; s < slices; s++) {
        const float ms = src[s * (kHeadDim + 2)], ls = src[s * (kHeadDim + 2) + 1], os = src[s * (kHeadDim + 2) + 2 + dim];
        const float w = expf(ms - m);
        l = fmaf(w, ls, l);
        o = fmaf(w, os, o);
    }
    a.o[b * a.o_sb + h * a.o_sh + dim] = o / l;
}

// ---- KV-cache append: the new tokens' keys and values go to positions pos .. pos + rows - 1 -------
// Every operand carries (batch, head, row) strides like the attention operands, so the projection
// output [batch * rows, heads * dim] is read in place and the cache may be the reference's
// [batch, heads, positions, dim] (rumus-serve/src/model.rs:11-14) or token-major.  One launch
// moves both tensors: blockIdx.z picks K or V; a thread moves 16 bytes.
struct KvAppendArgs {
    const float* src[2];
    float* dst[2];
    uint64_t sb[2], sh[2], sr[2];     // source strides: batch, head, row
    uint64_t db[2], dh[2], dr[2];     // cache strides
    uint32_t heads, rows, dim4, pos;  // dim4 = head_dim / 4
};

__global__ __launch_bounds__(256) void kv_append_kernel(KvAppendArgs a) {
    const uint32_t which = blockIdx.z;
    const uint32_t per_row = a.heads * a.dim4;
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;        // (row, head, chunk) of this batch entry
    if (i >= a.rows * per_row) return;
    const uint32_t row = i / per_row, rem = i % per_row, head = rem / a.dim4, c = rem % a.dim4;
    const uint32_t b = blockIdx.y;
    const float4 v = *reinterpret_cast<const float4*>(a.src[which] + b * a.sb[which] + head * a.sh[which] +
                                                      row * a.sr[which] + 4 * c);
    *reinterpret_cast<float4*>(a.dst[which] + b * a.db[which] + head * a.dh[which] +
                               (uint64_t)(a.pos + row) * a.dr[which] + 4 * c) = v;
}

}  // namespace rumus

// One query row per (batch, head): slices of 256 keys, or of 128 or 64 while that is what it takes to put two
// workgroups on every CU (32 heads at 2048 keys: 512 workgroups of 128 keys), merged by a second kernel.
static int launch_attention_decode(const rumus::AttnArgs& a, hipStream_t s) {
    using namespace rumus;
    const uint32_t bh = a.batch * a.heads;
    const uint32_t slice = (uint64_t)bh * ceil_div(a.kv_len, 256u) >= 512 ? 256 : (uint64_t)bh * ceil_div(a.kv_len, 128u) >= 512 ? 128 : 64;
    const uint32_t slices = ceil_div(a.kv_len, slice);
    void* ws = nullptr;
    WorkspaceLease lease;                                    // until both kernels are queued
    if (int rc = workspace_get(s, (size_t)bh * slices * (kHeadDim + 2) * sizeof(float), &ws, lease)) return rc;
    const dim3 grid(slices, bh);
    if (slice == 256) hipLaunchKernelGGL(attention_decode_kernel<256>, grid, dim3(256), 0, s, a, static_cast<float*>(ws));
    else if (slice == 128) hipLaunchKernelGGL(attention_decode_kernel<128>, grid, dim3(256), 0, s, a, static_cast<float*>(ws));
    else hipLaunchKernelGGL(attention_decode_kernel<64>, grid, dim3(256), 0, s, a, static_cast<float*>(ws));
    if (int rc = check_launch("attention_decode_kernel")) return rc;
    hipLaunchKernelGGL(attention_merge_kernel, dim3(bh), dim3(kHeadDim), 0, s, a, static_cast<const float*>(ws), slices);
    return check_launch("attention_merge_kernel");
}

using namespace rumus;

extern "C" {

int rumus_hip_rmsnorm(const float* x, const float* weight, float* y, uint32_t rows, uint32_t dim, float eps,
                      rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(rows == 0 || (x && weight && y), "rmsnorm: null buffer");
    RUMUS_REQUIRE(dim > 0, "rmsnorm: dim must be > 0");
    if (rows == 0) return RUMUS_HIP_OK;
    const bool vec = dim % 4 == 0 && dim <= 8192 &&
                     ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) |
                       reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    if (vec) hipLaunchKernelGGL((rmsnorm_kernel<true, false>), dim3(rows), dim3(256), 0, as_stream(stream), x, nullptr,
                                weight, nullptr, y, dim, eps);
    else hipLaunchKernelGGL((rmsnorm_kernel<false, false>), dim3(rows), dim3(256), 0, as_stream(stream), x, nullptr,
                            weight, nullptr, y, dim, eps);
    return check_launch("rmsnorm_kernel");
}

int rumus_hip_add_rmsnorm(const float* x, const float* delta, const float* weight, float* sum, float* y,
                          uint32_t rows, uint32_t dim, float eps, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(rows == 0 || (x && delta && weight && sum && y), "add_rmsnorm: null buffer");
    RUMUS_REQUIRE(dim > 0, "add_rmsnorm: dim must be positive");
    RUMUS_REQUIRE(rows == 0 || (y != x && y != delta && y != sum), "add_rmsnorm: y must not alias x, delta or sum");
    if (rows == 0) return RUMUS_HIP_OK;
    const bool vec = dim % 4 == 0 && dim <= 8192 &&
                     ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(delta) |
                       reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(sum) |
                       reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    if (vec) hipLaunchKernelGGL((rmsnorm_kernel<true, true>), dim3(rows), dim3(256), 0, as_stream(stream), x, delta,
                                weight, sum, y, dim, eps);
    else hipLaunchKernelGGL((rmsnorm_kernel<false, true>), dim3(rows), dim3(256), 0, as_stream(stream), x, delta,
                            weight, sum, y, dim, eps);
    return check_launch("rmsnorm_kernel");
}

int rumus_hip_swiglu(const float* gate, const float* up, float* out, uint64_t numel, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(numel == 0 || (gate && up && out), "swiglu: null buffer");
    if (numel == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(swiglu_kernel, dim3((uint32_t)((numel + 255) / 256)), dim3(256), 0, as_stream(stream), gate,
                       up, out, numel);
    return check_launch("swiglu_kernel");
}

int rumus_hip_swiglu_rows(const float* gate_up, float* out, uint32_t rows, uint32_t n, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(rows == 0 || n == 0 || (gate_up && out), "swiglu_rows: null buffer");
    RUMUS_REQUIRE(rows <= 65535, "swiglu_rows: rows %u beyond the grid limit", rows);
    if (rows == 0 || n == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(swiglu_rows_kernel, dim3(ceil_div(n, 256), rows), dim3(256), 0, as_stream(stream), gate_up, out,
                       n);
    return check_launch("swiglu_rows_kernel");
}

int rumus_hip_add(const float* a, const float* b, float* out, uint64_t numel, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(numel == 0 || (a && b && out), "add: null buffer");
    if (numel == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(add_kernel, dim3((uint32_t)((numel + 255) / 256)), dim3(256), 0, as_stream(stream), a, b, out,
                       numel);
    return check_launch("add_kernel");
}

int rumus_hip_attention(const float* q, const float* k, const float* v, float* out, uint32_t batch, uint32_t heads,
                        uint32_t q_len, uint32_t kv_len, uint32_t head_dim, const uint64_t* strides, int causal,
                        rumus_hip_stream_t stream) {
    RUMUS_REQUIRE((batch == 0 || heads == 0 || q_len == 0) || (q && k && v && out && strides), "attention: null buffer");
    RUMUS_REQUIRE(head_dim == kHeadDim, "attention: head_dim must be %d (got %u)", kHeadDim, head_dim);
    RUMUS_REQUIRE(q_len <= kv_len, "attention: q_len %u exceeds kv_len %u", q_len, kv_len);
    if (batch == 0 || heads == 0 || q_len == 0) return RUMUS_HIP_OK;
    for (int i = 0; i < 12; i++)
        RUMUS_REQUIRE(strides[i] % 4 == 0, "attention: stride %d (%llu) must be a multiple of 4 floats", i,
                      (unsigned long long)strides[i]);
    RUMUS_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                    reinterpret_cast<uintptr_t>(out)) & 15) == 0, "attention: operands must be 16-byte aligned");
    RUMUS_REQUIRE((uint64_t)batch * heads <= 65535, "attention: batch * heads beyond the grid limit");
    AttnArgs a{q, k, v, out, strides[0], strides[1], strides[2], strides[3], strides[4], strides[5],
               strides[6], strides[7], strides[8], strides[9], strides[10], strides[11],
               batch, heads, q_len, kv_len, 1.0f / sqrtf((float)head_dim), causal};
    hipStream_t s = as_stream(stream);
    if (q_len == 1) return launch_attention_decode(a, s);
    if (q_len >= 64) {                                       // enough rows to fill 32-row matrix-core tiles
        RUMUS_REQUIRE(ceil_div(q_len, 128) <= 65535, "attention: q_len %u beyond the grid limit", q_len);
        hipLaunchKernelGGL(attention_mfma_kernel, dim3(batch * heads, ceil_div(q_len, 128)), dim3(256), 0, s, a);
        return check_launch("attention_mfma_kernel");
    }
    hipLaunchKernelGGL(attention_rows_kernel, dim3(ceil_div(q_len, 64), batch * heads), dim3(256), 0, s, a);
    return check_launch("attention_rows_kernel");
}

int rumus_hip_kv_append(const float* k_new, const float* v_new, float* k_cache, float* v_cache, uint32_t batch,
                        uint32_t heads, uint32_t rows, uint32_t head_dim, uint32_t pos, uint32_t cache_len,
                        const uint64_t* strides, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE((batch == 0 || heads == 0 || rows == 0) || (k_new && v_new && k_cache && v_cache && strides),
                  "kv_append: null buffer");
    RUMUS_REQUIRE(head_dim > 0 && head_dim % 4 == 0, "kv_append: head_dim %u must be a positive multiple of 4", head_dim);
    RUMUS_REQUIRE((uint64_t)pos + rows <= cache_len, "kv_append: positions %u..%llu do not fit a cache of %u", pos,
                  (unsigned long long)pos + rows, cache_len);
    if (batch == 0 || heads == 0 || rows == 0) return RUMUS_HIP_OK;
    for (int i = 0; i < 12; i++)
        RUMUS_REQUIRE(strides[i] % 4 == 0, "kv_append: stride %d (%llu) must be a multiple of 4 floats", i,
                      (unsigned long long)strides[i]);
    RUMUS_REQUIRE(((reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new) |
                    reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache)) & 15) == 0,
                  "kv_append: operands must be 16-byte aligned");
    const uint64_t per_batch = (uint64_t)rows * heads * (head_dim / 4);
    RUMUS_REQUIRE(batch <= 65535 && per_batch < (1ull << 32), "kv_append: shape beyond the grid limit");
    KvAppendArgs a{{k_new, v_new}, {k_cache, v_cache},
                   {strides[0], strides[3]}, {strides[1], strides[4]}, {strides[2], strides[5]},
                   {strides[6], strides[9]}, {strides[7], strides[10]}, {strides[8], strides[11]},
                   heads, rows, head_dim / 4, pos};
    hipLaunchKernelGGL(kv_append_kernel, dim3((uint32_t)((per_batch + 255) / 256), batch, 2), dim3(256), 0,
                       as_stream(stream), a);
    return check_launch("kv_append_kernel");
}

// kv_append of one token at `pos` and attention of its query over positions 0 .. pos, in the two launches of
// the decode attention: the newest key / value are read from k_new / v_new and stored by the last slice's workgroup.
int rumus_hip_attention_decode_append(const float* q, const float* k_new, const float* v_new, float* k_cache,
                                      float* v_cache, float* out, uint32_t batch, uint32_t heads, uint32_t head_dim,
                                      uint32_t pos, uint32_t cache_len, const uint64_t* strides,
                                      rumus_hip_stream_t stream) {
    RUMUS_REQUIRE((batch == 0 || heads == 0) || (q && k_new && v_new && k_cache && v_cache && out && strides),
                  "attention_decode_append: null buffer");
    RUMUS_REQUIRE(head_dim == kHeadDim, "attention_decode_append: head_dim must be %d (got %u)", kHeadDim, head_dim);
    RUMUS_REQUIRE(pos < cache_len, "attention_decode_append: position %u does not fit a cache of %u", pos, cache_len);
    if (batch == 0 || heads == 0) return RUMUS_HIP_OK;
    for (int i = 0; i < 18; i++)
        RUMUS_REQUIRE(strides[i] % 4 == 0, "attention_decode_append: stride %d (%llu) must be a multiple of 4 floats", i,
                      (unsigned long long)strides[i]);
    RUMUS_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new) |
                    reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache) |
                    reinterpret_cast<uintptr_t>(out)) & 15) == 0, "attention_decode_append: operands must be 16-byte aligned");
    RUMUS_REQUIRE((uint64_t)batch * heads <= 65535, "attention_decode_append: batch * heads beyond the grid limit");
    // strides: {q, k_new, v_new, k_cache, v_cache, out} x {batch, head, row}; the rows of q, k_new, v_new and out
    // are single, their row strides unused
    AttnArgs a{q, k_cache, v_cache, out, strides[0], strides[1], strides[2], strides[9], strides[10], strides[11],
               strides[12], strides[13], strides[14], strides[15], strides[16], strides[17],
               batch, heads, 1, pos + 1, 1.0f / sqrtf((float)head_dim), 0};
    a.k_new = k_new;
    a.v_new = v_new;
    a.kn_sb = strides[3]; a.kn_sh = strides[4];
    a.vn_sb = strides[6]; a.vn_sh = strides[7];
    return launch_attention_decode(a, as_stream(stream));
}

}  // extern "C"
