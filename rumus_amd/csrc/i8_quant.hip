// W8A8 INT8 engine, quantizers: dynamic per-row activation quantizer and the
// per-output-channel weight quantizer.  Both apply the reference's symmetric
// rule (rumus/src/backend/gpu/shaders/quantize.wgsl:66-67,93) with the scale
// kept in f32: scale = amax/127 (1 if amax == 0), inv = 127/amax (0 if
// amax == 0), q = clamp(rint(v*inv), -128, 127).
#include "common.h"

namespace rumus {

__device__ __forceinline__ float wave_max64(float v) { return wave_max(v); }

__device__ __forceinline__ int q_i8(float v, float inv) {
    float t = rintf(__fmul_rn(v, inv));
    return (int)fminf(fmaxf(t, -128.0f), 127.0f);
}

// One workgroup per row.  A row of up to 1024 CACHE elements stays in registers between the two
// passes (all of a thread's loads in flight at once, the row read once: 2048 x 11008 29 -> 18 us);
// CACHE = 0 or longer rows: read twice (the second read hits L2).

__device__ __forceinline__ uint32_t pack_i8x4(const float4& v, float inv) {
    return ((uint32_t)q_i8(v.x, inv) & 0xFFu) | (((uint32_t)q_i8(v.y, inv) & 0xFFu) << 8) |
           (((uint32_t)q_i8(v.z, inv) & 0xFFu) << 16) | (((uint32_t)q_i8(v.w, inv) & 0xFFu) << 24);
}

template <int CACHE>
__global__ __launch_bounds__(256) void i8_quantize_rows_kernel(const float* __restrict__ x,
                                                               int8_t* __restrict__ xq,
                                                               float* __restrict__ scale,
                                                               uint32_t cols) {
    __shared__ float red[4];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const float* xr = x + (uint64_t)row * cols;
    int8_t* qr = xq + (uint64_t)row * cols;
    const bool vec = (cols % 4 == 0) && ((reinterpret_cast<uintptr_t>(xr) & 15) == 0) &&
                     ((reinterpret_cast<uintptr_t>(qr) & 3) == 0);
    const bool cached = CACHE > 0 && vec && cols <= 1024u * CACHE;
    const float4* p = reinterpret_cast<const float4*>(xr);
    float4 cache[CACHE > 0 ? CACHE : 1];
    float amax = 0.0f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; i++) {
            const uint32_t j = tid + 256 * i;
            cache[i] = j < cols / 4 ? p[j] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int i = 0; i < CACHE; i++)
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(cache[i].x), fabsf(cache[i].y)), fmaxf(fabsf(cache[i].z), fabsf(cache[i].w))));
    } else if (vec) {
        for (uint32_t i = tid; i < cols / 4; i += 256) {
            float4 v = p[i];
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    } else {
        for (uint32_t i = tid; i < cols; i += 256) amax = fmaxf(amax, fabsf(xr[i]));
    }
    amax = wave_max64(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float inv = amax == 0.0f ? 0.0f : __fdiv_rn(127.0f, amax);
    if (tid == 0) scale[row] = amax == 0.0f ? 1.0f : __fdiv_rn(amax, 127.0f);
    uint32_t* o = reinterpret_cast<uint32_t*>(qr);
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; i++) {
            const uint32_t j = tid + 256 * i;
            if (j < cols / 4) o[j] = pack_i8x4(cache[i], inv);
        }
    } else if (vec) {
        for (uint32_t i = tid; i < cols / 4; i += 256) o[i] = pack_i8x4(p[i], inv);
    } else {
        for (uint32_t i = tid; i < cols; i += 256) qr[i] = (int8_t)q_i8(xr[i], inv);
    }
}

// ---- per-output-channel weights: w[k,n] -> wq[n,k], sw[n] -----------------

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t* __restrict__ p, uint32_t n) {
    uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// Pass 1: column abs-max.  Thread = four adjacent columns (one 128-bit load per row), workgroup = 1024 columns x
// one K slice; slices combine with an integer atomic max on the float bits (exact and order-independent for
// non-negative floats).
__global__ __launch_bounds__(256) void col_absmax_kernel(const float* __restrict__ w,
                                                         uint32_t* __restrict__ amax_bits,
                                                         uint32_t k, uint32_t n, uint32_t kslice) {
    const uint32_t col = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (col >= n) return;
    const uint32_t k0 = blockIdx.y * kslice, k1 = min(k, k0 + kslice);
    float amax[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (n % 4 == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
        for (uint32_t r = k0; r < k1; r++) {
            const float4 v = *reinterpret_cast<const float4*>(w + (uint64_t)r * n + col);
            amax[0] = fmaxf(amax[0], fabsf(v.x)); amax[1] = fmaxf(amax[1], fabsf(v.y));
            amax[2] = fmaxf(amax[2], fabsf(v.z)); amax[3] = fmaxf(amax[3], fabsf(v.w));
        }
    } else {
        for (uint32_t r = k0; r < k1; r++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (col + j < n) amax[j] = fmaxf(amax[j], fabsf(w[(uint64_t)r * n + col + j]));
    }
#pragma unroll
    for (int j = 0; j < 4; j++)
        if (col + j < n) atomicMax(amax_bits + col + j, __float_as_uint(amax[j]));
}

// Pass 2: 64x64 tile, quantize with the column's inv and write transposed.  Reads are 128-bit over
// four adjacent columns, writes 128-bit over sixteen consecutive k of one column; the tile turns in LDS.
__global__ __launch_bounds__(256) void quantize_cols_t_kernel(const float* __restrict__ w,
                                                              const float* __restrict__ amax,
                                                              int8_t* __restrict__ wq, uint32_t k,
                                                              uint32_t n) {
    __shared__ __attribute__((aligned(16))) int8_t t[64][64 + 16];   // [col][k]; rows 16-byte aligned
    const uint32_t k0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;  // 16 groups of 4 columns x 16 rows
    const uint32_t col = c0 + 4 * tx;
    const bool vec = n % 4 == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0;   // then col + 3 < n whenever col < n
    float inv[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float am = col + j < n ? amax[col + j] : 0.0f;
        inv[j] = am == 0.0f ? 0.0f : __fdiv_rn(127.0f, am);
    }
#pragma unroll
    for (uint32_t r = ty; r < 64; r += 16) {
        const uint32_t kk = k0 + r;
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (kk < k) {
            if (vec && col < n) {
                const float4 q = *reinterpret_cast<const float4*>(w + (uint64_t)kk * n + col);
                v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (col + j < n) v[j] = w[(uint64_t)kk * n + col + j];
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) t[4 * tx + j][r] = (int8_t)q_i8(v[j], inv[j]);
    }
    __syncthreads();
    // write: thread handles one column row, 16 consecutive k bytes
    const uint32_t oc = threadIdx.x / 4, seg = (threadIdx.x % 4) * 16;
    if (c0 + oc < n && k0 + seg < k) {
        int8_t* dst = wq + (uint64_t)(c0 + oc) * k + k0 + seg;
        if (k % 16 == 0 && (reinterpret_cast<uintptr_t>(wq) & 15) == 0) {
            *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(&t[oc][seg]);
        } else {
            for (uint32_t i = 0; i < 16; i++)
                if (k0 + seg + i < k) dst[i] = t[oc][seg + i];
        }
    }
}

// Pass 3: abs-max -> scale, in place.
__global__ __launch_bounds__(256) void amax_to_scale_kernel(float* __restrict__ sw, uint32_t n) {
    uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        float am = sw[i];
        sw[i] = am == 0.0f ? 1.0f : __fdiv_rn(am, 127.0f);
    }
}

}  // namespace rumus

using namespace rumus;

extern "C" {

int rumus_hip_i8_quantize_rows(const float* x, int8_t* xq, float* scale, uint32_t rows,
                               uint32_t cols, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(rows == 0 || (x && xq && scale), "i8_quantize_rows: null buffer");
    if (rows == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(cols > 0, "i8_quantize_rows: cols must be > 0");
    hipStream_t s = as_stream(stream);
    if (cols <= 4096)
        hipLaunchKernelGGL(i8_quantize_rows_kernel<4>, dim3(rows), dim3(256), 0, s, x, xq, scale, cols);
    else if (cols <= 8192)
        hipLaunchKernelGGL(i8_quantize_rows_kernel<8>, dim3(rows), dim3(256), 0, s, x, xq, scale, cols);
    else if (cols <= 12288)
        hipLaunchKernelGGL(i8_quantize_rows_kernel<12>, dim3(rows), dim3(256), 0, s, x, xq, scale, cols);
    else
        hipLaunchKernelGGL(i8_quantize_rows_kernel<0>, dim3(rows), dim3(256), 0, s, x, xq, scale, cols);
    return check_launch("i8_quantize_rows_kernel");
}

int rumus_hip_i8_quantize_cols_t(const float* w, int8_t* wq, float* sw, uint32_t k, uint32_t n,
                                 rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(n == 0 || (w && wq && sw), "i8_quantize_cols_t: null buffer");
    if (n == 0) return RUMUS_HIP_OK;
    RUMUS_REQUIRE(k > 0, "i8_quantize_cols_t: k must be > 0");
    hipStream_t s = as_stream(stream);
    // sw doubles as the abs-max accumulator until pass 3 turns it into scales.
    hipLaunchKernelGGL(fill_zero_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, s,
                       reinterpret_cast<uint32_t*>(sw), n);
    const uint32_t kslice = 64;
    hipLaunchKernelGGL(col_absmax_kernel, dim3(ceil_div(n, 1024), ceil_div(k, kslice)), dim3(256), 0,
                       s, w, reinterpret_cast<uint32_t*>(sw), k, n, kslice);
    hipLaunchKernelGGL(quantize_cols_t_kernel, dim3(ceil_div(n, 64), ceil_div(k, 64)), dim3(256), 0,
                       s, w, sw, wq, k, n);
    hipLaunchKernelGGL(amax_to_scale_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, s, sw, n);
    return check_launch("i8_quantize_cols_t");
}

}  // extern "C"
