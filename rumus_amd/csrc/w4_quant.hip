// INT4 engine, weight preparation: min/max group quantizer + nibble packer
// (QuantizedTensor::from_f32, rumus-vision/src/quant.rs:42-102), its symmetric
// variant, and the one-time act-order row sort.
//
// Packed layout (quant.rs:98-100): word (row/8)*N + col holds rows
// 8*(row/8) .. +7 of column col, row r in bits 4*(r%8) .. +3.
#include <vector>

#include "common.h"

namespace rumus {

// Thread = one column of one group; workgroup = 256 adjacent columns, so every row read and
// every word store is one contiguous segment per wave.  GS = 32, 64 or 128: the group size is a
// compile-time constant and the group is read once, all loads issued before the first use, and
// kept in registers for the two passes (min/max, then quantize).  GS = 0: any group size, the
// group is read twice (the second read is served by L2).  The arithmetic is the same, in the
// same order, either way.
template <int GS>
struct GroupReader {
    const float* w;
    uint32_t k, n, col, r0;
    float cache[GS > 0 ? GS : 1];
    __device__ __forceinline__ GroupReader(const float* w_, uint32_t k_, uint32_t n_, uint32_t col_, uint32_t r0_)
        : w(w_), k(k_), n(n_), col(col_), r0(r0_) {
        if constexpr (GS > 0) {
#pragma unroll
            for (int i = 0; i < GS; i++) {
                const uint32_t r = r0 + i;
                const float v = w[(uint64_t)min(r, k - 1) * n + col];
                cache[i] = r < k ? v : 0.0f;                 // rows >= k: the zero padding of quant.rs:50-56
            }
        }
    }
    __device__ __forceinline__ float operator[](uint32_t i) const {
        if constexpr (GS > 0) return cache[i];
        const uint32_t r = r0 + i;
        return r < k ? w[(uint64_t)r * n + col] : 0.0f;
    }
};

template <bool SYM, int GS>
__global__ __launch_bounds__(256) void w4_quantize_pack_kernel(
    const float* __restrict__ w, uint32_t k, uint32_t n, uint32_t gs_arg,
    uint32_t* __restrict__ packed, float* __restrict__ scales, float* __restrict__ zps) {
    const uint32_t col = blockIdx.x * 256 + threadIdx.x;
    const uint32_t g = blockIdx.y;
    if (col >= n) return;
    const uint32_t gs = GS > 0 ? GS : gs_arg;
    const uint32_t r0 = g * gs;
    const GroupReader<GS> group(w, k, n, col, r0);

    float scale, zp;
    if (SYM) {
        float amax = 0.0f;
#pragma unroll
        for (uint32_t i = 0; i < gs; i++) amax = fmaxf(amax, fabsf(group[i]));
        scale = amax > 0.0f ? __fdiv_rn(amax, 7.0f) : 1.0f;
        zp = 8.0f;
    } else {
        // quant.rs:66-74
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
#pragma unroll
        for (uint32_t i = 0; i < gs; i++) {
            const float v = group[i];
            if (v < mn) mn = v;
            if (v > mx) mx = v;
        }
        const float range = __fsub_rn(mx, mn);
        const bool live = range > 1e-10f;                       // quant.rs:77-79
        scale = live ? __fdiv_rn(range, 15.0f) : 1.0f;
        zp = live ? __fdiv_rn(-mn, scale) : 0.0f;
    }
    scales[(uint64_t)g * n + col] = scale;
    if (zps) zps[(uint64_t)g * n + col] = zp;

#pragma unroll
    for (uint32_t wr = 0; wr < gs / 8; wr++) {
        uint32_t word = 0;
#pragma unroll
        for (uint32_t j = 0; j < 8; j++) {
            const float v = group[wr * 8 + j];
            float t;
            if (SYM) {
                t = __fadd_rn(roundf(__fdiv_rn(v, scale)), 8.0f);
            } else {
                t = roundf(__fadd_rn(__fdiv_rn(v, scale), zp));  // quant.rs:96, half away
            }
            t = fminf(fmaxf(t, 0.0f), 15.0f);                    // NaN -> 0 like `as i32`
            word |= (uint32_t)t << (4 * j);
        }
        packed[(uint64_t)(r0 / 8 + wr) * n + col] = word;
    }
}

// AWQ storage: integer zero-points packed eight per word along n.
//   scale = max(max - min, 1e-5) / 15;  z = clamp(-rint(min / scale), 0, 15);
//   q = clamp(rint(w / scale) + z, 0, 15)        (rint: half to even)
// Same thread layout as above; the eight lanes that share a zero-point word combine their
// nibbles with lane exchanges (n % 8 == 0, so the eight are all inside or all outside).
template <int GS>
__global__ __launch_bounds__(256) void w4_quantize_pack_awq_kernel(
    const float* __restrict__ w, uint32_t k, uint32_t n, uint32_t gs_arg,
    uint32_t* __restrict__ packed, float* __restrict__ scales, uint32_t* __restrict__ qzeros) {
    const uint32_t col = blockIdx.x * 256 + threadIdx.x;
    const uint32_t g = blockIdx.y;
    if (col >= n) return;
    const uint32_t gs = GS > 0 ? GS : gs_arg;
    const uint32_t r0 = g * gs;
    const GroupReader<GS> group(w, k, n, col, r0);
    float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
#pragma unroll
    for (uint32_t i = 0; i < gs; i++) {
        const float v = group[i];
        if (v < mn) mn = v;
        if (v > mx) mx = v;
    }
    float range = __fsub_rn(mx, mn);
    if (!(range > 1e-5f)) range = 1e-5f;
    const float scale = __fdiv_rn(range, 15.0f);
    const float zf = fminf(fmaxf(-rintf(__fdiv_rn(mn, scale)), 0.0f), 15.0f);   // NaN -> 0
    scales[(uint64_t)g * n + col] = scale;
    uint32_t zw = (uint32_t)zf << (4 * (col & 7));
    zw |= __shfl_xor(zw, 1);
    zw |= __shfl_xor(zw, 2);
    zw |= __shfl_xor(zw, 4);
    if ((col & 7) == 0) qzeros[(uint64_t)g * (n / 8) + col / 8] = zw;
#pragma unroll
    for (uint32_t wr = 0; wr < gs / 8; wr++) {
        uint32_t word = 0;
#pragma unroll
        for (uint32_t j = 0; j < 8; j++) {
            const float v = group[wr * 8 + j];
            float t = __fadd_rn(rintf(__fdiv_rn(v, scale)), zf);
            t = fminf(fmaxf(t, 0.0f), 15.0f);
            word |= (uint32_t)t << (4 * j);
        }
        packed[(uint64_t)(r0 / 8 + wr) * n + col] = word;
    }
}

// Decode layout: tile-major copy of a [rows, n] array of 32-bit words, tile = 16 columns:
// out[(c*rows + r)*16 + j] = in[r*n + 16*c + j].  One thread per 4 words.
__global__ __launch_bounds__(256) void w4_tile16_kernel(const uint4* __restrict__ in, uint4* __restrict__ out,
                                                        uint32_t rows, uint32_t n) {
    const uint32_t q = blockIdx.x * 256 + threadIdx.x, r = blockIdx.y;     // q: which group of 4 columns
    if (q * 4 >= n) return;
    out[((uint64_t)(q >> 2) * rows + r) * 4 + (q & 3)] = in[(uint64_t)r * (n / 4) + q];
}

// Decode layout of u4 zero-points [groups, n/8]: the two words of a tile's 16 columns side by
// side per group, out[(c*groups + g)*2 + h] = in[g*(n/8) + 2*c + h].
__global__ __launch_bounds__(256) void w4_tile16_zp4_kernel(const uint32_t* __restrict__ in,
                                                            uint32_t* __restrict__ out, uint32_t groups,
                                                            uint32_t words_per_row) {
    const uint32_t wd = blockIdx.x * 256 + threadIdx.x, g = blockIdx.y;
    if (wd >= words_per_row) return;
    out[((uint64_t)(wd >> 1) * groups + g) * 2 + (wd & 1)] = in[(uint64_t)g * words_per_row + wd];
}

// packed_sorted word (jr, col) gathers the nibbles of original rows
// perm[8*jr .. 8*jr+7].
__global__ __launch_bounds__(256) void w4_gather_rows_kernel(const uint32_t* __restrict__ packed,
                                                             const int32_t* __restrict__ perm,
                                                             uint32_t n,
                                                             uint32_t* __restrict__ out) {
    const uint32_t col = blockIdx.x * 256 + threadIdx.x;
    const uint32_t jr = blockIdx.y;
    if (col >= n) return;
    uint32_t word = 0;
#pragma unroll
    for (uint32_t i = 0; i < 8; i++) {
        const uint32_t r = (uint32_t)perm[jr * 8 + i];
        const uint32_t src = packed[(uint64_t)(r / 8) * n + col];
        word |= ((src >> (4 * (r % 8))) & 0xFu) << (4 * i);
    }
    out[(uint64_t)jr * n + col] = word;
}

// u4 zero-points, eight per word (nibble of column c at bits 4 * (c % 8) of word c / 8) -> one f32 each.
__global__ __launch_bounds__(256) void w4_qzeros_unpack_kernel(const uint32_t* __restrict__ qzeros,
                                                               float* __restrict__ zps, uint32_t n) {
    const uint32_t word = blockIdx.x * 256 + threadIdx.x, g = blockIdx.y;
    if (word >= n / 8) return;
    const uint32_t q = qzeros[(uint64_t)g * (n / 8) + word];
    float4 lo, hi;
    lo.x = (float)(q & 15u);         lo.y = (float)((q >> 4) & 15u);
    lo.z = (float)((q >> 8) & 15u);  lo.w = (float)((q >> 12) & 15u);
    hi.x = (float)((q >> 16) & 15u); hi.y = (float)((q >> 20) & 15u);
    hi.z = (float)((q >> 24) & 15u); hi.w = (float)(q >> 28);
    float4* dst = reinterpret_cast<float4*>(zps + (uint64_t)g * n + 8 * word);
    dst[0] = lo;
    dst[1] = hi;
}

// f16 -> f32 (exact): stored checkpoints often keep their scales in half precision.
__global__ __launch_bounds__(256) void f16_to_f32_kernel(const _Float16* __restrict__ in, float* __restrict__ out,
                                                         uint64_t numel) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < numel) out[i] = (float)in[i];
}

template <bool SYM>
static int quantize_pack(const float* w, uint32_t k, uint32_t n, uint32_t gs, uint32_t* packed,
                         float* scales, float* zps, hipStream_t s) {
    RUMUS_REQUIRE(gs > 0 && gs % 8 == 0, "group_size must be a multiple of 8 (got %u)", gs);
    RUMUS_REQUIRE(n == 0 || k == 0 || (w && packed && scales && (SYM || zps)), "w4_quantize_pack: null buffer");
    if (n == 0 || k == 0) return RUMUS_HIP_OK;
    const uint32_t groups = ceil_div(k, gs);
    const dim3 grid(ceil_div(n, 256), groups);
    switch (gs) {                                        // common sizes: one pass over the weights
        case 32: hipLaunchKernelGGL((w4_quantize_pack_kernel<SYM, 32>), grid, dim3(256), 0, s, w, k, n, gs, packed, scales, zps); break;
        case 64: hipLaunchKernelGGL((w4_quantize_pack_kernel<SYM, 64>), grid, dim3(256), 0, s, w, k, n, gs, packed, scales, zps); break;
        case 128: hipLaunchKernelGGL((w4_quantize_pack_kernel<SYM, 128>), grid, dim3(256), 0, s, w, k, n, gs, packed, scales, zps); break;
        default: hipLaunchKernelGGL((w4_quantize_pack_kernel<SYM, 0>), grid, dim3(256), 0, s, w, k, n, gs, packed, scales, zps);
    }
    return check_launch("w4_quantize_pack_kernel");
}

}  // namespace rumus

using namespace rumus;

extern "C" {

int rumus_hip_w4_quantize_pack(const float* w, uint32_t k, uint32_t n, uint32_t group_size,
                               uint32_t* packed, float* scales, float* zero_points,
                               rumus_hip_stream_t stream) {
    return quantize_pack<false>(w, k, n, group_size, packed, scales, zero_points, as_stream(stream));
}

static int decode_layout(const uint32_t* packed, const float* scales, const float* zero_points,
                         const uint32_t* qzeros, uint32_t padded_k, uint32_t n, uint32_t group_size,
                         uint32_t* packed_t, float* scales_t, float* zero_points_t, uint32_t* qzeros_t,
                         hipStream_t s) {
    RUMUS_REQUIRE(packed && scales && packed_t && scales_t && ((zero_points && zero_points_t) || (qzeros && qzeros_t)),
                  "w4_decode_layout: null buffer");
    RUMUS_REQUIRE(n % 16 == 0, "w4_decode_layout: n must be a multiple of 16 (got %u)", n);
    RUMUS_REQUIRE(group_size > 0 && padded_k % group_size == 0 && group_size % 8 == 0,
                  "w4_decode_layout: padded_k %u is not a whole number of groups of %u", padded_k, group_size);
    const uintptr_t bits = reinterpret_cast<uintptr_t>(packed) | reinterpret_cast<uintptr_t>(scales) |
                           reinterpret_cast<uintptr_t>(zero_points) | reinterpret_cast<uintptr_t>(packed_t) |
                           reinterpret_cast<uintptr_t>(scales_t) | reinterpret_cast<uintptr_t>(zero_points_t);
    RUMUS_REQUIRE((bits & 15) == 0, "w4_decode_layout: buffers must be 16-byte aligned");
    if (padded_k == 0 || n == 0) return RUMUS_HIP_OK;
    const uint32_t word_rows = padded_k / 8, groups = padded_k / group_size;
    RUMUS_REQUIRE(word_rows <= 65535, "w4_decode_layout: padded_k %u beyond the grid limit", padded_k);
    const dim3 gx(ceil_div(n / 4, 256));
    hipLaunchKernelGGL(w4_tile16_kernel, dim3(gx.x, word_rows), dim3(256), 0, s,
                       reinterpret_cast<const uint4*>(packed), reinterpret_cast<uint4*>(packed_t), word_rows, n);
    hipLaunchKernelGGL(w4_tile16_kernel, dim3(gx.x, groups), dim3(256), 0, s,
                       reinterpret_cast<const uint4*>(scales), reinterpret_cast<uint4*>(scales_t), groups, n);
    if (qzeros)
        hipLaunchKernelGGL(w4_tile16_zp4_kernel, dim3(ceil_div(n / 8, 256), groups), dim3(256), 0, s, qzeros, qzeros_t,
                           groups, n / 8);
    else
        hipLaunchKernelGGL(w4_tile16_kernel, dim3(gx.x, groups), dim3(256), 0, s,
                           reinterpret_cast<const uint4*>(zero_points), reinterpret_cast<uint4*>(zero_points_t), groups,
                           n);
    return check_launch("w4_tile16_kernel");
}

int rumus_hip_w4_decode_layout(const uint32_t* packed, const float* scales, const float* zero_points,
                               uint32_t padded_k, uint32_t n, uint32_t group_size, uint32_t* packed_t,
                               float* scales_t, float* zero_points_t, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(zero_points && zero_points_t, "w4_decode_layout: null buffer");
    return decode_layout(packed, scales, zero_points, nullptr, padded_k, n, group_size, packed_t, scales_t,
                         zero_points_t, nullptr, as_stream(stream));
}

int rumus_hip_w4_decode_layout_zp4(const uint32_t* packed, const float* scales, const uint32_t* qzeros,
                                   uint32_t padded_k, uint32_t n, uint32_t group_size, uint32_t* packed_t,
                                   float* scales_t, uint32_t* qzeros_t, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(qzeros && qzeros_t, "w4_decode_layout_zp4: null buffer");
    return decode_layout(packed, scales, nullptr, qzeros, padded_k, n, group_size, packed_t, scales_t, nullptr,
                         qzeros_t, as_stream(stream));
}

int rumus_hip_f16_to_f32(const uint16_t* in, float* out, uint64_t numel, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(numel == 0 || (in && out), "f16_to_f32: null buffer");
    RUMUS_REQUIRE(numel < (1ull << 39), "f16_to_f32: %llu elements are beyond the grid limit",
                  (unsigned long long)numel);
    if (numel == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(f16_to_f32_kernel, dim3((uint32_t)((numel + 255) / 256)), dim3(256), 0, as_stream(stream),
                       reinterpret_cast<const _Float16*>(in), out, numel);
    return check_launch("f16_to_f32_kernel");
}

int rumus_hip_w4_qzeros_unpack(const uint32_t* qzeros, uint32_t num_groups, uint32_t n, float* zero_points,
                               rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(qzeros && zero_points, "w4_qzeros_unpack: null buffer");
    RUMUS_REQUIRE(n % 8 == 0, "w4_qzeros_unpack: n must be a multiple of 8 (got %u)", n);
    RUMUS_REQUIRE((reinterpret_cast<uintptr_t>(zero_points) & 15) == 0,
                  "w4_qzeros_unpack: zero_points must be 16-byte aligned");
    RUMUS_REQUIRE(num_groups <= 65535, "w4_qzeros_unpack: %u groups are beyond the grid limit", num_groups);
    if (num_groups == 0 || n == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(w4_qzeros_unpack_kernel, dim3(ceil_div(n / 8, 256), num_groups), dim3(256), 0,
                       as_stream(stream), qzeros, zero_points, n);
    return check_launch("w4_qzeros_unpack_kernel");
}

int rumus_hip_w4_quantize_pack_awq(const float* w, uint32_t k, uint32_t n, uint32_t group_size,
                                   uint32_t* packed, float* scales, uint32_t* qzeros,
                                   rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(group_size > 0 && group_size % 8 == 0,
                  "w4_quantize_pack_awq: group_size must be a multiple of 8 (got %u)", group_size);
    RUMUS_REQUIRE(n % 8 == 0, "w4_quantize_pack_awq: n must be a multiple of 8 (got %u)", n);
    RUMUS_REQUIRE(n == 0 || k == 0 || (w && packed && scales && qzeros), "w4_quantize_pack_awq: null buffer");
    if (k == 0 || n == 0) return RUMUS_HIP_OK;
    const uint32_t groups = ceil_div(k, group_size);
    const dim3 grid(ceil_div(n, 256), groups);
    hipStream_t s = as_stream(stream);
    switch (group_size) {
        case 32: hipLaunchKernelGGL(w4_quantize_pack_awq_kernel<32>, grid, dim3(256), 0, s, w, k, n, group_size, packed, scales, qzeros); break;
        case 64: hipLaunchKernelGGL(w4_quantize_pack_awq_kernel<64>, grid, dim3(256), 0, s, w, k, n, group_size, packed, scales, qzeros); break;
        case 128: hipLaunchKernelGGL(w4_quantize_pack_awq_kernel<128>, grid, dim3(256), 0, s, w, k, n, group_size, packed, scales, qzeros); break;
        default: hipLaunchKernelGGL(w4_quantize_pack_awq_kernel<0>, grid, dim3(256), 0, s, w, k, n, group_size, packed, scales, qzeros);
    }
    return check_launch("w4_quantize_pack_awq_kernel");
}

int rumus_hip_w4_quantize_pack_sym(const float* w, uint32_t k, uint32_t n, uint32_t group_size,
                                   uint32_t* packed, float* scales, float* zero_points,
                                   rumus_hip_stream_t stream) {
    return quantize_pack<true>(w, k, n, group_size, packed, scales, zero_points, as_stream(stream));
}

// Synchronous by design (runs once per weight): g_idx is copied to the host,
// validated and stably sorted there, and the row gather runs on the device.
int rumus_hip_w4_actorder_prepare(const uint32_t* packed, const int32_t* g_idx, uint32_t padded_k,
                                  uint32_t n, uint32_t group_size, uint32_t* packed_sorted,
                                  int32_t* perm, rumus_hip_stream_t stream) {
    RUMUS_REQUIRE(group_size > 0 && group_size % 8 == 0,
                  "group_size must be a multiple of 8 (got %u)", group_size);
    RUMUS_REQUIRE(padded_k > 0 && padded_k % group_size == 0,
                  "actorder_prepare: padded_k %u is not a multiple of group_size %u", padded_k,
                  group_size);
    RUMUS_REQUIRE(packed && g_idx && packed_sorted && perm, "actorder_prepare: null buffer");
    RUMUS_REQUIRE(packed != packed_sorted, "actorder_prepare: cannot sort in place");
    hipStream_t s = as_stream(stream);
    const uint32_t groups = padded_k / group_size;
    std::vector<int32_t> gi(padded_k), pm(padded_k);
    if (int rc = check_hip(hipMemcpyAsync(gi.data(), g_idx, padded_k * sizeof(int32_t),
                                          hipMemcpyDeviceToHost, s), "copy g_idx"))
        return rc;
    if (int rc = check_hip(hipStreamSynchronize(s), "sync g_idx")) return rc;
    std::vector<uint32_t> count(groups, 0);
    for (uint32_t r = 0; r < padded_k; r++) {
        RUMUS_REQUIRE(gi[r] >= 0 && (uint32_t)gi[r] < groups, "actorder_prepare: g_idx[%u] = %d out of range",
                      r, gi[r]);
        count[gi[r]]++;
    }
    for (uint32_t g = 0; g < groups; g++)
        RUMUS_REQUIRE(count[g] == group_size, "actorder_prepare: group %u holds %u rows, expected %u", g,
                      count[g], group_size);
    std::vector<uint32_t> next(groups);
    for (uint32_t g = 0; g < groups; g++) next[g] = g * group_size;
    for (uint32_t r = 0; r < padded_k; r++) pm[next[gi[r]]++] = (int32_t)r;  // stable
    if (int rc = check_hip(hipMemcpyAsync(perm, pm.data(), padded_k * sizeof(int32_t),
                                          hipMemcpyHostToDevice, s), "copy perm"))
        return rc;
    if (int rc = check_hip(hipStreamSynchronize(s), "sync perm")) return rc;
    if (n == 0) return RUMUS_HIP_OK;
    hipLaunchKernelGGL(w4_gather_rows_kernel, dim3(ceil_div(n, 256), padded_k / 8), dim3(256), 0, s,
                       packed, perm, n, packed_sorted);
    if (int rc = check_launch("w4_gather_rows_kernel")) return rc;
    return check_hip(hipStreamSynchronize(s), "sync gather");
}

}  // extern "C"
