/*
 * rumus_oracle.c -- CPU restatement of the RUMUS quantized-Linear arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY (see rumus_oracle.h).  Scalar loops in the
 * reference's own loop order, single thread unless a `threads` argument asks
 * for OpenMP over output columns.  Build with -O2 -ffp-contract=off so that no
 * multiply-add is fused: every f32 operation below rounds once, as written.
 */
#include "rumus_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* small helpers                                                             */
/* ------------------------------------------------------------------------ */

/* Rust `f32 as i32`: saturating, NaN -> 0. */
static int32_t f32_as_i32_sat(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

static int32_t clamp_i32(int32_t v, int32_t lo, int32_t hi) {
    return v < lo ? lo : (v > hi ? hi : v);
}

/* IEEE binary32 -> binary16 bits, round-to-nearest-even (what numpy's
 * astype(float16) and the GPU's v_cvt_f16_f32 do). */
uint16_t orc_f32_to_f16_bits(float v) {
    uint32_t x;
    memcpy(&x, &v, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (absx > 0x7F800000u ? 0x0200u : 0));
    }
    if (absx >= 0x477FF000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x33000001u) { /* <= 2^-25 rounds to zero (tie at 2^-25 -> even = 0) */
        return (uint16_t)sign;
    }
    int32_t exp = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x007FFFFFu) | 0x00800000u; /* 24-bit significand */
    uint32_t shift;                                     /* bits dropped */
    uint32_t base;
    if (exp >= -14) { /* normal half */
        shift = 13;
        base = ((uint32_t)(exp + 15) << 10) - 0x400u; /* add man>>13 incl. hidden bit */
    } else { /* subnormal half: value = man * 2^(exp-23), unit = 2^-24 */
        shift = (uint32_t)(13 + (-14 - exp));
        base = 0;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1;
    return (uint16_t)(sign | (base + q));
}

float orc_f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* WGSL extract_i8 (matmul_q8.wgsl:32-35, dequantize.wgsl:26-30) */
static int32_t extract_i8(uint32_t word, uint32_t byte_pos) {
    uint32_t raw = (word >> (byte_pos * 8u)) & 0xFFu;
    return raw > 127u ? (int32_t)raw - 256 : (int32_t)raw;
}

/* ------------------------------------------------------------------------ */
/* INT4 engine                                                               */
/* ------------------------------------------------------------------------ */

/* quant.rs:42-102 */
int orc_w4_from_f32(const float* data, size_t k, size_t n, size_t group_size,
                    uint32_t* packed, float* scales, float* zero_points) {
    if (group_size == 0 || group_size % 8 != 0) return -1; /* quant.rs:43 */
    size_t padded_k = ((k + group_size - 1) / group_size) * group_size; /* :46 */
    size_t num_groups = padded_k / group_size;
    size_t num_words = (padded_k / 8) * n;

    /* :50-56 zero-padded copy */
    size_t padded_len = padded_k * n;
    float* padded = (float*)calloc(padded_len > 0 ? padded_len : 1, sizeof(float));
    if (!padded) return -2;
    for (size_t row = 0; row < k; row++)
        for (size_t col = 0; col < n; col++)
            padded[row * n + col] = data[row * n + col];

    /* :62-84 per (col, group) min/max -> scale, zp */
    for (size_t col = 0; col < n; col++) {
        for (size_t g = 0; g < num_groups; g++) {
            size_t start = g * group_size, end = start + group_size;
            float min_val = FLT_MAX;   /* f32::MAX */
            float max_val = -FLT_MAX;  /* f32::MIN */
            for (size_t row = start; row < end; row++) {
                float v = padded[row * n + col];
                if (v < min_val) min_val = v;
                if (v > max_val) max_val = v;
            }
            float range = max_val - min_val;
            float scale = range > 1e-10f ? range / 15.0f : 1.0f;
            float zp = range > 1e-10f ? -min_val / scale : 0.0f;
            scales[g * n + col] = scale;
            zero_points[g * n + col] = zp;
        }
    }

    /* :87-102 quantize + pack */
    memset(packed, 0, num_words * sizeof(uint32_t));
    for (size_t col = 0; col < n; col++) {
        for (size_t row = 0; row < padded_k; row++) {
            size_t g = row / group_size;
            float scale = scales[g * n + col];
            float zp = zero_points[g * n + col];
            float val = padded[row * n + col];
            float t = val / scale;
            t = t + zp;
            uint32_t q = (uint32_t)clamp_i32(f32_as_i32_sat(roundf(t)), 0, 15);
            size_t word_idx = (row / 8) * n + col;
            uint32_t nibble = (uint32_t)(row % 8);
            packed[word_idx] |= q << (nibble * 4u);
        }
    }
    free(padded);
    return 0;
}

/* EXTENSION: symmetric, zp = 8, scale = max|w|/7 (1.0 for an all-zero group). */
int orc_w4_sym_from_f32(const float* data, size_t k, size_t n, size_t group_size,
                        uint32_t* packed, float* scales, float* zero_points) {
    if (group_size == 0 || group_size % 8 != 0) return -1;
    size_t padded_k = ((k + group_size - 1) / group_size) * group_size;
    size_t num_groups = padded_k / group_size;
    size_t num_words = (padded_k / 8) * n;
    memset(packed, 0, num_words * sizeof(uint32_t));
    for (size_t col = 0; col < n; col++) {
        for (size_t g = 0; g < num_groups; g++) {
            float amax = 0.0f;
            for (size_t row = g * group_size; row < (g + 1) * group_size; row++) {
                float v = row < k ? fabsf(data[row * n + col]) : 0.0f;
                if (v > amax) amax = v;
            }
            float scale = amax > 0.0f ? amax / 7.0f : 1.0f;
            scales[g * n + col] = scale;
            if (zero_points) zero_points[g * n + col] = 8.0f;
            for (size_t row = g * group_size; row < (g + 1) * group_size; row++) {
                float v = row < k ? data[row * n + col] : 0.0f;
                float t = v / scale;
                int32_t q = clamp_i32(f32_as_i32_sat(roundf(t)) + 8, 0, 15);
                packed[(row / 8) * n + col] |= (uint32_t)q << ((row % 8) * 4u);
            }
        }
    }
    return 0;
}

/* EXTENSION: AWQ storage.  Integer zero-points, eight per u32 along N.
 *   scale = max(max - min, 1e-5) / 15;  z = clamp(-rint(min / scale), 0, 15)
 *   q = clamp(rint(w / scale) + z, 0, 15)          (rint: half to even)
 * which is AutoAWQ's pseudo_quantize_tensor with zero_point=True on w.view(-1, group).
 * qzeros[g * (n/8) + col/8] holds z of column col in bits 4*(col%8) .. +3. */
int orc_w4_awq_from_f32(const float* data, size_t k, size_t n, size_t group_size,
                        uint32_t* packed, float* scales, uint32_t* qzeros) {
    if (group_size == 0 || group_size % 8 != 0 || n % 8 != 0) return -1;
    size_t padded_k = ((k + group_size - 1) / group_size) * group_size;
    size_t num_groups = padded_k / group_size;
    memset(packed, 0, (padded_k / 8) * n * sizeof(uint32_t));
    memset(qzeros, 0, num_groups * (n / 8) * sizeof(uint32_t));
    for (size_t col = 0; col < n; col++) {
        for (size_t g = 0; g < num_groups; g++) {
            float mn = FLT_MAX, mx = -FLT_MAX;
            for (size_t row = g * group_size; row < (g + 1) * group_size; row++) {
                float v = row < k ? data[row * n + col] : 0.0f;
                if (v < mn) mn = v;
                if (v > mx) mx = v;
            }
            float range = mx - mn;
            if (!(range > 1e-5f)) range = 1e-5f;
            float scale = range / 15.0f;
            int32_t z = clamp_i32(-f32_as_i32_sat(rintf(mn / scale)), 0, 15);
            scales[g * n + col] = scale;
            qzeros[g * (n / 8) + col / 8] |= (uint32_t)z << ((col % 8) * 4u);
            for (size_t row = g * group_size; row < (g + 1) * group_size; row++) {
                float v = row < k ? data[row * n + col] : 0.0f;
                int32_t q = clamp_i32(f32_as_i32_sat(rintf(v / scale)) + z, 0, 15);
                packed[(row / 8) * n + col] |= (uint32_t)q << ((row % 8) * 4u);
            }
        }
    }
    return 0;
}

/* qmatmul_int4.wgsl:40-87 */
void orc_qmatmul_int4(const float* x, const uint32_t* packed, const float* scales,
                      const float* zp, const float* bias, const int32_t* g_idx,
                      float* y, uint32_t m, uint32_t k, uint32_t n,
                      uint32_t padded_k, uint32_t group_size, uint32_t num_groups,
                      int threads) {
    (void)padded_k;
    long long total = (long long)m * n;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
#else
    (void)threads;
#endif
    for (long long idx = 0; idx < total; idx++) {
        uint32_t row = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
        float sum = 0.0f;
        for (uint32_t g = 0; g < num_groups; g++) {
            size_t meta_idx = (size_t)g * n + col;
            float scale = scales[meta_idx];
            float z = zp[meta_idx];
            uint32_t k_start = g * group_size;
            uint32_t words_per_group = group_size / 8u;
            for (uint32_t w = 0; w < words_per_group; w++) {
                uint32_t k_base = k_start + w * 8u;
                size_t word_idx = (size_t)(k_base / 8u) * n + col;
                uint32_t word = packed[word_idx];
                for (uint32_t j = 0; j < 8u; j++) {
                    uint32_t kk = k_base + j;
                    if (kk >= k) break;
                    uint32_t q = (word >> (j * 4u)) & 0xFu;
                    if (g_idx) { /* EXTENSION: act-order metadata row */
                        size_t mi = (size_t)g_idx[kk] * n + col;
                        scale = scales[mi];
                        z = zp[mi];
                    }
                    float w_val = ((float)q - z) * scale;
                    float prod = x[(size_t)row * k + kk] * w_val;
                    sum = sum + prod;
                }
            }
        }
        if (bias) sum = sum + bias[col]; /* cpu.rs:73-81 */
        y[(size_t)row * n + col] = sum;
    }
}

/* qmatmul_int4_transpose.wgsl:37-74 */
void orc_qmatmul_int4_t(const float* a, const uint32_t* packed, const float* scales,
                        const float* zp, float* out, uint32_t m, uint32_t k,
                        uint32_t n, uint32_t padded_k, uint32_t group_size,
                        uint32_t num_groups, int threads) {
    (void)padded_k; (void)num_groups;
    long long total = (long long)m * k;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
#else
    (void)threads;
#endif
    for (long long idx = 0; idx < total; idx++) {
        uint32_t row = (uint32_t)(idx / k), k_col = (uint32_t)(idx % k);
        uint32_t word_row = k_col / 8u;
        uint32_t shift = (k_col % 8u) * 4u;
        uint32_t group = k_col / group_size;
        float sum = 0.0f;
        for (uint32_t c = 0; c < n; c++) {
            uint32_t word = packed[(size_t)word_row * n + c];
            uint32_t q = (word >> shift) & 0xFu;
            size_t meta_idx = (size_t)group * n + c;
            float w_val = ((float)q - zp[meta_idx]) * scales[meta_idx];
            float prod = a[(size_t)row * n + c] * w_val;
            sum = sum + prod;
        }
        out[(size_t)row * k + k_col] = sum;
    }
}

/* ------------------------------------------------------------------------ */
/* INT8 engine, reference format                                             */
/* ------------------------------------------------------------------------ */

/* core.rs:87-98 */
uint64_t orc_q8_buf_size(uint64_t numel, uint32_t block_size) {
    uint64_t num_blocks = (numel + block_size - 1) / block_size;
    uint64_t raw = num_blocks * (4 + (uint64_t)block_size);
    return (raw + 3) & ~(uint64_t)3;
}

/* quantize.wgsl:29-100 */
int orc_q8_quantize(const float* in, uint32_t* out, uint32_t numel, uint32_t block_size) {
    if (block_size == 0 || block_size % 4 != 0) return -1; /* ops.rs:2291 */
    uint32_t num_blocks = (numel + block_size - 1) / block_size;  /* compute.rs:1955 */
    uint32_t stride = (4 + block_size + 3) / 4;                   /* compute.rs:1956 */
    for (uint32_t b = 0; b < num_blocks; b++) {
        uint32_t elem_start = b * block_size;
        float abs_max = 0.0f;
        for (uint32_t i = 0; i < block_size; i++) {
            uint32_t gi = elem_start + i;
            if (gi < numel) {
                float av = fabsf(in[gi]);
                if (av > abs_max) abs_max = av;
            }
        }
        float scale = abs_max == 0.0f ? 1.0f : abs_max / 127.0f;     /* :66 */
        float inv_scale = abs_max == 0.0f ? 0.0f : 127.0f / abs_max; /* :67 */
        uint32_t base = b * stride;
        out[base] = (uint32_t)orc_f32_to_f16_bits(scale);            /* :71-74 */
        uint32_t num_data_words = (block_size + 3u) / 4u;
        for (uint32_t w = 0; w < num_data_words; w++) {
            uint32_t word = 0;
            for (uint32_t byte_idx = 0; byte_idx < 4u; byte_idx++) {
                uint32_t pos = w * 4u + byte_idx;
                uint32_t gi = elem_start + pos;
                int32_t q = 0;
                if (pos < block_size && gi < numel) {
                    float t = in[gi] * inv_scale;
                    q = clamp_i32(f32_as_i32_sat(nearbyintf(t)), -128, 127); /* :93 */
                }
                word |= ((uint32_t)q & 0xFFu) << (byte_idx * 8u);
            }
            out[base + 1u + w] = word;
        }
    }
    return 0;
}

/* dequantize.wgsl:32-52 */
void orc_q8_dequantize(const uint32_t* in, float* out, uint32_t numel, uint32_t block_size) {
    uint32_t stride = (4 + block_size + 3) / 4;
    for (uint32_t idx = 0; idx < numel; idx++) {
        uint32_t block_idx = idx / block_size;
        uint32_t pos = idx % block_size;
        uint32_t base = block_idx * stride;
        float scale = orc_f16_bits_to_f32((uint16_t)(in[base] & 0xFFFFu));
        int32_t q = extract_i8(in[base + 1u + pos / 4u], pos % 4u);
        out[idx] = (float)q * scale;
    }
}

/* matmul_q8.wgsl:37-98 */
void orc_matmul_q8(const float* a, const uint32_t* b, float* c, uint32_t m,
                   uint32_t k, uint32_t n, uint32_t block_size, int threads) {
    uint32_t blocks_per_col = (k + block_size - 1) / block_size; /* compute.rs:2029 */
    uint32_t stride = (4 + block_size + 3) / 4;                  /* compute.rs:2030 */
    long long total = (long long)m * n;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
#else
    (void)threads;
#endif
    for (long long idx = 0; idx < total; idx++) {
        uint32_t row = (uint32_t)(idx / n), col = (uint32_t)(idx % n);
        float sum = 0.0f;
        size_t col_base = (size_t)col * blocks_per_col * stride;
        uint32_t k_offset = 0;
        for (uint32_t blk = 0; blk < blocks_per_col; blk++) {
            size_t base = col_base + (size_t)blk * stride;
            float blk_scale = orc_f16_bits_to_f32((uint16_t)(b[base] & 0xFFFFu));
            uint32_t bs = block_size < k - k_offset ? block_size : k - k_offset;
            for (uint32_t r = 0; r < bs; r++) {
                int32_t q = extract_i8(b[base + 1u + r / 4u], r % 4u);
                float t = a[(size_t)row * k + k_offset + r] * (float)q;
                t = t * blk_scale;
                sum = sum + t;
            }
            k_offset += block_size;
        }
        c[(size_t)row * n + col] = sum;
    }
}

/* cpu.rs:73-81 */
void orc_add_bias(const float* mat, const float* bias, float* dst, size_t m, size_t n) {
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++)
            dst[i * n + j] = mat[i * n + j] + bias[j];
}

/* ops.rs:2307 (transpose + contiguous) */
void orc_transpose(const float* in, float* out, size_t rows, size_t cols) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++)
            out[c * rows + r] = in[r * cols + c];
}

/* ------------------------------------------------------------------------ */
/* INT8 engine, W8A8 extension                                               */
/* ------------------------------------------------------------------------ */

void orc_i8_quantize_rows(const float* x, int8_t* xq, float* scale,
                          size_t rows, size_t cols) {
    for (size_t r = 0; r < rows; r++) {
        const float* xr = x + r * cols;
        float abs_max = 0.0f;
        for (size_t c = 0; c < cols; c++) {
            float av = fabsf(xr[c]);
            if (av > abs_max) abs_max = av;
        }
        float s = abs_max == 0.0f ? 1.0f : abs_max / 127.0f;
        float inv = abs_max == 0.0f ? 0.0f : 127.0f / abs_max;
        scale[r] = s;
        for (size_t c = 0; c < cols; c++) {
            float t = xr[c] * inv;
            xq[r * cols + c] = (int8_t)clamp_i32(f32_as_i32_sat(nearbyintf(t)), -128, 127);
        }
    }
}

void orc_i8_gemm_i32(const int8_t* xq, const int8_t* wq, int32_t* acc,
                     size_t m, size_t k, size_t n, int threads) {
    long long total = (long long)m * (long long)n;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
#else
    (void)threads;
#endif
    for (long long idx = 0; idx < total; idx++) {
        size_t i = (size_t)(idx / (long long)n), j = (size_t)(idx % (long long)n);
        const int8_t* a = xq + i * k;
        const int8_t* b = wq + j * k;
        int32_t s = 0;
        for (size_t p = 0; p < k; p++) s += (int32_t)a[p] * (int32_t)b[p];
        acc[i * n + j] = s;
    }
}

void orc_i8_rescale_bias(const int32_t* acc, const float* sx, const float* sw,
                         const float* bias, float* y, size_t m, size_t n) {
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            float t = (float)acc[i * n + j] * sx[i];
            t = t * sw[j];
            if (bias) t = t + bias[j];
            y[i * n + j] = t;
        }
}
