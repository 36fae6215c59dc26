/*
 * rumus_oracle.h -- CPU restatement of the RUMUS quantized-Linear arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker for the HIP kernels:
 * it is linked/loaded by tests, by the smoke check and by the CPU-baseline leg
 * of the benchmark, and by nothing else.  The product library never calls it.
 *
 * Every function follows one reference source (paths relative to the RUMUS
 * checkout); functions marked EXTENSION have no reference code and restate the
 * closed form the HIP kernels implement.
 *
 * Pin status (what fixes the result independently of this file):
 *   orc_w4_from_f32         hand-computed known answers (exact power-of-two
 *                           scales, half-away ties, constant group, K padding)
 *                           + invariants (min->0, max->15, |err|<=scale/2)
 *   orc_qmatmul_int4(_t)    float64 numpy matmul of the dequantized matrix,
 *                           exact-integer special case, linearity
 *   orc_q8_quantize         hand-computed known answers (half-even ties,
 *                           zero block, f16 header vs numpy float16)
 *   orc_q8_dequantize       exact: numpy int8*float16 product
 *   orc_matmul_q8           float64 numpy matmul, exact-integer special case
 *   orc_add_bias            exact single add
 *   orc_i8_quantize_rows    EXTENSION: same known answers as orc_q8_quantize
 *   orc_i8_gemm_i32         EXTENSION: numpy int32/int64 matmul, bit-exact
 *   orc_i8_rescale_bias     EXTENSION: float64 closed form
 *   orc_w4_sym_from_f32     EXTENSION: known answers (zp=8, scale=max|w|/7)
 *   orc_w4_awq_from_f32     EXTENSION: known answers (exact power-of-two scale,
 *                           half-even ties, nibble order of qzeros) + numpy
 *                           restatement of the published AutoAWQ formula
 * The reference ships no test, fixture or golden vector for this path and its
 * Rust/WGSL sources cannot be built in this environment, so none of the above
 * is pinned by running the reference; f32 matmul outputs of the reference
 * depend on the WGSL driver's FMA contraction and are compared by tolerance.
 */
#ifndef RUMUS_ORACLE_H
#define RUMUS_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- INT4 engine ------------------------------------------------------- */

/* rumus-vision/src/quant.rs:42-102  QuantizedTensor::from_f32.
 * data [k,n] row-major; packed [(padded_k/8), n]; scales, zp [num_groups, n].
 * Returns 0, or -1 when group_size % 8 != 0 (the reference asserts). */
int orc_w4_from_f32(const float* data, size_t k, size_t n, size_t group_size,
                    uint32_t* packed, float* scales, float* zero_points);

/* EXTENSION: symmetric 4-bit, zero-point fixed at 8, scale = max|w|/7 per
 * (group, column), q = clamp(round_half_away(w/scale) + 8, 0, 15).
 * zero_points (may be NULL) is filled with 8.0f. */
int orc_w4_sym_from_f32(const float* data, size_t k, size_t n, size_t group_size,
                        uint32_t* packed, float* scales, float* zero_points);

/* EXTENSION: AWQ storage (integer zero-points, eight per u32 along N):
 * scale = max(max-min, 1e-5)/15, z = clamp(-rint(min/scale), 0, 15),
 * q = clamp(rint(w/scale) + z, 0, 15), rint = half to even.
 * qzeros [num_groups, n/8], column col in bits 4*(col%8).  -1 unless n % 8 == 0. */
int orc_w4_awq_from_f32(const float* data, size_t k, size_t n, size_t group_size,
                        uint32_t* packed, float* scales, uint32_t* qzeros);

/* rumus-vision/src/shaders/qmatmul_int4.wgsl:40-87 (one invocation per
 * (row, col); strictly ascending k; w=(f32(q)-zp)*scale, then sum += a*w).
 * EXTENSION: g_idx != NULL selects scale/zp row g_idx[k] per k (act-order);
 * g_idx == NULL is the reference.  bias != NULL adds bias[col] afterwards
 * (rumus/src/backend/cpu.rs:73-81).  threads>1 splits columns with OpenMP. */
void orc_qmatmul_int4(const float* x, const uint32_t* packed, const float* scales,
                      const float* zp, const float* bias, const int32_t* g_idx,
                      float* y, uint32_t m, uint32_t k, uint32_t n,
                      uint32_t padded_k, uint32_t group_size, uint32_t num_groups,
                      int threads);

/* rumus-vision/src/shaders/qmatmul_int4_transpose.wgsl:37-74.
 * a [m,n] -> out [m,k]; sum over n ascending. */
void orc_qmatmul_int4_t(const float* a, const uint32_t* packed, const float* scales,
                        const float* zp, float* out, uint32_t m, uint32_t k,
                        uint32_t n, uint32_t padded_k, uint32_t group_size,
                        uint32_t num_groups, int threads);

/* ---- INT8 engine (reference format: W8A32, f16 block header) ------------ */

/* rumus/src/tensor/core.rs:87-98: bytes of a Q8 buffer for numel elements. */
uint64_t orc_q8_buf_size(uint64_t numel, uint32_t block_size);

/* rumus/src/backend/gpu/shaders/quantize.wgsl:29-100 (+ compute.rs:1955-1956).
 * in: numel f32 (already in the order to be blocked); out: num_blocks *
 * ((4+bs+3)/4) words.  f32->f16 of the scale is round-to-nearest-even. */
int orc_q8_quantize(const float* in, uint32_t* out, uint32_t numel, uint32_t block_size);

/* rumus/src/backend/gpu/shaders/dequantize.wgsl:32-52 */
void orc_q8_dequantize(const uint32_t* in, float* out, uint32_t numel, uint32_t block_size);

/* rumus/src/backend/gpu/shaders/matmul_q8.wgsl:37-98: sum += (a*f32(q))*scale. */
void orc_matmul_q8(const float* a, const uint32_t* b, float* c, uint32_t m,
                   uint32_t k, uint32_t n, uint32_t block_size, int threads);

/* rumus/src/backend/cpu.rs:73-81 */
void orc_add_bias(const float* mat, const float* bias, float* dst, size_t m, size_t n);

/* rumus/src/tensor/ops.rs:2307: transpose [k,n] -> [n,k] before blocking. */
void orc_transpose(const float* in, float* out, size_t rows, size_t cols);

/* ---- INT8 engine (EXTENSION: W8A8, i32 accumulate) ---------------------- */

/* quantize.wgsl:66-67,93 applied to each row of x[rows,cols]; f32 scale out. */
void orc_i8_quantize_rows(const float* x, int8_t* xq, float* scale,
                          size_t rows, size_t cols);

/* acc[m,n] = sum_k xq[m,k] * wq[n,k]  (wq is [n,k], K contiguous). */
void orc_i8_gemm_i32(const int8_t* xq, const int8_t* wq, int32_t* acc,
                     size_t m, size_t k, size_t n, int threads);

/* y = (f32(acc)*sx[m])*sw[n] (+ bias[n]) */
void orc_i8_rescale_bias(const int32_t* acc, const float* sx, const float* sw,
                         const float* bias, float* y, size_t m, size_t n);

/* helpers exported for tests */
uint16_t orc_f32_to_f16_bits(float v);
float orc_f16_bits_to_f32(uint16_t h);

#ifdef __cplusplus
}
#endif
#endif
