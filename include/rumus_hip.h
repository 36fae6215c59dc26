/*
 * rumus_hip.h -- C ABI of librumus_hip.so: the MI355X (gfx950) device code for
 * RUMUS's quantized-Linear path.
 *
 * Every entry point is what a RUMUS dispatch function for this path would bind
 * through FFI; the reference interface each one replaces is cited as
 * file:line relative to the RUMUS checkout.  Entry points marked EXTENSION
 * have no reference counterpart (the W8A8 INT8 engine, symmetric / act-order
 * INT4) and follow the closed forms given in their comments.
 *
 * Conventions
 *   - every pointer is a caller-owned DEVICE pointer (hipMalloc'd) unless it
 *     is said to be a host pointer; the library never frees caller memory and
 *     allocates nothing on the launch path;
 *   - a call whose batch is empty (zero rows, zero elements) succeeds, queues
 *     nothing and reads no array: the pointers of such a call may be NULL, as
 *     the data pointer of an empty tensor is.  The scalar preconditions
 *     (group and block sizes, divisibility) are checked all the same;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     launches are asynchronous on that stream, like wgpu's queue.submit
 *     (rumus/src/backend/gpu/compute.rs:1981);
 *   - every function returns 0 on success or a RUMUS_HIP_E* code, and
 *     rumus_hip_last_error() then returns a thread-local message.  The
 *     reference panics on the same preconditions (assert!/expect); a Rust
 *     shim turns a non-zero status into panic! to keep that behaviour;
 *   - functions are re-entrant and thread-safe: any number of host threads may
 *     call any entry point at once, on the same or on different streams (the
 *     reference runs ops from several threads, rumus/src/nn/parallel.rs:84).  A
 *     call that queues several kernels which share the stream's workspace holds
 *     that stream's workspace lock until its last kernel is queued, so calls of
 *     two threads on one stream are queued one whole call after the other; calls
 *     on different streams never wait for each other.
 */
#ifndef RUMUS_HIP_H
#define RUMUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RUMUS_HIP_OK 0
#define RUMUS_HIP_EINVAL 1 /* a precondition the reference asserts does not hold */
#define RUMUS_HIP_EHIP 2   /* a HIP runtime call failed */

typedef void* rumus_hip_stream_t;

/* ---- runtime ------------------------------------------------------------ */

/* GpuContext::get() (rumus/src/backend/gpu/context.rs:779-820): select the
 * device and cache its properties.  Optional: launches work without it on the
 * current device. */
int rumus_hip_init(int device);

/* Message for the last non-zero status returned on this thread. */
const char* rumus_hip_last_error(void);

/* "rumus-hip <version> gfx950" */
const char* rumus_hip_version(void);

/* device.poll(Wait) (context.rs:840-850): block until `stream` is idle. */
int rumus_hip_sync(rumus_hip_stream_t stream);

/* Workspace.  The reference takes every temporary from its BufferPool
 * (rumus/src/backend/gpu/pool.rs:34-75) and returns it on drop; here the
 * temporaries live in one device buffer per (device, stream), grown on demand
 * inside the call that needs it.  A caller that must not allocate later
 * (graph capture, serving loop) reserves the largest size up front.  Upper
 * bounds per call, in bytes:
 *   qmatmul_int4 / _perm / _zp4, m > 5: 5 * (m + 64) * (padded_k + 128) (activations
 *       in matrix-core order and a scale factor per row) + 64 * m * n (partial
 *       sums, only while the output has fewer than 192 tiles of 64 x 512) + 1280
 *       (the last kilobyte: flags of the look at the zero-point table);
 *   qmatmul_int4_t, m >= 8: 64 * m * k (partial sums, only below 512 tiles of
 *       64 x 128) + 10 * num_groups * n + 4 * (m + num_groups) + 2048;
 *   i8_gemm: rumus_hip_i8_gemm_workspace_size(m, k, n) exactly; at most
 *       min(32 * m * n, 16 MiB);
 *   matmul_q8, m >= 5: 4 * m * k * 4 (digit planes of a) + 4 * m * n * 4 + 32 MiB
 *       (partial sums of the int8 GEMM inside); with one block per column from
 *       384 rows on also k * n + 4 * n;
 *   attention with q_len == 1: batch * heads * ceil(kv_len / 64) * 520.
 * rumus_hip_shutdown frees every workspace (no launch may be in flight). */
int rumus_hip_workspace_reserve(rumus_hip_stream_t stream, uint64_t bytes);
int rumus_hip_shutdown(void);

/* ---- INT8 engine, reference Q8 block format ----------------------------- */

/* DType::Q8{block_size}.gpu_buf_size(numel) (rumus/src/tensor/core.rs:87-98):
 * num_blocks*(4+block_size) bytes rounded up to 4. */
uint64_t rumus_hip_q8_buf_size(uint64_t numel, uint32_t block_size);

/* quantize_dispatch (compute.rs:1948-1982) + quantize_kernel
 * (shaders/quantize.wgsl:29-100).  in: numel f32, already in the order to be
 * blocked.  out: per block one header word (f16 scale in the low 16 bits) and
 * block_size/4 data words of little-endian signed bytes.
 * EINVAL unless block_size > 0 and block_size % 4 == 0 (ops.rs:2291). */
int rumus_hip_q8_quantize(const float* in, uint32_t* out, uint32_t numel,
                          uint32_t block_size, rumus_hip_stream_t stream);

/* dequantize_dispatch (compute.rs:1985-2018) + dequantize_kernel
 * (shaders/dequantize.wgsl:32-52): out[i] = f32(q[i]) * f16scale(block i/bs). */
int rumus_hip_q8_dequantize(const uint32_t* in, float* out, uint32_t numel,
                            uint32_t block_size, rumus_hip_stream_t stream);

/* The same values in the order of the tensor's shape: Tensor::quantize stores
 * the transposed [N,K] tensor (ops.rs:2307), so rumus_hip_q8_dequantize - like
 * Tensor::dequantize (ops.rs:2332-2352) - returns [N,K] order under the [K,N]
 * shape.  This returns out[kk*n + col] = value at flat index col*k + kk, i.e.
 * the dequantized [K,N] weight; bit-identical values, k*n = numel. */
int rumus_hip_q8_dequantize_kn(const uint32_t* in, float* out, uint32_t k, uint32_t n,
                               uint32_t block_size, rumus_hip_stream_t stream);

/* matmul_q8_dispatch (compute.rs:2021-2060) + matmul_q8_kernel
 * (shaders/matmul_q8.wgsl:37-98): c[m,n] = a[m,k] f32 x Q8 b, where column j
 * of b is the run of ceil(k/block_size) blocks starting at word
 * j*blocks_per_col*stride.  Results are within f32 summation error of the
 * reference's loop (block_size % 16 != 0: the same operations in the same
 * order).  Batches of 5 rows or more with block_size % 32 == 0 run on the
 * matrix cores and use the stream's internal workspace (4 bytes per element
 * of a, plus partial results for small m; one block per column from 384 rows
 * on: also a dense copy of b). */
int rumus_hip_matmul_q8(const float* a, const uint32_t* b, float* c, uint32_t m,
                        uint32_t k, uint32_t n, uint32_t block_size,
                        rumus_hip_stream_t stream);

/* The per-output-channel case of matmul_q8_dispatch (compute.rs:2021-2060 with
 * block_size >= k, one block per column) for a weight that is multiplied more
 * than once: rumus_hip_q8_dense_layout copies the Q8 buffer once into a dense
 * int8 matrix wq [n, k] (row j = the k quantized values of column j) and its n
 * block scales sw (the f16 header of block j, widened), and
 * rumus_hip_matmul_q8_dense multiplies against that copy without touching the
 * Q8 buffer: c[m,n] = a[m,k] x (wq, sw), bit for bit what rumus_hip_matmul_q8
 * returns on its matrix-core route for the same tensor (m >= 384 there; here
 * any m).  k % 16 == 0; a, wq, c 16-byte aligned; n <= 65535 for the layout
 * call.  Workspace of the stream: 4 bytes per element of a (+ 16 per row), and
 * below about a thousand rows also 16 bytes per element of c. */
int rumus_hip_q8_dense_layout(const uint32_t* b_q8, uint32_t k, uint32_t n, uint32_t block_size,
                              int8_t* wq, float* sw, rumus_hip_stream_t stream);
int rumus_hip_matmul_q8_dense(const float* a, const int8_t* wq, const float* sw, float* c,
                              uint32_t m, uint32_t k, uint32_t n, rumus_hip_stream_t stream);

/* Tensor::add_bias (rumus/src/tensor/ops.rs:885-931, shaders/bias.wgsl:18-25):
 * out[i,j] = mat[i,j] + bias[j].  out may alias mat. */
int rumus_hip_add_bias(const float* mat, const float* bias, float* out,
                       uint32_t m, uint32_t n, rumus_hip_stream_t stream);

/* transpose(-2,-1).contiguous() that Tensor::quantize runs first
 * (ops.rs:2307): out[c,r] = in[r,c]. */
int rumus_hip_transpose_f32(const float* in, float* out, uint32_t rows,
                            uint32_t cols, rumus_hip_stream_t stream);

/* ---- INT8 engine, W8A8 (EXTENSION) -------------------------------------- */

/* Dynamic per-row quantizer: for each row r of x[rows,cols]
 *   amax = max|x[r,:]|; scale[r] = amax==0 ? 1 : amax/127;
 *   inv = amax==0 ? 0 : 127/amax; xq[r,c] = clamp(rint(x[r,c]*inv),-128,127)
 * i.e. quantize.wgsl:66-67,93 per row, with the scale kept in f32. */
int rumus_hip_i8_quantize_rows(const float* x, int8_t* xq, float* scale,
                               uint32_t rows, uint32_t cols,
                               rumus_hip_stream_t stream);

/* Per-output-channel weight quantizer for a Linear weight w[k,n] ([in,out],
 * rumus/src/nn/linear.rs:39-46): same formula per COLUMN of w; the result is
 * written transposed, wq[n,k] (K contiguous), with sw[n]. */
int rumus_hip_i8_quantize_cols_t(const float* w, int8_t* wq, float* sw,
                                 uint32_t k, uint32_t n, rumus_hip_stream_t stream);

/* acc[m,n] = sum_k xq[m,k]*wq[n,k] on the i8 matrix cores (exact i32), then
 * y[m,n] = (f32(acc)*sx[m])*sw[n] (+ bias[n]).
 * acc may be NULL (accumulators not stored); y may be NULL (only acc stored,
 * sx/sw/bias ignored); bias may be NULL.  EINVAL unless k % 16 == 0. */
int rumus_hip_i8_gemm(const int8_t* xq, const int8_t* wq, const float* sx,
                      const float* sw, const float* bias, int32_t* acc, float* y,
                      uint32_t m, uint32_t k, uint32_t n, rumus_hip_stream_t stream);

/* Workspace bytes rumus_hip_i8_gemm takes on its stream for an m x k x n
 * product: i32 partial sums where K is shared over workgroups (outputs of few
 * tiles), 0 otherwise; never more than 16 MiB.  Host arithmetic only, for
 * rumus_hip_workspace_reserve.  No counterpart in the reference (its BufferPool
 * sizes temporaries inside the op, rumus/src/backend/gpu/pool.rs:34-75). */
uint64_t rumus_hip_i8_gemm_workspace_size(uint32_t m, uint32_t k, uint32_t n);

/* ---- INT4 engine --------------------------------------------------------- */

/* QuantizedTensor::from_f32 (rumus-vision/src/quant.rs:42-102) on the device:
 * w[k,n] f32 -> packed u32 [(padded_k/8), n], scales and zero_points f32
 * [num_groups, n], with padded_k = ceil(k/group_size)*group_size.
 * EINVAL unless group_size % 8 == 0 (quant.rs:43). */
int rumus_hip_w4_quantize_pack(const float* w, uint32_t k, uint32_t n,
                               uint32_t group_size, uint32_t* packed,
                               float* scales, float* zero_points,
                               rumus_hip_stream_t stream);

/* EXTENSION: symmetric 4-bit, zero-point 8: scale = max|w|/7 per (group,col)
 * (1 for an all-zero group), q = clamp(round_half_away(w/scale)+8, 0, 15).
 * zero_points (may be NULL) is filled with 8.0f. */
int rumus_hip_w4_quantize_pack_sym(const float* w, uint32_t k, uint32_t n,
                                   uint32_t group_size, uint32_t* packed,
                                   float* scales, float* zero_points,
                                   rumus_hip_stream_t stream);

/* EXTENSION: AWQ storage, integer zero-points packed eight per u32 along n
 * (the reference keeps an unrounded f32 zero-point per group and column,
 * quant.rs:77-79, which a u4 cannot hold, so this is a second format, not a
 * re-encoding):  scale = max(max-min, 1e-5)/15,
 *   z = clamp(-rint(min/scale), 0, 15),  q = clamp(rint(w/scale) + z, 0, 15),
 * rint = half to even (AutoAWQ's pseudo-quantizer).  packed and scales as
 * above; qzeros u32 [num_groups, n/8], column col in bits 4*(col%8) of word
 * col/8.  EINVAL unless group_size % 8 == 0 and n % 8 == 0. */
int rumus_hip_w4_quantize_pack_awq(const float* w, uint32_t k, uint32_t n,
                                   uint32_t group_size, uint32_t* packed,
                                   float* scales, uint32_t* qzeros,
                                   rumus_hip_stream_t stream);

/* EXTENSION: u4 zero-points of a stored checkpoint (qzeros u32 [num_groups,
 * n/8], column col in bits 4*(col%8) of word col/8) -> the f32 zero-point
 * array of the reference's QuantizedTensor (quant.rs:29-31,77-79), exactly.
 * EINVAL unless n % 8 == 0 and zero_points is 16-byte aligned. */
int rumus_hip_w4_qzeros_unpack(const uint32_t* qzeros, uint32_t num_groups,
                               uint32_t n, float* zero_points,
                               rumus_hip_stream_t stream);

/* EXTENSION: IEEE half -> f32, exact (scales of stored checkpoints kept in
 * half precision; the reference's scales are f32, quant.rs:29).  No
 * counterpart in the reference. */
int rumus_hip_f16_to_f32(const uint16_t* in, float* out, uint64_t numel,
                         rumus_hip_stream_t stream);

/* custom_forward(&QMatMulINT4FwdOp, [x, packed, scales, zp]) followed by
 * add_bias (rumus-vision/src/quant.rs:191-221,228-256; kernel
 * shaders/qmatmul_int4.wgsl:40-87).  The six scalars are the op's uniform
 * (quant.rs:243-249).  y[m,n] = x[m,k] . dequant(W) (+ bias[n]),
 * dequant = (q - zp[g,n]) * scales[g,n], g = row/group_size.
 * bias may be NULL.  EXTENSION: g_idx (device int32[k], may be NULL) replaces
 * g by g_idx[row] (act-order).
 * EINVAL unless group_size % 8 == 0, padded_k == num_groups*group_size,
 * k <= padded_k < k+group_size.
 * Numerics: within rel 1e-3 / abs 1e-4 of the reference's f32 loop; rows of
 * any magnitude; a NaN or an infinity in x poisons its own row only.  Up to
 * 128 rows (up to 1024 where the integer matrix-core kernel is the faster one:
 * group_size % 64 == 0 and enough columns to fill the chip) x is held in fixed
 * point below the largest magnitude of a part of the row (20 bits per 32 k up
 * to decode_max_rows rows, 22 bits per eighth of K beyond):
 * |error| <= max|x| * 2^-19 * sum|w| over that part.  Elements
 * that tower over their part by 2^8 or more are multiplied in f32 on their
 * own (all of a chunk of 32 k in the few-row kernel; up to 16 elements per
 * row and eighth of K beyond), so single outlier channels of thousands of
 * sigma keep the tolerance.  The u4-zero-point decode entry point
 * (rumus_hip_qmatmul_int4_decode_zp4) does not make that exception and keeps
 * the plain bound.  Larger batches, and those the f16 tile kernel takes, keep
 * 22 bits of every element and add in f32.  That kernel is faster on tables
 * of integer zero-points (what AWQ and GPTQ checkpoints hold; it looks before
 * it multiplies): an eighth of its work at groups of 128, more at smaller
 * groups, exists only for their fractional part. */
int rumus_hip_qmatmul_int4(const float* x, const uint32_t* packed,
                           const float* scales, const float* zero_points,
                           const float* bias, const int32_t* g_idx, float* y,
                           uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                           uint32_t group_size, uint32_t num_groups,
                           rumus_hip_stream_t stream);

/* The two quantized matmuls with half-precision activations.  The reference's
 * kernels are typed `scalar` = f32 or f16 as the activations are
 * (rumus/src/backend/gpu/shaders/matmul_q8.wgsl:1-5,26-28,
 * rumus-vision/src/shaders/qmatmul_int4.wgsl:33-38; the type is picked at
 * rumus/src/ext/mod.rs:132-150): in f16 mode activations, output and the
 * running sum are f16.  Here a / x and c / y are IEEE half (uint16_t bits),
 * the product runs in the f32 kernels of rumus_hip_matmul_q8 /
 * rumus_hip_qmatmul_int4 on the widened activations (same arguments, same
 * checks, same accuracy) and the result is rounded to f16 once, to nearest
 * even.  Scales, zero-points and bias stay f32 (convert stored f16 metadata
 * once with rumus_hip_f16_to_f32).  The f32 copies live in a staging buffer
 * per (device, stream) of 4 * m * (k + n) + 512 bytes, grown inside the call
 * like the workspace; rumus_hip_f16_staging_reserve sizes it up front for
 * callers that must not allocate later; rumus_hip_shutdown frees it. */
int rumus_hip_matmul_q8_f16(const uint16_t* a, const uint32_t* b, uint16_t* c,
                            uint32_t m, uint32_t k, uint32_t n, uint32_t block_size,
                            rumus_hip_stream_t stream);
int rumus_hip_qmatmul_int4_f16(const uint16_t* x, const uint32_t* packed,
                               const float* scales, const float* zero_points,
                               const float* bias, const int32_t* g_idx, uint16_t* y,
                               uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                               uint32_t group_size, uint32_t num_groups,
                               rumus_hip_stream_t stream);
int rumus_hip_f16_staging_reserve(rumus_hip_stream_t stream, uint64_t bytes);

/* rumus_hip_qmatmul_int4_perm for callers that cannot allocate (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments, same kernels and the same
 * bits as rumus_hip_qmatmul_int4_perm, but what that call parks in the
 * stream's workspace between its kernels (activations in matrix-core order,
 * partial tiles while K is shared over workgroups) lives in a static device
 * array of rumus_hip_static_scratch_bytes() = 32 MiB that each GPU holds
 * until the process ends; nothing is allocated or freed, on any call.
 * EINVAL ("needs ... bytes of scratch memory") when the shape needs more than
 * the array holds; the need is the qmatmul_int4 line of the workspace bounds
 * above and does not grow evenly with m: batches that share K over
 * workgroups of the f16 tile kernel (few output tiles) need room for their
 * partial sums.  With k = 4096, n = 11008 and groups of 128 every call up to
 * about 1900 rows runs; with groups of 32 (which the integer kernel does not
 * take) calls of 318 to 383 rows are refused.
 * All calls on one GPU share the one array, whatever their stream: calls that
 * overlap in time on one GPU race (calls on one stream do not overlap).
 * Nothing in the array has to start at zero: every byte a kernel reads from
 * it is written earlier in the same call. */
int rumus_hip_qmatmul_int4_perm_static(const float* x, const uint32_t* packed_sorted,
                                       const float* scales, const float* zero_points,
                                       const float* bias, const int32_t* perm, float* y,
                                       uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                                       uint32_t group_size, uint32_t num_groups,
                                       rumus_hip_stream_t stream);
uint64_t rumus_hip_static_scratch_bytes(void);

/* custom_forward(&QMatMulINT4TransposeOp, [grad_y, packed, scales, zp])
 * (quant.rs:262-317; kernel shaders/qmatmul_int4_transpose.wgsl:37-74):
 * out[m,k] = a[m,n] . dequant(W)^T. */
int rumus_hip_qmatmul_int4_t(const float* a, const uint32_t* packed,
                             const float* scales, const float* zero_points,
                             float* out, uint32_t m, uint32_t k, uint32_t n,
                             uint32_t padded_k, uint32_t group_size,
                             uint32_t num_groups, rumus_hip_stream_t stream);

/* EXTENSION (act-order, done once per weight): stable-sort the rows of W by
 * g_idx so that every group is contiguous.  perm[j] (int32[padded_k]) is the
 * original row stored at sorted position j; packed_sorted has the layout of
 * packed.  EINVAL unless every group holds exactly group_size rows. */
int rumus_hip_w4_actorder_prepare(const uint32_t* packed, const int32_t* g_idx,
                                  uint32_t padded_k, uint32_t n, uint32_t group_size,
                                  uint32_t* packed_sorted, int32_t* perm,
                                  rumus_hip_stream_t stream);

/* EXTENSION: qmatmul_int4 on a weight prepared by rumus_hip_w4_actorder_prepare:
 * y[m,n] = sum_j x[m,perm[j]] * (q_sorted[j,n]-zp[j/gs,n])*scales[j/gs,n].
 * perm == NULL means the identity.  Requires k == padded_k when perm != NULL. */
int rumus_hip_qmatmul_int4_perm(const float* x, const uint32_t* packed_sorted,
                                const float* scales, const float* zero_points,
                                const float* bias, const int32_t* perm, float* y,
                                uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                                uint32_t group_size, uint32_t num_groups,
                                rumus_hip_stream_t stream);

/* EXTENSION (decode layout, done once per weight): tile-major copies of the
 * three arrays of a QuantizedTensor, tile = 16 columns over all rows:
 *   packed_t[(c*(padded_k/8) + r)*16 + j] = packed[r*n + 16*c + j]
 *   scales_t[(c*num_groups + g)*16 + j]   = scales[g*n + 16*c + j]   (zero_points alike)
 * Same words, same sizes, another order: the decode kernel's workgroup (16
 * columns, all of K) then reads one contiguous slab.  EINVAL unless n % 16 == 0. */
int rumus_hip_w4_decode_layout(const uint32_t* packed, const float* scales,
                               const float* zero_points, uint32_t padded_k, uint32_t n,
                               uint32_t group_size, uint32_t* packed_t, float* scales_t,
                               float* zero_points_t, rumus_hip_stream_t stream);

/* EXTENSION: QLinear::forward for m <= 8 on the decode layout; same arithmetic
 * and results as rumus_hip_qmatmul_int4_perm (bit for bit).  perm may be NULL.
 * EINVAL unless m <= 8, n % 16 == 0, group_size % 32 == 0. */
int rumus_hip_qmatmul_int4_decode(const float* x, const uint32_t* packed_t,
                                  const float* scales_t, const float* zero_points_t,
                                  const float* bias, const int32_t* perm, float* y,
                                  uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                                  uint32_t group_size, uint32_t num_groups,
                                  rumus_hip_stream_t stream);

/* Rows of x up to which the decode entry points are the faster way to run a
 * [padded_k, n] weight (between 1 and 8, from measurements; beyond it
 * rumus_hip_qmatmul_int4 takes the matrix cores).  The dispatch inside
 * rumus_hip_qmatmul_int4 uses the same number.  No counterpart in the reference. */
uint32_t rumus_hip_qmatmul_int4_decode_max_rows(uint32_t padded_k, uint32_t n);

/* EXTENSION: the decode layout and its matmul for AWQ storage (u4 zero-points,
 * rumus_hip_w4_quantize_pack_awq): packed_t and scales_t as in
 * rumus_hip_w4_decode_layout; qzeros_t[(c*num_groups + g)*2 + h] =
 * qzeros[g*(n/8) + 2*c + h], the two zero-point words of tile c's 16 columns.
 * Same bits as rumus_hip_qmatmul_int4_zp4 on the row-major arrays while m is
 * within rumus_hip_qmatmul_int4_decode_max_rows, except for one row with
 * group_size % 64 == 0: that case fixes the point of x per 64 rows instead of
 * 32 here (same tolerance, other bits).
 * EINVAL as for the f32 zero-point forms.  No counterpart in the reference. */
int rumus_hip_w4_decode_layout_zp4(const uint32_t* packed, const float* scales,
                                   const uint32_t* qzeros, uint32_t padded_k, uint32_t n,
                                   uint32_t group_size, uint32_t* packed_t, float* scales_t,
                                   uint32_t* qzeros_t, rumus_hip_stream_t stream);
int rumus_hip_qmatmul_int4_decode_zp4(const float* x, const uint32_t* packed_t,
                                      const float* scales_t, const uint32_t* qzeros_t,
                                      const float* bias, const int32_t* perm, float* y,
                                      uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                                      uint32_t group_size, uint32_t num_groups,
                                      rumus_hip_stream_t stream);

/* EXTENSION: rumus_hip_qmatmul_int4_decode whose input is the output of a
 * fused gate|up projection: gate_up [m, 2k] (gate in columns 0..k-1, up in
 * k..2k-1), x[m, j] = silu(gate[m, j]) * up[m, j] computed on the way in, so the
 * SwiGLU of a decoder block costs no launch of its own.  Same bits as
 * rumus_hip_swiglu_rows followed by rumus_hip_qmatmul_int4_decode.
 * EINVAL unless m <= 8, n % 16 == 0, k % 8 == 0, group_size % 32 == 0 and
 * 16-byte aligned buffers.  No counterpart in the reference. */
int rumus_hip_qmatmul_int4_decode_swiglu(const float* gate_up, const uint32_t* packed_t,
                                         const float* scales_t, const float* zero_points_t,
                                         const float* bias, float* y, uint32_t m, uint32_t k,
                                         uint32_t n, uint32_t padded_k, uint32_t group_size,
                                         uint32_t num_groups, rumus_hip_stream_t stream);

/* EXTENSION: the decode projection with the neighbouring operators of a
 * pre-norm decoder block folded in, so that a decode step launches no kernel
 * for them:
 *   norm_weight non-NULL: x [m, k] goes through RMSNorm first,
 *       x * rsqrt(mean(x^2) + eps) * norm_weight (what rumus_hip_rmsnorm computes);
 *   swiglu != 0: x is gate_up [m, 2k] as in rumus_hip_qmatmul_int4_decode_swiglu
 *       (norm_weight must be NULL);
 *   residual non-NULL: residual [m, n] is added to the result (it may be y).
 * With none of the three it is rumus_hip_qmatmul_int4_decode without perm.
 * EINVAL unless m <= 8, n % 16 == 0, k % 8 == 0, group_size % 32 == 0, 16-byte
 * aligned buffers and y != x.  No counterpart in the reference. */
int rumus_hip_qmatmul_int4_decode_block(const float* x, const float* norm_weight, float eps,
                                        int swiglu, const uint32_t* packed_t,
                                        const float* scales_t, const float* zero_points_t,
                                        const float* bias, const float* residual, float* y,
                                        uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                                        uint32_t group_size, uint32_t num_groups,
                                        rumus_hip_stream_t stream);

/* EXTENSION: qmatmul_int4_perm on AWQ storage: zero-points come as qzeros
 * (layout above) instead of f32.  perm may be NULL (plain k order).
 * EINVAL also unless n % 8 == 0. */
int rumus_hip_qmatmul_int4_zp4(const float* x, const uint32_t* packed,
                               const float* scales, const uint32_t* qzeros,
                               const float* bias, const int32_t* perm, float* y,
                               uint32_t m, uint32_t k, uint32_t n, uint32_t padded_k,
                               uint32_t group_size, uint32_t num_groups,
                               rumus_hip_stream_t stream);

/* ---- f32 operators between the projections of a decoder block (EXTENSION) --
 * None of these is on the reference's quantized path; they exist so that a
 * block built from the matmuls above needs no other library.  Reference
 * analogue of the attention: flash_attention (rumus/src/tensor/ops.rs:2685-2743,
 * shaders/flash_attn.wgsl): same online-softmax result, f32, head_dim 128. */

/* y[r,:] = x[r,:] * rsqrt(mean(x[r,:]^2) + eps) * weight[:] */
int rumus_hip_rmsnorm(const float* x, const float* weight, float* y, uint32_t rows,
                      uint32_t dim, float eps, rumus_hip_stream_t stream);

/* sum = x + delta; y = rmsnorm(sum) with the formula above, in one launch (the
 * residual update and the norm that follows it in a pre-norm block).  sum may
 * alias x or delta; y must not alias any of them.  Same bits as rumus_hip_add
 * followed by rumus_hip_rmsnorm. */
int rumus_hip_add_rmsnorm(const float* x, const float* delta, const float* weight,
                          float* sum, float* y, uint32_t rows, uint32_t dim, float eps,
                          rumus_hip_stream_t stream);

/* out = silu(gate) * up, silu(t) = t / (1 + exp(-t)); out may alias gate or up */
int rumus_hip_swiglu(const float* gate, const float* up, float* out, uint64_t numel,
                     rumus_hip_stream_t stream);

/* out[r, c] = silu(gate_up[r, c]) * gate_up[r, n + c] for gate_up [rows, 2n]: the two
 * halves of a fused gate|up projection.  out [rows, n] must not alias gate_up. */
int rumus_hip_swiglu_rows(const float* gate_up, float* out, uint32_t rows, uint32_t n,
                          rumus_hip_stream_t stream);

/* out = a + b; out may alias a or b */
int rumus_hip_add(const float* a, const float* b, float* out, uint64_t numel,
                  rumus_hip_stream_t stream);

/* out = softmax(q k^T / sqrt(head_dim)) v per (batch, head).
 * strides: HOST array of 12 element strides (in floats, multiples of 4):
 * {q_batch, q_head, q_row, k_batch, k_head, k_row, v_batch, v_head, v_row,
 *  o_batch, o_head, o_row}; head_dim is contiguous.  A projection output
 * [batch*rows, heads*128] is {rows*heads*128, 128, heads*128}; the reference's
 * [B,H,N,d] is {H*N*128, N*128, 128}.
 * causal != 0: query row i is token kv_len - q_len + i and sees keys up to
 * itself.  q_len == 1 (decode) splits the keys over workgroups and uses the
 * workspace.  EINVAL unless head_dim == 128, q_len <= kv_len, 16-byte aligned. */
int rumus_hip_attention(const float* q, const float* k, const float* v, float* out,
                        uint32_t batch, uint32_t heads, uint32_t q_len, uint32_t kv_len,
                        uint32_t head_dim, const uint64_t* strides, int causal,
                        rumus_hip_stream_t stream);

/* KV-cache append of a decoder block: the keys and values of `rows` new tokens
 * (prefill: all of them, decode: one) are written at positions pos .. pos+rows-1
 * of the cache.  Shape contract of the cache: rumus-serve/src/model.rs:11-14,
 * K and V [batch, heads, cached_len, head_dim]; there the new entries are
 * concatenated by the tensor library, here they are written in place into a
 * cache allocated for cache_len positions.
 * strides: HOST array of 12 element strides (floats, multiples of 4), in the
 * order of rumus_hip_attention: {knew_batch, knew_head, knew_row, vnew_batch,
 * vnew_head, vnew_row, kcache_batch, kcache_head, kcache_row, vcache_batch,
 * vcache_head, vcache_row}; head_dim is contiguous.  The reference's layout is
 * {H*T*d, T*d, d}; a token-major cache [batch, T, heads, d] is {T*H*d, d, H*d}.
 * EINVAL unless head_dim % 4 == 0, pos + rows <= cache_len, 16-byte aligned. */
int rumus_hip_kv_append(const float* k_new, const float* v_new, float* k_cache, float* v_cache,
                        uint32_t batch, uint32_t heads, uint32_t rows, uint32_t head_dim,
                        uint32_t pos, uint32_t cache_len, const uint64_t* strides,
                        rumus_hip_stream_t stream);

/* EXTENSION: rumus_hip_kv_append of ONE new token at `pos` followed by
 * rumus_hip_attention of its query (q_len 1) over positions 0 .. pos, without
 * the launch for the append: the newest key and value are read from k_new /
 * v_new and the kernel writes them into the caches on its way.  Same bits in
 * `out` and in the caches as the two calls.
 * strides: HOST array of 18 element strides (floats, multiples of 4), {batch,
 * head, row} for q, k_new, v_new, k_cache, v_cache, out in that order (the row
 * strides of q, k_new, v_new and out are not used: one row each).
 * EINVAL unless head_dim == 128, pos < cache_len, 16-byte aligned operands.
 * Uses the stream's workspace like rumus_hip_attention with q_len == 1
 * (kv_len = pos + 1).  No counterpart in the reference. */
int rumus_hip_attention_decode_append(const float* q, const float* k_new, const float* v_new,
                                      float* k_cache, float* v_cache, float* out, uint32_t batch,
                                      uint32_t heads, uint32_t head_dim, uint32_t pos,
                                      uint32_t cache_len, const uint64_t* strides,
                                      rumus_hip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
