//! Bindings to `librumus_hip.so` (declared in `include/rumus_hip.h`).
//!
//! Written against the header, never compiled (no Rust toolchain where this was written).
//! The safe functions at the bottom have the argument lists of the RUMUS functions they
//! replace, with `wgpu::Buffer` swapped for a device pointer:
//!   * `quantize_dispatch` / `dequantize_dispatch` / `matmul_q8_dispatch`
//!     (rumus/src/backend/gpu/compute.rs:1948-2060)
//!   * `QuantizedTensor::from_f32` and `QLinear::forward` / `QLinearBackward::backward`
//!     (rumus-vision/src/quant.rs:42-127, 191-221, 298-317)
//! The reference panics on precondition failures (`assert!`, `expect`), so `check` does too.

use std::ffi::{c_char, c_int, c_void, CStr};

/// `hipStream_t`; null is the default stream.
pub type Stream = *mut c_void;

extern "C" {
    pub fn rumus_hip_init(device: c_int) -> c_int;
    pub fn rumus_hip_last_error() -> *const c_char;
    pub fn rumus_hip_version() -> *const c_char;
    pub fn rumus_hip_sync(stream: Stream) -> c_int;
    pub fn rumus_hip_workspace_reserve(stream: Stream, bytes: u64) -> c_int;
    pub fn rumus_hip_shutdown() -> c_int;

    pub fn rumus_hip_q8_buf_size(numel: u64, block_size: u32) -> u64;
    pub fn rumus_hip_q8_quantize(input: *const f32, out: *mut u32, numel: u32, block_size: u32, s: Stream) -> c_int;
    pub fn rumus_hip_q8_dequantize(input: *const u32, out: *mut f32, numel: u32, block_size: u32, s: Stream) -> c_int;
    pub fn rumus_hip_q8_dequantize_kn(input: *const u32, out: *mut f32, k: u32, n: u32, block_size: u32, s: Stream) -> c_int;
    pub fn rumus_hip_matmul_q8(a: *const f32, b: *const u32, c: *mut f32, m: u32, k: u32, n: u32,
                               block_size: u32, s: Stream) -> c_int;
    pub fn rumus_hip_add_bias(mat: *const f32, bias: *const f32, out: *mut f32, m: u32, n: u32, s: Stream) -> c_int;
    pub fn rumus_hip_transpose_f32(input: *const f32, out: *mut f32, rows: u32, cols: u32, s: Stream) -> c_int;

    pub fn rumus_hip_i8_quantize_rows(x: *const f32, xq: *mut i8, scale: *mut f32, rows: u32, cols: u32,
                                      s: Stream) -> c_int;
    pub fn rumus_hip_i8_quantize_cols_t(w: *const f32, wq: *mut i8, sw: *mut f32, k: u32, n: u32, s: Stream) -> c_int;
    pub fn rumus_hip_i8_gemm(xq: *const i8, wq: *const i8, sx: *const f32, sw: *const f32, bias: *const f32,
                             acc: *mut i32, y: *mut f32, m: u32, k: u32, n: u32, s: Stream) -> c_int;

    pub fn rumus_hip_w4_quantize_pack(w: *const f32, k: u32, n: u32, group_size: u32, packed: *mut u32,
                                      scales: *mut f32, zero_points: *mut f32, s: Stream) -> c_int;
    pub fn rumus_hip_w4_quantize_pack_sym(w: *const f32, k: u32, n: u32, group_size: u32, packed: *mut u32,
                                          scales: *mut f32, zero_points: *mut f32, s: Stream) -> c_int;
    pub fn rumus_hip_w4_quantize_pack_awq(w: *const f32, k: u32, n: u32, group_size: u32, packed: *mut u32,
                                          scales: *mut f32, qzeros: *mut u32, s: Stream) -> c_int;
    pub fn rumus_hip_f16_to_f32(input: *const u16, out: *mut f32, numel: u64, s: Stream) -> c_int;
    pub fn rumus_hip_matmul_q8_f16(a: *const u16, b: *const u32, c: *mut u16, m: u32, k: u32, n: u32, block_size: u32,
                                   s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_f16(x: *const u16, packed: *const u32, scales: *const f32, zero_points: *const f32,
                                      bias: *const f32, g_idx: *const i32, y: *mut u16, m: u32, k: u32, n: u32,
                                      padded_k: u32, group_size: u32, num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_f16_staging_reserve(s: Stream, bytes: u64) -> c_int;
    pub fn rumus_hip_w4_qzeros_unpack(qzeros: *const u32, num_groups: u32, n: u32, zero_points: *mut f32,
                                      s: Stream) -> c_int;
    pub fn rumus_hip_w4_decode_layout(packed: *const u32, scales: *const f32, zero_points: *const f32,
                                      padded_k: u32, n: u32, group_size: u32, packed_t: *mut u32,
                                      scales_t: *mut f32, zero_points_t: *mut f32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_decode(x: *const f32, packed_t: *const u32, scales_t: *const f32,
                                         zero_points_t: *const f32, bias: *const f32, perm: *const i32,
                                         y: *mut f32, m: u32, k: u32, n: u32, padded_k: u32, group_size: u32,
                                         num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_decode_max_rows(padded_k: u32, n: u32) -> u32;
    pub fn rumus_hip_w4_decode_layout_zp4(packed: *const u32, scales: *const f32, qzeros: *const u32, padded_k: u32,
                                          n: u32, group_size: u32, packed_t: *mut u32, scales_t: *mut f32,
                                          qzeros_t: *mut u32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_decode_zp4(x: *const f32, packed_t: *const u32, scales_t: *const f32,
                                             qzeros_t: *const u32, bias: *const f32, perm: *const i32,
                                             y: *mut f32, m: u32, k: u32, n: u32, padded_k: u32, group_size: u32,
                                             num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_decode_swiglu(gate_up: *const f32, packed_t: *const u32, scales_t: *const f32,
                                                zero_points_t: *const f32, bias: *const f32, y: *mut f32,
                                                m: u32, k: u32, n: u32, padded_k: u32, group_size: u32,
                                                num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_decode_block(x: *const f32, norm_weight: *const f32, eps: f32, swiglu: c_int,
                                               packed_t: *const u32, scales_t: *const f32,
                                               zero_points_t: *const f32, bias: *const f32, residual: *const f32,
                                               y: *mut f32, m: u32, k: u32, n: u32, padded_k: u32, group_size: u32,
                                               num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_add_rmsnorm(x: *const f32, delta: *const f32, weight: *const f32, sum: *mut f32, y: *mut f32,
                                 rows: u32, dim: u32, eps: f32, s: Stream) -> c_int;
    pub fn rumus_hip_rmsnorm(x: *const f32, weight: *const f32, y: *mut f32, rows: u32, dim: u32, eps: f32,
                             s: Stream) -> c_int;
    pub fn rumus_hip_swiglu(gate: *const f32, up: *const f32, out: *mut f32, numel: u64, s: Stream) -> c_int;
    pub fn rumus_hip_swiglu_rows(gate_up: *const f32, out: *mut f32, rows: u32, n: u32, s: Stream) -> c_int;
    pub fn rumus_hip_add(a: *const f32, b: *const f32, out: *mut f32, numel: u64, s: Stream) -> c_int;
    pub fn rumus_hip_attention_decode_append(q: *const f32, k_new: *const f32, v_new: *const f32, k_cache: *mut f32,
                                             v_cache: *mut f32, out: *mut f32, batch: u32, heads: u32, head_dim: u32,
                                             pos: u32, cache_len: u32, strides: *const u64, s: Stream) -> c_int;
    pub fn rumus_hip_attention(q: *const f32, k: *const f32, v: *const f32, out: *mut f32, batch: u32,
                               heads: u32, q_len: u32, kv_len: u32, head_dim: u32, strides: *const u64,
                               causal: c_int, s: Stream) -> c_int;
    pub fn rumus_hip_kv_append(k_new: *const f32, v_new: *const f32, k_cache: *mut f32, v_cache: *mut f32, batch: u32,
                               heads: u32, rows: u32, head_dim: u32, pos: u32, cache_len: u32, strides: *const u64,
                               s: Stream) -> c_int;
    pub fn rumus_hip_q8_dense_layout(b_q8: *const u32, k: u32, n: u32, block_size: u32, wq: *mut i8, sw: *mut f32,
                                     s: Stream) -> c_int;
    pub fn rumus_hip_matmul_q8_dense(a: *const f32, wq: *const i8, sw: *const f32, c: *mut f32, m: u32, k: u32,
                                     n: u32, s: Stream) -> c_int;
    pub fn rumus_hip_i8_gemm_workspace_size(m: u32, k: u32, n: u32) -> u64;
    pub fn rumus_hip_qmatmul_int4_perm_static(x: *const f32, packed_sorted: *const u32, scales: *const f32,
                                              zp: *const f32, bias: *const f32, perm: *const i32, y: *mut f32,
                                              m: u32, k: u32, n: u32, padded_k: u32, group_size: u32,
                                              num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_static_scratch_bytes() -> u64;
    pub fn rumus_hip_qmatmul_int4_zp4(x: *const f32, packed: *const u32, scales: *const f32, qzeros: *const u32,
                                      bias: *const f32, perm: *const i32, y: *mut f32, m: u32, k: u32, n: u32,
                                      padded_k: u32, group_size: u32, num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4(x: *const f32, packed: *const u32, scales: *const f32, zp: *const f32,
                                  bias: *const f32, g_idx: *const i32, y: *mut f32, m: u32, k: u32, n: u32,
                                  padded_k: u32, group_size: u32, num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_t(a: *const f32, packed: *const u32, scales: *const f32, zp: *const f32,
                                    out: *mut f32, m: u32, k: u32, n: u32, padded_k: u32, group_size: u32,
                                    num_groups: u32, s: Stream) -> c_int;
    pub fn rumus_hip_w4_actorder_prepare(packed: *const u32, g_idx: *const i32, padded_k: u32, n: u32,
                                         group_size: u32, packed_sorted: *mut u32, perm: *mut i32, s: Stream) -> c_int;
    pub fn rumus_hip_qmatmul_int4_perm(x: *const f32, packed_sorted: *const u32, scales: *const f32,
                                       zp: *const f32, bias: *const f32, perm: *const i32, y: *mut f32, m: u32,
                                       k: u32, n: u32, padded_k: u32, group_size: u32, num_groups: u32,
                                       s: Stream) -> c_int;
}

/// Panics with the library's message on a non-zero status, like the reference's asserts.
pub fn check(status: c_int) {
    if status != 0 {
        let msg = unsafe { CStr::from_ptr(rumus_hip_last_error()) }.to_string_lossy().into_owned();
        panic!("rumus_hip: {msg}");
    }
}

/// A device allocation handed out by the HIP build of RUMUS's `BufferPool`.
#[derive(Clone, Copy)]
pub struct DevPtr(pub *mut c_void);

/// `quantize_dispatch(ctx, input, output, numel, block_size)` (compute.rs:1948-1954).
pub fn quantize_dispatch(stream: Stream, input: DevPtr, output: DevPtr, numel: u32, block_size: u32) {
    check(unsafe { rumus_hip_q8_quantize(input.0 as *const f32, output.0 as *mut u32, numel, block_size, stream) });
}

/// `dequantize_dispatch(ctx, input, output, numel, block_size)` (compute.rs:1985-1991).
pub fn dequantize_dispatch(stream: Stream, input: DevPtr, output: DevPtr, numel: u32, block_size: u32) {
    check(unsafe { rumus_hip_q8_dequantize(input.0 as *const u32, output.0 as *mut f32, numel, block_size, stream) });
}

/// The dequantized `[k, n]` tensor in the order of its shape (the Q8 buffer holds the transposed tensor).
pub fn dequantize_kn_dispatch(stream: Stream, input: DevPtr, output: DevPtr, k: u32, n: u32, block_size: u32) {
    check(unsafe { rumus_hip_q8_dequantize_kn(input.0 as *const u32, output.0 as *mut f32, k, n, block_size, stream) });
}

/// `matmul_q8_dispatch(ctx, a, b, c, m, k, n, block_size)` (compute.rs:2021-2028).
#[allow(clippy::too_many_arguments)]
pub fn matmul_q8_dispatch(stream: Stream, a: DevPtr, b: DevPtr, c: DevPtr, m: u32, k: u32, n: u32, block_size: u32) {
    check(unsafe {
        rumus_hip_matmul_q8(a.0 as *const f32, b.0 as *const u32, c.0 as *mut f32, m, k, n, block_size, stream)
    });
}

/// The three device arrays of a `QuantizedTensor` plus its public metadata (quant.rs:24-38).
pub struct QuantizedTensorHip {
    pub packed: DevPtr,
    pub scales: DevPtr,
    pub zero_points: DevPtr,
    pub k: u32,
    pub n: u32,
    pub padded_k: u32,
    pub group_size: u32,
    pub num_groups: u32,
}

impl QuantizedTensorHip {
    /// `QuantizedTensor::from_f32` (quant.rs:42-127) with `data` already on the device; the
    /// caller provides the three output allocations: `(padded_k/8)*n` u32, `num_groups*n` f32 twice.
    pub fn from_f32(stream: Stream, data: DevPtr, k: u32, n: u32, group_size: u32, packed: DevPtr, scales: DevPtr,
                    zero_points: DevPtr) -> Self {
        assert!(group_size % 8 == 0, "group_size must be a multiple of 8");
        let num_groups = (k + group_size - 1) / group_size;
        check(unsafe {
            rumus_hip_w4_quantize_pack(data.0 as *const f32, k, n, group_size, packed.0 as *mut u32,
                                       scales.0 as *mut f32, zero_points.0 as *mut f32, stream)
        });
        Self { packed, scales, zero_points, k, n, padded_k: num_groups * group_size, group_size, num_groups }
    }
}

/// `QLinear` (quant.rs:165-221): `y = x . dequant(W) (+ bias)`.
pub struct QLinearHip {
    pub weight: QuantizedTensorHip,
    pub bias: Option<DevPtr>,
}

impl QLinearHip {
    /// `QLinear::forward` (quant.rs:191-221): x is `[m, k]`, y is `[m, n]`, both on the device.
    pub fn forward(&self, stream: Stream, x: DevPtr, y: DevPtr, m: u32) {
        let w = &self.weight;
        let bias = self.bias.map_or(std::ptr::null(), |b| b.0 as *const f32);
        check(unsafe {
            rumus_hip_qmatmul_int4(x.0 as *const f32, w.packed.0 as *const u32, w.scales.0 as *const f32,
                                   w.zero_points.0 as *const f32, bias, std::ptr::null(), y.0 as *mut f32, m, w.k,
                                   w.n, w.padded_k, w.group_size, w.num_groups, stream)
        });
    }

    /// `QLinearBackward::backward` (quant.rs:298-317): grad_x `[m, k]` from grad_y `[m, n]`.
    pub fn backward_input(&self, stream: Stream, grad_y: DevPtr, grad_x: DevPtr, m: u32) {
        let w = &self.weight;
        check(unsafe {
            rumus_hip_qmatmul_int4_t(grad_y.0 as *const f32, w.packed.0 as *const u32, w.scales.0 as *const f32,
                                     w.zero_points.0 as *const f32, grad_x.0 as *mut f32, m, w.k, w.n, w.padded_k,
                                     w.group_size, w.num_groups, stream)
        });
    }
}
