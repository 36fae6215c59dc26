// rumus_hip.hpp -- header-only C++ mirror of RUMUS's module API for the
// quantized-Linear path, over the C ABI of rumus_hip.h.
//
// Same names, argument meaning and error behaviour as the reference (which
// panics; here a failed precondition throws rumus_hip::Error):
//   Linear             rumus/src/nn/linear.rs:44-104       (weight [in, out])
//   QuantizedTensor    rumus-vision/src/quant.rs:24-127
//   QLinear            rumus-vision/src/quant.rs:165-222
//   Q8Tensor + quantize / dequantize / matmul
//                      rumus/src/tensor/ops.rs:516-545,2290-2357 (DType::Q8)
//   Int8Linear         the W8A8 engine (no reference counterpart)
// Device memory is owned through DeviceBuffer (hipMalloc / hipFree), the
// counterpart of the reference's pooled wgpu::Buffer + StorageHandle.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "rumus_hip.h"

namespace rumus_hip {

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string& what) : std::runtime_error(what), code(c) {}
};

inline void check(int status) {
    if (status != RUMUS_HIP_OK) throw Error(status, rumus_hip_last_error());
}
inline void check_hip(hipError_t e, const char* what) {
    if (e != hipSuccess) throw Error(RUMUS_HIP_EHIP, std::string(what) + ": " + hipGetErrorString(e));
}
inline void require(bool ok, const char* what) {
    if (!ok) throw Error(RUMUS_HIP_EINVAL, what);
}

// Owned device allocation of `count` elements of T.
template <typename T>
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t count) : count_(count) {
        if (count) check_hip(hipMalloc(reinterpret_cast<void**>(&ptr_), count * sizeof(T)), "hipMalloc");
    }
    DeviceBuffer(const std::vector<T>& host) : DeviceBuffer(host.size()) { upload(host.data(), host.size()); }
    DeviceBuffer(DeviceBuffer&& o) noexcept : ptr_(o.ptr_), count_(o.count_) { o.ptr_ = nullptr; o.count_ = 0; }
    DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
        if (this != &o) { release(); ptr_ = o.ptr_; count_ = o.count_; o.ptr_ = nullptr; o.count_ = 0; }
        return *this;
    }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer() { release(); }

    T* data() { return ptr_; }
    const T* data() const { return ptr_; }
    size_t size() const { return count_; }
    void upload(const T* host, size_t count) {
        require(count <= count_, "upload: buffer too small");
        if (count) check_hip(hipMemcpy(ptr_, host, count * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy H2D");
    }
    std::vector<T> download() const {
        std::vector<T> out(count_);
        if (count_) check_hip(hipMemcpy(out.data(), ptr_, count_ * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy D2H");
        return out;
    }

private:
    void release() { if (ptr_) (void)hipFree(ptr_); ptr_ = nullptr; }
    T* ptr_ = nullptr;
    size_t count_ = 0;
};

// y = x @ weight + bias, weight [in_features, out_features] row-major.
struct Linear {
    DeviceBuffer<float> weight;
    DeviceBuffer<float> bias;   // empty = no bias
    uint32_t in_features = 0, out_features = 0;
    Linear(const std::vector<float>& w, uint32_t in, uint32_t out, const std::vector<float>& b = {})
        : weight(w), bias(b), in_features(in), out_features(out) {
        require(w.size() == (size_t)in * out, "Linear: weight length mismatch");
        require(b.empty() || b.size() == out, "Linear: bias length mismatch");
    }
};

// ---- INT4 -------------------------------------------------------------------

// INT4 weight with group-wise metadata (quant.rs:24-38).
struct QuantizedTensor {
    uint32_t k = 0, n = 0, padded_k = 0, group_size = 0, num_groups = 0;
    DeviceBuffer<uint32_t> packed;    // [(padded_k/8), n]
    DeviceBuffer<float> scales, zp;   // [num_groups, n]
    // Tile-major copies of the three arrays for the decode kernel (16 columns per tile), built
    // when the shape allows (n % 16 == 0, group_size % 32 == 0); empty otherwise.
    DeviceBuffer<uint32_t> packed_t;
    DeviceBuffer<float> scales_t, zp_t;
    bool has_decode_layout() const { return packed_t.size() != 0; }

    // Act-order: original input feature held by each stored row (rows sorted by group); empty =
    // rows in their natural order.
    DeviceBuffer<int32_t> perm;

    // quant.rs:42-102 on the device; `data` is a device pointer to [k, n] f32.
    static QuantizedTensor from_f32(const float* data, size_t len, uint32_t k, uint32_t n, uint32_t group_size,
                                    hipStream_t stream = nullptr) {
        require(group_size > 0 && group_size % 8 == 0, "group_size must be a multiple of 8");
        require((size_t)k * n == len, "data length mismatch");
        QuantizedTensor q;
        q.set_geometry(k, n, group_size);
        q.packed = DeviceBuffer<uint32_t>((size_t)(q.padded_k / 8) * n);
        q.scales = DeviceBuffer<float>((size_t)q.num_groups * n);
        q.zp = DeviceBuffer<float>((size_t)q.num_groups * n);
        check(rumus_hip_w4_quantize_pack(data, k, n, group_size, q.packed.data(), q.scales.data(), q.zp.data(),
                                         stream));
        q.build_decode_layout(stream);
        return q;
    }

    // Adopt pre-quantized device arrays (GPTQ/AWQ style).  With g_idx (group of each of the k
    // rows, rows in their original order) the rows are sorted once so that groups are contiguous.
    static QuantizedTensor from_packed(DeviceBuffer<uint32_t>&& packed, DeviceBuffer<float>&& scales,
                                       DeviceBuffer<float>&& zp, uint32_t k, uint32_t n, uint32_t group_size,
                                       const int32_t* g_idx = nullptr, hipStream_t stream = nullptr) {
        require(group_size > 0 && group_size % 8 == 0, "group_size must be a multiple of 8");
        QuantizedTensor q;
        q.set_geometry(k, n, group_size);
        require(packed.size() == (size_t)(q.padded_k / 8) * n && scales.size() == (size_t)q.num_groups * n &&
                    zp.size() == scales.size(), "from_packed: array sizes do not match k / n / group_size");
        q.scales = std::move(scales);
        q.zp = std::move(zp);
        if (g_idx) {
            require(k == q.padded_k, "act-order needs k to be a multiple of group_size");
            q.packed = DeviceBuffer<uint32_t>(packed.size());
            q.perm = DeviceBuffer<int32_t>(k);
            check(rumus_hip_w4_actorder_prepare(packed.data(), g_idx, q.padded_k, n, group_size, q.packed.data(),
                                                q.perm.data(), stream));
            check(rumus_hip_sync(stream));   // `packed` is released on return
        } else {
            q.packed = std::move(packed);
        }
        q.build_decode_layout(stream);
        return q;
    }

    void set_geometry(uint32_t k_, uint32_t n_, uint32_t group_size_) {
        k = k_; n = n_; group_size = group_size_;
        padded_k = ((k + group_size - 1) / group_size) * group_size;
        num_groups = padded_k / group_size;
    }
    void build_decode_layout(hipStream_t stream = nullptr) {
        if (n % 16 != 0 || group_size % 32 != 0 || packed.size() == 0) return;
        packed_t = DeviceBuffer<uint32_t>(packed.size());
        scales_t = DeviceBuffer<float>(scales.size());
        zp_t = DeviceBuffer<float>(zp.size());
        check(rumus_hip_w4_decode_layout(packed.data(), scales.data(), zp.data(), padded_k, n, group_size,
                                         packed_t.data(), scales_t.data(), zp_t.data(), stream));
    }
    // Gives the second copy back (no launch that reads it may be in flight): decode batches then run on the
    // reference's arrays, about 15 % slower at 4096 x 4096, and the weight costs its 4.5 bits per value only.
    void drop_decode_layout() {
        packed_t = DeviceBuffer<uint32_t>();
        scales_t = DeviceBuffer<float>();
        zp_t = DeviceBuffer<float>();
    }
};

// Linear layer with frozen INT4 weights and optional bias (quant.rs:165-222).
struct QLinear {
    QuantizedTensor weight;
    DeviceBuffer<float> bias;
    uint32_t in_features = 0, out_features = 0;

    static QLinear from_linear(const Linear& linear, uint32_t group_size, hipStream_t stream = nullptr) {
        QLinear q;
        q.weight = QuantizedTensor::from_f32(linear.weight.data(), linear.weight.size(), linear.in_features,
                                             linear.out_features, group_size, stream);
        q.in_features = linear.in_features;
        q.out_features = linear.out_features;
        if (linear.bias.size()) {
            q.bias = DeviceBuffer<float>(linear.bias.size());
            check_hip(hipMemcpyAsync(q.bias.data(), linear.bias.data(), linear.bias.size() * sizeof(float),
                                     hipMemcpyDeviceToDevice, stream), "copy bias");
        }
        return q;
    }

    // y[m, out] = x[m, in] . dequant(W) + bias; x and y are device pointers.
    // Few rows take the decode kernel on the tile-major copy (same result bit for bit).
    void forward(const float* x, uint32_t m, float* y, hipStream_t stream = nullptr) const {
        const int32_t* perm = weight.perm.size() ? weight.perm.data() : nullptr;
        if (weight.has_decode_layout() && m <= rumus_hip_qmatmul_int4_decode_max_rows(weight.padded_k, weight.n)) {
            check(rumus_hip_qmatmul_int4_decode(x, weight.packed_t.data(), weight.scales_t.data(), weight.zp_t.data(),
                                                bias.size() ? bias.data() : nullptr, perm, y, m, weight.k,
                                                weight.n, weight.padded_k, weight.group_size, weight.num_groups,
                                                stream));
            return;
        }
        check(rumus_hip_qmatmul_int4_perm(x, weight.packed.data(), weight.scales.data(), weight.zp.data(),
                                          bias.size() ? bias.data() : nullptr, perm, y, m, weight.k, weight.n,
                                          weight.padded_k, weight.group_size, weight.num_groups, stream));
    }
    DeviceBuffer<float> forward(const DeviceBuffer<float>& x, hipStream_t stream = nullptr) const {
        require(in_features && x.size() % in_features == 0, "QLinear::forward: x must be [m, in_features]");
        const uint32_t m = (uint32_t)(x.size() / in_features);
        DeviceBuffer<float> y((size_t)m * out_features);
        forward(x.data(), m, y.data(), stream);
        return y;
    }
    // grad_x[m, in] = grad_y[m, out] . dequant(W)^T (QLinearBackward, quant.rs:298-317)
    DeviceBuffer<float> backward_input(const DeviceBuffer<float>& grad_y, hipStream_t stream = nullptr) const {
        require(out_features && grad_y.size() % out_features == 0, "QLinear::backward: grad_y must be [m, out]");
        require(weight.perm.size() == 0, "QLinear::backward: grad_x for act-order weights is not implemented");
        const uint32_t m = (uint32_t)(grad_y.size() / out_features);
        DeviceBuffer<float> gx((size_t)m * in_features);
        check(rumus_hip_qmatmul_int4_t(grad_y.data(), weight.packed.data(), weight.scales.data(), weight.zp.data(),
                                       gx.data(), m, weight.k, weight.n, weight.padded_k, weight.group_size,
                                       weight.num_groups, stream));
        return gx;
    }
};

// ---- INT8, reference block format ------------------------------------------------

// A DType::Q8{block_size} tensor of logical shape [K, N]: fused header + data buffer.
struct Q8Tensor {
    DeviceBuffer<uint32_t> buffer;
    uint32_t k = 0, n = 0, block_size = 0;
    size_t numel() const { return (size_t)k * n; }
};

// Tensor::quantize (ops.rs:2290-2327): transpose [K,N] -> [N,K], then block-quantize.
inline Q8Tensor quantize(const float* w, uint32_t k, uint32_t n, uint32_t block_size, hipStream_t stream = nullptr) {
    require(block_size > 0 && block_size % 4 == 0, "quantize: block_size must be > 0 and divisible by 4");
    Q8Tensor q;
    q.k = k; q.n = n; q.block_size = block_size;
    DeviceBuffer<float> t((size_t)k * n);
    check(rumus_hip_transpose_f32(w, t.data(), k, n, stream));
    q.buffer = DeviceBuffer<uint32_t>(rumus_hip_q8_buf_size((uint64_t)k * n, block_size) / 4);
    check(rumus_hip_q8_quantize(t.data(), q.buffer.data(), k * n, block_size, stream));
    check(rumus_hip_sync(stream));   // `t` is released on return
    return q;
}

// Tensor::dequantize (ops.rs:2332-2357): buffer order ([N,K]) under the [K,N] shape, as in the reference.
inline DeviceBuffer<float> dequantize(const Q8Tensor& q, hipStream_t stream = nullptr) {
    DeviceBuffer<float> out(q.numel());
    check(rumus_hip_q8_dequantize(q.buffer.data(), out.data(), (uint32_t)q.numel(), q.block_size, stream));
    return out;
}

// Tensor::data() on a Q8 tensor (core.rs:612-691): dequantize on the GPU, then download.
inline std::vector<float> data(const Q8Tensor& q, hipStream_t stream = nullptr) {
    DeviceBuffer<float> f = dequantize(q, stream);
    check(rumus_hip_sync(stream));
    return f.download();
}

// The dequantized [K, N] tensor with every value where the shape says it is (the buffer holds the
// transposed tensor; Tensor::dequantize does not undo that).
inline DeviceBuffer<float> dequantize_kn(const Q8Tensor& q, hipStream_t stream = nullptr) {
    DeviceBuffer<float> out(q.numel());
    check(rumus_hip_q8_dequantize_kn(q.buffer.data(), out.data(), q.k, q.n, q.block_size, stream));
    return out;
}

// Tensor::matmul with a Q8 right-hand side (ops.rs:516-545): c[m,n] = a[m,k] x Q8.
inline DeviceBuffer<float> matmul(const DeviceBuffer<float>& a, uint32_t m, const Q8Tensor& b,
                                  hipStream_t stream = nullptr) {
    require(a.size() == (size_t)m * b.k, "matmul: inner dimension mismatch");
    // the kernel, like matmul_q8.wgsl:47-52, reads ceil(k / block_size) whole blocks per column; Tensor::quantize
    // blocks the flat transposed tensor, which is that many only when k % block_size == 0 (or one block holds it all)
    require(b.block_size > 0 && b.buffer.size() >= (size_t)b.n * ((b.k + b.block_size - 1) / b.block_size) *
                                                       ((4 + (size_t)b.block_size + 3) / 4),
            "matmul: the Q8 buffer is shorter than n columns of whole blocks (k % block_size != 0?)");
    DeviceBuffer<float> c((size_t)m * b.n);
    check(rumus_hip_matmul_q8(a.data(), b.buffer.data(), c.data(), m, b.k, b.n, b.block_size, stream));
    return c;
}

// A per-output-channel Q8 weight (block_size >= k) in the layout the matrix cores read: made once with
// prepare_dense, multiplied many times.  Same results as matmul() on the Q8 tensor from 384 rows on.
struct Q8Dense {
    DeviceBuffer<int8_t> wq;     // [n, k]
    DeviceBuffer<float> sw;      // [n]
    uint32_t k = 0, n = 0;
};

inline Q8Dense prepare_dense(const Q8Tensor& q, hipStream_t stream = nullptr) {
    require(q.block_size > 0 && q.block_size >= q.k, "prepare_dense: one block per column wanted (block_size >= k)");
    require(q.buffer.size() >= (size_t)q.n * ((4 + (size_t)q.block_size + 3) / 4),
            "prepare_dense: the Q8 buffer is shorter than n blocks");
    Q8Dense d;
    d.k = q.k; d.n = q.n;
    d.wq = DeviceBuffer<int8_t>((size_t)q.n * q.k);
    d.sw = DeviceBuffer<float>(q.n);
    check(rumus_hip_q8_dense_layout(q.buffer.data(), q.k, q.n, q.block_size, d.wq.data(), d.sw.data(), stream));
    return d;
}

inline DeviceBuffer<float> matmul(const DeviceBuffer<float>& a, uint32_t m, const Q8Dense& b,
                                  hipStream_t stream = nullptr) {
    require(a.size() == (size_t)m * b.k, "matmul: inner dimension mismatch");
    DeviceBuffer<float> c((size_t)m * b.n);
    check(rumus_hip_matmul_q8_dense(a.data(), b.wq.data(), b.sw.data(), c.data(), m, b.k, b.n, stream));
    return c;
}

// ---- INT8, W8A8 --------------------------------------------------------------------

// Per-output-channel int8 weights, dynamic per-row int8 activations, i32 accumulate.
struct Int8Linear {
    DeviceBuffer<int8_t> wq;     // [out, in]
    DeviceBuffer<float> sw, bias;
    uint32_t in_features = 0, out_features = 0;

    static Int8Linear from_linear(const Linear& linear, hipStream_t stream = nullptr) {
        Int8Linear l;
        l.in_features = linear.in_features;
        l.out_features = linear.out_features;
        l.wq = DeviceBuffer<int8_t>(linear.weight.size());
        l.sw = DeviceBuffer<float>(linear.out_features);
        check(rumus_hip_i8_quantize_cols_t(linear.weight.data(), l.wq.data(), l.sw.data(), linear.in_features,
                                           linear.out_features, stream));
        if (linear.bias.size()) {
            l.bias = DeviceBuffer<float>(linear.bias.size());
            check_hip(hipMemcpyAsync(l.bias.data(), linear.bias.data(), linear.bias.size() * sizeof(float),
                                     hipMemcpyDeviceToDevice, stream), "copy bias");
        }
        return l;
    }

    // y[m, out] (and optionally the exact i32 accumulators) for x[m, in] on the device.
    DeviceBuffer<float> forward(const DeviceBuffer<float>& x, DeviceBuffer<int32_t>* acc = nullptr,
                                hipStream_t stream = nullptr) const {
        require(in_features && x.size() % in_features == 0, "Int8Linear::forward: x must be [m, in_features]");
        const uint32_t m = (uint32_t)(x.size() / in_features);
        DeviceBuffer<int8_t> xq(x.size());
        DeviceBuffer<float> sx(m), y((size_t)m * out_features);
        check(rumus_hip_i8_quantize_rows(x.data(), xq.data(), sx.data(), m, in_features, stream));
        if (acc) *acc = DeviceBuffer<int32_t>((size_t)m * out_features);
        check(rumus_hip_i8_gemm(xq.data(), wq.data(), sx.data(), sw.data(), bias.size() ? bias.data() : nullptr,
                                acc ? acc->data() : nullptr, y.data(), m, in_features, out_features, stream));
        check(rumus_hip_sync(stream));   // xq / sx are released on return
        return y;
    }
};

}  // namespace rumus_hip
