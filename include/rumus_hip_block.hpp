// rumus_hip_block.hpp -- a Llama-shaped pre-norm decoder block on the C ABI of rumus_hip.h, for C++ hosts:
//   RMSNorm -> q | k | v -> attention (f32, no rotary embedding) -> o -> residual ->
//   RMSNorm -> gate | up -> SwiGLU -> down -> residual,
// the seven projections INT4 QLinear layers (rumus-vision/src/quant.rs:165-222).  The reference serves such
// blocks through `trait ModelForward` with a K/V cache per layer (rumus-serve/src/model.rs:11-45: K and V
// [batch, heads, cached_len, head_dim]); here the cache is token-major, [batch, cache_len, heads, 128], so that
// the projection output of a new token is one contiguous run per position.
//
// Activations stay [tokens, features] between the layers; the attention and the cache write read the fused
// q|k|v output through strides, so nothing is permuted or copied.  q|k|v and gate|up run as one launch each
// over the column-wise concatenation of their weights.
#pragma once

#include <map>
#include <string>
#include <vector>

#include "rumus_hip.hpp"

namespace rumus_hip {

struct DecoderBlockW4 {
    QLinear qkv, o, gate_up, down;
    DeviceBuffer<float> norm1, norm2;      // [dim]
    uint32_t dim = 0, heads = 0, ffn = 0;
    float eps = 1e-6f;

    // Column-wise concatenation of layers that read the same activations: packed words, scales and zero-points
    // are all [rows, n] arrays.  Equal k and group_size, no act-order, no bias.
    static QLinear concat(const std::vector<const QLinear*>& layers, hipStream_t stream = nullptr) {
        require(!layers.empty(), "concat: no layers");
        const QuantizedTensor& w0 = layers[0]->weight;
        uint32_t n = 0;
        for (const QLinear* l : layers) {
            require(l->weight.k == w0.k && l->weight.group_size == w0.group_size && l->weight.perm.size() == 0 &&
                        l->bias.size() == 0,
                    "DecoderBlockW4: fused projections need equal k / group_size, no act-order, no bias");
            n += l->weight.n;
        }
        QLinear out;
        out.weight.set_geometry(w0.k, n, w0.group_size);
        out.weight.packed = DeviceBuffer<uint32_t>((size_t)(w0.padded_k / 8) * n);
        out.weight.scales = DeviceBuffer<float>((size_t)w0.num_groups * n);
        out.weight.zp = DeviceBuffer<float>((size_t)w0.num_groups * n);
        uint32_t col = 0;
        for (const QLinear* l : layers) {
            const QuantizedTensor& w = l->weight;
            const size_t pitch = (size_t)n * 4, width = (size_t)w.n * 4;
            check_hip(hipMemcpy2DAsync(out.weight.packed.data() + col, pitch, w.packed.data(), width, width,
                                       w.padded_k / 8, hipMemcpyDeviceToDevice, stream), "concat packed");
            check_hip(hipMemcpy2DAsync(out.weight.scales.data() + col, pitch, w.scales.data(), width, width,
                                       w.num_groups, hipMemcpyDeviceToDevice, stream), "concat scales");
            check_hip(hipMemcpy2DAsync(out.weight.zp.data() + col, pitch, w.zp.data(), width, width, w.num_groups,
                                       hipMemcpyDeviceToDevice, stream), "concat zero-points");
            col += w.n;
        }
        out.weight.build_decode_layout(stream);
        out.in_features = w0.k;
        out.out_features = n;
        return out;
    }

    // `layers` holds the projections under the names q, k, v, o, gate, up, down (e.g. from load_w4); o and down
    // are moved out of it.  norm weights: [dim] on the host.
    static DecoderBlockW4 from_layers(std::map<std::string, QLinear>& layers, const std::vector<float>& norm1,
                                      const std::vector<float>& norm2, uint32_t heads, float eps = 1e-6f,
                                      hipStream_t stream = nullptr) {
        for (const char* name : {"q", "k", "v", "o", "gate", "up", "down"})
            require(layers.count(name) == 1, "DecoderBlockW4: a projection is missing");
        DecoderBlockW4 b;
        b.dim = layers.at("q").in_features;
        b.ffn = layers.at("gate").out_features;
        b.heads = heads;
        b.eps = eps;
        require(b.dim == heads * 128, "DecoderBlockW4: head_dim must be 128");
        require(layers.at("q").out_features == b.dim && layers.at("k").out_features == b.dim &&
                    layers.at("v").out_features == b.dim && layers.at("o").in_features == b.dim &&
                    layers.at("o").out_features == b.dim && layers.at("up").out_features == b.ffn &&
                    layers.at("down").in_features == b.ffn && layers.at("down").out_features == b.dim,
                "DecoderBlockW4: projection shapes do not make a block");
        require(norm1.size() == b.dim && norm2.size() == b.dim, "DecoderBlockW4: norm weights must be [dim]");
        b.qkv = concat({&layers.at("q"), &layers.at("k"), &layers.at("v")}, stream);
        b.gate_up = concat({&layers.at("gate"), &layers.at("up")}, stream);
        check(rumus_hip_sync(stream));       // the sources may be released by the caller
        b.o = std::move(layers.at("o"));
        b.down = std::move(layers.at("down"));
        b.norm1 = DeviceBuffer<float>(norm1);
        b.norm2 = DeviceBuffer<float>(norm2);
        return b;
    }

    // x, y: device [batch * n, dim].  k_cache, v_cache: device [batch, cache_len, heads, 128], valid below `pos`
    // (may be null for a prefill that keeps no cache).  pos == 0: causal self-attention over the n tokens, whose
    // keys and values are also written to the caches at 0 .. n-1.  pos > 0: n must be 1; the token's key and value
    // are written at `pos` and it attends positions 0 .. pos.
    static bool folds(const QLinear& lin, uint32_t rows) {
        const QuantizedTensor& w = lin.weight;
        return w.has_decode_layout() && w.perm.size() == 0 && w.k % 8 == 0 &&
               rows <= rumus_hip_qmatmul_int4_decode_max_rows(w.padded_k, w.n);
    }

    // The block's temporaries, [rows, ...] each.  A caller that runs many steps keeps one, sized once for its
    // largest batch * n: forward() on it allocates nothing, frees nothing and does not wait for the stream (so a
    // decode step can be queued behind the previous one, or captured into a HIP graph once the stream's workspace
    // is reserved).  Calls that share a Scratch must be ordered on one stream.
    struct Scratch {
        DeviceBuffer<float> hn, qkv_out, att, ob, gu, dn, sw;
        uint32_t rows = 0;
        Scratch() = default;
        Scratch(const DecoderBlockW4& b, uint32_t max_rows) { reserve(b, max_rows); }
        void reserve(const DecoderBlockW4& b, uint32_t max_rows) {
            if (max_rows <= rows) return;
            const size_t r = max_rows, d = b.dim, f = b.ffn;
            hn = DeviceBuffer<float>(r * d);
            qkv_out = DeviceBuffer<float>(r * 3 * d);
            att = DeviceBuffer<float>(r * d);
            ob = DeviceBuffer<float>(r * d);
            gu = DeviceBuffer<float>(r * 2 * f);
            dn = DeviceBuffer<float>(r * d);
            sw = DeviceBuffer<float>(r * f);
            rows = max_rows;
        }
    };

    // One call with temporaries of its own: allocates them, waits for the stream and frees them.
    void forward(const float* x, uint32_t batch, uint32_t n, float* y, float* k_cache, float* v_cache,
                 uint32_t cache_len, uint32_t pos, hipStream_t stream = nullptr) const {
        require(batch > 0 && n > 0, "DecoderBlockW4: empty input");
        Scratch scratch(*this, batch * n);
        forward(x, batch, n, y, k_cache, v_cache, cache_len, pos, scratch, stream);
        check(rumus_hip_sync(stream));       // the temporaries are released on return
    }

    // The same on the caller's temporaries: asynchronous on `stream`, no allocation.
    void forward(const float* x, uint32_t batch, uint32_t n, float* y, float* k_cache, float* v_cache,
                 uint32_t cache_len, uint32_t pos, Scratch& scratch, hipStream_t stream = nullptr) const {
        require(batch > 0 && n > 0, "DecoderBlockW4: empty input");
        require(pos == 0 || n == 1, "DecoderBlockW4: decode takes one token per sequence");
        require(pos == 0 || (k_cache && v_cache), "DecoderBlockW4: decode needs the caches");
        const uint32_t rows = batch * n, h = heads;
        const uint64_t d = dim;
        require(rows <= scratch.rows, "DecoderBlockW4: the scratch holds fewer rows than batch * n");
        DeviceBuffer<float>&hn = scratch.hn, &qkv_out = scratch.qkv_out, &att = scratch.att, &ob = scratch.ob,
                           &gu = scratch.gu, &dn = scratch.dn, &sw = scratch.sw;
        // a decode step whose rows suit every projection's decode kernel: the norms, the SwiGLU and the residual adds
        // ride on the projections (rumus_hip_qmatmul_int4_decode_block), six launches in all
        const bool folded = pos != 0 && folds(qkv, rows) && folds(o, rows) && folds(gate_up, rows) && folds(down, rows);
        auto project = [&](const QLinear& lin, const float* in, const float* norm_w, int swiglu, const float* resid,
                           float* out) {
            const QuantizedTensor& w = lin.weight;
            check(rumus_hip_qmatmul_int4_decode_block(in, norm_w, eps, swiglu, w.packed_t.data(), w.scales_t.data(),
                                                      w.zp_t.data(), lin.bias.size() ? lin.bias.data() : nullptr, resid,
                                                      out, rows, w.k, w.n, w.padded_k, w.group_size, w.num_groups, stream));
        };
        if (folded) project(qkv, x, norm1.data(), 0, nullptr, qkv_out.data());
        else {
            check(rumus_hip_rmsnorm(x, norm1.data(), hn.data(), rows, dim, eps, stream));
            qkv.forward(hn.data(), rows, qkv_out.data(), stream);
        }
        const float* q = qkv_out.data();
        const float* k = q + d;
        const float* v = q + 2 * d;
        const uint64_t pb = (uint64_t)n * 3 * d, pr = 3 * d;                 // fused projection output
        const uint64_t cb = (uint64_t)cache_len * h * 128, cr = (uint64_t)h * 128;   // token-major cache
        if (k_cache && v_cache && pos == 0) {
            const uint64_t st[12] = {pb, 128, pr, pb, 128, pr, cb, 128, cr, cb, 128, cr};
            check(rumus_hip_kv_append(k, v, k_cache, v_cache, batch, h, n, 128, pos, cache_len, st, stream));
        }
        if (pos == 0) {
            const uint64_t st[12] = {pb, 128, pr, pb, 128, pr, pb, 128, pr, (uint64_t)n * d, 128, d};
            check(rumus_hip_attention(q, k, v, att.data(), batch, h, n, n, 128, st, 1, stream));
        } else {
            // the cache write of the new token rides on the attention
            const uint64_t st[18] = {pb, 128, pr, pb, 128, pr, pb, 128, pr, cb, 128, cr, cb, 128, cr, (uint64_t)n * d, 128, d};
            check(rumus_hip_attention_decode_append(q, k, v, k_cache, v_cache, att.data(), batch, h, 128, pos, cache_len,
                                                    st, stream));
        }
        if (folded) {
            project(o, att.data(), nullptr, 0, x, ob.data());                   // x1 = x + o
            project(gate_up, ob.data(), norm2.data(), 0, nullptr, gu.data());
            project(down, gu.data(), nullptr, 1, ob.data(), y);                 // y = x1 + down(swiglu)
            return;
        }
        o.forward(att.data(), rows, ob.data(), stream);
        // x1 = x + o (kept in `ob`), h2 = rmsnorm(x1) (kept in `hn`)
        check(rumus_hip_add_rmsnorm(x, ob.data(), norm2.data(), ob.data(), hn.data(), rows, dim, eps, stream));
        gate_up.forward(hn.data(), rows, gu.data(), stream);
        const QuantizedTensor& dw = down.weight;
        if (dw.has_decode_layout() && dw.perm.size() == 0 &&
            rows <= rumus_hip_qmatmul_int4_decode_max_rows(dw.padded_k, dw.n)) {
            // decode rows: the SwiGLU happens while the down projection reads its input
            check(rumus_hip_qmatmul_int4_decode_swiglu(gu.data(), dw.packed_t.data(), dw.scales_t.data(), dw.zp_t.data(),
                                                       down.bias.size() ? down.bias.data() : nullptr, dn.data(), rows,
                                                       dw.k, dw.n, dw.padded_k, dw.group_size, dw.num_groups, stream));
        } else {
            check(rumus_hip_swiglu_rows(gu.data(), sw.data(), rows, ffn, stream));
            down.forward(sw.data(), rows, dn.data(), stream);
        }
        check(rumus_hip_add(ob.data(), dn.data(), y, (uint64_t)rows * d, stream));
    }
};

}  // namespace rumus_hip
