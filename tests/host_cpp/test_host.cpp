// GPU parity test of the C++ host mirror (include/rumus_hip.hpp) against the CPU
// oracle: reads like a RUMUS integration test (build a Linear, quantize it, run
// forward, compare).  Exit status 0 = every check passed.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <random>
#include <string>
#include <vector>

#include "rumus_hip.hpp"
#include "rumus_hip_block.hpp"
#include "rumus_hip_file.hpp"
#include "rumus_oracle.h"

using namespace rumus_hip;

static int g_fail = 0;
#define CHECK(cond, ...)                                   \
    do {                                                   \
        if (!(cond)) { g_fail++; printf("FAIL %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); } \
    } while (0)

static std::vector<float> normal(size_t n, float sigma, uint32_t seed) {
    std::mt19937 gen(seed);
    std::normal_distribution<float> d(0.0f, sigma);
    std::vector<float> v(n);
    for (auto& x : v) x = d(gen);
    return v;
}

static bool close(const std::vector<float>& got, const std::vector<float>& want, const char* what) {
    size_t bad = 0;
    double worst = 0;
    for (size_t i = 0; i < got.size(); i++) {
        double err = std::fabs((double)got[i] - want[i]), tol = 1e-4 + 1e-3 * std::fabs(want[i]);
        if (!(err <= tol)) bad++;
        worst = std::fmax(worst, err);
    }
    printf("  %-34s max abs err %.3g, %zu of %zu outside rel 1e-3 / abs 1e-4\n", what, worst, bad, got.size());
    return bad == 0;
}

static void test_qlinear(uint32_t m, uint32_t k, uint32_t n, uint32_t g) {
    printf("[host-cpp] QLinear m=%u k=%u n=%u g=%u\n", m, k, n, g);
    fflush(stdout);
    auto w = normal((size_t)k * n, 0.02f, 1), b = normal(n, 0.01f, 2), x = normal((size_t)m * k, 1.0f, 3);
    Linear linear(w, k, n, b);
    QLinear q = QLinear::from_linear(linear, g);
    CHECK(q.in_features == k && q.out_features == n, "feature sizes");
    // oracle: QuantizedTensor::from_f32 then the WGSL kernel's loop
    const uint32_t padded_k = ((k + g - 1) / g) * g, groups = padded_k / g;
    std::vector<uint32_t> packed((size_t)(padded_k / 8) * n);
    std::vector<float> scales((size_t)groups * n), zp((size_t)groups * n), want((size_t)m * n);
    CHECK(orc_w4_from_f32(w.data(), k, n, g, packed.data(), scales.data(), zp.data()) == 0, "oracle from_f32");
    CHECK(q.weight.padded_k == padded_k && q.weight.num_groups == groups, "padding metadata");
    CHECK(q.weight.packed.download() == packed, "nibble pack is not bit-exact");
    CHECK(q.weight.scales.download() == scales, "scales are not bit-exact");
    CHECK(q.weight.zp.download() == zp, "zero-points are not bit-exact");
    orc_qmatmul_int4(x.data(), packed.data(), scales.data(), zp.data(), b.data(), nullptr, want.data(), m, k, n,
                     padded_k, g, groups, 8);
    DeviceBuffer<float> dx(x);
    CHECK(close(q.forward(dx).download(), want, "forward"), "QLinear::forward");
    // grad_x
    auto gy = normal((size_t)m * n, 1.0f, 4);
    std::vector<float> want_gx((size_t)m * k);
    orc_qmatmul_int4_t(gy.data(), packed.data(), scales.data(), zp.data(), want_gx.data(), m, k, n, padded_k, g,
                       groups, 8);
    CHECK(close(q.backward_input(DeviceBuffer<float>(gy)).download(), want_gx, "backward_input"), "grad_x");
}

static void test_q8(uint32_t m, uint32_t k, uint32_t n, uint32_t bs) {
    printf("[host-cpp] Q8 quantize/matmul m=%u k=%u n=%u bs=%u\n", m, k, n, bs);
    fflush(stdout);
    auto w = normal((size_t)k * n, 0.02f, 5), a = normal((size_t)m * k, 1.0f, 6);
    DeviceBuffer<float> dw(w), da(a);
    Q8Tensor q = quantize(dw.data(), k, n, bs);
    std::vector<float> wt((size_t)k * n);
    orc_transpose(w.data(), wt.data(), k, n);
    std::vector<uint32_t> words(orc_q8_buf_size((uint64_t)k * n, bs) / 4);
    CHECK(orc_q8_quantize(wt.data(), words.data(), k * n, bs) == 0, "oracle quantize");
    CHECK(q.buffer.download() == words, "Q8 buffer is not bit-exact");
    std::vector<float> want((size_t)m * n), deq((size_t)k * n);
    orc_matmul_q8(a.data(), words.data(), want.data(), m, k, n, bs, 8);
    CHECK(close(matmul(da, m, q).download(), want, "matmul (Q8 rhs)"), "matmul_q8");
    orc_q8_dequantize(words.data(), deq.data(), k * n, bs);
    CHECK(dequantize(q).download() == deq, "dequantize is not bit-exact");
    CHECK(data(q) == deq, "data() of a Q8 tensor is not the dequantized buffer");
    {
        std::vector<float> kn = dequantize_kn(q).download();
        bool same = kn.size() == deq.size();
        for (uint32_t r = 0; same && r < k; r++)
            for (uint32_t c = 0; c < n; c++)
                if (kn[(size_t)r * n + c] != deq[(size_t)c * k + r]) { same = false; break; }
        CHECK(same, "dequantize_kn is not the transposed dequantize");
    }
}

static void test_int8_linear(uint32_t m, uint32_t k, uint32_t n) {
    printf("[host-cpp] Int8Linear m=%u k=%u n=%u\n", m, k, n);
    fflush(stdout);
    auto w = normal((size_t)k * n, 0.02f, 7), b = normal(n, 0.01f, 8), x = normal((size_t)m * k, 1.0f, 9);
    Linear linear(w, k, n, b);
    Int8Linear l = Int8Linear::from_linear(linear);
    std::vector<float> wt((size_t)k * n), sw(n), sx(m), want((size_t)m * n);
    std::vector<int8_t> wq((size_t)k * n), xq((size_t)m * k);
    std::vector<int32_t> acc((size_t)m * n);
    orc_transpose(w.data(), wt.data(), k, n);
    orc_i8_quantize_rows(wt.data(), wq.data(), sw.data(), n, k);
    orc_i8_quantize_rows(x.data(), xq.data(), sx.data(), m, k);
    orc_i8_gemm_i32(xq.data(), wq.data(), acc.data(), m, k, n, 8);
    orc_i8_rescale_bias(acc.data(), sx.data(), sw.data(), b.data(), want.data(), m, n);
    CHECK(l.wq.download() == wq, "int8 weights are not bit-exact");
    CHECK(l.sw.download() == sw, "weight scales are not bit-exact");
    DeviceBuffer<int32_t> dacc;
    auto y = l.forward(DeviceBuffer<float>(x), &dacc).download();
    CHECK(dacc.download() == acc, "i32 accumulators are not bit-exact");
    CHECK(close(y, want, "forward"), "Int8Linear::forward");
}


static std::vector<char> slurp(const std::string& path) {
    std::vector<char> out;
    if (FILE* f = fopen(path.c_str(), "rb")) {
        char buf[1 << 16];
        size_t got;
        while ((got = fread(buf, 1, sizeof buf, f)) > 0) out.insert(out.end(), buf, buf + got);
        fclose(f);
    }
    return out;
}

static void spill(const std::string& path, const void* data, size_t nbytes) {
    FILE* f = fopen(path.c_str(), "wb");
    CHECK(f && fwrite(data, 1, nbytes, f) == nbytes, "cannot write %s", path.c_str());
    if (f) fclose(f);
}

// Layers through the on-disk form and back: same bits, same outputs; an act-order layer built
// from g_idx matches the oracle.  With a directory argument the file and one forward pass are
// left there for the Python loader to check, and a file the Python writer left is loaded and run.
static void test_file(const std::string& dir) {
    printf("[host-cpp] save_w4 / load_w4 in %s\n", dir.c_str());
    fflush(stdout);
    const uint32_t k = 512, n = 272, g = 128, m = 3;
    auto w = normal((size_t)k * n, 0.02f, 11), b = normal(n, 0.01f, 12), x = normal((size_t)m * k, 1.0f, 13);
    Linear linear(w, k, n, b);
    QLinear plain = QLinear::from_linear(linear, g);
    // act-order: the same quantized rows, announced in a shuffled group order
    std::vector<int32_t> g_idx(k);
    {
        std::vector<uint32_t> order(k);
        for (uint32_t i = 0; i < k; i++) order[i] = i;
        std::mt19937 gen(14);
        std::shuffle(order.begin(), order.end(), gen);
        for (uint32_t i = 0; i < k; i++) g_idx[order[i]] = (int32_t)(i / g);
    }
    auto hp = plain.weight.packed.download();
    auto hs = plain.weight.scales.download(), hz = plain.weight.zp.download();
    QLinear ao;
    {
        DeviceBuffer<int32_t> dg(g_idx);
        ao.weight = QuantizedTensor::from_packed(DeviceBuffer<uint32_t>(hp), DeviceBuffer<float>(hs),
                                                 DeviceBuffer<float>(hz), k, n, g, dg.data());
        check(rumus_hip_sync(nullptr));
    }
    ao.in_features = k;
    ao.out_features = n;
    std::vector<float> want((size_t)m * n);
    orc_qmatmul_int4(x.data(), hp.data(), hs.data(), hz.data(), nullptr, g_idx.data(), want.data(), m, k, n, k, g,
                     k / g, 8);
    DeviceBuffer<float> dx(x);
    CHECK(close(ao.forward(dx).download(), want, "act-order forward (from g_idx)"), "from_packed with g_idx");

    const std::string path = dir + "/cpp.safetensors";
    save_w4(path, {{"blk.plain", &plain}, {"blk.act_order", &ao}});
    auto back = load_w4(path, nullptr, 40000);             // odd chunk size: many pieces per tensor
    CHECK(back.size() == 2 && back.count("blk.plain") && back.count("blk.act_order"), "layer names");
    if (back.size() == 2) {
        const QLinear& p2 = back.at("blk.plain");
        const QLinear& a2 = back.at("blk.act_order");
        CHECK(p2.weight.packed.download() == hp && p2.weight.scales.download() == hs && p2.weight.zp.download() == hz,
              "plain layer arrays changed");
        CHECK(p2.bias.download() == b, "bias changed");
        CHECK(p2.weight.k == k && p2.weight.n == n && p2.weight.group_size == g && p2.in_features == k, "metadata");
        CHECK(p2.forward(dx).download() == plain.forward(dx).download(), "plain forward differs after reload");
        CHECK(a2.weight.perm.download() == ao.weight.perm.download(), "perm changed");
        CHECK(a2.weight.packed.download() == ao.weight.packed.download(), "sorted rows changed");
        CHECK(a2.forward(dx).download() == ao.forward(dx).download(), "act-order forward differs after reload");
    }
    // refusals: a cut file, a header that is not JSON
    auto bytes = slurp(path);
    spill(dir + "/cut.safetensors", bytes.data(), bytes.size() - 100);
    bool threw = false;
    try { load_w4(dir + "/cut.safetensors"); } catch (const Error& e) { threw = e.code == RUMUS_HIP_EINVAL; }
    CHECK(threw, "a truncated file must be refused");
    auto bad = bytes;
    bad[8] = '[';
    spill(dir + "/bad.safetensors", bad.data(), bad.size());
    threw = false;
    try { load_w4(dir + "/bad.safetensors"); } catch (const Error& e) { threw = e.code == RUMUS_HIP_EINVAL; }
    CHECK(threw, "a malformed header must be refused");
    remove((dir + "/cut.safetensors").c_str());
    remove((dir + "/bad.safetensors").c_str());

    // exchange with the Python side
    spill(dir + "/cpp_x.bin", x.data(), x.size() * 4);
    auto y = plain.forward(dx).download();
    spill(dir + "/cpp_y.bin", y.data(), y.size() * 4);
    const auto px = slurp(dir + "/py_x.bin");
    if (!px.empty()) {
        auto layers = load_w4(dir + "/py.safetensors");
        CHECK(!layers.empty(), "py.safetensors holds no layer");
        for (const auto& kv : layers) {
            const QLinear& lin = kv.second;
            const uint32_t rows = (uint32_t)(px.size() / 4 / lin.in_features);
            std::vector<float> hx(px.size() / 4);
            memcpy(hx.data(), px.data(), px.size());
            auto out = lin.forward(DeviceBuffer<float>(hx)).download();
            spill(dir + "/py_y_" + kv.first + ".bin", out.data(), out.size() * 4);
            printf("  loaded %s: k=%u n=%u g=%u rows=%u perm=%zu\n", kv.first.c_str(), lin.weight.k, lin.weight.n,
                   lin.weight.group_size, rows, lin.weight.perm.size());
        }
    }
}

// The decoder block on layers the Python side stored (block.safetensors: q, k, v, o, gate, up, down; block_x.bin:
// [batch, n, dim] f32): a prefill that fills the caches, then one decode step at position n on block_x1.bin
// ([batch, 1, dim]).  Outputs go back as files; the Python test compares them bit for bit with its own block.
static void test_block(const std::string& dir) {
    const auto px = slurp(dir + "/block_x.bin"), px1 = slurp(dir + "/block_x1.bin"), cfg = slurp(dir + "/block_cfg.txt");
    if (px.empty() || px1.empty() || cfg.empty()) return;
    uint32_t batch = 0, n = 0, heads = 0, cache_len = 0;
    CHECK(sscanf(std::string(cfg.begin(), cfg.end()).c_str(), "%u %u %u %u", &batch, &n, &heads, &cache_len) == 4,
          "block_cfg.txt: batch n heads cache_len");
    printf("[host-cpp] decoder block: batch %u, %u tokens, %u heads\n", batch, n, heads);
    fflush(stdout);
    auto layers = load_w4(dir + "/block.safetensors");
    const uint32_t dim = heads * 128;
    std::vector<float> ones(dim, 1.0f);
    DecoderBlockW4 blk = DecoderBlockW4::from_layers(layers, ones, ones, heads);
    std::vector<float> hx(px.size() / 4), hx1(px1.size() / 4);
    memcpy(hx.data(), px.data(), px.size());
    memcpy(hx1.data(), px1.data(), px1.size());
    CHECK(hx.size() == (size_t)batch * n * dim && hx1.size() == (size_t)batch * dim, "block input sizes");
    DeviceBuffer<float> x(hx), x1(hx1), y(hx.size()), y1(hx1.size());
    DeviceBuffer<float> kc(std::vector<float>((size_t)batch * cache_len * dim, 0.0f)),
        vc(std::vector<float>((size_t)batch * cache_len * dim, 0.0f));
    blk.forward(x.data(), batch, n, y.data(), kc.data(), vc.data(), cache_len, 0);
    blk.forward(x1.data(), batch, 1, y1.data(), kc.data(), vc.data(), cache_len, n);
    const auto hy = y.download(), hy1 = y1.download(), hk = kc.download();
    spill(dir + "/block_y.bin", hy.data(), hy.size() * 4);
    spill(dir + "/block_y1.bin", hy1.data(), hy1.size() * 4);
    spill(dir + "/block_k.bin", hk.data(), hk.size() * 4);
    // the same two calls on temporaries the caller keeps (no allocation, no wait inside): same bits, twice in a row
    DecoderBlockW4::Scratch scratch(blk, batch * n);
    DeviceBuffer<float> y2(hx.size()), y3(hx1.size());
    blk.forward(x.data(), batch, n, y2.data(), kc.data(), vc.data(), cache_len, 0, scratch);
    for (int rep = 0; rep < 2; rep++) blk.forward(x1.data(), batch, 1, y3.data(), kc.data(), vc.data(), cache_len, n, scratch);
    check(rumus_hip_sync(nullptr));
    CHECK(y2.download() == hy && y3.download() == hy1 && kc.download() == hk, "block on a kept Scratch differs");
    bool threw = false;
    try { blk.forward(x.data(), batch, n, y.data(), kc.data(), vc.data(), cache_len, 1); } catch (const Error& e) { threw = e.code == RUMUS_HIP_EINVAL; }
    CHECK(threw, "several tokens at pos > 0 must be rejected");
    threw = false;
    DecoderBlockW4::Scratch small(blk, 1);
    try { blk.forward(x.data(), batch, n, y.data(), kc.data(), vc.data(), cache_len, 0, small); } catch (const Error& e) { threw = e.code == RUMUS_HIP_EINVAL; }
    CHECK(threw || batch * n <= 1, "a Scratch of fewer rows must be rejected");
}

static void test_errors() {
    printf("[host-cpp] preconditions\n");
    fflush(stdout);
    DeviceBuffer<float> w(std::vector<float>(64, 0.0f));
    bool threw = false;
    try { QuantizedTensor::from_f32(w.data(), 64, 8, 8, 12); } catch (const Error& e) { threw = e.code == RUMUS_HIP_EINVAL; }
    CHECK(threw, "group_size 12 must be rejected");
    threw = false;
    try { quantize(w.data(), 8, 8, 6); } catch (const Error& e) { threw = e.code == RUMUS_HIP_EINVAL; }
    CHECK(threw, "block_size 6 must be rejected");
    threw = false;
    try { QuantizedTensor::from_f32(w.data(), 60, 8, 8, 8); } catch (const Error&) { threw = true; }
    CHECK(threw, "length mismatch must be rejected");
}

int main(int argc, char** argv) {
    check(rumus_hip_init(0));
    test_qlinear(1, 1024, 512, 128);
    test_qlinear(4, 200, 52, 8);
    test_qlinear(16, 512, 256, 128);
    test_q8(32, 512, 512, 512);
    test_q8(3, 96, 7, 32);
    test_int8_linear(32, 512, 512);
    test_int8_linear(300, 1024, 260);
    test_errors();
    test_file(argc > 1 ? argv[1] : "/tmp");
    test_block(argc > 1 ? argv[1] : "/tmp");
    printf(g_fail ? "host-cpp: %d FAILED\n" : "host-cpp: all passed\n", g_fail);
    return g_fail ? 1 : 0;
}
