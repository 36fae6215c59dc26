// rumus_hip_file.hpp -- INT4 layers on disk, for the C++ mirror of rumus_hip.hpp.
//
// The reference keeps QuantizedTensor / QLinear (rumus-vision/src/quant.rs:24-38,165-170) in
// memory only.  This is the stored form of exactly those fields in one safetensors file, under
// the tensor names GPTQ/AWQ checkpoints use:
//
//   <name>.qweight  I32 [padded_k/8, n]  word (r, c) holds rows 8r..8r+7 of column c, row 8r+j in
//                                        bits 4j..4j+3 (quant.rs:98-100)
//   <name>.scales   F32 [groups, n]      (F16 is accepted and widened on the device, exactly)
//   <name>.zeros    F32 [groups, n]      the reference's unrounded zero-points (quant.rs:77-79), or
//   <name>.qzeros   I32 [groups, n/8]    u4 zero-points, column c in bits 4*(c%8) of word c/8
//   <name>.bias     F32 [n]              optional
//   <name>.perm     I32 [k]              optional: input feature held by each stored row, or
//   <name>.g_idx    I32 [k]              optional: group of each row, rows in original order
//
// __metadata__: format = rumus-w4, version = 1, and per layer <name>.k, <name>.group_size.
// The container: 8-byte little-endian header length, a JSON header, raw little-endian tensors.
// Files are read through two pinned staging buffers: while one chunk travels to the device the
// next is read from disk.  Only the header is interpreted on the host.
#pragma once

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "rumus_hip.hpp"

namespace rumus_hip {

struct FileTensor {
    std::string dtype;             // "F32", "F16", "I32"
    std::vector<uint64_t> shape;
    uint64_t begin = 0, end = 0;   // byte range inside the data region
    uint64_t numel() const { uint64_t c = 1; for (uint64_t d : shape) c *= d; return c; }
};

struct FileHeader {
    std::map<std::string, FileTensor> tensors;
    std::map<std::string, std::string> metadata;
    uint64_t data_start = 0;
};

namespace detail {

inline size_t dtype_size(const std::string& d) {
    if (d == "F32" || d == "I32") return 4;
    if (d == "F16") return 2;
    return 0;
}

// The subset of JSON a safetensors header uses: objects, arrays, strings, non-negative integers.
class HeaderParser {
public:
    HeaderParser(const std::string& text, const std::string& path) : s_(text), path_(path) {}

    FileHeader parse() {
        FileHeader h;
        expect('{');
        if (!peek('}')) {
            do {
                const std::string name = string();
                expect(':');
                if (name == "__metadata__") metadata(h.metadata);
                else h.tensors[name] = tensor(name);
            } while (accept(','));
        }
        expect('}');
        skip();
        if (pos_ != s_.size()) fail("text after the header object");
        return h;
    }

private:
    [[noreturn]] void fail(const std::string& what) const {
        throw Error(RUMUS_HIP_EINVAL, path_ + ": malformed header (" + what + " at byte " + std::to_string(pos_) + ")");
    }
    void skip() { while (pos_ < s_.size() && (s_[pos_] == ' ' || s_[pos_] == '\n' || s_[pos_] == '\t' || s_[pos_] == '\r')) pos_++; }
    bool peek(char c) { skip(); return pos_ < s_.size() && s_[pos_] == c; }
    bool accept(char c) { if (peek(c)) { pos_++; return true; } return false; }
    void expect(char c) { if (!accept(c)) fail(std::string("expected '") + c + "'"); }

    std::string string() {
        expect('"');
        std::string out;
        while (true) {
            if (pos_ >= s_.size()) fail("unterminated string");
            char c = s_[pos_++];
            if (c == '"') return out;
            if (c != '\\') { out.push_back(c); continue; }
            if (pos_ >= s_.size()) fail("unterminated escape");
            c = s_[pos_++];
            switch (c) {
                case '"': case '\\': case '/': out.push_back(c); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'n': out.push_back('\n'); break;
                case 'r': out.push_back('\r'); break;
                case 't': out.push_back('\t'); break;
                case 'u': {
                    if (pos_ + 4 > s_.size()) fail("short \\u escape");
                    unsigned cp = 0;
                    for (int i = 0; i < 4; i++) {
                        const char h = s_[pos_++];
                        cp = cp * 16 + (h >= '0' && h <= '9' ? h - '0' : h >= 'a' && h <= 'f' ? h - 'a' + 10 :
                                        h >= 'A' && h <= 'F' ? h - 'A' + 10 : (fail("bad \\u escape"), 0));
                    }
                    if (cp < 0x80) out.push_back((char)cp);          // names and metadata here are ASCII;
                    else if (cp < 0x800) { out.push_back((char)(0xC0 | (cp >> 6))); out.push_back((char)(0x80 | (cp & 63))); }
                    else { out.push_back((char)(0xE0 | (cp >> 12))); out.push_back((char)(0x80 | ((cp >> 6) & 63))); out.push_back((char)(0x80 | (cp & 63))); }
                    break;
                }
                default: fail("unknown escape");
            }
        }
    }
    uint64_t integer() {
        skip();
        if (pos_ >= s_.size() || s_[pos_] < '0' || s_[pos_] > '9') fail("expected a non-negative integer");
        uint64_t v = 0;
        while (pos_ < s_.size() && s_[pos_] >= '0' && s_[pos_] <= '9') {
            if (v > (UINT64_MAX - 9) / 10) fail("integer overflow");
            v = v * 10 + (uint64_t)(s_[pos_++] - '0');
        }
        return v;
    }
    std::vector<uint64_t> integers() {
        std::vector<uint64_t> out;
        expect('[');
        if (!peek(']')) do out.push_back(integer()); while (accept(','));
        expect(']');
        return out;
    }
    void metadata(std::map<std::string, std::string>& out) {
        expect('{');
        if (!peek('}')) do { const std::string k = string(); expect(':'); out[k] = string(); } while (accept(','));
        expect('}');
    }
    FileTensor tensor(const std::string& name) {
        FileTensor t;
        bool have_dtype = false, have_shape = false, have_offsets = false;
        expect('{');
        do {
            const std::string key = string();
            expect(':');
            if (key == "dtype") { t.dtype = string(); have_dtype = true; }
            else if (key == "shape") { t.shape = integers(); have_shape = true; }
            else if (key == "data_offsets") {
                const auto o = integers();
                if (o.size() != 2) fail(name + ": data_offsets needs two entries");
                t.begin = o[0]; t.end = o[1]; have_offsets = true;
            } else fail(name + ": unknown key " + key);
        } while (accept(','));
        expect('}');
        if (!have_dtype || !have_shape || !have_offsets) fail(name + ": dtype, shape and data_offsets are required");
        return t;
    }

    const std::string& s_;
    std::string path_;
    size_t pos_ = 0;
};

struct FileCloser { void operator()(FILE* f) const { if (f) fclose(f); } };
using File = std::unique_ptr<FILE, FileCloser>;

inline File open_file(const std::string& path, const char* mode) {
    File f(fopen(path.c_str(), mode));
    if (!f) throw Error(RUMUS_HIP_EINVAL, path + ": cannot open");
    return f;
}

inline std::string json_string(const std::string& v) {
    std::string out = "\"";
    for (char c : v) {
        if (c == '"' || c == '\\') { out.push_back('\\'); out.push_back(c); }
        else if ((unsigned char)c < 0x20) { char buf[8]; snprintf(buf, sizeof buf, "\\u%04x", c); out += buf; }
        else out.push_back(c);
    }
    return out + "\"";
}

}  // namespace detail

// Header of a safetensors file; refuses what a truncated or foreign file would show (offsets
// outside the file, sizes that do not match shape x dtype, dtypes this library does not read).
inline FileHeader read_header(const std::string& path) {
    detail::File f = detail::open_file(path, "rb");
    require(fseek(f.get(), 0, SEEK_END) == 0, "seek failed");
    const long size_l = ftell(f.get());
    require(size_l >= 0 && fseek(f.get(), 0, SEEK_SET) == 0, "seek failed");
    const uint64_t size = (uint64_t)size_l;
    unsigned char len[8];
    if (fread(len, 1, 8, f.get()) != 8)
        throw Error(RUMUS_HIP_EINVAL, path + ": not a safetensors file (shorter than its length field)");
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; i--) hlen = (hlen << 8) | len[i];
    if (hlen > size - 8 || hlen > (100ull << 20))
        throw Error(RUMUS_HIP_EINVAL, path + ": header length " + std::to_string(hlen) + " does not fit the file");
    std::string text(hlen, '\0');
    if (hlen && fread(&text[0], 1, hlen, f.get()) != hlen) throw Error(RUMUS_HIP_EINVAL, path + ": short read");
    FileHeader h = detail::HeaderParser(text, path).parse();
    h.data_start = 8 + hlen;
    for (const auto& kv : h.tensors) {
        const FileTensor& t = kv.second;
        const size_t es = detail::dtype_size(t.dtype);
        if (!es) throw Error(RUMUS_HIP_EINVAL, path + ": " + kv.first + " has dtype " + t.dtype + ", which this loader does not read");
        if (t.end < t.begin || t.end - t.begin != t.numel() * es || h.data_start + t.end > size)
            throw Error(RUMUS_HIP_EINVAL, path + ": " + kv.first + " has offsets [" + std::to_string(t.begin) + ", " +
                                              std::to_string(t.end) + ") for " + std::to_string(t.numel() * es) +
                                              " bytes in a file of " + std::to_string(size));
    }
    return h;
}

// File ranges -> device memory through two pinned buffers.
class Uploader {
public:
    explicit Uploader(FILE* f, hipStream_t stream = nullptr, size_t chunk = (size_t)64 << 20)
        : f_(f), stream_(stream), chunk_(chunk) {
        for (int i = 0; i < 2; i++) {
            check_hip(hipHostMalloc(&pinned_[i], chunk_, hipHostMallocDefault), "hipHostMalloc");
            check_hip(hipEventCreateWithFlags(&done_[i], hipEventDisableTiming), "hipEventCreate");
        }
    }
    ~Uploader() {
        for (int i = 0; i < 2; i++) {
            if (used_[i]) (void)hipEventSynchronize(done_[i]);
            if (done_[i]) (void)hipEventDestroy(done_[i]);
            if (pinned_[i]) (void)hipHostFree(pinned_[i]);
        }
    }
    Uploader(const Uploader&) = delete;
    Uploader& operator=(const Uploader&) = delete;

    void fetch(uint64_t offset, uint64_t nbytes, void* device_dst) {
        require(fseek(f_, (long)offset, SEEK_SET) == 0, "seek failed");
        uint64_t pos = 0;
        while (pos < nbytes) {
            const size_t n = (size_t)std::min<uint64_t>(chunk_, nbytes - pos);
            const int slot = turn_;
            turn_ ^= 1;
            if (used_[slot]) check_hip(hipEventSynchronize(done_[slot]), "hipEventSynchronize");
            if (fread(pinned_[slot], 1, n, f_) != n) throw Error(RUMUS_HIP_EINVAL, "file ended early");
            check_hip(hipMemcpyAsync(static_cast<char*>(device_dst) + pos, pinned_[slot], n, hipMemcpyHostToDevice,
                                     stream_), "hipMemcpyAsync H2D");
            check_hip(hipEventRecord(done_[slot], stream_), "hipEventRecord");
            used_[slot] = true;
            pos += n;
        }
    }
    void finish() {
        for (int i = 0; i < 2; i++)
            if (used_[i]) check_hip(hipEventSynchronize(done_[i]), "hipEventSynchronize");
    }

private:
    FILE* f_;
    hipStream_t stream_;
    size_t chunk_;
    void* pinned_[2] = {nullptr, nullptr};
    hipEvent_t done_[2] = {nullptr, nullptr};
    bool used_[2] = {false, false};
    int turn_ = 0;
};

// Read every layer of the file into device memory: name -> QLinear, ready to run.
inline std::map<std::string, QLinear> load_w4(const std::string& path, hipStream_t stream = nullptr,
                                              size_t chunk_bytes = (size_t)64 << 20) {
    const FileHeader h = read_header(path);
    auto meta = [&](const std::string& key) -> const std::string* {
        auto it = h.metadata.find(key);
        return it == h.metadata.end() ? nullptr : &it->second;
    };
    if (!meta("format") || *meta("format") != "rumus-w4") throw Error(RUMUS_HIP_EINVAL, path + ": not a rumus-w4 file");
    if (!meta("version") || *meta("version") != "1") throw Error(RUMUS_HIP_EINVAL, path + ": unknown version");
    detail::File f = detail::open_file(path, "rb");
    Uploader up(f.get(), stream, chunk_bytes);

    auto find = [&](const std::string& name, const char* dtypes, std::vector<uint64_t> shape) -> const FileTensor* {
        auto it = h.tensors.find(name);
        if (it == h.tensors.end()) return nullptr;
        const FileTensor& t = it->second;
        if (std::string(dtypes).find(t.dtype) == std::string::npos)
            throw Error(RUMUS_HIP_EINVAL, path + ": " + name + " is " + t.dtype + ", expected " + dtypes);
        if (t.shape != shape) throw Error(RUMUS_HIP_EINVAL, path + ": " + name + " has an unexpected shape");
        return &t;
    };
    auto parse_u32 = [&](const std::string& key) -> uint32_t {
        const std::string* v = meta(key);
        if (!v || v->empty() || v->size() > 9 || v->find_first_not_of("0123456789") != std::string::npos)
            throw Error(RUMUS_HIP_EINVAL, path + ": metadata lacks " + key);
        return (uint32_t)std::stoul(*v);
    };

    std::map<std::string, QLinear> layers;
    const std::string suffix = ".qweight";
    for (const auto& kv : h.tensors) {
        const std::string& tname = kv.first;
        if (tname.size() <= suffix.size() || tname.compare(tname.size() - suffix.size(), suffix.size(), suffix) != 0)
            continue;
        const std::string name = tname.substr(0, tname.size() - suffix.size());
        const uint32_t k = parse_u32(name + ".k"), gs = parse_u32(name + ".group_size");
        if (gs == 0 || gs % 8 != 0) throw Error(RUMUS_HIP_EINVAL, path + ": " + name + ".group_size is not a multiple of 8");
        const uint32_t padded_k = ((k + gs - 1) / gs) * gs, groups = padded_k / gs;
        const FileTensor& qw = kv.second;
        if (qw.dtype != "I32" || qw.shape.size() != 2 || qw.shape[0] * 8 != padded_k || qw.shape[1] > UINT32_MAX)
            throw Error(RUMUS_HIP_EINVAL, path + ": " + tname + " must be I32 [" + std::to_string(padded_k / 8) + ", n]");
        const uint32_t n = (uint32_t)qw.shape[1];

        DeviceBuffer<uint32_t> packed(qw.numel());
        up.fetch(h.data_start + qw.begin, qw.end - qw.begin, packed.data());

        const FileTensor* sc = find(name + ".scales", "F32 F16", {groups, n});
        if (!sc) throw Error(RUMUS_HIP_EINVAL, path + ": " + name + ".scales is missing");
        DeviceBuffer<float> scales(sc->numel());
        if (sc->dtype == "F16") {
            DeviceBuffer<uint16_t> half(sc->numel());
            up.fetch(h.data_start + sc->begin, sc->end - sc->begin, half.data());
            check(rumus_hip_f16_to_f32(half.data(), scales.data(), sc->numel(), stream));
            check(rumus_hip_sync(stream));   // `half` is released here
        } else {
            up.fetch(h.data_start + sc->begin, sc->end - sc->begin, scales.data());
        }

        DeviceBuffer<float> zp((size_t)groups * n);
        if (const FileTensor* z = find(name + ".zeros", "F32", {groups, n})) {
            up.fetch(h.data_start + z->begin, z->end - z->begin, zp.data());
        } else {
            const FileTensor* qz = n % 8 == 0 ? find(name + ".qzeros", "I32", {groups, n / 8}) : nullptr;
            if (!qz) throw Error(RUMUS_HIP_EINVAL, path + ": " + name + " has neither zeros [groups, n] nor qzeros [groups, n/8]");
            DeviceBuffer<uint32_t> words(qz->numel());
            up.fetch(h.data_start + qz->begin, qz->end - qz->begin, words.data());
            check(rumus_hip_w4_qzeros_unpack(words.data(), groups, n, zp.data(), stream));
            check(rumus_hip_sync(stream));   // `words` is released here
        }

        QLinear layer;
        if (const FileTensor* b = find(name + ".bias", "F32", {n})) {
            layer.bias = DeviceBuffer<float>(n);
            up.fetch(h.data_start + b->begin, b->end - b->begin, layer.bias.data());
        }
        const FileTensor* pm = find(name + ".perm", "I32", {k});
        const FileTensor* gi = find(name + ".g_idx", "I32", {k});
        if (pm && gi) throw Error(RUMUS_HIP_EINVAL, path + ": " + name + " has both perm and g_idx");
        if (gi) {
            DeviceBuffer<int32_t> g_idx(k);
            up.fetch(h.data_start + gi->begin, gi->end - gi->begin, g_idx.data());
            layer.weight = QuantizedTensor::from_packed(std::move(packed), std::move(scales), std::move(zp), k, n, gs,
                                                        g_idx.data(), stream);
            check(rumus_hip_sync(stream));   // `g_idx` is released here
        } else {
            layer.weight = QuantizedTensor::from_packed(std::move(packed), std::move(scales), std::move(zp), k, n, gs,
                                                        nullptr, stream);
            if (pm) {
                require(k == padded_k, "perm needs k to be a multiple of group_size");
                // the kernels gather activations through perm without a bounds check of their own: every
                // input feature 0..k-1 must appear exactly once (checked on the host, before the upload)
                std::vector<int32_t> host_perm(k);
                require(fseek(f.get(), (long)(h.data_start + pm->begin), SEEK_SET) == 0, "seek failed");
                require(fread(host_perm.data(), 4, k, f.get()) == k, "file ended early");
                std::vector<char> seen(k, 0);
                for (uint32_t j = 0; j < k; j++) {
                    const int32_t v = host_perm[j];
                    require(v >= 0 && (uint32_t)v < k && !seen[v], "perm is not a permutation of 0..k-1");
                    seen[v] = 1;
                }
                layer.weight.perm = DeviceBuffer<int32_t>(k);
                up.fetch(h.data_start + pm->begin, pm->end - pm->begin, layer.weight.perm.data());
            }
        }
        layer.in_features = k;
        layer.out_features = n;
        layers.emplace(name, std::move(layer));
    }
    up.finish();
    check(rumus_hip_sync(stream));
    return layers;
}

// Write layers (name -> layer) with f32 zero-points, the reference's own fields.
inline void save_w4(const std::string& path, const std::map<std::string, const QLinear*>& layers) {
    struct Item { std::string name, dtype; std::vector<uint64_t> shape; std::vector<char> bytes; };
    std::vector<Item> items;
    auto add = [&](const std::string& name, const char* dtype, std::vector<uint64_t> shape, const void* dev, size_t nbytes) {
        Item it{name, dtype, std::move(shape), std::vector<char>(nbytes)};
        if (nbytes) check_hip(hipMemcpy(it.bytes.data(), dev, nbytes, hipMemcpyDeviceToHost), "hipMemcpy D2H");
        items.push_back(std::move(it));
    };
    std::string meta = "\"format\":\"rumus-w4\",\"version\":\"1\"";
    for (const auto& kv : layers) {                       // std::map: names in sorted order
        const QuantizedTensor& w = kv.second->weight;
        const std::string& name = kv.first;
        if (kv.second->bias.size()) add(name + ".bias", "F32", {w.n}, kv.second->bias.data(), (size_t)w.n * 4);
        if (w.perm.size()) add(name + ".perm", "I32", {w.k}, w.perm.data(), (size_t)w.k * 4);
        add(name + ".qweight", "I32", {w.padded_k / 8, w.n}, w.packed.data(), w.packed.size() * 4);
        add(name + ".scales", "F32", {w.num_groups, w.n}, w.scales.data(), w.scales.size() * 4);
        add(name + ".zeros", "F32", {w.num_groups, w.n}, w.zp.data(), w.zp.size() * 4);
        meta += "," + detail::json_string(name + ".k") + ":\"" + std::to_string(w.k) + "\"";
        meta += "," + detail::json_string(name + ".group_size") + ":\"" + std::to_string(w.group_size) + "\"";
    }
    std::string header = "{\"__metadata__\":{" + meta + "}";
    uint64_t offset = 0;
    for (const Item& it : items) {
        header += "," + detail::json_string(it.name) + ":{\"dtype\":\"" + it.dtype + "\",\"shape\":[";
        for (size_t i = 0; i < it.shape.size(); i++) header += (i ? "," : "") + std::to_string(it.shape[i]);
        header += "],\"data_offsets\":[" + std::to_string(offset) + "," + std::to_string(offset + it.bytes.size()) + "]}";
        offset += it.bytes.size();
    }
    header += "}";
    header.append((64 - (8 + header.size()) % 64) % 64, ' ');     // data start on a 64-byte boundary
    const std::string tmp = path + ".tmp";
    {
        detail::File f = detail::open_file(tmp, "wb");
        unsigned char len[8];
        for (int i = 0; i < 8; i++) len[i] = (unsigned char)((uint64_t)header.size() >> (8 * i));
        bool ok = fwrite(len, 1, 8, f.get()) == 8 && fwrite(header.data(), 1, header.size(), f.get()) == header.size();
        for (const Item& it : items)
            ok = ok && (it.bytes.empty() || fwrite(it.bytes.data(), 1, it.bytes.size(), f.get()) == it.bytes.size());
        ok = ok && fflush(f.get()) == 0;
        if (!ok) throw Error(RUMUS_HIP_EINVAL, tmp + ": write failed");
    }
    if (rename(tmp.c_str(), path.c_str()) != 0) throw Error(RUMUS_HIP_EINVAL, path + ": rename failed");
}

}  // namespace rumus_hip
