// GGUF side of the HIP loader in C++: what crates/luminal_hip/src/loader.rs does in Rust, which in turn is what
// `q8_load` of examples/llama/src/loader.rs:99-165 does for CUDA over the example's own reader
// (examples/llama/src/gguf.rs:190-263: header, key/value metadata, tensor infos; dtype numbers :283-303; the data
// section starts at the next multiple of `general.alignment`, default 32, :9,246-255).
//
// The reader keeps what the loader needs per tensor (element count, offset, ggml dtype) and skips the metadata
// values, except for `general.alignment`, which only the integer types of at most 32 bits can set.  Where the
// reference panics (unknown magic, unsupported version, unknown value type, unsupported tensor dtype) these throw
// luminal_hip::Panic.  Header-only; needs luminal_hip.hpp.
#pragma once

#include <cstdio>
#include <fstream>
#include <istream>

#include "luminal_hip.hpp"

namespace luminal_hip {

constexpr uint32_t kGgmlF32 = 0, kGgmlQ8_0 = 8;

struct GgufTensorInfo {
    uint64_t n_elements = 1;
    uint64_t offset = 0;  // from the start of the data section
    uint32_t dtype = 0;
};

struct GgufHeader {
    uint32_t version = 0;
    uint64_t alignment = 32;
    uint64_t data_offset = 0;
    std::map<std::string, GgufTensorInfo> tensors;
};

class GgufReader {
  public:
    explicit GgufReader(std::istream &in) : in_(in) {}

    GgufHeader read_header() {
        GgufHeader h;
        const uint32_t magic = u32();
        if (magic != 0x46554747u && magic != 0x47475546u) throw Panic("unknown magic " + hex(magic));
        h.version = u32();
        if (h.version < 1 || h.version > 3) throw Panic("gguf: unsupported version " + std::to_string(h.version));
        wide_ = h.version > 1;  // versions 2 and 3 hold 64-bit counts and lengths, version 1 32-bit ones
        const uint64_t tensor_count = size(), kv_count = size();
        for (uint64_t i = 0; i < kv_count; ++i) {
            const std::string key = string();
            const uint32_t type = u32();
            int64_t small = 0;
            const bool is_small_int = value(type, small);
            if (key == "general.alignment" && is_small_int && small > 0) h.alignment = static_cast<uint64_t>(small);
        }
        for (uint64_t i = 0; i < tensor_count; ++i) {
            const std::string name = string();
            GgufTensorInfo t;
            const uint32_t n_dims = u32();
            for (uint32_t d = 0; d < n_dims; ++d) t.n_elements *= size();
            t.dtype = u32();
            t.offset = u64();
            h.tensors[name] = t;
        }
        const uint64_t pos = static_cast<uint64_t>(in_.tellg());
        h.data_offset = (pos + h.alignment - 1) / h.alignment * h.alignment;
        return h;
    }

  private:
    template <typename T>
    T raw() {
        T v{};
        in_.read(reinterpret_cast<char *>(&v), sizeof(T));  // the format and the hosts this runs on are little-endian
        if (!in_) throw Panic("gguf: unexpected end of file");
        return v;
    }
    uint32_t u32() { return raw<uint32_t>(); }
    uint64_t u64() { return raw<uint64_t>(); }
    uint64_t size() { return wide_ ? u64() : u32(); }
    std::string string() {
        const uint64_t n = size();
        if (n > (uint64_t{1} << 30)) throw Panic("gguf: unreasonable string length");
        std::string s(n, '\0');
        in_.read(s.data(), static_cast<std::streamsize>(n));
        if (!in_) throw Panic("gguf: unexpected end of file");
        while (!s.empty() && s.back() == '\0') s.pop_back();  // version-1 files may carry a terminator
        return s;
    }
    // Reads one metadata value of type `type`; true (and the value) when it is an integer of at most 32 bits.
    bool value(uint32_t type, int64_t &small) {
        switch (type) {
            case 0: small = raw<uint8_t>(); return true;
            case 1: small = raw<int8_t>(); return true;
            case 2: small = raw<uint16_t>(); return true;
            case 3: small = raw<int16_t>(); return true;
            case 4: small = raw<uint32_t>(); return true;
            case 5: small = raw<int32_t>(); return true;
            case 6: raw<float>(); return false;
            case 7: {
                const uint8_t b = raw<uint8_t>();
                if (b > 1) throw Panic("unexpected bool value " + std::to_string(b));
                return false;
            }
            case 8: string(); return false;
            case 9: {
                const uint32_t element = u32();
                const uint64_t n = size();
                int64_t ignored;
                for (uint64_t i = 0; i < n; ++i) value(element, ignored);
                return false;
            }
            case 10: case 11: raw<uint64_t>(); return false;
            case 12: raw<double>(); return false;
            default: throw Panic("unrecognized value-type " + hex(type));
        }
    }
    static std::string hex(uint32_t v) {
        char buf[16];
        std::snprintf(buf, sizeof buf, "0x%08x", v);
        return buf;
    }
    std::istream &in_;
    bool wide_ = true;
};

// Points every named parameter of the graph at its tensor in the GGUF file: F32 tensors become host vectors, Q8_0
// tensors (n + n/16 bytes) are uploaded and re-arranged into the planar form (which depends on the number of blocks
// only, so (n_elements / 32, 32) is as good a shape as the tensor's own); any other dtype panics like the reference
// loader.  Returns the nodes that hold Q8_0 weights, for HipQuantizedCompiler.  Unlike the reference (and the Rust
// crate), which read a tensor when the graph first runs its node, this reads at once: the graph model here has
// no lazily evaluated inputs.
inline std::vector<NodeIndex> q8_load_hip_file(const std::string &path, Graph &g, const std::map<std::string, NodeIndex> &params) {
    std::ifstream file(path, std::ios::binary);
    if (!file) throw Panic("cannot open " + path);
    const GgufHeader h = GgufReader(file).read_header();
    std::vector<NodeIndex> q_weights;
    for (auto &[name, node] : params) {
        auto *f = dynamic_cast<Function *>(g.nodes.at(node).get());
        if (!f) throw Panic("loader target is not a graph input");
        std::string key = name;
        std::replace(key.begin(), key.end(), '/', '.');  // loader.rs:43
        auto it = h.tensors.find(key);
        if (it == h.tensors.end()) throw Panic("tensor " + key + " is not in the file");
        const GgufTensorInfo &t = it->second;
        size_t n_bytes;
        if (t.dtype == kGgmlF32) n_bytes = t.n_elements * 4;
        else if (t.dtype == kGgmlQ8_0) n_bytes = t.n_elements + t.n_elements / 16;
        else throw Panic("Unsupported dtype: " + std::to_string(t.dtype));
        std::vector<uint8_t> bytes(n_bytes);
        file.seekg(static_cast<std::streamoff>(h.data_offset + t.offset));
        file.read(reinterpret_cast<char *>(bytes.data()), static_cast<std::streamsize>(n_bytes));
        if (!file) throw Panic("gguf: tensor " + key + " runs past the end of the file");
        if (t.dtype == kGgmlF32) {
            std::vector<float> v(t.n_elements);
            std::memcpy(v.data(), bytes.data(), n_bytes);
            f->value = host_tensor(std::move(v));
        } else {
            if (t.n_elements % 32 != 0) throw Panic("Q8_0 tensors hold whole blocks of 32");
            f->value = Tensor{HipData::q8_0_from_raw(bytes, static_cast<int64_t>(t.n_elements / 32), 32)};
            q_weights.push_back(node);
        }
    }
    return q_weights;
}

}  // namespace luminal_hip
