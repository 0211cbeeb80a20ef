// C++ host side of the luminal_hip backend: what the Rust crate `luminal_hip` does above the C ABI, restated in
// C++ because the reference's own toolchain (cargo) is not available where this library is built.
//
// Names, argument meaning and failure behaviour follow the reference:
//   HipData                 <- CudaData<T>                         crates/luminal_cuda/src/lib.rs:83-100
//   Operator::process       <- trait Operator                      src/op.rs:82-90
//   QuantizedMatmul         <- QuantizedMatmul<T>, T = f32 | f16   crates/luminal_cuda/src/quantized.rs:111-168
//   QuantizedGather         <- QuantizedGather<T>                  crates/luminal_cuda/src/quantized.rs:170-233
//   HipCopyToDevice / HipCopyFromDevice <- CudaCopyToDevice / CudaCopyFromDevice   crates/luminal_cuda/src/prim.rs:20-75
//   HipQuantizedCompiler    <- CudaQuantizedCompiler<T>            crates/luminal_cuda/src/quantized.rs:235-272
//   downstream              <- luminal::module::downstream         src/module.rs:84-113
// Where the reference panics (unwrap / assert! / panic!), these throw luminal_hip::Panic with the same message.
//
// Unlike the CUDA pass, which runs behind a dense CUDA compiler and finds ready-made Matmul<T> / CudaGather<T>
// nodes, this pass is meant to run directly behind the generic compiler: (GenericCompiler, HipQuantizedCompiler).
// The graph then still holds luminal's primitive operators, which execute on host f32 vectors (src/op.rs), so the
// pass itself
//   * recognises the matmul as the primitives spell it, Mul -> SumReduce over fake-expanded operands
//     (src/hl_ops/matmul.rs:4-33; the pattern crates/luminal_cpu/src/matmul.rs:11-59,97-146 matches), and the row
//     gather as Mul(one-hot, table) -> SumReduce(1) (src/hl_ops/other.rs:114-123), downstream of each Q8_0 weight;
//   * replaces them by QuantizedMatmul / QuantizedGather nodes, and
//   * puts copy nodes around those (activations host -> device in front, device -> host behind, as
//     crates/luminal_cuda/src/prim.rs:687-767 does around the host-side Function nodes), so that every other node
//     keeps seeing host vectors.
// The graph model below is the minimum that takes: primitive operators with their host execution, stride-based
// shape trackers with fake (expanded) dimensions, data edges carrying (input_order, shape), to_retrieve marks and
// a topological executor.  Header-only; links against libluminal_hip.so only.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <functional>
#include <iterator>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <utility>
#include <variant>
#include <vector>

#include "../../include/luminal_hip.h"

namespace luminal_hip {

struct Panic : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline void check(lhip_status s, const char *what) {
    if (s != LHIP_OK)
        throw Panic(std::string(what) + ": " + lhip_status_string(s) + " (hipError_t " +
                    std::to_string(lhip_last_hip_error()) + ")");
}

// Owned device allocation.
class HipData {
  public:
    explicit HipData(size_t bytes) : bytes_(bytes) { check(lhip_malloc(&ptr_, bytes ? bytes : 1), "lhip_malloc"); }
    HipData(const HipData &) = delete;
    HipData &operator=(const HipData &) = delete;
    ~HipData() { lhip_free(ptr_); }
    template <typename T>
    static std::shared_ptr<HipData> from_host(const std::vector<T> &host) {
        auto d = std::make_shared<HipData>(host.size() * sizeof(T));
        check(lhip_memcpy_h2d(d->ptr_, host.data(), d->bytes_, nullptr), "lhip_memcpy_h2d");
        return d;
    }
    std::vector<float> to_host_f32() const {
        std::vector<float> v(bytes_ / sizeof(float));
        check(lhip_memcpy_d2h(v.data(), ptr_, bytes_, nullptr), "lhip_memcpy_d2h");
        return v;
    }
    std::vector<uint16_t> to_host_f16_codes() const {
        std::vector<uint16_t> v(bytes_ / sizeof(uint16_t));
        check(lhip_memcpy_d2h(v.data(), ptr_, bytes_, nullptr), "lhip_memcpy_d2h");
        return v;
    }
    // Raw GGUF Q8_0 blocks of an (n, k) weight -> planar device buffer: what the HIP loader keeps per tensor
    // (q8_load_hip below; examples/llama/src/loader.rs:124-158 copies the same bytes to the device untouched).
    static std::shared_ptr<HipData> q8_0_from_raw(const std::vector<uint8_t> &raw_blocks, int64_t n, int64_t k) {
        if (raw_blocks.size() != lhip_q8_0_raw_nbytes(n, k) || raw_blocks.empty())
            throw Panic("Q8_0 tensor has " + std::to_string(raw_blocks.size()) + " bytes, expected n + n/16");
        auto staged = from_host(raw_blocks);
        auto planar = std::make_shared<HipData>(lhip_q8_0_planar_nbytes(n, k));
        check(lhip_q8_0_repack(staged->ptr(), planar->ptr(), n, k, nullptr), "lhip_q8_0_repack");
        check(lhip_stream_sync(nullptr), "lhip_stream_sync");
        return planar;
    }
    void *ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }

  private:
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
};

// A tensor's payload: host f32 (what the primitive operators and the token ids use) or a device buffer.
using HostVec = std::shared_ptr<std::vector<float>>;
using Data = std::variant<std::monostate, HostVec, std::shared_ptr<HipData>>;

struct Tensor {
    Data data;
};

inline Tensor host_tensor(std::vector<float> v) { return Tensor{std::make_shared<std::vector<float>>(std::move(v))}; }

// The part of luminal's ShapeTracker this path reads: dimensions, strides into the source's storage, and which
// dimensions are fake (expanded: stride 0).  A view is contiguous when its strides are the row-major ones of its
// dimensions (no permutation, no fake dimension).
struct ShapeTracker {
    std::vector<int64_t> dims, strides;
    ShapeTracker() = default;
    ShapeTracker(std::vector<int64_t> d) : dims(std::move(d)), strides(dims.size()) {  // contiguous
        int64_t s = 1;
        for (size_t i = dims.size(); i-- > 0;) {
            strides[i] = s;
            s *= dims[i];
        }
    }
    int64_t n_elements() const {
        int64_t n = 1;
        for (auto d : dims) n *= d;
        return n;
    }
    size_t rank() const { return dims.size(); }
    bool is_fake(size_t axis) const { return strides.at(axis) == 0; }
    bool is_contiguous() const { return strides == ShapeTracker(dims).strides; }
    ShapeTracker expand_dim(size_t axis, int64_t size) const {
        ShapeTracker r = *this;
        r.dims.insert(r.dims.begin() + axis, size);
        r.strides.insert(r.strides.begin() + axis, 0);
        return r;
    }
    ShapeTracker remove_dim(size_t axis) const {
        ShapeTracker r = *this;
        r.dims.erase(r.dims.begin() + axis);
        r.strides.erase(r.strides.begin() + axis);
        return r;
    }
    ShapeTracker permute(const std::vector<size_t> &order) const {
        ShapeTracker r;
        for (size_t a : order) {
            r.dims.push_back(dims.at(a));
            r.strides.push_back(strides.at(a));
        }
        return r;
    }
    // storage index of logical element i (row-major over dims)
    int64_t index(int64_t i) const {
        int64_t at = 0;
        for (size_t a = dims.size(); a-- > 0;) {
            at += (i % dims[a]) * strides[a];
            i /= dims[a];
        }
        return at;
    }
};

using Input = std::pair<const Tensor *, ShapeTracker>;

struct Operator {
    virtual ~Operator() = default;
    // One tensor per output (src/op.rs:82-90 returns Vec<Tensor>); most operators have one.
    virtual std::vector<Tensor> process(const std::vector<Input> &inp) = 0;
    virtual std::string name() const = 0;
};

inline const HipData &device_operand(const Tensor &t, const char *what) {
    auto p = std::get_if<std::shared_ptr<HipData>>(&t.data);
    if (!p || !*p) throw Panic(std::string(what) + " is not a HIP buffer");
    return **p;
}
inline const std::vector<float> &host_operand(const Tensor &t, const char *what) {
    auto p = std::get_if<HostVec>(&t.data);
    if (!p || !*p) throw Panic(std::string(what) + " is not a host f32 vector");  // downcast_ref::<Vec<f32>>().unwrap()
    return **p;
}

// The reference's operators are generic over the activation type T (f32 or f16); here it is a run-time tag.
enum class DType { F32, F16 };
inline size_t dtype_size(DType t) { return t == DType::F32 ? 4 : 2; }

// (batch.., m, K) T x Q8_0 (N, K) -> (batch.., m, N) T.  inp[0] = activations, a device buffer of T (the pass puts
// a HipCopyToDevice in front of a host producer); inp[1] = weight with dims [.., K, N], necessarily a permuted
// (non-contiguous) view.  Launches and returns: nothing here waits for the device.
class QuantizedMatmul : public Operator {
  public:
    explicit QuantizedMatmul(DType dtype = DType::F32) : dtype(dtype) {}
    DType dtype;
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        const ShapeTracker &a = inp.at(0).second, &b = inp.at(1).second;
        if (b.is_contiguous()) throw Panic("Weight matrix must be column-major");
        if (a.dims.empty() || b.dims.size() < 2) throw Panic("QuantizedMatmul: operands need at least 1 and 2 dims");
        const int64_t k = b.dims[b.dims.size() - 2], n = b.dims[b.dims.size() - 1];
        if (a.dims.back() != k) throw Panic("QuantizedMatmul: inner dimensions differ");
        const int64_t rows = std::max<int64_t>(a.n_elements() / k, 1);  // batch * m
        const void *x = device_operand(*inp[0].first, "activation").ptr();
        auto out = std::make_shared<HipData>(static_cast<size_t>(rows * n) * dtype_size(dtype));
        const void *w = device_operand(*inp[1].first, "weight").ptr();
        if (dtype == DType::F32)
            check(lhip_q8_0_matmul_f32(w, static_cast<const float *>(x), static_cast<float *>(out->ptr()), rows, n, k,
                                       nullptr),
                  "lhip_q8_0_matmul_f32");
        else
            check(lhip_q8_0_matmul_f16(w, x, out->ptr(), rows, n, k, nullptr), "lhip_q8_0_matmul_f16");
        return {Tensor{out}};
    }
    std::string name() const override { return "QuantizedMatmul"; }
};

// Row gather from a Q8_0 embedding table; indices arrive as host f32, as in every luminal backend, and are copied
// to the device here (quantized.rs:205-208).  The staged indices stay alive in the operator until its next call,
// so nothing waits for the device.
class QuantizedGather : public Operator {
  public:
    explicit QuantizedGather(int64_t embed_dim, DType dtype = DType::F32) : embed_dim(embed_dim), dtype(dtype) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        const std::vector<float> &idx = host_operand(*inp.at(0).first, "gather indices");
        const int64_t vocab = inp.at(1).second.n_elements() / embed_dim;
        staged_ = HipData::from_host(idx);
        auto out = std::make_shared<HipData>(idx.size() * embed_dim * dtype_size(dtype));
        const void *table = device_operand(*inp[1].first, "table").ptr();
        const auto *ids = static_cast<const float *>(staged_->ptr());
        const auto count = static_cast<int64_t>(idx.size());
        if (dtype == DType::F32)
            check(lhip_q8_0_gather_f32(table, ids, static_cast<float *>(out->ptr()), count, vocab, embed_dim, nullptr),
                  "lhip_q8_0_gather_f32");
        else
            check(lhip_q8_0_gather_f16(table, ids, out->ptr(), count, vocab, embed_dim, nullptr), "lhip_q8_0_gather_f16");
        return {Tensor{out}};
    }
    std::string name() const override { return "QuantizedGather"; }
    int64_t embed_dim;
    DType dtype;

  private:
    std::shared_ptr<HipData> staged_;
};

// f32 <-> IEEE binary16 on the host (T::from_f32 / T::to_f32 of the reference's copy operators for T = f16):
// round to nearest even, subnormals and overflow to infinity included.
inline uint16_t f32_to_f16_code(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) return static_cast<uint16_t>(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u : 0));  // inf / NaN
    if (mag >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);                                    // rounds to inf
    if (mag < 0x33000001u) return static_cast<uint16_t>(sign);                                               // rounds to zero
    int e = static_cast<int>(mag >> 23) - 127 + 15;
    uint32_t m = (mag & 0x7fffffu) | 0x800000u;  // 24-bit significand
    int shift = 13;
    if (e <= 0) {  // subnormal result
        shift += 1 - e;
        e = 0;
    }
    uint32_t h = m >> shift;
    const uint32_t rest = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rest > half || (rest == half && (h & 1u))) ++h;
    h += static_cast<uint32_t>(e > 0 ? e - 1 : 0) << 10;  // the hidden bit carries into the exponent field
    return static_cast<uint16_t>(sign | h);
}
inline float f16_code_to_f32(uint16_t c) {
    const int e = (c >> 10) & 31, m = c & 1023;
    float v;
    if (e == 31) v = m ? NAN : INFINITY;
    else v = e == 0 ? std::ldexp(static_cast<float>(m), -24) : std::ldexp(1.0f + m / 1024.0f, e - 15);
    return (c & 0x8000) ? -v : v;
}

// Host vector -> device buffer of T (a tensor already on the device passes through), prim.rs:31-46.
struct HipCopyToDevice : Operator {
    DType dtype;
    explicit HipCopyToDevice(DType t = DType::F32) : dtype(t) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        if (std::holds_alternative<std::shared_ptr<HipData>>(inp.at(0).first->data)) return {*inp[0].first};
        const std::vector<float> &v = host_operand(*inp[0].first, "copy source");
        if (dtype == DType::F32) return {Tensor{HipData::from_host(v)}};
        std::vector<uint16_t> codes(v.size());
        for (size_t i = 0; i < v.size(); ++i) codes[i] = f32_to_f16_code(v[i]);
        return {Tensor{HipData::from_host(codes)}};
    }
    std::string name() const override { return "HipCopyToDevice"; }
};
// Device buffer of T -> host f32 vector (a host tensor passes through), prim.rs:60-75.  The copy waits for the
// stream: the one place where host and device meet, as memcpy_dtov is in the reference.
struct HipCopyFromDevice : Operator {
    DType dtype;
    explicit HipCopyFromDevice(DType t = DType::F32) : dtype(t) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        if (std::holds_alternative<HostVec>(inp.at(0).first->data)) return {*inp[0].first};
        const HipData &d = device_operand(*inp[0].first, "copy source");
        if (dtype == DType::F32) return {host_tensor(d.to_host_f32())};
        std::vector<float> v;
        for (uint16_t c : d.to_host_f16_codes()) v.push_back(f16_code_to_f32(c));
        return {host_tensor(std::move(v))};
    }
    std::string name() const override { return "HipCopyFromDevice"; }
};

// ---- luminal's primitive operators, executing on host f32 like src/op.rs ------------------------------------
struct Function : Operator {  // graph input: yields the tensor set on it (weights, activations, token ids)
    Tensor value;
    std::vector<Tensor> process(const std::vector<Input> &) override { return {value}; }
    std::string name() const override { return "Function"; }
};
struct Constant : Operator {  // src/op.rs:157-190
    float value;
    explicit Constant(float v) : value(v) {}
    std::vector<Tensor> process(const std::vector<Input> &) override { return {host_tensor({value})}; }
    std::string name() const override { return "Constant(" + std::to_string(value) + ")"; }
};
struct ARange : Operator {  // 0 .. n-1 (luminal builds it from a constant and a cumulative sum, src/hl_ops/other.rs:63-71)
    int64_t n;
    explicit ARange(int64_t n) : n(n) {}
    std::vector<Tensor> process(const std::vector<Input> &) override {
        std::vector<float> v(n);
        for (int64_t i = 0; i < n; ++i) v[i] = static_cast<float>(i);
        return {host_tensor(std::move(v))};
    }
    std::string name() const override { return "ARange"; }
};
// Element-wise binary primitives over two views of equal dims (src/op.rs:278-357): the result is contiguous.
struct Binary : Operator {
    enum Kind { Add, Mul, LessThan } kind;
    explicit Binary(Kind k) : kind(k) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        const auto &a = host_operand(*inp.at(0).first, "lhs"), &b = host_operand(*inp.at(1).first, "rhs");
        const ShapeTracker &sa = inp[0].second, &sb = inp[1].second;
        if (sa.dims != sb.dims) throw Panic("Dims must match");
        std::vector<float> out(sa.n_elements());
        for (int64_t i = 0; i < static_cast<int64_t>(out.size()); ++i) {
            const float x = a[sa.index(i)], y = b[sb.index(i)];
            out[i] = kind == Add ? x + y : kind == Mul ? x * y : (x < y ? 1.f : 0.f);
        }
        return {host_tensor(std::move(out))};
    }
    std::string name() const override { return kind == Add ? "Add" : kind == Mul ? "Mul" : "LessThan"; }
};
struct SumReduce : Operator {  // src/op.rs:361-382: f32 sum in increasing index along `dim`
    size_t dim;
    explicit SumReduce(size_t d) : dim(d) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        const auto &a = host_operand(*inp.at(0).first, "input");
        const ShapeTracker &s = inp[0].second;
        int64_t front = 1, back = 1;
        for (size_t i = 0; i < dim; ++i) front *= s.dims[i];
        for (size_t i = dim + 1; i < s.rank(); ++i) back *= s.dims[i];
        const int64_t len = s.dims.at(dim);
        std::vector<float> out(front * back, 0.f);
        for (int64_t f = 0; f < front; ++f)
            for (int64_t b = 0; b < back; ++b)
                for (int64_t j = 0; j < len; ++j) out[f * back + b] += a[s.index((f * len + j) * back + b)];
        return {host_tensor(std::move(out))};
    }
    std::string name() const override { return "SumReduce(" + std::to_string(dim) + ")"; }
};
struct Unary : Operator {  // any single-input host op, e.g. the contiguous copy a loader may leave behind a weight
    std::string label;
    std::function<float(float)> fn;
    explicit Unary(std::string l, std::function<float(float)> f = nullptr) : label(std::move(l)), fn(std::move(f)) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        if (!fn) return {*inp.at(0).first};
        const auto &a = host_operand(*inp.at(0).first, "input");  // a device buffer here is the reference's unwrap panic
        const ShapeTracker &s = inp[0].second;
        std::vector<float> out(s.n_elements());
        for (int64_t i = 0; i < static_cast<int64_t>(out.size()); ++i) out[i] = fn(a[s.index(i)]);
        return {host_tensor(std::move(out))};
    }
    std::string name() const override { return label; }
};

using NodeIndex = int;

struct Edge {  // Dependency::Data { input_order, output_order, shape } of src/graph.rs
    NodeIndex src, dst;
    int input_order;
    ShapeTracker shape;
    int output_order = 0;
};

struct Graph {
    std::vector<std::unique_ptr<Operator>> nodes;  // a removed node leaves a null slot
    std::vector<Edge> edges;
    std::set<NodeIndex> to_retrieve;               // nodes whose results the caller reads as host vectors
    std::set<NodeIndex> no_delete;                 // nodes whose results outlive an execution (weights and what is made of them once)
    std::map<NodeIndex, Tensor> results;           // output 0 of every executed node
    std::map<std::pair<NodeIndex, int>, Tensor> more_results;  // outputs 1.. of the operators that have them

    NodeIndex add(std::unique_ptr<Operator> op) {
        nodes.push_back(std::move(op));
        return static_cast<NodeIndex>(nodes.size()) - 1;
    }
    void connect(NodeIndex src, NodeIndex dst, int input_order, ShapeTracker shape, int output_order = 0) {
        edges.push_back({src, dst, input_order, std::move(shape), output_order});
    }
    const Tensor &result(NodeIndex n, int output_order = 0) const {
        return output_order == 0 ? results.at(n) : more_results.at({n, output_order});
    }
    void remove_node(NodeIndex n) {
        nodes.at(n).reset();
        edges.erase(std::remove_if(edges.begin(), edges.end(), [&](const Edge &e) { return e.src == n || e.dst == n; }),
                    edges.end());
    }
    std::vector<const Edge *> outgoing(NodeIndex n) const {
        std::vector<const Edge *> v;
        for (auto &e : edges)
            if (e.src == n) v.push_back(&e);
        return v;
    }
    std::vector<const Edge *> incoming(NodeIndex n) const {
        std::vector<const Edge *> v;
        for (auto &e : edges)
            if (e.dst == n) v.push_back(&e);
        std::sort(v.begin(), v.end(), [](auto a, auto b) { return a->input_order < b->input_order; });
        return v;
    }
    // Forward execution in topological order.  As in src/graph.rs:199-202 a node whose result is already there is
    // not run again; only the results of no_delete nodes are there when an execution starts.
    void execute() {
        for (auto it = results.begin(); it != results.end();) it = no_delete.count(it->first) ? std::next(it) : results.erase(it);
        for (auto it = more_results.begin(); it != more_results.end();)
            it = no_delete.count(it->first.first) ? std::next(it) : more_results.erase(it);
        std::vector<int> pending(nodes.size(), 0);
        for (auto &e : edges) ++pending[e.dst];
        std::vector<NodeIndex> ready;
        for (NodeIndex n = 0; n < static_cast<NodeIndex>(nodes.size()); ++n)
            if (nodes[n] && pending[n] == 0) ready.push_back(n);
        size_t done = 0, live = 0;
        for (auto &n : nodes) live += n != nullptr;
        while (!ready.empty()) {
            const NodeIndex n = ready.back();
            ready.pop_back();
            if (!results.count(n)) {
                std::vector<Input> inp;
                for (auto e : incoming(n)) inp.emplace_back(&result(e->src, e->output_order), e->shape);
                std::vector<Tensor> out = nodes[n]->process(inp);
                results[n] = out.at(0);
                for (size_t i = 1; i < out.size(); ++i) more_results[{n, static_cast<int>(i)}] = out[i];
            }
            ++done;
            for (auto e : outgoing(n))
                if (--pending[e->dst] == 0) ready.push_back(e->dst);
        }
        if (done != live) throw Panic("graph has a cycle");
    }
};

// luminal::module::downstream: follow each node along single-consumer edges while the consumer depends on nothing
// but the original set; the returned nodes are the ones whose consumers the pass rewrites.
inline std::vector<NodeIndex> downstream(const std::vector<NodeIndex> &nodes, const Graph &g) {
    const std::set<NodeIndex> orig(nodes.begin(), nodes.end());
    std::function<bool(NodeIndex)> from_set = [&](NodeIndex n) {
        if (orig.count(n)) return true;
        auto in = g.incoming(n);
        if (in.empty()) return false;
        return std::all_of(in.begin(), in.end(), [&](const Edge *e) { return from_set(e->src); });
    };
    std::vector<NodeIndex> fin;
    std::set<NodeIndex> added;
    for (NodeIndex node : nodes) {
        while (g.outgoing(node).size() == 1) {
            const NodeIndex next = g.outgoing(node)[0]->dst;
            if (!from_set(next)) break;
            node = next;
        }
        if (added.insert(node).second) fin.push_back(node);
    }
    return fin;
}

// Rewrites the consumers of the given Q8_0 weight nodes into the HIP quantized operators.
class HipQuantizedCompiler {
  public:
    explicit HipQuantizedCompiler(std::vector<NodeIndex> weights, DType dtype = DType::F32)
        : weights_(std::move(weights)), dtype_(dtype) {}

    // init_device = false leaves device selection to the caller (and lets the rewrite be exercised without a GPU).
    void compile(Graph &graph, bool init_device = true) const {
        if (init_device) check(lhip_init(0), "lhip_init");
        std::vector<NodeIndex> quantized;
        for (NodeIndex weight : downstream(weights_, graph)) {
            // copied: the rewrite below edits the edge list
            std::vector<Edge> uses;
            for (const Edge *e : graph.outgoing(weight)) uses.push_back(*e);
            for (const Edge &e : uses) {
                const std::string target = "NodeIndex(" + std::to_string(e.dst) + ")";
                if (e.input_order != 1) throw Panic("Quantized weight " + target + " is the wrong input!");
                NodeIndex made = -1;
                auto *mul = dynamic_cast<Binary *>(graph.nodes[e.dst].get());
                if (mul && mul->kind == Binary::Mul) made = rewrite_mul(graph, e);
                if (made < 0)
                    throw Panic("Quantized weight " + target + " is an input to a node that isn't a matmul or gather (" +
                                graph.nodes[e.dst]->name() + ")");
                quantized.push_back(made);
            }
        }
        for (NodeIndex q : quantized) insert_copies(graph, q, dtype_);
    }

  private:
    // The Mul that consumes a weight, together with the SumReduce behind it, as a matmul or a gather: returns the new
    // node, or -1 if the shapes spell neither.
    //   matmul  (src/hl_ops/matmul.rs:4-33): rank r >= 3, activations [.., M, N(fake), K], weight [..(fake), M(fake), N, K],
    //           SumReduce(r - 1); the weight storage is (N, K) row-major.  As crates/luminal_cpu/src/matmul.rs:37-41 the fake
    //           dimensions are taken off and the weight's last two dimensions swapped, which makes its view [K, N].
    //   gather  (src/hl_ops/other.rs:114-123): one-hot [B, V, D(fake)] times table [B(fake), V, D], SumReduce(1); the
    //           indices are found above the one-hot as the operand that was expanded over the vocabulary, [B, V(fake)].
    NodeIndex rewrite_mul(Graph &g, const Edge &w_edge) const {
        const NodeIndex mul = w_edge.dst;
        auto outs = g.outgoing(mul);
        if (outs.size() != 1) return -1;
        const NodeIndex red = outs[0]->dst;
        auto *sum = dynamic_cast<SumReduce *>(g.nodes[red].get());
        auto ins = g.incoming(mul);
        if (!sum || ins.size() != 2) return -1;
        const Edge a_edge = *ins[0];
        const ShapeTracker &a = a_edge.shape, &w = w_edge.shape;
        const size_t r = w.rank();
        if (a.rank() != r || a.dims != w.dims || r < 3) return -1;
        NodeIndex made = -1;
        bool w_lead_fake = true, a_lead_real = true;
        for (size_t i = 0; i + 2 < r; ++i) {
            w_lead_fake &= w.is_fake(i);
            a_lead_real &= !a.is_fake(i);
        }
        if (sum->dim == r - 1 && w_lead_fake && a_lead_real && a.is_fake(r - 2) && !a.is_fake(r - 1) && !w.is_fake(r - 2) &&
            !w.is_fake(r - 1)) {
            ShapeTracker as = a.remove_dim(r - 2), ws = w;
            for (size_t i = 0; i + 2 < r; ++i) ws = ws.remove_dim(0);
            ws = ws.permute({1, 0});
            made = g.add(std::make_unique<QuantizedMatmul>(dtype_));
            g.connect(a_edge.src, made, 0, as);
            g.connect(w_edge.src, made, 1, ws);
        } else if (r == 3 && sum->dim == 1 && w.is_fake(0) && !w.is_fake(1) && !w.is_fake(2) && a.is_fake(2) &&
                   !a.is_fake(0) && !a.is_fake(1)) {
            const Edge *idx = find_indices(g, a_edge.src, w.dims[0], w.dims[1]);
            if (!idx) return -1;
            made = g.add(std::make_unique<QuantizedGather>(w.dims[2], dtype_));
            g.connect(idx->src, made, 0, idx->shape.remove_dim(1));
            g.connect(w_edge.src, made, 1, w.remove_dim(0));
        } else {
            return -1;
        }
        // the consumers of the SumReduce now read the new node; Mul and SumReduce go, and what only fed them with it
        std::vector<Edge> moved;
        for (const Edge *e : g.outgoing(red)) moved.push_back(*e);
        if (g.to_retrieve.erase(red)) g.to_retrieve.insert(made);
        g.remove_node(red);
        const NodeIndex a_src = a_edge.src;
        g.remove_node(mul);
        for (Edge e : moved) g.connect(made, e.dst, e.input_order, e.shape);
        prune_dead(g, a_src);
        return made;
    }

    // Above the one-hot mask: the operand that is not derived from constants alone and enters as [B, V(fake)].
    static const Edge *find_indices(const Graph &g, NodeIndex from, int64_t batch, int64_t vocab) {
        std::function<bool(NodeIndex)> constant_only = [&](NodeIndex n) {
            if (dynamic_cast<Constant *>(g.nodes[n].get()) || dynamic_cast<ARange *>(g.nodes[n].get())) return true;
            auto in = g.incoming(n);
            if (in.empty()) return false;
            return std::all_of(in.begin(), in.end(), [&](const Edge *e) { return constant_only(e->src); });
        };
        std::vector<NodeIndex> stack{from};
        std::set<NodeIndex> seen;
        const Edge *found = nullptr;
        while (!stack.empty()) {
            const NodeIndex n = stack.back();
            stack.pop_back();
            if (!seen.insert(n).second) continue;
            for (const Edge *e : g.incoming(n)) {
                if (constant_only(e->src)) continue;
                const ShapeTracker &s = e->shape;
                if (s.rank() == 2 && s.dims[0] == batch && s.dims[1] == vocab && s.is_fake(1) && !s.is_fake(0)) {
                    if (found && found->src != e->src) return nullptr;  // two candidates: not the gather pattern
                    found = e;
                } else {
                    stack.push_back(e->src);
                }
            }
        }
        return found;
    }

    // Removes nodes that have lost their last consumer (the one-hot subgraph of a gather), walking upwards.
    static void prune_dead(Graph &g, NodeIndex n) {
        if (!g.nodes.at(n) || !g.outgoing(n).empty() || g.to_retrieve.count(n)) return;
        if (dynamic_cast<Function *>(g.nodes[n].get())) return;  // graph inputs stay
        std::vector<NodeIndex> parents;
        for (const Edge *e : g.incoming(n)) parents.push_back(e->src);
        g.remove_node(n);
        for (NodeIndex p : parents) prune_dead(g, p);
    }

    // Copy nodes around a quantized node (prim.rs:687-767 does the same around host Function nodes): a host
    // producer of the matmul's activations gets a HipCopyToDevice behind it; every consumer that is not itself a
    // quantized node reads through one HipCopyFromDevice, and a retrieved result is retrieved from that copy.
    static void insert_copies(Graph &g, NodeIndex q, DType dtype) {
        auto on_device = [&](NodeIndex n) {
            Operator *op = g.nodes[n].get();
            return dynamic_cast<QuantizedMatmul *>(op) || dynamic_cast<QuantizedGather *>(op) ||
                   dynamic_cast<HipCopyToDevice *>(op);
        };
        if (dynamic_cast<QuantizedMatmul *>(g.nodes[q].get())) {
            const Edge act = *g.incoming(q).at(0);
            if (!on_device(act.src)) {
                const NodeIndex up = g.add(std::make_unique<HipCopyToDevice>(dtype));
                // the copy takes the producer's whole result; the view stays on the edge into the matmul
                g.edges.erase(std::remove_if(g.edges.begin(), g.edges.end(),
                                             [&](const Edge &e) { return e.dst == q && e.input_order == 0; }),
                              g.edges.end());
                g.connect(act.src, up, 0, ShapeTracker());
                g.connect(up, q, 0, act.shape);
            }
        }
        std::vector<Edge> host_uses;
        for (const Edge *e : g.outgoing(q))
            if (!on_device(e->dst) && !dynamic_cast<HipCopyFromDevice *>(g.nodes[e->dst].get())) host_uses.push_back(*e);
        if (host_uses.empty() && !g.to_retrieve.count(q)) return;
        const NodeIndex down = g.add(std::make_unique<HipCopyFromDevice>(dtype));
        for (const Edge &e : host_uses) {
            g.edges.erase(std::remove_if(g.edges.begin(), g.edges.end(),
                                         [&](const Edge &x) {
                                             return x.src == q && x.dst == e.dst && x.input_order == e.input_order;
                                         }),
                          g.edges.end());
            g.connect(down, e.dst, e.input_order, e.shape);
        }
        g.connect(q, down, 0, ShapeTracker());
        if (g.to_retrieve.erase(q)) g.to_retrieve.insert(down);
    }

    std::vector<NodeIndex> weights_;
    DType dtype_;
};

// What the HIP loader does per tensor of a GGUF file (examples/llama/src/loader.rs:99-165, which reads each tensor's
// bytes and copies Q8_0 ones to the device untouched): F32 tensors become host vectors, Q8_0 tensors planar device
// buffers; the Q8_0 nodes are returned for HipQuantizedCompiler.  `tensors`: node -> (is_q8_0, n, k, bytes).
struct GgufTensor {
    bool q8_0;
    int64_t n, k;
    const std::vector<uint8_t> *bytes;
};
inline std::vector<NodeIndex> q8_load_hip(Graph &g, const std::map<NodeIndex, GgufTensor> &tensors) {
    std::vector<NodeIndex> q_weights;
    for (auto &[node, t] : tensors) {
        auto *f = dynamic_cast<Function *>(g.nodes.at(node).get());
        if (!f) throw Panic("loader target is not a graph input");
        if (t.q8_0) {
            f->value = Tensor{HipData::q8_0_from_raw(*t.bytes, t.n, t.k)};
            q_weights.push_back(node);
        } else {
            if (t.bytes->size() != static_cast<size_t>(t.n * t.k) * 4) throw Panic("F32 tensor has the wrong size");
            std::vector<float> v(t.n * t.k);
            std::memcpy(v.data(), t.bytes->data(), t.bytes->size());
            f->value = host_tensor(std::move(v));
        }
    }
    return q_weights;
}

}  // namespace luminal_hip
