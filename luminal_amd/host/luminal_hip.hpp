// C++ host side of the luminal_hip backend: what the Rust crate `luminal_hip` does above the C ABI, restated in
// C++ because the reference's own toolchain (cargo) is not available where this library is built.
//
// Names, argument meaning and failure behaviour follow the reference:
//   HipData                 <- CudaData<T>                         crates/luminal_cuda/src/lib.rs:83-100
//   Operator::process       <- trait Operator                      src/op.rs:82-90
//   QuantizedMatmul         <- QuantizedMatmul<T>, T = f32 | f16   crates/luminal_cuda/src/quantized.rs:111-168
//   QuantizedGather         <- QuantizedGather<T>                  crates/luminal_cuda/src/quantized.rs:170-233
//   HipQuantizedCompiler    <- CudaQuantizedCompiler<T>            crates/luminal_cuda/src/quantized.rs:235-272
//   downstream              <- luminal::module::downstream         src/module.rs:84-113
// Where the reference panics (unwrap / assert! / panic!), these throw luminal_hip::Panic with the same message.
// The graph model is the minimum the compiler pass and a forward execution need: nodes holding an operator,
// data edges carrying (input_order, shape).  Header-only; links against libluminal_hip.so only.
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <functional>
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
    // Raw GGUF Q8_0 blocks of an (n, k) weight -> planar device buffer (what the HIP loader keeps per tensor).
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

// A tensor's payload: host f32 (what the CPU operators and the token ids use) or a device buffer.
using Data = std::variant<std::monostate, std::shared_ptr<std::vector<float>>, std::shared_ptr<HipData>>;

struct Tensor {
    Data data;
};

// The part of ShapeTracker the quantized operators read: dimensions and whether the view is contiguous.
struct ShapeTracker {
    std::vector<int64_t> dims;
    bool contiguous = true;
    int64_t n_elements() const {
        int64_t n = 1;
        for (auto d : dims) n *= d;
        return n;
    }
};

using Input = std::pair<const Tensor *, ShapeTracker>;

struct Operator {
    virtual ~Operator() = default;
    virtual std::vector<Tensor> process(const std::vector<Input> &inp) = 0;
    virtual std::string name() const = 0;
};

inline const HipData &device_operand(const Tensor &t, const char *what) {
    auto p = std::get_if<std::shared_ptr<HipData>>(&t.data);
    if (!p || !*p) throw Panic(std::string(what) + " is not a HIP buffer");
    return **p;
}

// The reference's operators are generic over the activation type T (f32 or f16); here it is a run-time tag.
enum class DType { F32, F16 };
inline size_t dtype_size(DType t) { return t == DType::F32 ? 4 : 2; }

// (batch.., m, K) T x Q8_0 (N, K) -> (batch.., m, N) T.  inp[0] = activations (a device buffer of T, or, for f32,
// host f32 which is uploaded for the call), inp[1] = weight with dims [.., K, N], necessarily a permuted
// (non-contiguous) view.
class QuantizedMatmul : public Operator {
  public:
    explicit QuantizedMatmul(DType dtype = DType::F32) : dtype(dtype) {}
    DType dtype;
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        const ShapeTracker &a = inp.at(0).second, &b = inp.at(1).second;
        if (b.contiguous) throw Panic("Weight matrix must be column-major");
        if (a.dims.empty() || b.dims.size() < 2) throw Panic("QuantizedMatmul: operands need at least 1 and 2 dims");
        const int64_t k = b.dims[b.dims.size() - 2], n = b.dims[b.dims.size() - 1];
        if (a.dims.back() != k) throw Panic("QuantizedMatmul: inner dimensions differ");
        const int64_t rows = std::max<int64_t>(a.n_elements() / k, 1);  // batch * m
        std::shared_ptr<HipData> staged;
        const void *x;
        if (auto host = std::get_if<std::shared_ptr<std::vector<float>>>(&inp[0].first->data)) {
            if (dtype != DType::F32) throw Panic("QuantizedMatmul<f16>: host activations are f32");
            staged = HipData::from_host(**host);
            x = staged->ptr();
        } else {
            x = device_operand(*inp[0].first, "activation").ptr();
        }
        auto out = std::make_shared<HipData>(static_cast<size_t>(rows * n) * dtype_size(dtype));
        const void *w = device_operand(*inp[1].first, "weight").ptr();
        if (dtype == DType::F32)
            check(lhip_q8_0_matmul_f32(w, static_cast<const float *>(x), static_cast<float *>(out->ptr()), rows, n, k,
                                       nullptr),
                  "lhip_q8_0_matmul_f32");
        else
            check(lhip_q8_0_matmul_f16(w, x, out->ptr(), rows, n, k, nullptr), "lhip_q8_0_matmul_f16");
        check(lhip_stream_sync(nullptr), "lhip_stream_sync");  // a staged activation is released on return
        return {Tensor{out}};
    }
    std::string name() const override { return "QuantizedMatmul"; }
};

// Row gather from a Q8_0 embedding table; indices arrive as host f32, as in every luminal backend.
class QuantizedGather : public Operator {
  public:
    explicit QuantizedGather(int64_t embed_dim, DType dtype = DType::F32) : embed_dim(embed_dim), dtype(dtype) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        auto idx = std::get_if<std::shared_ptr<std::vector<float>>>(&inp.at(0).first->data);
        if (!idx) throw Panic("gather indices are host f32");
        const int64_t vocab = inp.at(1).second.n_elements() / embed_dim;
        auto idx_dev = HipData::from_host(**idx);
        auto out = std::make_shared<HipData>((*idx)->size() * embed_dim * dtype_size(dtype));
        const void *table = device_operand(*inp[1].first, "table").ptr();
        const auto *ids = static_cast<const float *>(idx_dev->ptr());
        const auto count = static_cast<int64_t>((*idx)->size());
        if (dtype == DType::F32)
            check(lhip_q8_0_gather_f32(table, ids, static_cast<float *>(out->ptr()), count, vocab, embed_dim, nullptr),
                  "lhip_q8_0_gather_f32");
        else
            check(lhip_q8_0_gather_f16(table, ids, out->ptr(), count, vocab, embed_dim, nullptr), "lhip_q8_0_gather_f16");
        check(lhip_stream_sync(nullptr), "lhip_stream_sync");
        return {Tensor{out}};
    }
    std::string name() const override { return "QuantizedGather"; }
    int64_t embed_dim;
    DType dtype;
};

// ---- the operators a graph holds before the pass runs (markers; a CPU backend would execute them) -------------
struct Function : Operator {  // graph input: yields the tensor set on it (weights, activations, token ids)
    Tensor value;
    std::vector<Tensor> process(const std::vector<Input> &) override { return {value}; }
    std::string name() const override { return "Function"; }
};
struct MatMul2D : Operator {  // dense matmul node produced by the pattern pass (crates/luminal_cpu/src/matmul.rs:62)
    std::vector<Tensor> process(const std::vector<Input> &) override { throw Panic("dense MatMul2D is not executed here"); }
    std::string name() const override { return "MatMul2D"; }
};
struct Gather : Operator {  // crates/luminal_cpu/src/binary.rs:170-173
    explicit Gather(int64_t e) : embed_dim(e) {}
    int64_t embed_dim;
    std::vector<Tensor> process(const std::vector<Input> &) override { throw Panic("dense Gather is not executed here"); }
    std::string name() const override { return "Gather { embed_dim: " + std::to_string(embed_dim) + " }"; }
};
struct Unary : Operator {  // any single-input op, e.g. the contiguous copy a loader may leave behind a weight
    std::string label;
    explicit Unary(std::string l) : label(std::move(l)) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override { return {*inp.at(0).first}; }
    std::string name() const override { return label; }
};

using NodeIndex = int;

struct Edge {
    NodeIndex src, dst;
    int input_order;
    ShapeTracker shape;
};

struct Graph {
    std::vector<std::unique_ptr<Operator>> nodes;
    std::vector<Edge> edges;
    std::map<NodeIndex, Tensor> results;

    NodeIndex add(std::unique_ptr<Operator> op) {
        nodes.push_back(std::move(op));
        return static_cast<NodeIndex>(nodes.size()) - 1;
    }
    void connect(NodeIndex src, NodeIndex dst, int input_order, ShapeTracker shape) {
        edges.push_back({src, dst, input_order, std::move(shape)});
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
    // Forward execution in node order (nodes are added producers-first in these tests).
    void execute() {
        results.clear();
        for (NodeIndex n = 0; n < static_cast<NodeIndex>(nodes.size()); ++n) {
            std::vector<Input> inp;
            for (auto e : incoming(n)) inp.emplace_back(&results.at(e->src), e->shape);
            results[n] = nodes[n]->process(inp).at(0);
        }
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
        for (NodeIndex weight : downstream(weights_, graph)) {
            for (const Edge *e : graph.outgoing(weight)) {
                const std::string target = "NodeIndex(" + std::to_string(e->dst) + ")";
                if (e->input_order != 1) throw Panic("Quantized weight " + target + " is the wrong input!");
                auto &op = graph.nodes[e->dst];
                if (auto gather = dynamic_cast<Gather *>(op.get())) {
                    op = std::make_unique<QuantizedGather>(gather->embed_dim, dtype_);
                } else if (dynamic_cast<MatMul2D *>(op.get())) {
                    op = std::make_unique<QuantizedMatmul>(dtype_);
                } else {
                    throw Panic("Quantized weight " + target + " is an input to a node that isn't a matmul or gather (" +
                                op->name() + ")");
                }
            }
        }
    }

  private:
    std::vector<NodeIndex> weights_;
    DType dtype_;
};

}  // namespace luminal_hip
