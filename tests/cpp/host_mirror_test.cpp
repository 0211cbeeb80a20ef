// Tests of the C++ host mirror (luminal_amd/host/luminal_hip.hpp), written after the reference's own tests of the
// quantized path and of the matmul it replaces:
//   test_quantized_matvec / test_quantized_matmul   crates/luminal_metal/src/quantized.rs:888-986
//                                                   (same, commented out, crates/luminal_cuda/src/quantized.rs:307-451)
//   the literal matmul case                         crates/luminal_cpu/src/lib.rs:177-192
//   the compiler pass' two panics                   crates/luminal_cuda/src/quantized.rs:256-267
//   the "column-major" assert                       crates/luminal_cuda/src/quantized.rs:118-121
// The graphs are built the way luminal's high-level ops spell them (src/hl_ops/matmul.rs:4-33, src/hl_ops/other.rs:114-123):
// primitive Mul / SumReduce / LessThan / Add nodes over fake-expanded views, which the pass has to recognise by itself.
// Usage: host_mirror_test cpu   (primitives, graph rewrite and error paths, no device)
//        host_mirror_test gpu   (everything)
#include <cmath>
#include <cstdio>
#include <random>

#include <fstream>
#include <sstream>

#include "../../luminal_amd/host/luminal_hip.hpp"
#include "../../luminal_amd/host/luminal_hip_fusion.hpp"
#include "../../luminal_amd/host/luminal_hip_gguf.hpp"

using namespace luminal_hip;

static int checks = 0, failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        ++checks;                                                           \
        if (!(cond)) {                                                      \
            ++failures;                                                     \
            std::printf("FAIL %s:%d  %s\n", __FILE__, __LINE__, #cond);     \
        }                                                                   \
    } while (0)

template <typename F>
static std::string panic_message(F f) {
    try {
        f();
    } catch (const Panic &p) {
        return p.what();
    }
    return "";
}

// (n, k) quants + per-block scales -> raw GGUF Q8_0 blocks {f16 d; i8 qs[32]}.
static std::vector<uint8_t> q8_0_blocks(const std::vector<int8_t> &q, const std::vector<float> &d) {
    std::vector<uint8_t> raw(q.size() / 32 * 34);
    for (size_t b = 0; b < q.size() / 32; ++b) {
        const uint16_t c = f32_to_f16_code(d[b]);
        std::memcpy(&raw[b * 34], &c, 2);
        std::memcpy(&raw[b * 34 + 2], &q[b * 32], 32);
    }
    return raw;
}
static std::vector<uint8_t> f32_bytes(const std::vector<float> &v) {
    std::vector<uint8_t> b(v.size() * 4);
    std::memcpy(b.data(), v.data(), b.size());
    return b;
}

static double max_abs_diff(const std::vector<float> &got, const std::vector<float> &want) {
    double m = got.size() == want.size() ? 0 : 1e30;
    for (size_t i = 0; i < want.size() && i < got.size(); ++i) m = std::max(m, std::fabs(static_cast<double>(got[i]) - want[i]));
    return m;
}
static double rms(const std::vector<float> &v) {
    double s = 0;
    for (float x : v) s += static_cast<double>(x) * x;
    return std::sqrt(s / std::max<size_t>(v.size(), 1));
}

static Function *fn(Graph &g, NodeIndex n) { return dynamic_cast<Function *>(g.nodes[n].get()); }
static int count_nodes(const Graph &g, const std::string &name) {
    int c = 0;
    for (auto &n : g.nodes) c += n && n->name() == name;
    return c;
}

// ---- graph builders: what luminal's high-level ops put on the graph ------------------------------------------
// x (.., m, k) . w^T with w stored (n, k): x.matmul(w.permute((1, 0))) as src/hl_ops/matmul.rs:4-33 expands it.
static NodeIndex build_matmul(Graph &g, NodeIndex x, std::vector<int64_t> x_dims, NodeIndex w, int64_t n) {
    const size_t r = x_dims.size();
    const int64_t k = x_dims.back();
    ShapeTracker xs = ShapeTracker(x_dims).expand_dim(r - 1, n);  // [.., m, n(fake), k]
    ShapeTracker ws({n, k});
    for (size_t i = 0; i + 1 < r; ++i) ws = ws.expand_dim(0, x_dims[r - 2 - i]);  // [..(fake), m(fake), n, k]
    const NodeIndex mul = g.add(std::make_unique<Binary>(Binary::Mul));
    g.connect(x, mul, 0, xs);
    g.connect(w, mul, 1, ws);
    const NodeIndex red = g.add(std::make_unique<SumReduce>(r));
    std::vector<int64_t> prod = xs.dims;
    g.connect(mul, red, 0, ShapeTracker(prod));
    return red;
}
// table.gather(idx) as src/hl_ops/other.rs:114-123: one_hot = arange(V).expand(0, B).eq(idx.expand(1, V)) with
// eq = -(a < b + b < a) + 1 (src/hl_ops/binary.rs:232-261); (one_hot.expand(2, D) * table.expand(0, B)).sum(1).
static NodeIndex build_gather(Graph &g, NodeIndex idx, int64_t batch, NodeIndex table, int64_t vocab, int64_t dim) {
    const NodeIndex ar = g.add(std::make_unique<ARange>(vocab));
    const ShapeTracker ar_s = ShapeTracker({vocab}).expand_dim(0, batch), idx_s = ShapeTracker({batch}).expand_dim(1, vocab);
    const ShapeTracker bv({batch, vocab}), scalar = ShapeTracker().expand_dim(0, batch).expand_dim(1, vocab);
    auto binary = [&](Binary::Kind kind, NodeIndex a, ShapeTracker as, NodeIndex b, ShapeTracker bs) {
        const NodeIndex n = g.add(std::make_unique<Binary>(kind));
        g.connect(a, n, 0, as);
        g.connect(b, n, 1, bs);
        return n;
    };
    const NodeIndex lt = binary(Binary::LessThan, ar, ar_s, idx, idx_s), gt = binary(Binary::LessThan, idx, idx_s, ar, ar_s);
    const NodeIndex ne = binary(Binary::Add, lt, bv, gt, bv);
    const NodeIndex neg = binary(Binary::Mul, ne, bv, g.add(std::make_unique<Constant>(-1.f)), scalar);
    const NodeIndex eq = binary(Binary::Add, neg, bv, g.add(std::make_unique<Constant>(1.f)), scalar);
    const NodeIndex mul = binary(Binary::Mul, eq, bv.expand_dim(2, dim), table, ShapeTracker({vocab, dim}).expand_dim(0, batch));
    const NodeIndex red = g.add(std::make_unique<SumReduce>(1));
    g.connect(mul, red, 0, ShapeTracker({batch, vocab, dim}));
    return red;
}
static NodeIndex build_relu(Graph &g, NodeIndex src, std::vector<int64_t> dims) {
    const NodeIndex n = g.add(std::make_unique<Unary>("Relu", [](float v) { return v > 0 ? v : 0.f; }));
    g.connect(src, n, 0, ShapeTracker(std::move(dims)));
    return n;
}

static NodeIndex binary(Graph &g, Binary::Kind kind, NodeIndex a, ShapeTracker as, NodeIndex b, ShapeTracker bs) {
    const NodeIndex n = g.add(std::make_unique<Binary>(kind));
    g.connect(a, n, 0, std::move(as));
    g.connect(b, n, 1, std::move(bs));
    return n;
}
static NodeIndex unary(Graph &g, const char *label, std::function<float(float)> f, NodeIndex src, ShapeTracker s) {
    const NodeIndex n = g.add(std::make_unique<Unary>(label, std::move(f)));
    g.connect(src, n, 0, std::move(s));
    return n;
}
static ShapeTracker expanded_scalar(const std::vector<int64_t> &dims) {
    ShapeTracker s;
    for (size_t i = 0; i < dims.size(); ++i) s = s.expand_dim(i, dims[i]);
    return s;
}
// LayerNorm(weight, no bias, no mean_norm).forward(x) as crates/luminal_nn/src/norm.rs:56-70 puts it on the graph:
// std_norm (src/hl_ops/unary.rs:93-104) with mean = sum / D (src/hl_ops/reduction.rs:38-45, a division by an
// Expression: times Recip(expand(Constant(D)))), then times expand(weight).  x has dims [.., D].
static NodeIndex build_rms_norm(Graph &g, NodeIndex x, std::vector<int64_t> dims, NodeIndex w, float eps) {
    const size_t r = dims.size();
    const int64_t d = dims.back();
    const ShapeTracker full(dims);
    std::vector<int64_t> lead(dims.begin(), dims.end() - 1);
    const ShapeTracker red(lead), c = expanded_scalar(lead);
    const NodeIndex sq = binary(g, Binary::Mul, x, full, x, full);
    const NodeIndex sum = g.add(std::make_unique<SumReduce>(r - 1));
    g.connect(sq, sum, 0, full);
    const NodeIndex inv_d = unary(g, "Recip", [](float v) { return 1.f / v; }, g.add(std::make_unique<Constant>(static_cast<float>(d))), c);
    const NodeIndex mean = binary(g, Binary::Mul, sum, red, inv_d, red);
    const NodeIndex plus = binary(g, Binary::Add, mean, red, g.add(std::make_unique<Constant>(eps)), c);
    const NodeIndex root = unary(g, "Sqrt", [](float v) { return std::sqrt(v); }, plus, red);
    const NodeIndex factor = unary(g, "Recip", [](float v) { return 1.f / v; }, root, red);
    const NodeIndex scaled = binary(g, Binary::Mul, factor, red.expand_dim(r - 1, d), x, full);
    ShapeTracker ws({d});
    for (size_t i = 0; i + 1 < r; ++i) ws = ws.expand_dim(0, dims[r - 2 - i]);
    return binary(g, Binary::Mul, scaled, full, w, ws);
}
// up * gate.swish() (examples/llama/src/model.rs:27-29) in primitives: swish = gate * sigmoid(gate),
// sigmoid(t) = 1. / (1. + (-t).exp()), exp(t) = (t * (1/ln 2)).exp2() (src/hl_ops/unary.rs:4-10,33-36,168-177), with
// `f32 op tensor` spelled as `tensor op constant` (src/hl_ops/binary.rs:35-41,90-96,113-120).
static NodeIndex build_swiglu(Graph &g, NodeIndex gate, NodeIndex up, std::vector<int64_t> dims) {
    const ShapeTracker full(dims), c = expanded_scalar(dims);
    const NodeIndex neg = binary(g, Binary::Mul, gate, full, g.add(std::make_unique<Constant>(-1.f)), c);
    const NodeIndex scaled = binary(g, Binary::Mul, neg, full, g.add(std::make_unique<Constant>(1.f / std::log(2.f))), c);
    const NodeIndex e = unary(g, "Exp2", [](float v) { return std::exp2(v); }, scaled, full);
    const NodeIndex plus = binary(g, Binary::Add, e, full, g.add(std::make_unique<Constant>(1.f)), c);
    const NodeIndex rec = unary(g, "Recip", [](float v) { return 1.f / v; }, plus, full);
    const NodeIndex sig = binary(g, Binary::Mul, rec, full, g.add(std::make_unique<Constant>(1.f)), c);
    const NodeIndex swish = binary(g, Binary::Mul, gate, full, sig, full);
    return binary(g, Binary::Mul, up, full, swish, full);
}

// One decoder layer at one position the way examples/llama/src/model.rs:150-175 strings it together, with the
// attention itself (model.rs:112-139, no weights in it) stood in for by a host operator on q; k and v are
// retrieved like the cache rows they become.
struct LayerNodes {
    NodeIndex x, attn_norm, ffn_norm, wq, wk, wv, wo, wg, wu, wd, k, v, out;
};
static LayerNodes build_decoder_layer(Graph &g, int64_t dim, int64_t kv_dim, int64_t ffn, float eps) {
    LayerNodes n{};
    for (NodeIndex *f : {&n.x, &n.attn_norm, &n.ffn_norm, &n.wq, &n.wk, &n.wv, &n.wo, &n.wg, &n.wu, &n.wd}) *f = g.add(std::make_unique<Function>());
    const std::vector<int64_t> row{1, 1, dim};
    const NodeIndex normed = build_rms_norm(g, n.x, row, n.attn_norm, eps);
    const NodeIndex q = build_matmul(g, normed, row, n.wq, dim);
    n.k = build_matmul(g, normed, row, n.wk, kv_dim);
    n.v = build_matmul(g, normed, row, n.wv, kv_dim);
    const NodeIndex attn = unary(g, "AttentionStandIn", [](float v) { return std::tanh(v); }, q, ShapeTracker(row));
    const NodeIndex o = build_matmul(g, attn, row, n.wo, dim);
    const NodeIndex mid = binary(g, Binary::Add, n.x, ShapeTracker(row), o, ShapeTracker(row));  // x += y
    const NodeIndex normed2 = build_rms_norm(g, mid, row, n.ffn_norm, eps);
    const NodeIndex gate = build_matmul(g, normed2, row, n.wg, ffn);
    const NodeIndex up = build_matmul(g, normed2, row, n.wu, ffn);
    const NodeIndex act = build_swiglu(g, gate, up, {1, 1, ffn});
    const NodeIndex down = build_matmul(g, act, {1, 1, ffn}, n.wd, dim);
    n.out = binary(g, Binary::Add, mid, ShapeTracker(row), down, ShapeTracker(row));
    g.to_retrieve.insert(n.k);
    g.to_retrieve.insert(n.v);
    g.to_retrieve.insert(n.out);
    return n;
}

// ---------------------------------------------------------------- primitives and graph rewrite, no device
static void test_primitives_on_the_host() {
    // crates/luminal_cpu/src/lib.rs:177-192: [[1,2,3],[1,2,3]] . [[1,2,3,1],[2,3,1,2],[3,1,2,3]] = [[14,11,11,14]] x 2;
    // here the right operand is stored transposed, (n, k) = (4, 3), like a Linear's weight.
    Graph g;
    auto x = g.add(std::make_unique<Function>()), w = g.add(std::make_unique<Function>());
    auto y = build_matmul(g, x, {2, 3}, w, 4);
    g.to_retrieve.insert(y);
    fn(g, x)->value = host_tensor({1, 2, 3, 1, 2, 3});
    fn(g, w)->value = host_tensor({1, 2, 3, 2, 3, 1, 3, 1, 2, 1, 2, 3});
    g.execute();
    EXPECT((host_operand(g.results.at(y), "y") == std::vector<float>{14, 11, 11, 14, 14, 11, 11, 14}));
    // gather on the host: rows 2, 0, 2 of a 3 x 2 table
    Graph h;
    auto idx = h.add(std::make_unique<Function>()), table = h.add(std::make_unique<Function>());
    auto rows = build_gather(h, idx, 3, table, 3, 2);
    fn(h, idx)->value = host_tensor({2, 0, 2});
    fn(h, table)->value = host_tensor({10, 11, 20, 21, 30, 31});
    h.execute();
    EXPECT((host_operand(h.results.at(rows), "rows") == std::vector<float>{30, 31, 10, 11, 30, 31}));
    // f16 codes: round to nearest even, subnormals, overflow
    EXPECT(f32_to_f16_code(1.0f) == 0x3c00 && f32_to_f16_code(-2.0f) == 0xc000 && f32_to_f16_code(65504.f) == 0x7bff);
    EXPECT(f32_to_f16_code(1.0f + 1.0f / 2048) == 0x3c00 && f32_to_f16_code(1.0f + 3.0f / 2048) == 0x3c02);  // ties to even
    EXPECT(f32_to_f16_code(65520.f) == 0x7c00 && f32_to_f16_code(std::ldexp(1.0f, -24)) == 0x0001 &&
           f32_to_f16_code(std::ldexp(1.0f, -25)) == 0x0000 && f32_to_f16_code(std::ldexp(3.0f, -25)) == 0x0002);
    for (uint32_t c = 0; c < 0x7c00; c += 7) EXPECT(f32_to_f16_code(f16_code_to_f32(static_cast<uint16_t>(c))) == c);
}

static void test_compiler_pass_cpu() {
    // tokens -> gather(embed) -> matmul(w) -> relu (host) -> matmul(w2 behind a contiguous copy) -> retrieved
    Graph g;
    auto tok = g.add(std::make_unique<Function>());
    auto embed = g.add(std::make_unique<Function>());
    auto w = g.add(std::make_unique<Function>());
    auto w2 = g.add(std::make_unique<Function>());
    auto w2_copy = g.add(std::make_unique<Unary>("Contiguous"));
    g.connect(w2, w2_copy, 0, ShapeTracker({32, 32}));
    auto rows = build_gather(g, tok, 3, embed, 100, 64);
    auto h1 = build_matmul(g, rows, {3, 64}, w, 32);
    auto act = build_relu(g, h1, {3, 32});
    auto h2 = build_matmul(g, act, {3, 32}, w2_copy, 32);
    g.to_retrieve.insert(h2);
    const size_t before = g.nodes.size();
    EXPECT((downstream({embed, w, w2}, g) == std::vector<NodeIndex>{embed, w, w2_copy}));
    HipQuantizedCompiler({embed, w, w2}).compile(g, /*init_device=*/false);
    EXPECT(count_nodes(g, "QuantizedGather") == 1 && count_nodes(g, "QuantizedMatmul") == 2);
    EXPECT(count_nodes(g, "Mul") == 0 && count_nodes(g, "SumReduce(1)") == 0 && count_nodes(g, "SumReduce(2)") == 0);
    EXPECT(count_nodes(g, "LessThan") == 0 && count_nodes(g, "ARange") == 0 && count_nodes(g, "Add") == 0);  // the one-hot went
    EXPECT(count_nodes(g, "Contiguous") == 1 && count_nodes(g, "Relu") == 1);  // nodes around the pattern are left alone
    // gather -> matmul stays on the device; matmul -> relu -> matmul crosses to the host and back; the retrieved
    // result is read from a copy
    EXPECT(count_nodes(g, "HipCopyToDevice") == 1 && count_nodes(g, "HipCopyFromDevice") == 2);
    EXPECT(g.to_retrieve.size() == 1 && g.nodes[*g.to_retrieve.begin()]->name() == "HipCopyFromDevice");
    NodeIndex qg = -1, q1 = -1;
    for (NodeIndex n = static_cast<NodeIndex>(before); n < static_cast<NodeIndex>(g.nodes.size()); ++n) {
        if (g.nodes[n] && g.nodes[n]->name() == "QuantizedGather") qg = n;
        if (g.nodes[n] && g.nodes[n]->name() == "QuantizedMatmul" && q1 < 0) q1 = n;
    }
    EXPECT(dynamic_cast<QuantizedGather *>(g.nodes[qg].get())->embed_dim == 64);
    auto gi = g.incoming(qg);
    EXPECT(gi.size() == 2 && gi[0]->src == tok && gi[0]->shape.dims == std::vector<int64_t>{3} && gi[1]->src == embed &&
           (gi[1]->shape.dims == std::vector<int64_t>{100, 64}) && gi[1]->shape.is_contiguous());
    auto mi = g.incoming(q1);
    EXPECT(mi.size() == 2 && mi[0]->src == qg && (mi[0]->shape.dims == std::vector<int64_t>{3, 64}) && mi[1]->src == w &&
           (mi[1]->shape.dims == std::vector<int64_t>{64, 32}) && !mi[1]->shape.is_contiguous());

    // a batched matmul, (1, s, k) x (n, k): rank-4 product, SumReduce(3)
    Graph b;
    auto bx = b.add(std::make_unique<Function>()), bw = b.add(std::make_unique<Function>());
    auto by = build_matmul(b, bx, {1, 5, 64}, bw, 96);
    b.to_retrieve.insert(by);
    HipQuantizedCompiler({bw}).compile(b, false);
    EXPECT(count_nodes(b, "QuantizedMatmul") == 1 && count_nodes(b, "Mul") == 0 && count_nodes(b, "SumReduce(3)") == 0);
    for (NodeIndex n = 0; n < static_cast<NodeIndex>(b.nodes.size()); ++n)
        if (b.nodes[n] && b.nodes[n]->name() == "QuantizedMatmul") {
            auto in = b.incoming(n);
            EXPECT((in[0]->shape.dims == std::vector<int64_t>{1, 5, 64}) && (in[1]->shape.dims == std::vector<int64_t>{64, 96}) &&
                   !in[1]->shape.is_contiguous());
        }

    // weight as input 0: "Quantized weight .. is the wrong input!"
    Graph bad;
    auto badw = bad.add(std::make_unique<Function>()), badx = bad.add(std::make_unique<Function>());
    auto bmul = bad.add(std::make_unique<Binary>(Binary::Mul));
    bad.connect(badw, bmul, 0, ShapeTracker({8, 32}).expand_dim(0, 1));
    bad.connect(badx, bmul, 1, ShapeTracker({1, 32}).expand_dim(1, 8));
    EXPECT(panic_message([&] { HipQuantizedCompiler({badw}).compile(bad, false); }).find("is the wrong input!") != std::string::npos);

    // weight into something that is neither matmul nor gather: another operator, or a Mul of another shape
    Graph odd;
    auto ow = odd.add(std::make_unique<Function>()), ox = odd.add(std::make_unique<Function>());
    auto oadd = odd.add(std::make_unique<Binary>(Binary::Add));
    odd.connect(ox, oadd, 0, ShapeTracker({32}));
    odd.connect(ow, oadd, 1, ShapeTracker({32}));
    EXPECT(panic_message([&] { HipQuantizedCompiler({ow}).compile(odd, false); }).find("isn't a matmul or gather (Add)") !=
           std::string::npos);
    Graph odd2;
    auto pw = odd2.add(std::make_unique<Function>()), px = odd2.add(std::make_unique<Function>());
    auto pmul = odd2.add(std::make_unique<Binary>(Binary::Mul));  // element-wise product, no reduction behind it
    odd2.connect(px, pmul, 0, ShapeTracker({4, 32}));
    odd2.connect(pw, pmul, 1, ShapeTracker({4, 32}));
    EXPECT(panic_message([&] { HipQuantizedCompiler({pw}).compile(odd2, false); }).find("isn't a matmul or gather (Mul)") !=
           std::string::npos);

    // operator-level asserts that need no device: contiguous weight view, mismatched K, wrong byte count, host operand
    QuantizedMatmul op;
    Tensor dummy;
    EXPECT(panic_message([&] { op.process({{&dummy, ShapeTracker({1, 32})}, {&dummy, ShapeTracker({32, 8})}}); }) ==
           "Weight matrix must be column-major");
    EXPECT(panic_message([&] {
               op.process({{&dummy, ShapeTracker({1, 64})}, {&dummy, ShapeTracker({8, 32}).permute({1, 0})}});
           }).find("inner dimensions") != std::string::npos);
    Tensor host = host_tensor({1.f});
    EXPECT(panic_message([&] {
               op.process({{&host, ShapeTracker({1, 32})}, {&dummy, ShapeTracker({8, 32}).permute({1, 0})}});
           }).find("activation is not a HIP buffer") != std::string::npos);
    EXPECT(panic_message([&] { HipData::q8_0_from_raw(std::vector<uint8_t>(33), 1, 32); }).find("n + n/16") != std::string::npos);
}

static std::vector<FusedMatvec *> fused_nodes(Graph &g) {
    std::vector<FusedMatvec *> v;
    for (auto &n : g.nodes)
        if (auto *f = dynamic_cast<FusedMatvec *>(n.get())) v.push_back(f);
    return v;
}

static void test_fusion_pass_cpu() {
    // a decoder layer at one position: seven projections become four fused launches
    Graph g;
    const LayerNodes n = build_decoder_layer(g, 1024, 256, 2048, 1e-5f);
    HipQuantizedCompiler({n.wq, n.wk, n.wv, n.wo, n.wg, n.wu, n.wd}).compile(g, false);
    EXPECT(count_nodes(g, "QuantizedMatmul") == 7);
    HipFusedMatvecCompiler().compile(g);
    EXPECT(count_nodes(g, "QuantizedMatmul") == 0 && count_nodes(g, "FusedMatvec") == 4 && count_nodes(g, "Q8InterleaveRows") == 1);
    // both norms and the SwiGLU are gone from the host side; the two residual adds went into epilogues
    EXPECT(count_nodes(g, "Mul") == 0 && count_nodes(g, "Add") == 0 && count_nodes(g, "Sqrt") == 0 && count_nodes(g, "Recip") == 0 &&
           count_nodes(g, "Exp2") == 0 && count_nodes(g, "SumReduce(2)") == 0);
    EXPECT(count_nodes(g, "AttentionStandIn") == 1);
    int qkv = 0, o = 0, gate_up = 0, down = 0;
    for (FusedMatvec *f : fused_nodes(g)) {
        if (f->n == std::vector<int64_t>{1024, 256, 256} && f->k == 1024 && f->norm && f->epilogue == FusedMatvec::None && f->eps == 1e-5f) ++qkv;
        if (f->n == std::vector<int64_t>{1024} && f->k == 1024 && !f->norm && f->epilogue == FusedMatvec::Residual) ++o;
        if (f->n == std::vector<int64_t>{4096} && f->k == 1024 && f->norm && f->epilogue == FusedMatvec::SwiGLU) ++gate_up;
        if (f->n == std::vector<int64_t>{1024} && f->k == 2048 && !f->norm && f->epilogue == FusedMatvec::Residual) ++down;
    }
    EXPECT(qkv == 1 && o == 1 && gate_up == 1 && down == 1);
    // host <-> device crossings left: x up (once, shared), the two norm weights up (kept), the stand-in's input
    // down and its result up, k, v and the layer output down
    EXPECT(count_nodes(g, "HipCopyToDevice") == 4 && count_nodes(g, "HipCopyFromDevice") == 4);
    EXPECT(g.no_delete.size() == 3);  // two norm weights on the device, the interleaved gate|up weight
    EXPECT(g.to_retrieve.size() == 3);
    for (NodeIndex r : g.to_retrieve) EXPECT(g.nodes[r] && g.nodes[r]->name() == "HipCopyFromDevice");
    // o -> (residual) -> gate|up -> down never leave the device: the gate|up launch reads the o launch's output, the
    // down launch reads gate|up's output and o's output (its residual)
    for (NodeIndex i = 0; i < static_cast<NodeIndex>(g.nodes.size()); ++i) {
        auto *f = dynamic_cast<FusedMatvec *>(g.nodes[i].get());
        if (!f || f->epilogue == FusedMatvec::None) continue;
        auto in = g.incoming(i);
        if (f->epilogue == FusedMatvec::SwiGLU) EXPECT(g.nodes[in.at(0)->src]->name() == "FusedMatvec" && g.nodes[in.at(1)->src]->name() == "Q8InterleaveRows");
        if (f->k == 2048) EXPECT(g.nodes[in.at(0)->src]->name() == "FusedMatvec" && g.nodes[in.at(2)->src]->name() == "FusedMatvec");
    }

    // patterns that must NOT fuse: a norm whose result something else reads too; a projection of several rows; K not
    // a multiple of 1024; a gate whose swish is read elsewhere too
    {
        Graph h;
        auto x = h.add(std::make_unique<Function>()), nw = h.add(std::make_unique<Function>()), w = h.add(std::make_unique<Function>());
        const NodeIndex normed = build_rms_norm(h, x, {1, 1, 1024}, nw, 1e-5f);
        const NodeIndex y = build_matmul(h, normed, {1, 1, 1024}, w, 64);
        const NodeIndex side = build_relu(h, normed, {1, 1, 1024});
        h.to_retrieve.insert(y);
        h.to_retrieve.insert(side);
        HipQuantizedCompiler({w}).compile(h, false);
        HipFusedMatvecCompiler().compile(h);
        EXPECT(count_nodes(h, "FusedMatvec") == 0 && count_nodes(h, "QuantizedMatmul") == 1 && count_nodes(h, "Sqrt") == 1);
    }
    {
        Graph h;
        auto x = h.add(std::make_unique<Function>()), wa = h.add(std::make_unique<Function>()), wb = h.add(std::make_unique<Function>());
        h.to_retrieve.insert(build_matmul(h, x, {1, 4, 1024}, wa, 64));  // four rows
        h.to_retrieve.insert(build_matmul(h, x, {1, 4, 1024}, wb, 64));
        auto x2 = h.add(std::make_unique<Function>()), wc = h.add(std::make_unique<Function>()), wd = h.add(std::make_unique<Function>());
        h.to_retrieve.insert(build_matmul(h, x2, {1, 1, 512}, wc, 64));  // K = 512
        h.to_retrieve.insert(build_matmul(h, x2, {1, 1, 512}, wd, 64));
        HipQuantizedCompiler({wa, wb, wc, wd}).compile(h, false);
        HipFusedMatvecCompiler().compile(h);
        EXPECT(count_nodes(h, "FusedMatvec") == 0 && count_nodes(h, "QuantizedMatmul") == 4);
    }
    {
        // siblings without norm or epilogue still share one launch and one upload of x; five siblings make 4 + 1
        Graph h;
        auto x = h.add(std::make_unique<Function>());
        std::vector<NodeIndex> ws;
        for (int i = 0; i < 5; ++i) {
            ws.push_back(h.add(std::make_unique<Function>()));
            h.to_retrieve.insert(build_matmul(h, x, {1, 1, 2048}, ws.back(), 32 * (i + 1)));
        }
        HipQuantizedCompiler(ws).compile(h, false);
        HipFusedMatvecCompiler().compile(h);
        EXPECT(count_nodes(h, "FusedMatvec") == 1 && count_nodes(h, "QuantizedMatmul") == 1);
        for (FusedMatvec *f : fused_nodes(h)) EXPECT((f->n == std::vector<int64_t>{32, 64, 96, 128}) && !f->norm && f->epilogue == FusedMatvec::None);
        EXPECT(h.to_retrieve.size() == 5);
    }
    {
        // the swish of the gate is read by a second consumer: gate and up still share a launch, the SwiGLU stays on the host
        Graph h;
        auto x = h.add(std::make_unique<Function>()), wg = h.add(std::make_unique<Function>()), wu = h.add(std::make_unique<Function>());
        const NodeIndex gate = build_matmul(h, x, {1, 1, 1024}, wg, 64), up = build_matmul(h, x, {1, 1, 1024}, wu, 64);
        const NodeIndex act = build_swiglu(h, gate, up, {1, 1, 64});
        h.to_retrieve.insert(act);
        const NodeIndex swish = h.incoming(act).at(1)->src;
        h.to_retrieve.insert(build_relu(h, swish, {1, 1, 64}));
        HipQuantizedCompiler({wg, wu}).compile(h, false);
        HipFusedMatvecCompiler().compile(h);
        EXPECT(count_nodes(h, "FusedMatvec") == 1 && count_nodes(h, "Exp2") == 1 && count_nodes(h, "Q8InterleaveRows") == 0);
        for (FusedMatvec *f : fused_nodes(h)) EXPECT(f->epilogue == FusedMatvec::None && f->n.size() == 2);
    }
    // operator-level checks without a device
    FusedMatvec op({64}, 1024, false, 0.f, FusedMatvec::None);
    Tensor dummy;
    EXPECT(panic_message([&] { op.process({{&dummy, ShapeTracker({1024})}}); }).find("wrong number of inputs") != std::string::npos);
    EXPECT(panic_message([&] { op.process({{&dummy, ShapeTracker({2, 1024})}, {&dummy, ShapeTracker({64, 1024}).permute({1, 0})}}); })
               .find("one contiguous row") != std::string::npos);
}

// tests/golden/gguf_v3_literal.hex: 644 bytes assembled by hand from examples/llama/src/gguf.rs:190-263 (hex pairs,
// '#' starts a comment): a v3 header, one key of every value type, alignment 64, one F32 and one Q8_0 tensor.
static std::string literal_gguf_bytes() {
    std::string path = __FILE__;
    path = path.substr(0, path.rfind('/')) + "/../golden/gguf_v3_literal.hex";
    std::ifstream f(path);
    std::string line, out;
    while (std::getline(f, line)) {
        line = line.substr(0, line.find('#'));
        int hi = -1;
        for (char ch : line) {
            const int v = ch >= '0' && ch <= '9' ? ch - '0' : ch >= 'a' && ch <= 'f' ? ch - 'a' + 10 : ch >= 'A' && ch <= 'F' ? ch - 'A' + 10 : -1;
            if (v < 0) continue;
            if (hi < 0) hi = v;
            else {
                out.push_back(static_cast<char>(hi * 16 + v));
                hi = -1;
            }
        }
    }
    return out;
}

static void test_gguf_reader_cpu() {
    const std::string bytes = literal_gguf_bytes();
    EXPECT(bytes.size() == 644);
    std::istringstream in(bytes);
    const GgufHeader h = GgufReader(in).read_header();
    EXPECT(h.version == 3 && h.alignment == 64 && h.data_offset == 512 && h.tensors.size() == 2);  // 477 header bytes rounded up to 64
    const GgufTensorInfo &a = h.tensors.at("a.weight"), &q = h.tensors.at("blk.0.attn_q.weight");
    EXPECT(a.n_elements == 3 && a.offset == 0 && a.dtype == kGgmlF32);
    EXPECT(q.n_elements == 64 && q.offset == 64 && q.dtype == kGgmlQ8_0);
    // only integer types of at most 32 bits set the alignment (gguf.rs:246-255): the same key as a u64 is ignored
    const size_t at = bytes.find("general.alignment") + 17;
    {
        std::string head = bytes.substr(0, at);
        const uint32_t type_u64 = 10;
        const uint64_t v = 64;
        head.append(reinterpret_cast<const char *>(&type_u64), 4).append(reinterpret_cast<const char *>(&v), 8);
        head += bytes.substr(at + 8, 477 - (at + 8));
        std::istringstream in2(head);
        const GgufHeader h2 = GgufReader(in2).read_header();
        EXPECT(h2.alignment == 32 && h2.data_offset == (head.size() + 31) / 32 * 32 && h2.tensors.size() == 2);
    }
    // the reference's panics
    {
        std::string bad = bytes;
        bad[0] = 'X';
        std::istringstream s1(bad);
        EXPECT(panic_message([&] { GgufReader(s1).read_header(); }).find("unknown magic") != std::string::npos);
        bad = bytes;
        bad[4] = 4;  // version
        std::istringstream s2(bad);
        EXPECT(panic_message([&] { GgufReader(s2).read_header(); }).find("unsupported version 4") != std::string::npos);
        bad = bytes.substr(0, 100);
        std::istringstream s3(bad);
        EXPECT(panic_message([&] { GgufReader(s3).read_header(); }).find("unexpected end of file") != std::string::npos);
    }
}

static void test_gguf_file_to_graph() {
    // the literal file through the loader and the pass: the F32 tensor lands on the host, the Q8_0 tensor (2 x 32:
    // row 0 = 0.5 * [0..31], row 1 = -2 * [-16..15]) on the device in planar form and multiplies a row of ones
    const std::string bytes = literal_gguf_bytes();
    const std::string path = "/tmp/luminal_hip_literal.gguf";
    {
        std::ofstream out(path, std::ios::binary);
        out.write(bytes.data(), static_cast<std::streamsize>(bytes.size()));
    }
    Graph g;
    const NodeIndex a = g.add(std::make_unique<Function>()), w = g.add(std::make_unique<Function>()), x = g.add(std::make_unique<Function>());
    const NodeIndex y = build_matmul(g, x, {1, 32}, w, 2);
    g.to_retrieve.insert(y);
    fn(g, x)->value = host_tensor(std::vector<float>(32, 1.f));
    const auto q_weights = q8_load_hip_file(path, g, {{"a/weight", a}, {"blk/0/attn_q/weight", w}});
    EXPECT((q_weights == std::vector<NodeIndex>{w}));
    EXPECT((host_operand(fn(g, a)->value, "a") == std::vector<float>{1.f, -2.f, 0.5f}));
    HipQuantizedCompiler(q_weights).compile(g);
    g.execute();
    const std::vector<float> got = host_operand(g.results.at(*g.to_retrieve.begin()), "y");
    EXPECT((got == std::vector<float>{248.f, 32.f}));
    EXPECT(panic_message([&] { q8_load_hip_file(path, g, {{"missing", a}}); }).find("is not in the file") != std::string::npos);
    EXPECT(panic_message([&] { q8_load_hip_file("/tmp/no_such_file.gguf", g, {{"a/weight", a}}); }).find("cannot open") != std::string::npos);
    std::remove(path.c_str());
}

// ---------------------------------------------------------------- device
struct Q8 {
    std::vector<int8_t> q;
    std::vector<float> d, dense;  // dense = the weights as luminal_cpu holds them after its load-time dequantisation
    std::vector<uint8_t> raw;
};
static Q8 random_q8(std::mt19937 &rng, int rows, int cols, float floor_scale) {
    Q8 w;
    std::normal_distribution<float> gauss(0.f, 0.02f);
    w.q.resize(static_cast<size_t>(rows) * cols);
    w.d.resize(w.q.size() / 32);
    for (auto &v : w.q) v = static_cast<int8_t>(static_cast<int>(rng() % 255) - 127);
    for (auto &v : w.d) v = f16_code_to_f32(f32_to_f16_code(std::fabs(gauss(rng)) / 127.f + floor_scale));
    w.raw = q8_0_blocks(w.q, w.d);
    w.dense.resize(w.q.size());
    for (size_t i = 0; i < w.q.size(); ++i) w.dense[i] = static_cast<float>(w.q[i]) * w.d[i / 32];
    return w;
}

static void test_quantized_matvec_like_the_reference() {
    // W 512 x 1024 of small non-negative ints with d = 1, x random: the reference compares the quantized graph with
    // the f32 graph at 1e-3 (crates/luminal_metal/src/quantized.rs:888-935).  Both graphs are built here: the f32 one
    // runs on the host primitives, the other goes through the loader and the pass.
    std::mt19937 rng(1);
    const int n = 512, k = 1024;
    Q8 w;
    w.q.resize(static_cast<size_t>(n) * k);
    for (auto &v : w.q) v = static_cast<int8_t>(rng() % 5);
    w.d.assign(w.q.size() / 32, 1.0f);
    w.raw = q8_0_blocks(w.q, w.d);
    std::vector<float> dense(w.q.begin(), w.q.end()), x(k);
    std::uniform_real_distribution<float> u(-0.5f, 0.5f);
    for (auto &v : x) v = u(rng);
    auto build = [&](Graph &g, NodeIndex &xi, NodeIndex &wi) {
        xi = g.add(std::make_unique<Function>());
        wi = g.add(std::make_unique<Function>());
        const NodeIndex y = build_matmul(g, xi, {1, k}, wi, n);
        g.to_retrieve.insert(y);
        fn(g, xi)->value = host_tensor(x);
    };
    Graph f32g, q8g;
    NodeIndex xi, wi;
    build(f32g, xi, wi);
    fn(f32g, wi)->value = host_tensor(dense);
    f32g.execute();
    const std::vector<float> want = host_operand(f32g.results.at(*f32g.to_retrieve.begin()), "y");
    build(q8g, xi, wi);
    auto q_weights = q8_load_hip(q8g, {{wi, GgufTensor{true, n, k, &w.raw}}});
    HipQuantizedCompiler(q_weights).compile(q8g);
    q8g.execute();
    EXPECT(max_abs_diff(host_operand(q8g.results.at(*q8g.to_retrieve.begin()), "y"), want) < 1e-3);
}

static void test_graph_end_to_end(DType dtype) {
    // tokens -> gather(Q8_0 table 100 x 64) -> matmul(Q8_0 96 x 64) -> relu on the HOST -> matmul(Q8_0 40 x 96), 16 rows
    // like the reference's matmul test, real scales and negative quants; and a second consumer of the first matmul
    // that stays on the host.  The same graph with dequantised f32 weights runs on the host primitives as the check.
    std::mt19937 rng(2);
    const int vocab = 100, dim = 64, n1 = 96, n2 = 40, m = 16;
    const Q8 table = random_q8(rng, vocab, dim, 1e-3f), w1 = random_q8(rng, n1, dim, 1e-3f), w2 = random_q8(rng, n2, n1, 1e-3f);
    std::vector<float> ids(m);
    for (auto &v : ids) v = static_cast<float>(rng() % vocab);
    NodeIndex tok, ti, w1i, w2i, y2, side;
    auto build = [&](Graph &g) {
        tok = g.add(std::make_unique<Function>());
        ti = g.add(std::make_unique<Function>());
        w1i = g.add(std::make_unique<Function>());
        w2i = g.add(std::make_unique<Function>());
        const NodeIndex rows = build_gather(g, tok, m, ti, vocab, dim);
        const NodeIndex y1 = build_matmul(g, rows, {m, dim}, w1i, n1);
        const NodeIndex act = build_relu(g, y1, {m, n1});
        y2 = build_matmul(g, act, {m, n1}, w2i, n2);
        side = g.add(std::make_unique<Unary>("Double", [](float v) { return 2 * v; }));
        g.connect(y1, side, 0, ShapeTracker({m, n1}));
        g.to_retrieve.insert(y2);
        g.to_retrieve.insert(side);
        fn(g, tok)->value = host_tensor(ids);
    };
    Graph host;
    build(host);
    fn(host, ti)->value = host_tensor(table.dense);
    fn(host, w1i)->value = host_tensor(w1.dense);
    fn(host, w2i)->value = host_tensor(w2.dense);
    host.execute();
    const std::vector<float> want2 = host_operand(host.results.at(y2), "y2"), want_side = host_operand(host.results.at(side), "side");

    Graph dev;
    build(dev);
    const NodeIndex side_dev = side;
    auto q_weights = q8_load_hip(dev, {{ti, GgufTensor{true, vocab, dim, &table.raw}},
                                       {w1i, GgufTensor{true, n1, dim, &w1.raw}},
                                       {w2i, GgufTensor{true, n2, n1, &w2.raw}}});
    EXPECT(q_weights.size() == 3);
    HipQuantizedCompiler(q_weights, dtype).compile(dev);
    dev.execute();
    std::vector<float> got2;
    for (NodeIndex r : dev.to_retrieve)
        if (r != side_dev) got2 = host_operand(dev.results.at(r), "retrieved y2");
    const std::vector<float> got_side = host_operand(dev.results.at(side_dev), "side");
    // f32: the operators' 2e-3 bar; f16: one rounding of every intermediate (2^-11 relative each)
    const double tol = dtype == DType::F32 ? 2e-3 : 1e-2;
    EXPECT(max_abs_diff(got2, want2) < tol * rms(want2));
    EXPECT(max_abs_diff(got_side, want_side) < tol * rms(want_side));
    if (dtype == DType::F32) {
        // the gather itself is exact: read it back from the quantized node
        for (NodeIndex n = 0; n < static_cast<NodeIndex>(dev.nodes.size()); ++n)
            if (dev.nodes[n] && dev.nodes[n]->name() == "QuantizedGather") {
                auto rows = device_operand(dev.results.at(n), "gather").to_host_f32();
                bool exact = rows.size() == static_cast<size_t>(m) * dim;
                for (int t = 0; exact && t < m; ++t)
                    for (int c = 0; c < dim; ++c)
                        exact &= rows[static_cast<size_t>(t) * dim + c] == table.dense[static_cast<size_t>(ids[t]) * dim + c];
                EXPECT(exact);
            }
    }
}

// The retrieved node that holds the projection by `weight` (a host copy behind a QuantizedMatmul or behind one output
// of a FusedMatvec); -1 if there is none.
static NodeIndex retrieved_projection(const Graph &g, NodeIndex weight) {
    for (NodeIndex r : g.to_retrieve) {
        if (!g.nodes[r] || g.nodes[r]->name() != "HipCopyFromDevice") continue;
        const Edge *e = g.incoming(r).at(0);
        const std::string producer = g.nodes[e->src]->name();
        if (producer == "QuantizedMatmul" && g.incoming(e->src).at(1)->src == weight) return r;
        if (producer == "FusedMatvec" && g.incoming(e->src).at(1 + e->output_order)->src == weight) return r;
    }
    return -1;
}

static void test_fused_decoder_layer(const int dim, const int kv, const int ffn, const bool with_host) {
    // The decoder layer of test_fusion_pass_cpu with real Q8_0 weights: host primitives on the dequantised weights
    // (left out at the dimensions of Llama-3-8B, where they would take minutes), the device graph operator by
    // operator, and the fused graph, twice with different activations (what is kept between executions - the
    // interleaved gate|up weight, the norm weights on the device - is made once).
    std::mt19937 rng(7);
    const float eps = 1e-5f;
    const Q8 wq = random_q8(rng, dim, dim, 1e-3f), wk = random_q8(rng, kv, dim, 1e-3f), wv = random_q8(rng, kv, dim, 1e-3f),
             wo = random_q8(rng, dim, dim, 1e-3f), wg = random_q8(rng, ffn, dim, 1e-3f), wu = random_q8(rng, ffn, dim, 1e-3f),
             wd = random_q8(rng, dim, ffn, 1e-3f);
    std::normal_distribution<float> gauss(0.f, 1.f);
    std::vector<float> norm1(dim), norm2(dim);
    for (auto &v : norm1) v = 1.f + 0.1f * gauss(rng);
    for (auto &v : norm2) v = 1.f + 0.1f * gauss(rng);
    auto activations = [&] {
        std::vector<float> x(dim);
        for (auto &v : x) v = gauss(rng);
        return x;
    };
    Graph host, plain, fused;
    const LayerNodes hn = build_decoder_layer(host, dim, kv, ffn, eps);
    struct Weight { NodeIndex node; const Q8 *w; int64_t n, k; };
    const std::vector<Weight> weights{{hn.wq, &wq, dim, dim}, {hn.wk, &wk, kv, dim}, {hn.wv, &wv, kv, dim}, {hn.wo, &wo, dim, dim},
                                      {hn.wg, &wg, ffn, dim}, {hn.wu, &wu, ffn, dim}, {hn.wd, &wd, dim, ffn}};
    if (with_host)
        for (const Weight &w : weights) fn(host, w.node)->value = host_tensor(w.w->dense);
    auto prepare_device = [&](Graph &g, bool fuse) {
        const LayerNodes n = build_decoder_layer(g, dim, kv, ffn, eps);
        EXPECT(n.wd == hn.wd && n.out == hn.out);  // same construction order, same node numbers
        std::map<NodeIndex, GgufTensor> tensors;
        for (const Weight &w : weights) tensors[w.node] = GgufTensor{true, w.n, w.k, &w.w->raw};
        HipQuantizedCompiler(q8_load_hip(g, tensors)).compile(g);
        if (fuse) HipFusedMatvecCompiler().compile(g);
    };
    prepare_device(plain, false);
    prepare_device(fused, true);
    EXPECT(count_nodes(plain, "QuantizedMatmul") == 7 && count_nodes(fused, "FusedMatvec") == 4 && count_nodes(fused, "QuantizedMatmul") == 0);
    for (Graph *g : {&host, &plain, &fused}) {
        fn(*g, hn.attn_norm)->value = host_tensor(norm1);
        fn(*g, hn.ffn_norm)->value = host_tensor(norm2);
    }
    const Tensor *kept_weight = nullptr;
    const void *first_buffer = nullptr;
    for (int round = 0; round < 2; ++round) {
        const std::vector<float> x = activations();
        for (Graph *g : {&host, &plain, &fused}) {
            if (g == &host && !with_host) continue;
            fn(*g, hn.x)->value = host_tensor(x);
            g->execute();
        }
        struct Out { const char *what; NodeIndex host_node, weight; };
        for (const Out &o : {Out{"k", hn.k, hn.wk}, Out{"v", hn.v, hn.wv}, Out{"out", hn.out, -1}}) {
            const bool have_want = with_host;
            const std::vector<float> want = have_want ? host_operand(host.results.at(o.host_node), o.what) : std::vector<float>();
            auto device_result = [&](Graph &g) {
                NodeIndex r = o.weight >= 0 ? retrieved_projection(g, o.weight) : -1;
                if (o.weight < 0)  // the layer output: the retrieved node that is neither k nor v
                    for (NodeIndex c : g.to_retrieve)
                        if (c != retrieved_projection(g, hn.wk) && c != retrieved_projection(g, hn.wv)) r = c;
                return host_operand(g.results.at(r), o.what);
            };
            const std::vector<float> got_plain = device_result(plain), got_fused = device_result(fused);
            EXPECT(got_plain.size() == got_fused.size() && !got_fused.empty());
            // operators' bar against the dequantised-weight host graph; fused against unfused differs only by f32
            // summation order (norm, dot products) and the exponential's last bits
            if (have_want) {
                EXPECT(got_plain.size() == want.size());
                EXPECT(max_abs_diff(got_plain, want) < 2e-3 * rms(want));
                EXPECT(max_abs_diff(got_fused, want) < 2e-3 * rms(want));
            }
            EXPECT(rms(got_plain) > 0 && max_abs_diff(got_fused, got_plain) < 1e-4 * rms(got_plain));
        }
        for (NodeIndex n = 0; n < static_cast<NodeIndex>(fused.nodes.size()); ++n)
            if (fused.nodes[n] && fused.nodes[n]->name() == "Q8InterleaveRows") {
                const Tensor *now = &fused.results.at(n);
                const void *buffer = device_operand(*now, "gate|up").ptr();
                if (round == 0) first_buffer = buffer;
                else EXPECT(buffer == first_buffer);  // not made again
                kept_weight = now;
            }
    }
    EXPECT(kept_weight != nullptr);
    // the interleaved weight row by row: unpack it and compare with the two sources' raw blocks
    {
        const HipData &both = device_operand(*kept_weight, "gate|up");
        HipData raw(lhip_q8_0_raw_nbytes(2 * ffn, dim));
        check(lhip_q8_0_unpack(both.ptr(), raw.ptr(), 2 * ffn, dim, nullptr), "lhip_q8_0_unpack");
        std::vector<uint8_t> bytes(raw.bytes());
        check(lhip_memcpy_d2h(bytes.data(), raw.ptr(), bytes.size(), nullptr), "lhip_memcpy_d2h");
        const size_t row = static_cast<size_t>(dim) / 32 * 34;
        bool same = true;
        for (int j = 0; j < ffn && same; ++j)
            same = std::memcmp(&bytes[(2 * j) * row], &wg.raw[j * row], row) == 0 && std::memcmp(&bytes[(2 * j + 1) * row], &wu.raw[j * row], row) == 0;
        EXPECT(same);
    }
}

static void test_device_errors_surface_as_panics() {
    // K = 40 is not a multiple of 32: the status of the C ABI becomes a Panic carrying its name
    std::mt19937 rng(4);
    const Q8 w = random_q8(rng, 8, 64, 1e-3f);
    Tensor wt{HipData::q8_0_from_raw(w.raw, 8, 64)};
    Tensor xt{HipData::from_host(std::vector<float>(40, 1.f))};
    QuantizedMatmul op;
    const std::string msg =
        panic_message([&] { op.process({{&xt, ShapeTracker({1, 40})}, {&wt, ShapeTracker({8, 40}).permute({1, 0})}}); });
    EXPECT(msg.find("lhip_q8_0_matmul_f32") != std::string::npos && msg.find("INVALID_SHAPE") != std::string::npos);
    // a host operator fed a device buffer fails the way the reference's downcast_ref::<Vec<f32>>().unwrap() does
    Unary relu("Relu", [](float v) { return v; });
    EXPECT(panic_message([&] { relu.process({{&xt, ShapeTracker({40})}}); }).find("not a host f32 vector") != std::string::npos);
    // F32 tensors of a file go to the host through the same loader
    Graph g;
    auto a = g.add(std::make_unique<Function>());
    const std::vector<uint8_t> bytes = f32_bytes({1.f, 2.f, 3.f, 4.f});
    EXPECT(q8_load_hip(g, {{a, GgufTensor{false, 2, 2, &bytes}}}).empty());
    EXPECT((host_operand(fn(g, a)->value, "a") == std::vector<float>{1, 2, 3, 4}));
}

int main(int argc, char **argv) {
    const std::string mode = argc > 1 ? argv[1] : "cpu";
    if (mode == "gguf-header" && argc > 2) {
        // the header of a file as this reader sees it, one line per fact, for a caller that compares it with its own
        try {
            std::ifstream f(argv[2], std::ios::binary);
            const GgufHeader h = GgufReader(f).read_header();
            std::printf("version %u\nalignment %llu\ndata_offset %llu\n", h.version, (unsigned long long)h.alignment,
                        (unsigned long long)h.data_offset);
            for (auto &[name, t] : h.tensors)
                std::printf("tensor %s %llu %llu %u\n", name.c_str(), (unsigned long long)t.n_elements,
                            (unsigned long long)t.offset, t.dtype);
            return 0;
        } catch (const std::exception &e) {
            std::printf("panic %s\n", e.what());
            return 3;
        }
    }
    try {
        test_primitives_on_the_host();
        test_compiler_pass_cpu();
        test_fusion_pass_cpu();
        test_gguf_reader_cpu();
        if (mode == "gpu") {
            check(lhip_init(0), "lhip_init");
            test_quantized_matvec_like_the_reference();
            test_graph_end_to_end(DType::F32);
            test_graph_end_to_end(DType::F16);
            test_gguf_file_to_graph();
            test_fused_decoder_layer(1024, 256, 2048, true);
            test_fused_decoder_layer(4096, 1024, 14336, false);  // the projections of a Llama-3-8B layer
            test_device_errors_surface_as_panics();
        }
    } catch (const std::exception &e) {
        std::printf("FAIL unexpected exception: %s\n", e.what());
        return 1;
    }
    std::printf("%s: %d checks, %d failures\n", mode.c_str(), checks, failures);
    return failures ? 1 : 0;
}
