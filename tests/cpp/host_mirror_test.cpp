// Tests of the C++ host mirror (luminal_amd/host/luminal_hip.hpp), written after the reference's own tests of the
// quantized path:
//   test_quantized_matvec / test_quantized_matmul   crates/luminal_metal/src/quantized.rs:888-986
//                                                   (same, commented out, crates/luminal_cuda/src/quantized.rs:307-451)
//   the compiler pass' two panics                   crates/luminal_cuda/src/quantized.rs:256-267
//   the "column-major" assert                       crates/luminal_cuda/src/quantized.rs:118-121
// Usage: host_mirror_test cpu   (graph rewrite and error paths, no device)
//        host_mirror_test gpu   (everything)
#include <cmath>
#include <cstdio>
#include <random>

#include "../../luminal_amd/host/luminal_hip.hpp"

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

// f32 -> IEEE binary16 code, round to nearest even (normal range and zero are all these tests need).
static uint16_t f16_code(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    int e = static_cast<int>((x >> 23) & 0xff) - 127 + 15;
    uint32_t m = x & 0x7fffffu;
    if ((x & 0x7fffffffu) == 0) return static_cast<uint16_t>(sign);
    if (e <= 0 || e >= 31) throw std::runtime_error("f16_code: out of the range these tests use");
    uint32_t h = (static_cast<uint32_t>(e) << 10) | (m >> 13);
    const uint32_t rest = m & 0x1fffu;
    if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) ++h;
    return static_cast<uint16_t>(sign | h);
}
static float f16_value(uint16_t c) {
    const int e = (c >> 10) & 31, m = c & 1023;
    const float v = e == 0 ? std::ldexp(static_cast<float>(m), -24) : std::ldexp(1.0f + m / 1024.0f, e - 15);
    return (c & 0x8000) ? -v : v;
}

// (n, k) quants + per-block scales -> raw GGUF Q8_0 blocks {f16 d; i8 qs[32]}.
static std::vector<uint8_t> q8_0_blocks(const std::vector<int8_t> &q, const std::vector<float> &d) {
    std::vector<uint8_t> raw(q.size() / 32 * 34);
    for (size_t b = 0; b < q.size() / 32; ++b) {
        const uint16_t c = f16_code(d[b]);
        std::memcpy(&raw[b * 34], &c, 2);
        std::memcpy(&raw[b * 34 + 2], &q[b * 32], 32);
    }
    return raw;
}

static double max_abs_diff(const std::vector<float> &got, const std::vector<double> &want) {
    double m = 0;
    for (size_t i = 0; i < want.size(); ++i) m = std::max(m, std::fabs(got[i] - want[i]));
    return m;
}

// ---------------------------------------------------------------- graph rewrite, no device
static void test_compiler_pass_cpu() {
    // tokens -> Gather(embed) -> ... ; x -> MatMul2D(w) ; a weight behind a unary copy ; the pass rewrites all three
    Graph g;
    auto tok = g.add(std::make_unique<Function>());
    auto embed = g.add(std::make_unique<Function>());
    auto w = g.add(std::make_unique<Function>());
    auto w2 = g.add(std::make_unique<Function>());
    auto w2_copy = g.add(std::make_unique<Unary>("Contiguous"));
    auto gather = g.add(std::make_unique<Gather>(64));
    auto mm = g.add(std::make_unique<MatMul2D>());
    auto mm2 = g.add(std::make_unique<MatMul2D>());
    g.connect(tok, gather, 0, {{3}, true});
    g.connect(embed, gather, 1, {{100, 64}, true});
    g.connect(gather, mm, 0, {{3, 64}, true});
    g.connect(w, mm, 1, {{64, 32}, false});
    g.connect(w2, w2_copy, 0, {{32, 32}, true});
    g.connect(mm, mm2, 0, {{3, 32}, true});
    g.connect(w2_copy, mm2, 1, {{32, 32}, false});
    EXPECT((downstream({embed, w, w2}, g) == std::vector<NodeIndex>{embed, w, w2_copy}));
    HipQuantizedCompiler({embed, w, w2}).compile(g, /*init_device=*/false);
    EXPECT(g.nodes[gather]->name() == "QuantizedGather");
    EXPECT(dynamic_cast<QuantizedGather *>(g.nodes[gather].get())->embed_dim == 64);
    EXPECT(g.nodes[mm]->name() == "QuantizedMatmul" && g.nodes[mm2]->name() == "QuantizedMatmul");
    EXPECT(g.nodes[w2_copy]->name() == "Contiguous");  // nodes on the way to the consumer are left alone

    // weight as input 0: "Quantized weight .. is the wrong input!"
    Graph bad;
    auto bw = bad.add(std::make_unique<Function>());
    auto bx = bad.add(std::make_unique<Function>());
    auto bmm = bad.add(std::make_unique<MatMul2D>());
    bad.connect(bw, bmm, 0, {{8, 32}, false});
    bad.connect(bx, bmm, 1, {{1, 32}, true});
    EXPECT(panic_message([&] { HipQuantizedCompiler({bw}).compile(bad, false); }).find("is the wrong input!") != std::string::npos);

    // weight into something that is neither matmul nor gather
    Graph odd;
    auto ow = odd.add(std::make_unique<Function>());
    auto ox = odd.add(std::make_unique<Function>());
    auto oadd = odd.add(std::make_unique<Unary>("Add"));
    odd.connect(ox, oadd, 0, {{32}, true});
    odd.connect(ow, oadd, 1, {{32}, true});
    const std::string msg = panic_message([&] { HipQuantizedCompiler({ow}).compile(odd, false); });
    EXPECT(msg.find("isn't a matmul or gather (Add)") != std::string::npos);

    // operator-level asserts that need no device: contiguous weight view, mismatched K
    QuantizedMatmul op;
    Tensor dummy;
    EXPECT(panic_message([&] { op.process({{&dummy, {{1, 32}, true}}, {&dummy, {{32, 8}, true}}}); }) ==
           "Weight matrix must be column-major");
    EXPECT(panic_message([&] { op.process({{&dummy, {{1, 64}, true}}, {&dummy, {{32, 8}, false}}}); }).find("inner dimensions") !=
           std::string::npos);
    EXPECT(panic_message([&] { HipData::q8_0_from_raw(std::vector<uint8_t>(33), 1, 32); }).find("n + n/16") != std::string::npos);
}

// ---------------------------------------------------------------- device
static void test_quantized_matvec_like_the_reference() {
    // W 512 x 1024 of small non-negative ints with d = 1, x random: the reference compares with the f32 graph at 1e-3.
    std::mt19937 rng(1);
    const int n = 512, k = 1024;
    std::vector<int8_t> q(static_cast<size_t>(n) * k);
    for (auto &v : q) v = static_cast<int8_t>(rng() % 5);
    std::vector<float> d(q.size() / 32, 1.0f), x(k);
    std::uniform_real_distribution<float> u(-0.5f, 0.5f);
    for (auto &v : x) v = u(rng);
    Tensor w{HipData::q8_0_from_raw(q8_0_blocks(q, d), n, k)};
    Tensor xt{std::make_shared<std::vector<float>>(x)};
    QuantizedMatmul op;
    auto out = op.process({{&xt, {{k}, true}}, {&w, {{k, n}, false}}});
    std::vector<double> want(n, 0.0);
    for (int r = 0; r < n; ++r)
        for (int c = 0; c < k; ++c) want[r] += static_cast<double>(q[static_cast<size_t>(r) * k + c]) * x[c];
    EXPECT(max_abs_diff(device_operand(out[0], "out").to_host_f32(), want) < 1e-3);
}

static void test_quantized_matmul_and_graph_execution() {
    // tokens -> QuantizedGather(embed 100 x 64) -> QuantizedMatmul(w 96 x 64), real scales and negative quants,
    // through compile() + execute(); M = 16 rows like the reference's matmul test.
    std::mt19937 rng(2);
    const int vocab = 100, dim = 64, n = 96, m = 16;
    std::normal_distribution<float> gauss(0.f, 0.02f);
    auto make = [&](int rows, int cols, std::vector<int8_t> &q, std::vector<float> &d) {
        q.resize(static_cast<size_t>(rows) * cols);
        d.resize(q.size() / 32);
        for (auto &v : q) v = static_cast<int8_t>(static_cast<int>(rng() % 255) - 127);
        for (auto &v : d) v = f16_value(f16_code(std::fabs(gauss(rng)) / 127.f + 1e-4f));
        return q8_0_blocks(q, d);
    };
    std::vector<int8_t> eq, wq;
    std::vector<float> ed, wd;
    auto e_raw = make(vocab, dim, eq, ed), w_raw = make(n, dim, wq, wd);
    std::vector<float> ids(m);
    for (auto &v : ids) v = static_cast<float>(rng() % vocab);

    Graph g;
    auto tok = g.add(std::make_unique<Function>());
    auto embed = g.add(std::make_unique<Function>());
    auto w = g.add(std::make_unique<Function>());
    auto gather = g.add(std::make_unique<Gather>(dim));
    auto mm = g.add(std::make_unique<MatMul2D>());
    g.connect(tok, gather, 0, {{m}, true});
    g.connect(embed, gather, 1, {{vocab, dim}, true});
    g.connect(gather, mm, 0, {{m, dim}, true});
    g.connect(w, mm, 1, {{dim, n}, false});
    HipQuantizedCompiler({embed, w}).compile(g);
    dynamic_cast<Function *>(g.nodes[tok].get())->value = Tensor{std::make_shared<std::vector<float>>(ids)};
    dynamic_cast<Function *>(g.nodes[embed].get())->value = Tensor{HipData::q8_0_from_raw(e_raw, vocab, dim)};
    dynamic_cast<Function *>(g.nodes[w].get())->value = Tensor{HipData::q8_0_from_raw(w_raw, n, dim)};
    g.execute();

    auto deq = [](const std::vector<int8_t> &q, const std::vector<float> &d, size_t i) {
        return static_cast<double>(q[i]) * static_cast<double>(d[i / 32]);
    };
    // gather is exact
    auto rows = device_operand(g.results.at(gather), "gather").to_host_f32();
    bool exact = true;
    for (int t = 0; t < m; ++t)
        for (int c = 0; c < dim; ++c)
            exact &= rows[static_cast<size_t>(t) * dim + c] ==
                     static_cast<float>(deq(eq, ed, static_cast<size_t>(ids[t]) * dim + c));
    EXPECT(exact);
    std::vector<double> want(static_cast<size_t>(m) * n, 0.0);
    double rms = 0;
    for (int t = 0; t < m; ++t)
        for (int r = 0; r < n; ++r) {
            double s = 0;
            for (int c = 0; c < dim; ++c)
                s += deq(eq, ed, static_cast<size_t>(ids[t]) * dim + c) * deq(wq, wd, static_cast<size_t>(r) * dim + c);
            want[static_cast<size_t>(t) * n + r] = s;
            rms += s * s;
        }
    rms = std::sqrt(rms / want.size());
    EXPECT(max_abs_diff(device_operand(g.results.at(mm), "matmul").to_host_f32(), want) < 2e-3 * rms);

    // device-side failure surfaces as a Panic carrying the status name (K not a multiple of 32)
    Tensor xt{std::make_shared<std::vector<float>>(std::vector<float>(40, 1.f))};
    QuantizedMatmul op;
    const std::string msg = panic_message([&] { op.process({{&xt, {{40}, true}}, {&g.results.at(w), {{40, 8}, false}}}); });
    EXPECT(msg.find("lhip_q8_0_matmul_f32") != std::string::npos && msg.find("INVALID_SHAPE") != std::string::npos);
}

static void test_f16_graph() {
    // The same two-node graph compiled for T = f16 (the type the reference's llama example runs in):
    // gather -> f16 rows (exact rows rounded once), matmul -> f32 sums rounded once to f16.
    std::mt19937 rng(3);
    const int vocab = 50, dim = 64, n = 40, m = 5;
    std::normal_distribution<float> gauss(0.f, 0.02f);
    auto make = [&](int rows, int cols, std::vector<int8_t> &q, std::vector<float> &d) {
        q.resize(static_cast<size_t>(rows) * cols);
        d.resize(q.size() / 32);
        for (auto &v : q) v = static_cast<int8_t>(static_cast<int>(rng() % 255) - 127);
        for (auto &v : d) v = f16_value(f16_code(std::fabs(gauss(rng)) / 127.f + 1e-3f));
        return q8_0_blocks(q, d);
    };
    std::vector<int8_t> eq, wq;
    std::vector<float> ed, wd;
    auto e_raw = make(vocab, dim, eq, ed), w_raw = make(n, dim, wq, wd);
    std::vector<float> ids(m);
    for (auto &v : ids) v = static_cast<float>(rng() % vocab);
    Graph g;
    auto tok = g.add(std::make_unique<Function>());
    auto embed = g.add(std::make_unique<Function>());
    auto w = g.add(std::make_unique<Function>());
    auto gather = g.add(std::make_unique<Gather>(dim));
    auto mm = g.add(std::make_unique<MatMul2D>());
    g.connect(tok, gather, 0, {{m}, true});
    g.connect(embed, gather, 1, {{vocab, dim}, true});
    g.connect(gather, mm, 0, {{m, dim}, true});
    g.connect(w, mm, 1, {{dim, n}, false});
    HipQuantizedCompiler({embed, w}, DType::F16).compile(g);
    EXPECT(dynamic_cast<QuantizedMatmul *>(g.nodes[mm].get())->dtype == DType::F16);
    dynamic_cast<Function *>(g.nodes[tok].get())->value = Tensor{std::make_shared<std::vector<float>>(ids)};
    dynamic_cast<Function *>(g.nodes[embed].get())->value = Tensor{HipData::q8_0_from_raw(e_raw, vocab, dim)};
    dynamic_cast<Function *>(g.nodes[w].get())->value = Tensor{HipData::q8_0_from_raw(w_raw, n, dim)};
    g.execute();
    auto rows = device_operand(g.results.at(gather), "gather").to_host_f16_codes();
    bool exact = rows.size() == static_cast<size_t>(m) * dim;
    for (int t = 0; exact && t < m; ++t)
        for (int c = 0; c < dim; ++c) {
            const size_t i = static_cast<size_t>(ids[t]) * dim + c;
            exact &= rows[static_cast<size_t>(t) * dim + c] == f16_code(static_cast<float>(eq[i]) * ed[i / 32]);
        }
    EXPECT(exact);
    auto out = device_operand(g.results.at(mm), "matmul").to_host_f16_codes();
    double worst = 0, rms = 0;
    for (int t = 0; t < m; ++t)
        for (int r = 0; r < n; ++r) {
            double s = 0;
            for (int c = 0; c < dim; ++c)
                s += static_cast<double>(f16_value(rows[static_cast<size_t>(t) * dim + c])) *
                     (static_cast<double>(wq[static_cast<size_t>(r) * dim + c]) * wd[(static_cast<size_t>(r) * dim + c) / 32]);
            worst = std::max(worst, std::fabs(f16_value(out[static_cast<size_t>(t) * n + r]) - s));
            rms += s * s;
        }
    EXPECT(worst < 2e-3 * std::sqrt(rms / (m * n)));
}

int main(int argc, char **argv) {
    const std::string mode = argc > 1 ? argv[1] : "cpu";
    try {
        test_compiler_pass_cpu();
        if (mode == "gpu") {
            check(lhip_init(0), "lhip_init");
            test_quantized_matvec_like_the_reference();
            test_quantized_matmul_and_graph_execution();
            test_f16_graph();
        }
    } catch (const std::exception &e) {
        std::printf("FAIL unexpected exception: %s\n", e.what());
        return 1;
    }
    std::printf("%s: %d checks, %d failures\n", mode.c_str(), checks, failures);
    return failures ? 1 : 0;
}
