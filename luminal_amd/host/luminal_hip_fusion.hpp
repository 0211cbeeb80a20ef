// Batch-1 decode fusions above HipQuantizedCompiler: a second pass that finds, around the QuantizedMatmul nodes of a
// one-row (matvec) graph, the patterns that lhip_q8_0_matvec_fused_f32 runs as one launch, and replaces each by a
// FusedMatvec node:
//   * sibling projections: up to four QuantizedMatmul nodes reading the same activations (q, k, v of
//     examples/llama/src/model.rs:95-110; gate and up of model.rs:24-32);
//   * norm prologue: the activations are the RMS norm of x as luminal_nn spells it in primitives
//     (crates/luminal_nn/src/norm.rs:56-70 over src/hl_ops/unary.rs:93-104 and src/hl_ops/reduction.rs:38-45):
//         Mul(Mul(expand(Recip(Sqrt(Add(Mul(SumReduce(Mul(x, x)), Recip(Constant(D))), Constant(eps))))), x), expand(w));
//   * residual epilogue: the projection's only consumer is Add(residual, y) (model.rs:163-172, `x += y`);
//   * SwiGLU epilogue: up * (gate * sigmoid(gate)) with sigmoid = 1 / (1 + exp(-gate)), exp(t) = exp2(t / ln 2)
//     (model.rs:27-29 over src/hl_ops/unary.rs:33-36,168-177); the two weights are interleaved row by row once, by a
//     Q8InterleaveRows node whose result is kept.
// The reference has no such pass (its graph runs one operator per launch); the patterns are the reference's own
// spellings, so a graph built by its model code is what this pass is written against.  f32 activations only.
// Header-only; needs luminal_hip.hpp.
#pragma once

#include "luminal_hip.hpp"

namespace luminal_hip {

// Planar (n, k) gate and up weights -> planar (2n, k), rows alternating (gate_j, up_j).  Runs once: the pass marks
// the node no_delete.
class Q8InterleaveRows : public Operator {
  public:
    Q8InterleaveRows(int64_t n, int64_t k) : n(n), k(k) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        const void *a = device_operand(*inp.at(0).first, "gate weight").ptr();
        const void *b = device_operand(*inp.at(1).first, "up weight").ptr();
        auto out = std::make_shared<HipData>(lhip_q8_0_planar_nbytes(2 * n, k));
        check(lhip_q8_0_interleave_rows(a, b, out->ptr(), n, k, nullptr), "lhip_q8_0_interleave_rows");
        return {Tensor{out}};
    }
    std::string name() const override { return "Q8InterleaveRows"; }
    int64_t n, k;
};

// One launch of lhip_q8_0_matvec_fused_f32.  Inputs by input_order: 0 activations x (device f32, k values),
// 1..count the planar weights, then the norm weight (device f32, k values) if `norm`, then the residual (device
// f32, n[0] values) if epilogue == Residual.  Outputs: one device f32 vector per weight; with SwiGLU the single
// weight holds (gate, up) row pairs and the output has n[0] / 2 values.
class FusedMatvec : public Operator {
  public:
    enum Epilogue { None = 0, Residual = 1, SwiGLU = 2 };
    FusedMatvec(std::vector<int64_t> n, int64_t k, bool norm, float eps, Epilogue epilogue)
        : n(std::move(n)), k(k), norm(norm), eps(eps), epilogue(epilogue) {}
    std::vector<Tensor> process(const std::vector<Input> &inp) override {
        const size_t count = n.size();
        if (inp.size() != 1 + count + (norm ? 1 : 0) + (epilogue == Residual ? 1 : 0))
            throw Panic("FusedMatvec: wrong number of inputs");
        if (!inp[0].second.is_contiguous() || inp[0].second.n_elements() != k)
            throw Panic("FusedMatvec: activations must be one contiguous row of K values");
        const auto *x = static_cast<const float *>(device_operand(*inp[0].first, "activation").ptr());
        std::vector<const void *> w(count);
        std::vector<float *> y(count);
        std::vector<std::shared_ptr<HipData>> out(count);
        for (size_t i = 0; i < count; ++i) {
            w[i] = device_operand(*inp[1 + i].first, "weight").ptr();
            const int64_t values = epilogue == SwiGLU ? n[i] / 2 : n[i];
            out[i] = std::make_shared<HipData>(static_cast<size_t>(values) * sizeof(float));
            y[i] = static_cast<float *>(out[i]->ptr());
        }
        size_t at = 1 + count;
        const float *norm_w = norm ? static_cast<const float *>(device_operand(*inp[at++].first, "norm weight").ptr()) : nullptr;
        const float *residual =
            epilogue == Residual ? static_cast<const float *>(device_operand(*inp[at++].first, "residual").ptr()) : nullptr;
        check(lhip_q8_0_matvec_fused_f32(w.data(), y.data(), n.data(), static_cast<int>(count), x, k, norm_w, eps, residual,
                                         static_cast<int>(epilogue), nullptr),
              "lhip_q8_0_matvec_fused_f32");
        std::vector<Tensor> result;
        for (auto &o : out) result.push_back(Tensor{o});
        return result;
    }
    std::string name() const override { return "FusedMatvec"; }
    std::vector<int64_t> n;
    int64_t k;
    bool norm;
    float eps;
    Epilogue epilogue;
};

class HipFusedMatvecCompiler {
  public:
    // Runs behind HipQuantizedCompiler on the same graph.  Touches no device.
    void compile(Graph &g) const {
        // Groups of one-row f32 QuantizedMatmul nodes by the node that produces their activations.
        std::map<NodeIndex, std::vector<NodeIndex>> groups;
        for (NodeIndex q = 0; q < static_cast<NodeIndex>(g.nodes.size()); ++q) {
            auto *mm = dynamic_cast<QuantizedMatmul *>(g.nodes[q].get());
            if (!mm || mm->dtype != DType::F32) continue;
            auto in = g.incoming(q);
            if (in.size() != 2) continue;
            const int64_t k = in[1]->shape.dims.at(in[1]->shape.rank() - 2);
            if (!in[0]->shape.is_contiguous() || in[0]->shape.n_elements() != k) continue;  // not a single row
            if (k % 1024 != 0 || k > 16384) continue;                                       // lhip_q8_0_matvec_fused_f32's K
            groups[producer_of(g, in[0]->src)].push_back(q);
        }
        for (auto &[producer, members] : groups)
            for (size_t first = 0; first < members.size(); first += 4)
                fuse(g, producer, std::vector<NodeIndex>(members.begin() + first,
                                                         members.begin() + std::min(members.size(), first + 4)));
        // An upload whose source has meanwhile become a device node only hands the buffer on: take it out.
        for (NodeIndex c = 0; c < static_cast<NodeIndex>(g.nodes.size()); ++c) {
            if (!as<HipCopyToDevice>(g, c) || g.no_delete.count(c)) continue;
            const Edge from = *g.incoming(c).at(0);
            if (!as<FusedMatvec>(g, from.src) && !as<QuantizedMatmul>(g, from.src) && !as<QuantizedGather>(g, from.src)) continue;
            std::vector<Edge> uses;
            for (const Edge *e : g.outgoing(c)) uses.push_back(*e);
            for (const Edge &e : uses) g.connect(from.src, e.dst, e.input_order, e.shape, from.output_order);
            g.remove_node(c);
        }
    }

  private:
    template <typename T>
    static T *as(const Graph &g, NodeIndex n) {
        return n >= 0 && g.nodes.at(n) ? dynamic_cast<T *>(g.nodes[n].get()) : nullptr;
    }
    static bool is_unary(const Graph &g, NodeIndex n, const char *label) {
        auto *u = as<Unary>(g, n);
        return u && u->label == label;
    }
    static bool is_binary(const Graph &g, NodeIndex n, Binary::Kind kind) {
        auto *b = as<Binary>(g, n);
        return b && b->kind == kind;
    }
    static bool all_fake(const ShapeTracker &s) {
        for (size_t i = 0; i < s.rank(); ++i)
            if (!s.is_fake(i)) return false;
        return true;
    }
    // A Constant entering through a fully expanded view: its value, else no value.
    static bool constant_operand(const Graph &g, const Edge *e, float &value) {
        auto *c = as<Constant>(g, e->src);
        if (!c || !all_fake(e->shape)) return false;
        value = c->value;
        return true;
    }
    static bool only_consumer(const Graph &g, NodeIndex n, NodeIndex consumer) {
        if (g.to_retrieve.count(n)) return false;
        auto out = g.outgoing(n);
        return std::all_of(out.begin(), out.end(), [&](const Edge *e) { return e->dst == consumer; }) && !out.empty();
    }
    // The node whose result a device operand is a copy of: through HipCopyToDevice to the host producer, and
    // through a HipCopyFromDevice -> HipCopyToDevice round trip back to the device producer.
    static NodeIndex producer_of(const Graph &g, NodeIndex n) {
        while (as<HipCopyToDevice>(g, n) || as<HipCopyFromDevice>(g, n)) n = g.incoming(n).at(0)->src;
        return n;
    }
    // Where to read node n's result (output `out`) on the device: the device node behind a HipCopyFromDevice, the
    // node itself if it runs on the device, else a new HipCopyToDevice behind the host node.
    static std::pair<NodeIndex, int> on_device(Graph &g, NodeIndex n, bool keep = false) {
        if (as<HipCopyFromDevice>(g, n)) {
            const Edge *e = g.incoming(n).at(0);
            return {e->src, e->output_order};
        }
        if (as<QuantizedMatmul>(g, n) || as<QuantizedGather>(g, n) || as<FusedMatvec>(g, n) || as<HipCopyToDevice>(g, n) ||
            as<Q8InterleaveRows>(g, n))
            return {n, 0};
        for (const Edge *e : g.outgoing(n))  // an upload of the whole result that is already there
            if (auto *c = as<HipCopyToDevice>(g, e->dst); c && c->dtype == DType::F32 && e->shape.rank() == 0) {
                if (keep) g.no_delete.insert(e->dst);
                return {e->dst, 0};
            }
        const NodeIndex up = g.add(std::make_unique<HipCopyToDevice>(DType::F32));
        g.connect(n, up, 0, ShapeTracker());
        if (keep) g.no_delete.insert(up);
        return {up, 0};
    }

    struct Norm {
        NodeIndex x = -1, weight = -1;  // the normalised tensor's producer, the Function holding the norm weight
        float eps = 0.f;
    };
    // `p` as the RMS norm of a K-vector; every node of the pattern below p must feed the pattern only.
    static bool match_rms_norm(const Graph &g, NodeIndex p, int64_t k, Norm &norm) {
        if (!is_binary(g, p, Binary::Mul)) return false;
        auto in = g.incoming(p);
        if (in.size() != 2) return false;
        // (normalised x) * expand(weight): the weight enters with every dimension but the last expanded
        auto weight_view = [&](const Edge *e) {
            const ShapeTracker &s = e->shape;
            if (!as<Function>(g, e->src) || s.rank() == 0 || s.dims.back() != k || s.strides.back() != 1) return false;
            for (size_t i = 0; i + 1 < s.rank(); ++i)
                if (!s.is_fake(i)) return false;
            return true;
        };
        const Edge *w_edge = weight_view(in[1]) ? in[1] : weight_view(in[0]) ? in[0] : nullptr;
        if (!w_edge) return false;
        const Edge *n_edge = w_edge == in[1] ? in[0] : in[1];
        const NodeIndex scaled = n_edge->src;  // expand(1 / sqrt(mean(x^2) + eps)) * x
        if (!is_binary(g, scaled, Binary::Mul) || !only_consumer(g, scaled, p) || !n_edge->shape.is_contiguous()) return false;
        auto sin = g.incoming(scaled);
        if (sin.size() != 2) return false;
        auto factor_view = [&](const Edge *e) { return e->shape.rank() > 0 && e->shape.is_fake(e->shape.rank() - 1); };
        const Edge *f_edge = factor_view(sin[0]) ? sin[0] : factor_view(sin[1]) ? sin[1] : nullptr;
        if (!f_edge) return false;
        const Edge *x_edge = f_edge == sin[0] ? sin[1] : sin[0];
        if (!x_edge->shape.is_contiguous() || x_edge->shape.n_elements() != k) return false;
        // upwards from the factor: Recip <- Sqrt <- Add(mean, eps) <- Mul(sum, 1/D) <- SumReduce(last) <- Mul(x, x)
        NodeIndex at = f_edge->src;
        if (!is_unary(g, at, "Recip") || !only_consumer(g, at, scaled)) return false;
        NodeIndex below = at;
        at = g.incoming(at).at(0)->src;
        if (!is_unary(g, at, "Sqrt") || !only_consumer(g, at, below)) return false;
        below = at;
        at = g.incoming(at).at(0)->src;
        if (!is_binary(g, at, Binary::Add) || !only_consumer(g, at, below)) return false;
        auto ain = g.incoming(at);
        float eps = 0.f;
        const Edge *mean_edge = nullptr;
        if (constant_operand(g, ain.at(1), eps)) mean_edge = ain[0];
        else if (constant_operand(g, ain.at(0), eps)) mean_edge = ain[1];
        else return false;
        below = at;
        at = mean_edge->src;
        if (!is_binary(g, at, Binary::Mul) || !only_consumer(g, at, below)) return false;
        auto min = g.incoming(at);
        // the divisor: `tensor / Expression` spells it Recip(expand(Constant(D))); `tensor / f32` Constant(1/D)
        auto inverse_of_k = [&](const Edge *e) {
            float v = 0.f;
            if (constant_operand(g, e, v)) return std::fabs(v * static_cast<float>(k) - 1.f) < 1e-5f;
            if (!is_unary(g, e->src, "Recip") || !only_consumer(g, e->src, at)) return false;
            return constant_operand(g, g.incoming(e->src).at(0), v) && v == static_cast<float>(k);
        };
        const Edge *sum_edge = inverse_of_k(min.at(1)) ? min[0] : inverse_of_k(min.at(0)) ? min[1] : nullptr;
        if (!sum_edge) return false;
        below = at;
        at = sum_edge->src;
        auto *sum = as<SumReduce>(g, at);
        if (!sum || !only_consumer(g, at, below)) return false;
        const Edge *sq_edge = g.incoming(at).at(0);
        if (sum->dim + 1 != sq_edge->shape.rank()) return false;
        below = at;
        at = sq_edge->src;
        if (!is_binary(g, at, Binary::Mul) || !only_consumer(g, at, below)) return false;
        auto qin = g.incoming(at);
        if (qin.size() != 2 || qin[0]->src != x_edge->src || qin[1]->src != x_edge->src) return false;
        if (qin[0]->output_order != x_edge->output_order || qin[1]->output_order != x_edge->output_order) return false;
        if (qin[0]->shape.strides != x_edge->shape.strides || qin[1]->shape.strides != x_edge->shape.strides) return false;
        norm.x = x_edge->src;
        norm.weight = w_edge->src;
        norm.eps = eps;
        return true;
    }

    // up * (gate * (1 / (1 + exp2(-gate / ln 2)))) behind the host copies `gate` and `up`: the node that holds the
    // product, or -1.
    static NodeIndex match_swiglu(const Graph &g, NodeIndex gate, NodeIndex up) {
        if (g.to_retrieve.count(gate) || g.to_retrieve.count(up)) return -1;
        auto gate_uses = g.outgoing(gate);
        if (gate_uses.size() != 2) return -1;
        // a Mul of `from` by a fully expanded Constant of the given value, in either operand order
        auto scaled_by = [&](NodeIndex from, float value, float tolerance) -> NodeIndex {
            for (const Edge *e : g.outgoing(from)) {
                if (!is_binary(g, e->dst, Binary::Mul)) continue;
                auto in = g.incoming(e->dst);
                float v = 0.f;
                const Edge *other = in.at(0)->src == from ? in.at(1) : in.at(0);
                if (constant_operand(g, other, v) && std::fabs(v - value) <= tolerance) return e->dst;
            }
            return -1;
        };
        const NodeIndex neg = scaled_by(gate, -1.f, 0.f);
        if (neg < 0) return -1;
        const NodeIndex scaled = scaled_by(neg, 1.f / std::log(2.f), 1e-6f);
        if (scaled < 0 || !only_consumer(g, neg, scaled)) return -1;
        auto single_next = [&](NodeIndex n) { return g.outgoing(n).size() == 1 && !g.to_retrieve.count(n) ? g.outgoing(n)[0]->dst : -1; };
        const NodeIndex e2 = single_next(scaled);
        if (!is_unary(g, e2, "Exp2")) return -1;
        const NodeIndex plus = single_next(e2);
        if (!is_binary(g, plus, Binary::Add)) return -1;
        {
            auto in = g.incoming(plus);
            float one = 0.f;
            const Edge *other = in.at(0)->src == e2 ? in.at(1) : in.at(0);
            if (!constant_operand(g, other, one) || one != 1.f) return -1;
        }
        NodeIndex sig = single_next(plus);
        if (!is_unary(g, sig, "Recip")) return -1;
        // `1. / t` is spelled 1.0 * recip(t): a Mul by Constant(1) may follow
        if (const NodeIndex times_one = scaled_by(sig, 1.f, 0.f); times_one >= 0 && only_consumer(g, sig, times_one)) sig = times_one;
        const NodeIndex swish = single_next(sig);
        if (!is_binary(g, swish, Binary::Mul)) return -1;
        {
            auto in = g.incoming(swish);
            const NodeIndex other = in.at(0)->src == sig ? in.at(1)->src : in.at(0)->src;
            if (other != gate) return -1;
        }
        for (const Edge *e : gate_uses)
            if (e->dst != neg && e->dst != swish) return -1;
        const NodeIndex out = single_next(swish);
        if (!is_binary(g, out, Binary::Mul) || !only_consumer(g, up, out)) return -1;
        auto in = g.incoming(out);
        const NodeIndex other = in.at(0)->src == swish ? in.at(1)->src : in.at(0)->src;
        return other == up ? out : -1;
    }

    // The host copy behind a quantized node, if that copy is the node's only consumer.
    static NodeIndex sole_host_copy(const Graph &g, NodeIndex q) {
        auto out = g.outgoing(q);
        if (out.size() != 1 || g.to_retrieve.count(q) || !as<HipCopyFromDevice>(g, out[0]->dst)) return -1;
        return out[0]->dst;
    }

    // Consumers of host node `old` read output `out` of device node `dev` instead: device-side consumers directly,
    // the others (and a retrieval) through one HipCopyFromDevice.
    static void replace_with_device_output(Graph &g, NodeIndex old, NodeIndex dev, int out) {
        std::vector<Edge> uses;
        for (const Edge *e : g.outgoing(old)) uses.push_back(*e);
        NodeIndex down = -1;
        auto host_copy = [&] {
            if (down < 0) {
                down = g.add(std::make_unique<HipCopyFromDevice>(DType::F32));
                g.connect(dev, down, 0, ShapeTracker(), out);
            }
            return down;
        };
        for (const Edge &e : uses) {
            const bool device_side = as<HipCopyToDevice>(g, e.dst) || as<FusedMatvec>(g, e.dst) ||
                                     (as<QuantizedMatmul>(g, e.dst) && e.input_order == 0);
            if (device_side) g.connect(dev, e.dst, e.input_order, e.shape, out);
            else g.connect(host_copy(), e.dst, e.input_order, e.shape);
        }
        if (g.to_retrieve.erase(old)) g.to_retrieve.insert(host_copy());
        g.edges.erase(std::remove_if(g.edges.begin(), g.edges.end(), [&](const Edge &e) { return e.src == old; }), g.edges.end());
    }

    static void prune_dead(Graph &g, NodeIndex n) {
        if (n < 0 || !g.nodes.at(n) || !g.outgoing(n).empty() || g.to_retrieve.count(n)) return;
        if (as<Function>(g, n)) return;
        std::vector<NodeIndex> parents;
        for (const Edge *e : g.incoming(n)) parents.push_back(e->src);
        g.remove_node(n);
        for (NodeIndex p : parents) prune_dead(g, p);
    }

    static void fuse(Graph &g, NodeIndex producer, const std::vector<NodeIndex> &members) {
        const int64_t k = g.incoming(members[0]).at(1)->shape.dims.at(g.incoming(members[0])[1]->shape.rank() - 2);
        Norm norm;
        const bool has_norm = match_rms_norm(g, producer, k, norm) && [&] {
            // the normalised vector must feed these projections only, or it has to be computed anyway
            std::set<NodeIndex> readers;
            for (NodeIndex q : members) readers.insert(g.incoming(q).at(0)->src), readers.insert(q);
            for (const Edge *e : g.outgoing(producer))
                if (!readers.count(e->dst)) return false;
            return !g.to_retrieve.count(producer);
        }();
        FusedMatvec::Epilogue epilogue = FusedMatvec::None;
        NodeIndex replaced = -1, residual = -1;  // the host node whose result the fused launch produces instead
        if (members.size() == 2) {
            const NodeIndex gate = sole_host_copy(g, members[0]), up = sole_host_copy(g, members[1]);
            const int64_t n0 = g.incoming(members[0])[1]->shape.dims.back(), n1 = g.incoming(members[1])[1]->shape.dims.back();
            if (gate >= 0 && up >= 0 && n0 == n1) {
                if ((replaced = match_swiglu(g, gate, up)) >= 0) epilogue = FusedMatvec::SwiGLU;
                else if (match_swiglu(g, up, gate) >= 0) return fuse(g, producer, {members[1], members[0]});  // (gate, up) order
            }
        } else if (members.size() == 1) {
            const NodeIndex y = sole_host_copy(g, members[0]);
            if (y >= 0 && g.outgoing(y).size() == 1 && !g.to_retrieve.count(y) && is_binary(g, g.outgoing(y)[0]->dst, Binary::Add)) {
                const NodeIndex add = g.outgoing(y)[0]->dst;
                auto in = g.incoming(add);
                const Edge *other = in.at(0)->src == y ? in.at(1) : in.at(0);
                const int64_t n = g.incoming(members[0])[1]->shape.dims.back();
                if (other->src != y && other->shape.is_contiguous() && other->shape.n_elements() == n) {
                    epilogue = FusedMatvec::Residual;
                    replaced = add;
                    residual = other->src;
                }
            }
        }
        if (members.size() == 1 && !has_norm && epilogue == FusedMatvec::None) return;  // nothing to gain

        // inputs
        std::vector<int64_t> n;
        std::vector<std::pair<NodeIndex, ShapeTracker>> weights;
        for (NodeIndex q : members) {
            const Edge *w = g.incoming(q).at(1);
            n.push_back(w->shape.dims.back());
            weights.emplace_back(w->src, w->shape);
        }
        const Edge act = *g.incoming(members[0]).at(0);
        const std::pair<NodeIndex, int> x = has_norm ? on_device(g, norm.x) : std::pair<NodeIndex, int>{act.src, act.output_order};
        if (epilogue == FusedMatvec::SwiGLU) {
            const NodeIndex both = g.add(std::make_unique<Q8InterleaveRows>(n[0], k));
            g.connect(weights[0].first, both, 0, weights[0].second);
            g.connect(weights[1].first, both, 1, weights[1].second);
            g.no_delete.insert(both);
            ShapeTracker view({2 * n[0], k});
            weights = {{both, view.permute({1, 0})}};
            n = {2 * n[0]};
        }
        const NodeIndex fused = g.add(std::make_unique<FusedMatvec>(n, k, has_norm, norm.eps, epilogue));
        int order = 0;
        g.connect(x.first, fused, order++, ShapeTracker({k}), x.second);
        for (auto &[node, shape] : weights) g.connect(node, fused, order++, shape);
        if (has_norm) g.connect(on_device(g, norm.weight, /*keep=*/true).first, fused, order++, ShapeTracker({k}));
        if (epilogue == FusedMatvec::Residual) {
            const auto r = on_device(g, residual);
            g.connect(r.first, fused, order++, ShapeTracker({n[0]}), r.second);
        }

        // outputs
        std::vector<NodeIndex> feeders;
        for (NodeIndex q : members) feeders.push_back(g.incoming(q).at(0)->src);
        if (epilogue == FusedMatvec::None) {
            for (size_t i = 0; i < members.size(); ++i) {
                std::vector<Edge> uses;
                for (const Edge *e : g.outgoing(members[i])) uses.push_back(*e);
                for (const Edge &e : uses) g.connect(fused, e.dst, e.input_order, e.shape, static_cast<int>(i));
                if (g.to_retrieve.erase(members[i])) {
                    const NodeIndex down = g.add(std::make_unique<HipCopyFromDevice>(DType::F32));
                    g.connect(fused, down, 0, ShapeTracker(), static_cast<int>(i));
                    g.to_retrieve.insert(down);
                }
                g.remove_node(members[i]);
            }
        } else {
            // the epilogue's host nodes go from the bottom up; the projections and their host copies lose their
            // last consumer on the way
            replace_with_device_output(g, replaced, fused, 0);
            prune_dead(g, replaced);
        }
        for (NodeIndex f : feeders) prune_dead(g, f);
        prune_dead(g, producer);
    }
};

}  // namespace luminal_hip
