//! Batch-1 decode fusions: a second pass, behind `HipQuantizedCompiler::<f32>`, that finds around the
//! `QuantizedMatmul<f32>` nodes of a one-row graph the patterns `lhip_q8_0_matvec_fused_f32` runs as one launch and
//! replaces each by a `FusedMatvec` node:
//!   * sibling projections: up to four matmuls reading the same activations (q, k, v of
//!     examples/llama/src/model.rs:95-110; gate and up of model.rs:24-32);
//!   * norm prologue: the activations are the RMS norm of x as luminal_nn spells it in primitives
//!     (crates/luminal_nn/src/norm.rs:56-70 over src/hl_ops/unary.rs:93-104 and src/hl_ops/reduction.rs:38-45):
//!     `Mul(Mul(expand(Recip(Sqrt(Add(Mul(SumReduce(Mul(x, x)), Recip(Constant(D))), Constant(eps))))), x), expand(w))`;
//!   * residual epilogue: the projection's only consumer is `Add(residual, y)` (model.rs:163-172, `x += y`);
//!   * SwiGLU epilogue: `up * (gate * sigmoid(gate))`, sigmoid = 1 / (1 + exp(-gate)), exp(t) = exp2(t / ln 2)
//!     (model.rs:27-29 over src/hl_ops/unary.rs:33-36,168-177); the two weights are interleaved row by row once, by
//!     a `Q8InterleaveRows` node whose result is kept (`no_delete`).
//! The reference has no such pass (its graph runs one operator per launch).  Usage:
//! ```ignore
//! cx.compile(
//!     (GenericCompiler::default(), HipQuantizedCompiler::<f32>::new(q_weights), HipFusedMatvecCompiler),
//!     (&mut logits, &mut cache),
//! );
//! ```
//! Like the rest of the crate this file has not met a compiler; it follows, function by function,
//! luminal_amd/host/luminal_hip_fusion.hpp, which is compiled and tested (tests/cpp/host_mirror_test.cpp).
use std::ptr::null_mut;

use luminal::{
    op::{Add, Constant, ConstantValue, Exp2, Function, InputTensor, Mul, Operator, Recip, Sqrt, SumReduce},
    prelude::*,
};
use petgraph::{visit::EdgeRef, Direction};
use rustc_hash::FxHashMap;

use crate::ffi::{self, check};
use crate::quantized::{HipCopyFromDevice, HipCopyToDevice, HipData, QuantizedGather, QuantizedMatmul};

fn device(t: &InputTensor, what: &str) -> HipData {
    t.borrowed().downcast_ref::<HipData>().unwrap_or_else(|| panic!("{what} is not a HIP buffer")).clone()
}

/// Planar (n, k) gate and up weights -> planar (2n, k), rows alternating (gate_j, up_j).  Runs once: the pass
/// marks the node `no_delete`, and the executor skips a node whose result is there (src/graph.rs:199-202).
#[derive(Clone, Debug)]
pub struct Q8InterleaveRows {
    pub n: usize,
    pub k: usize,
}

impl Operator for Q8InterleaveRows {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        let (a, b) = (device(&inp[0].0, "gate weight"), device(&inp[1].0, "up weight"));
        let (n, k) = (self.n as i64, self.k as i64);
        let out = HipData::alloc(unsafe { ffi::lhip_q8_0_planar_nbytes(2 * n, k) });
        check(unsafe { ffi::lhip_q8_0_interleave_rows(a.ptr(), b.ptr(), out.ptr(), n, k, null_mut()) }, "lhip_q8_0_interleave_rows");
        vec![Tensor::new(out)]
    }
}

#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum Epilogue {
    None = 0,
    Residual = 1,
    SwiGlu = 2,
}

/// One launch of `lhip_q8_0_matvec_fused_f32`.  Inputs by slot: 0 activations (device f32, k values), 1..=count
/// the planar weights, then the norm weight (device f32, k values) if `norm`, then the residual (device f32,
/// n[0] values) if the epilogue is `Residual`.  Outputs: one device f32 vector per weight; with `SwiGlu` the single
/// weight holds (gate, up) row pairs and the output has n[0] / 2 values.
#[derive(Clone, Debug)]
pub struct FusedMatvec {
    pub n: Vec<i64>,
    pub k: i64,
    pub norm: bool,
    pub eps: f32,
    pub epilogue: Epilogue,
}

impl Operator for FusedMatvec {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        let count = self.n.len();
        assert_eq!(
            inp.len(),
            1 + count + self.norm as usize + (self.epilogue == Epilogue::Residual) as usize,
            "FusedMatvec: wrong number of inputs"
        );
        assert!(
            inp[0].1.is_contiguous() && inp[0].1.n_elements().to_usize() == Some(self.k as usize),
            "FusedMatvec: activations must be one contiguous row of K values"
        );
        let x = device(&inp[0].0, "activation");
        let weights: Vec<HipData> = (0..count).map(|i| device(&inp[1 + i].0, "weight")).collect();
        let outs: Vec<HipData> = self
            .n
            .iter()
            .map(|&n| HipData::alloc((if self.epilogue == Epilogue::SwiGlu { n / 2 } else { n }) as usize * 4))
            .collect();
        let w_ptrs: Vec<*const std::ffi::c_void> = weights.iter().map(|w| w.ptr() as *const _).collect();
        let y_ptrs: Vec<*mut f32> = outs.iter().map(|o| o.ptr() as *mut f32).collect();
        let mut at = 1 + count;
        let norm_w = self.norm.then(|| {
            at += 1;
            device(&inp[at - 1].0, "norm weight")
        });
        let residual = (self.epilogue == Epilogue::Residual).then(|| device(&inp[at].0, "residual"));
        check(
            unsafe {
                ffi::lhip_q8_0_matvec_fused_f32(
                    w_ptrs.as_ptr(),
                    y_ptrs.as_ptr(),
                    self.n.as_ptr(),
                    count as i32,
                    x.ptr() as *const f32,
                    self.k,
                    norm_w.as_ref().map_or(std::ptr::null(), |w| w.ptr() as *const f32),
                    self.eps,
                    residual.as_ref().map_or(std::ptr::null(), |r| r.ptr() as *const f32),
                    self.epilogue as i32,
                    null_mut(),
                )
            },
            "lhip_q8_0_matvec_fused_f32",
        );
        outs.into_iter().map(Tensor::new).collect()
    }
}

// ---- graph helpers ---------------------------------------------------------------------------------------------

type Use = (petgraph::graph::EdgeIndex, NodeIndex, u8, u8, ShapeTracker); // edge, consumer, input slot, output, view

fn uses(graph: &Graph, node: NodeIndex) -> Vec<Use> {
    graph
        .edges_directed(node, Direction::Outgoing)
        .filter_map(|e| e.weight().as_data().map(|(slot, out, shape)| (e.id(), e.target(), slot, out, shape)))
        .collect()
}

fn is_fake(s: &ShapeTracker, axis: usize) -> bool {
    s.fake[s.indexes[axis]]
}

fn all_fake(s: &ShapeTracker) -> bool {
    (0..s.len()).all(|i| is_fake(s, i))
}

fn elements(s: &ShapeTracker) -> Option<usize> {
    s.n_elements().to_usize()
}

/// A `Constant` entering through a fully expanded view: its value.
fn constant_operand(graph: &Graph, (src, _, view): &(NodeIndex, u8, ShapeTracker)) -> Option<f32> {
    let c = graph.try_get_op::<Constant>(*src)?;
    if !all_fake(view) {
        return None;
    }
    match &c.0 {
        ConstantValue::Float(v) => Some(*v),
        ConstantValue::Expression(e) => e.to_usize().map(|v| v as f32),
    }
}

fn retrieved(graph: &Graph, node: NodeIndex) -> bool {
    graph.to_retrieve.contains_key(&node)
}

fn only_consumer(graph: &Graph, node: NodeIndex, consumer: NodeIndex) -> bool {
    let out = uses(graph, node);
    !retrieved(graph, node) && !out.is_empty() && out.iter().all(|u| u.1 == consumer)
}

fn single_next(graph: &Graph, node: NodeIndex) -> Option<NodeIndex> {
    let out = uses(graph, node);
    (out.len() == 1 && !retrieved(graph, node)).then(|| out[0].1)
}

fn is_copy(graph: &Graph, node: NodeIndex) -> bool {
    graph.check_node_type::<HipCopyToDevice<f32>>(node) || graph.check_node_type::<HipCopyFromDevice<f32>>(node)
}

fn runs_on_device(graph: &Graph, node: NodeIndex) -> bool {
    graph.check_node_type::<QuantizedMatmul<f32>>(node)
        || graph.check_node_type::<QuantizedGather<f32>>(node)
        || graph.check_node_type::<FusedMatvec>(node)
        || graph.check_node_type::<Q8InterleaveRows>(node)
        || graph.check_node_type::<HipCopyToDevice<f32>>(node)
}

/// The node whose result a device operand is a copy of.
fn producer_of(graph: &Graph, mut node: NodeIndex) -> NodeIndex {
    while is_copy(graph, node) {
        node = graph.get_sources(node)[0].0;
    }
    node
}

/// Where to read `node`'s result on the device: the device node behind a HipCopyFromDevice, the node itself if it
/// runs on the device, an upload of the whole result that is already there, else a new one.
fn on_device(graph: &mut Graph, node: NodeIndex, keep: bool) -> (NodeIndex, u8) {
    if graph.check_node_type::<HipCopyFromDevice<f32>>(node) {
        let (src, out, _) = graph.get_sources(node)[0];
        return (src, out);
    }
    if runs_on_device(graph, node) {
        return (node, 0);
    }
    let existing = uses(graph, node)
        .into_iter()
        .find(|u| graph.check_node_type::<HipCopyToDevice<f32>>(u.1) && u.4.len() == 0)
        .map(|u| u.1);
    let up = existing
        .unwrap_or_else(|| graph.add_op(HipCopyToDevice::<f32>::default()).input(node, 0, ShapeTracker::new(())).finish());
    if keep {
        graph.no_delete.insert(up);
    }
    (up, 0)
}

fn prune_dead(graph: &mut Graph, node: NodeIndex) {
    if graph.node_weight(node).is_none()
        || graph.edges_directed(node, Direction::Outgoing).next().is_some()
        || retrieved(graph, node)
        || graph.no_delete.contains(&node)
        || graph.check_node_type::<Function>(node)
    {
        return;
    }
    let parents: Vec<NodeIndex> = graph.get_sources(node).into_iter().map(|(src, _, _)| src).collect();
    graph.graph.remove_node(node);
    for parent in parents {
        prune_dead(graph, parent);
    }
}

struct Norm {
    x: NodeIndex,
    weight: NodeIndex,
    eps: f32,
}

/// `p` as the RMS norm of a K-vector; every node of the pattern below `p` must feed the pattern only.
fn match_rms_norm(graph: &Graph, p: NodeIndex, k: usize) -> Option<Norm> {
    if !graph.check_node_type::<Mul>(p) {
        return None;
    }
    let inp = graph.get_sources(p);
    if inp.len() != 2 {
        return None;
    }
    // (normalised x) * expand(weight): the weight enters with every dimension but the last expanded
    let weight_view = |(src, _, s): &(NodeIndex, u8, ShapeTracker)| {
        let r = s.len();
        graph.check_node_type::<Function>(*src)
            && r > 0
            && s.dims()[r - 1].to_usize() == Some(k)
            && !is_fake(s, r - 1)
            && (0..r - 1).all(|i| is_fake(s, i))
    };
    let w_at = if weight_view(&inp[1]) { 1 } else if weight_view(&inp[0]) { 0 } else { return None };
    let (scaled, _, n_view) = inp[1 - w_at];
    if !graph.check_node_type::<Mul>(scaled) || !only_consumer(graph, scaled, p) || !n_view.is_contiguous() {
        return None;
    }
    let sin = graph.get_sources(scaled);
    if sin.len() != 2 {
        return None;
    }
    let factor_view = |(_, _, s): &(NodeIndex, u8, ShapeTracker)| s.len() > 0 && is_fake(s, s.len() - 1);
    let f_at = if factor_view(&sin[0]) { 0 } else if factor_view(&sin[1]) { 1 } else { return None };
    let (x_src, x_out, x_view) = sin[1 - f_at];
    if !x_view.is_contiguous() || elements(&x_view) != Some(k) {
        return None;
    }
    // upwards from the factor: Recip <- Sqrt <- Add(mean, eps) <- Mul(sum, 1/D) <- SumReduce(last) <- Mul(x, x)
    let recip = sin[f_at].0;
    if !graph.check_node_type::<Recip>(recip) || !only_consumer(graph, recip, scaled) {
        return None;
    }
    let root = graph.get_sources(recip)[0].0;
    if !graph.check_node_type::<Sqrt>(root) || !only_consumer(graph, root, recip) {
        return None;
    }
    let plus = graph.get_sources(root)[0].0;
    if !graph.check_node_type::<Add>(plus) || !only_consumer(graph, plus, root) {
        return None;
    }
    let ain = graph.get_sources(plus);
    let (eps, mean) = match (constant_operand(graph, &ain[1]), constant_operand(graph, &ain[0])) {
        (Some(eps), _) => (eps, ain[0].0),
        (None, Some(eps)) => (eps, ain[1].0),
        _ => return None,
    };
    if !graph.check_node_type::<Mul>(mean) || !only_consumer(graph, mean, plus) {
        return None;
    }
    let min = graph.get_sources(mean);
    // the divisor: `tensor / Expression` spells it Recip(expand(Constant(D))); `tensor / f32` Constant(1/D)
    let inverse_of_k = |operand: &(NodeIndex, u8, ShapeTracker)| {
        if let Some(v) = constant_operand(graph, operand) {
            return (v * k as f32 - 1.0).abs() < 1e-5;
        }
        graph.check_node_type::<Recip>(operand.0)
            && only_consumer(graph, operand.0, mean)
            && constant_operand(graph, &graph.get_sources(operand.0)[0]) == Some(k as f32)
    };
    let sum = if inverse_of_k(&min[1]) { min[0].0 } else if inverse_of_k(&min[0]) { min[1].0 } else { return None };
    let reduce_dim = graph.try_get_op::<SumReduce>(sum)?.0;
    if !only_consumer(graph, sum, mean) {
        return None;
    }
    let (square, _, sq_view) = graph.get_sources(sum)[0];
    if reduce_dim + 1 != sq_view.len() || !graph.check_node_type::<Mul>(square) || !only_consumer(graph, square, sum) {
        return None;
    }
    let qin = graph.get_sources(square);
    let same_x = |(src, out, view): &(NodeIndex, u8, ShapeTracker)| {
        *src == x_src && *out == x_out && view.is_contiguous() && elements(view) == Some(k)
    };
    if qin.len() != 2 || !same_x(&qin[0]) || !same_x(&qin[1]) {
        return None;
    }
    Some(Norm { x: x_src, weight: inp[w_at].0, eps })
}

/// `up * (gate * (1 / (1 + exp2(-gate / ln 2))))` behind the host copies `gate` and `up`: the node that holds the
/// product.
fn match_swiglu(graph: &Graph, gate: NodeIndex, up: NodeIndex) -> Option<NodeIndex> {
    if retrieved(graph, gate) || retrieved(graph, up) {
        return None;
    }
    let gate_uses = uses(graph, gate);
    if gate_uses.len() != 2 {
        return None;
    }
    // a Mul of `from` by a fully expanded Constant of the given value, in either operand order
    let scaled_by = |from: NodeIndex, value: f32, tolerance: f32| -> Option<NodeIndex> {
        uses(graph, from).into_iter().map(|u| u.1).find(|&dst| {
            if !graph.check_node_type::<Mul>(dst) {
                return false;
            }
            let inp = graph.get_sources(dst);
            let other = if inp[0].0 == from { &inp[1] } else { &inp[0] };
            constant_operand(graph, other).is_some_and(|v| (v - value).abs() <= tolerance)
        })
    };
    let neg = scaled_by(gate, -1.0, 0.0)?;
    let scaled = scaled_by(neg, 1.0 / f32::ln(2.0), 1e-6)?;
    if !only_consumer(graph, neg, scaled) {
        return None;
    }
    let e2 = single_next(graph, scaled).filter(|&n| graph.check_node_type::<Exp2>(n))?;
    let plus = single_next(graph, e2).filter(|&n| graph.check_node_type::<Add>(n))?;
    {
        let inp = graph.get_sources(plus);
        let other = if inp[0].0 == e2 { &inp[1] } else { &inp[0] };
        if constant_operand(graph, other) != Some(1.0) {
            return None;
        }
    }
    let mut sig = single_next(graph, plus).filter(|&n| graph.check_node_type::<Recip>(n))?;
    // `1. / t` is spelled 1.0 * recip(t): a Mul by Constant(1) may follow
    if let Some(times_one) = scaled_by(sig, 1.0, 0.0).filter(|&n| only_consumer(graph, sig, n)) {
        sig = times_one;
    }
    let swish = single_next(graph, sig).filter(|&n| graph.check_node_type::<Mul>(n))?;
    {
        let inp = graph.get_sources(swish);
        let other = if inp[0].0 == sig { inp[1].0 } else { inp[0].0 };
        if other != gate {
            return None;
        }
    }
    if gate_uses.iter().any(|u| u.1 != neg && u.1 != swish) {
        return None;
    }
    let out = single_next(graph, swish).filter(|&n| graph.check_node_type::<Mul>(n))?;
    if !only_consumer(graph, up, out) {
        return None;
    }
    let inp = graph.get_sources(out);
    let other = if inp[0].0 == swish { inp[1].0 } else { inp[0].0 };
    (other == up).then_some(out)
}

/// The host copy behind a quantized node, if that copy is the node's only consumer.
fn sole_host_copy(graph: &Graph, q: NodeIndex) -> Option<NodeIndex> {
    let out = uses(graph, q);
    (out.len() == 1 && !retrieved(graph, q) && graph.check_node_type::<HipCopyFromDevice<f32>>(out[0].1)).then(|| out[0].1)
}

/// Weight operand of a QuantizedMatmul: (source, output, [K, N] view, K, N).
fn weight_of(graph: &Graph, q: NodeIndex) -> (NodeIndex, u8, ShapeTracker, usize, usize) {
    let (src, out, view) = graph.get_sources(q)[1];
    let dims = view.shape_usize();
    (src, out, view, dims[dims.len() - 2], dims[dims.len() - 1])
}

/// Pass object: `(GenericCompiler::default(), HipQuantizedCompiler::<f32>::new(w), HipFusedMatvecCompiler)`.
#[derive(Debug, Default)]
pub struct HipFusedMatvecCompiler;

impl HipFusedMatvecCompiler {
    /// Consumers of host node `old` read output `out` of device node `dev` instead: device-side consumers directly,
    /// the others (and a retrieval, with the caller's handles) through one HipCopyFromDevice.
    fn replace_with_device_output<To: ToIdsMut>(graph: &mut Graph, ids: &mut To, old: NodeIndex, dev: NodeIndex, out: u8) {
        let mut down: Option<NodeIndex> = None;
        let mut host_copy = |graph: &mut Graph| {
            *down.get_or_insert_with(|| graph.add_op(HipCopyFromDevice::<f32>::default()).input(dev, out, ShapeTracker::new(())).finish())
        };
        for (edge, dst, slot, _, shape) in uses(graph, old) {
            let device_side = graph.check_node_type::<HipCopyToDevice<f32>>(dst)
                || graph.check_node_type::<FusedMatvec>(dst)
                || (graph.check_node_type::<QuantizedMatmul<f32>>(dst) && slot == 0);
            graph.remove_edge(edge);
            if device_side {
                graph.add_edge(dev, dst, Dependency::Data { input_order: slot, output_order: out, shape });
            } else {
                let copy = host_copy(graph);
                graph.add_edge(copy, dst, Dependency::Data { input_order: slot, output_order: 0, shape });
            }
        }
        if retrieved(graph, old) || graph.no_delete.contains(&old) {
            let copy = host_copy(graph);
            remap(old, copy, &mut *ids, graph);
        }
    }

    fn fuse<To: ToIdsMut>(graph: &mut Graph, ids: &mut To, producer: NodeIndex, members: Vec<NodeIndex>) {
        let k = weight_of(graph, members[0]).3;
        let norm = (graph.node_weight(producer).is_some())
            .then(|| match_rms_norm(graph, producer, k))
            .flatten()
            .filter(|_| {
                // the normalised vector must feed these projections only, or it has to be computed anyway
                let readers: Vec<NodeIndex> = members.iter().flat_map(|&q| [q, graph.get_sources(q)[0].0]).collect();
                !retrieved(graph, producer) && uses(graph, producer).iter().all(|u| readers.contains(&u.1))
            });
        let mut epilogue = Epilogue::None;
        let (mut replaced, mut residual) = (None, None); // the host node whose result the fused launch produces instead
        if members.len() == 2 {
            let (n0, n1) = (weight_of(graph, members[0]).4, weight_of(graph, members[1]).4);
            if let (Some(gate), Some(up), true) = (sole_host_copy(graph, members[0]), sole_host_copy(graph, members[1]), n0 == n1) {
                if let Some(out) = match_swiglu(graph, gate, up) {
                    epilogue = Epilogue::SwiGlu;
                    replaced = Some(out);
                } else if match_swiglu(graph, up, gate).is_some() {
                    return Self::fuse(graph, ids, producer, vec![members[1], members[0]]); // (gate, up) order
                }
            }
        } else if members.len() == 1 {
            if let Some(y) = sole_host_copy(graph, members[0]) {
                if let Some(add) = single_next(graph, y).filter(|&n| graph.check_node_type::<Add>(n)) {
                    let inp = graph.get_sources(add);
                    let other = if inp[0].0 == y { inp[1] } else { inp[0] };
                    let n = weight_of(graph, members[0]).4;
                    if other.0 != y && other.2.is_contiguous() && elements(&other.2) == Some(n) {
                        epilogue = Epilogue::Residual;
                        replaced = Some(add);
                        residual = Some(other.0);
                    }
                }
            }
        }
        if members.len() == 1 && norm.is_none() && epilogue == Epilogue::None {
            return; // nothing to gain
        }

        // inputs
        let mut n: Vec<i64> = members.iter().map(|&q| weight_of(graph, q).4 as i64).collect();
        let mut weights: Vec<(NodeIndex, u8, ShapeTracker)> = members
            .iter()
            .map(|&q| {
                let (src, out, view, _, _) = weight_of(graph, q);
                (src, out, view)
            })
            .collect();
        let (act_src, act_out, _) = graph.get_sources(members[0])[0];
        let x = match &norm {
            Some(found) => on_device(graph, found.x, false),
            None => (act_src, act_out),
        };
        if epilogue == Epilogue::SwiGlu {
            let rows = n[0] as usize;
            let both = graph
                .add_op(Q8InterleaveRows { n: rows, k })
                .input(weights[0].0, weights[0].1, weights[0].2)
                .input(weights[1].0, weights[1].1, weights[1].2)
                .finish();
            graph.no_delete.insert(both);
            let mut view = ShapeTracker::new((2 * rows, k));
            view.permute(&[1, 0]);
            weights = vec![(both, 0, view)];
            n = vec![2 * n[0]];
        }
        let feeders: Vec<NodeIndex> = members.iter().map(|&q| graph.get_sources(q)[0].0).collect();
        // (source, output, view) of every input in slot order; the builder borrows the graph, so they are found first
        let mut inputs: Vec<(NodeIndex, u8, ShapeTracker)> = vec![(x.0, x.1, ShapeTracker::new(k))];
        inputs.extend(weights.iter().copied());
        if let Some(found) = &norm {
            let (w, out) = on_device(graph, found.weight, true);
            inputs.push((w, out, ShapeTracker::new(k)));
        }
        if let Some(other) = residual {
            let (r, out) = on_device(graph, other, false);
            inputs.push((r, out, ShapeTracker::new(n[0] as usize)));
        }
        let mut node = graph.add_op(FusedMatvec {
            n: n.clone(),
            k: k as i64,
            norm: norm.is_some(),
            eps: norm.as_ref().map_or(0.0, |f| f.eps),
            epilogue,
        });
        for (src, out, view) in inputs {
            node = node.input(src, out, view);
        }
        let fused = node.finish();

        // outputs
        match replaced {
            None => {
                for (i, &q) in members.iter().enumerate() {
                    for (_, dst, slot, _, shape) in uses(graph, q) {
                        graph.add_edge(fused, dst, Dependency::Data { input_order: slot, output_order: i as u8, shape });
                    }
                    if retrieved(graph, q) || graph.no_delete.contains(&q) {
                        let down = graph.add_op(HipCopyFromDevice::<f32>::default()).input(fused, i as u8, ShapeTracker::new(())).finish();
                        remap(q, down, &mut *ids, graph);
                    }
                    graph.graph.remove_node(q);
                }
            }
            Some(host_node) => {
                // the epilogue's host nodes go from the bottom up; the projections and their host copies lose
                // their last consumer on the way
                Self::replace_with_device_output(graph, ids, host_node, fused, 0);
                prune_dead(graph, host_node);
            }
        }
        for feeder in feeders {
            prune_dead(graph, feeder);
        }
        prune_dead(graph, producer);
    }
}

impl Compiler for HipFusedMatvecCompiler {
    type Output = ();
    fn compile<To: ToIdsMut>(&self, graph: &mut Graph, mut ids: To) {
        // groups of one-row QuantizedMatmul<f32> nodes by the node that produces their activations
        let mut groups: FxHashMap<NodeIndex, Vec<NodeIndex>> = FxHashMap::default();
        let mut order: Vec<NodeIndex> = vec![];
        for q in graph.node_indices().collect::<Vec<_>>() {
            if !graph.check_node_type::<QuantizedMatmul<f32>>(q) {
                continue;
            }
            let sources = graph.get_sources(q);
            if sources.len() != 2 {
                continue;
            }
            let k = weight_of(graph, q).3;
            let (act_src, _, act_view) = sources[0];
            if !act_view.is_contiguous() || elements(&act_view) != Some(k) {
                continue; // not a single row
            }
            if k % 1024 != 0 || k > 16384 {
                continue; // lhip_q8_0_matvec_fused_f32's K
            }
            let producer = producer_of(graph, act_src);
            if !groups.contains_key(&producer) {
                order.push(producer);
            }
            groups.entry(producer).or_default().push(q);
        }
        for producer in order {
            for members in groups[&producer].chunks(4) {
                Self::fuse(graph, &mut ids, producer, members.to_vec());
            }
        }
        // an upload whose source has meanwhile become a device node only hands the buffer on: take it out
        for copy in graph.node_indices().collect::<Vec<_>>() {
            if !graph.check_node_type::<HipCopyToDevice<f32>>(copy) || graph.no_delete.contains(&copy) {
                continue;
            }
            let (src, out, _) = graph.get_sources(copy)[0];
            if !(graph.check_node_type::<FusedMatvec>(src)
                || graph.check_node_type::<QuantizedMatmul<f32>>(src)
                || graph.check_node_type::<QuantizedGather<f32>>(src))
            {
                continue;
            }
            for (_, dst, slot, _, shape) in uses(graph, copy) {
                graph.add_edge(src, dst, Dependency::Data { input_order: slot, output_order: out, shape });
            }
            graph.graph.remove_node(copy);
        }
    }
}
