//! Operators and compiler pass over the C ABI.
//!
//! Differences from the CUDA backend this stands in for: kernels are precompiled in the shared library (nothing is
//! compiled per weight node), Q8_0 weights live on the device in the planar form produced once by
//! `lhip_q8_0_repack`, the pass matches luminal's primitive operators rather than a dense backend's matmul nodes,
//! and it brings its own host <-> device copy nodes.  All work goes to the default stream in program order, so an
//! operator returns without waiting for its kernel; the only waits are inside the copies (`lhip_memcpy_*` return
//! when the copy has landed).
use std::{any::Any, ffi::c_void, marker::PhantomData, ptr::null_mut, sync::Arc};

use half::f16;

use luminal::{
    op::{Constant, Function, InputTensor, Mul, Operator, SumReduce},
    prelude::*,
};
use petgraph::{visit::EdgeRef, Direction};
use rustc_hash::FxHashSet;

use crate::ffi::{self, check};

/// One device allocation, freed when its last holder lets go.
#[derive(Debug)]
struct HipBuffer {
    ptr: *mut c_void,
    bytes: usize,
}

impl Drop for HipBuffer {
    fn drop(&mut self) {
        unsafe { ffi::lhip_free(self.ptr) };
    }
}

/// The `Data` a tensor carries between HIP operators.  Operators never write into a buffer they received, so a
/// clone (the `Data` trait asks for one) shares the allocation instead of copying it.
#[derive(Clone, Debug)]
pub struct HipData(Arc<HipBuffer>);

impl HipData {
    pub fn alloc(bytes: usize) -> Self {
        let mut ptr = null_mut();
        check(unsafe { ffi::lhip_malloc(&mut ptr, bytes.max(1)) }, "lhip_malloc");
        Self(Arc::new(HipBuffer { ptr, bytes }))
    }
    pub fn ptr(&self) -> *mut c_void {
        self.0.ptr
    }
    pub fn bytes(&self) -> usize {
        self.0.bytes
    }
    pub fn from_host<E: Copy>(host: &[E]) -> Self {
        let out = Self::alloc(std::mem::size_of_val(host));
        check(unsafe { ffi::lhip_memcpy_h2d(out.ptr(), host.as_ptr() as _, std::mem::size_of_val(host), null_mut()) }, "lhip_memcpy_h2d");
        out
    }
    pub fn to_host<E: Copy + Default>(&self) -> Vec<E> {
        let mut v = vec![E::default(); self.bytes() / std::mem::size_of::<E>()];
        check(unsafe { ffi::lhip_memcpy_d2h(v.as_mut_ptr() as _, self.ptr(), std::mem::size_of_val(&v[..]), null_mut()) }, "lhip_memcpy_d2h");
        v
    }
    /// Raw GGUF Q8_0 blocks (34 bytes per 32 weights, in file order) -> planar device buffer.  The planar form puts
    /// all quants before all scales and so depends on the number of blocks only, not on the tensor's (n, k).
    pub fn q8_0_from_raw(raw_blocks: &[u8], n_elements: usize) -> Self {
        assert_eq!(n_elements % 32, 0, "Q8_0 tensors hold whole blocks of 32");
        let (n, k) = ((n_elements / 32) as i64, 32i64);
        assert_eq!(raw_blocks.len(), unsafe { ffi::lhip_q8_0_raw_nbytes(n, k) }, "Q8_0 size law n + n/16");
        let staged = Self::from_host(raw_blocks);
        let planar = Self::alloc(unsafe { ffi::lhip_q8_0_planar_nbytes(n, k) });
        check(unsafe { ffi::lhip_q8_0_repack(staged.ptr(), planar.ptr(), n, k, null_mut()) }, "lhip_q8_0_repack");
        // `staged` is freed on return; the free waits for the repack, which was queued before it
        planar
    }
}

impl Data for HipData {
    fn as_any(&self) -> &dyn Any {
        self
    }
    fn as_any_mut(&mut self) -> &mut dyn Any {
        self
    }
}

fn device(t: &InputTensor, what: &str) -> HipData {
    t.borrowed()
        .downcast_ref::<HipData>()
        .unwrap_or_else(|| panic!("{what} is not a HIP buffer (a copy node is missing in front of this operator)"))
        .clone()
}

fn is_fake(s: &ShapeTracker, axis: usize) -> bool {
    s.fake[s.indexes[axis]]
}

/// The activation types the operators exist for: what the C ABI calls the f32 and the f16 entry points.
pub trait HipFloat: 'static + Copy + Default + std::fmt::Debug {
    fn from_f32(v: f32) -> Self;
    fn to_f32(self) -> f32;
    /// # Safety
    /// plain FFI: device pointers of the sizes the C header states
    unsafe fn matmul(w: *const c_void, x: *const c_void, y: *mut c_void, m: i64, n: i64, k: i64) -> ffi::Status;
    /// # Safety
    /// as `matmul`
    unsafe fn gather(w: *const c_void, idx: *const f32, out: *mut c_void, n_idx: i64, n: i64, k: i64) -> ffi::Status;
}

impl HipFloat for f32 {
    fn from_f32(v: f32) -> Self {
        v
    }
    fn to_f32(self) -> f32 {
        self
    }
    unsafe fn matmul(w: *const c_void, x: *const c_void, y: *mut c_void, m: i64, n: i64, k: i64) -> ffi::Status {
        ffi::lhip_q8_0_matmul_f32(w, x as _, y as _, m, n, k, null_mut())
    }
    unsafe fn gather(w: *const c_void, idx: *const f32, out: *mut c_void, n_idx: i64, n: i64, k: i64) -> ffi::Status {
        ffi::lhip_q8_0_gather_f32(w, idx, out as _, n_idx, n, k, null_mut())
    }
}

impl HipFloat for f16 {
    fn from_f32(v: f32) -> Self {
        f16::from_f32(v)
    }
    fn to_f32(self) -> f32 {
        f16::to_f32(self)
    }
    unsafe fn matmul(w: *const c_void, x: *const c_void, y: *mut c_void, m: i64, n: i64, k: i64) -> ffi::Status {
        ffi::lhip_q8_0_matmul_f16(w, x, y, m, n, k, null_mut())
    }
    unsafe fn gather(w: *const c_void, idx: *const f32, out: *mut c_void, n_idx: i64, n: i64, k: i64) -> ffi::Status {
        ffi::lhip_q8_0_gather_f16(w, idx, out, n_idx, n, k, null_mut())
    }
}

/// (.., M, K) activations x Q8_0 (N, K) weight -> (.., M, N), both operands on the device; sums are f32 inside the
/// kernel for either `T`.  Stands in for crates/luminal_cuda/src/quantized.rs:16-149.
#[derive(Clone, Debug, Default)]
pub struct QuantizedMatmul<T>(PhantomData<T>);

impl<T: HipFloat> Operator for QuantizedMatmul<T> {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        // the weight storage is (N, K) row-major and reaches this node as the [K, N] view of it (quantized.rs:99-102)
        assert!(!inp[1].1.is_contiguous(), "Weight matrix must be column-major");
        assert!(inp[0].1.is_contiguous(), "Activations must be contiguous");
        let (a, b) = (inp[0].1.shape_usize(), inp[1].1.shape_usize());
        let rows: usize = a[..a.len() - 1].iter().product::<usize>().max(1); // batch * m
        let (k, n) = (b[b.len() - 2], b[b.len() - 1]);
        assert_eq!(a[a.len() - 1], k, "inner dimensions differ");
        let (x, w) = (device(&inp[0].0, "activation"), device(&inp[1].0, "weight"));
        let out = HipData::alloc(rows * n * std::mem::size_of::<T>());
        check(unsafe { T::matmul(w.ptr(), x.ptr(), out.ptr(), rows as i64, n as i64, k as i64) }, "lhip_q8_0_matmul");
        vec![Tensor::new(out)]
    }
}

/// Row gather from a Q8_0 embedding table (crates/luminal_cuda/src/quantized.rs:151-236).  The indices are the
/// host f32 vector the graph input holds; their device copy is kept until the next call, so the kernel that reads
/// it is never waited for here.
#[derive(Clone, Debug)]
pub struct QuantizedGather<T> {
    pub embed_dim: usize,
    staged: Option<HipData>,
    _t: PhantomData<T>,
}

impl<T> QuantizedGather<T> {
    pub fn new(embed_dim: usize) -> Self {
        Self { embed_dim, staged: None, _t: PhantomData }
    }
}

impl<T: HipFloat> Operator for QuantizedGather<T> {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        let idx_dev = {
            let any = inp[0].0.borrowed();
            match any.downcast_ref::<Vec<f32>>() {
                Some(host) => HipData::from_host(host),
                None => any.downcast_ref::<HipData>().expect("gather indices are neither host f32 nor a HIP buffer").clone(),
            }
        };
        let n_idx = inp[0].1.shape_usize().iter().product::<usize>().max(1);
        let vocab = inp[1].1.shape_usize().iter().product::<usize>() / self.embed_dim;
        let table = device(&inp[1].0, "embedding table");
        let out = HipData::alloc(n_idx * self.embed_dim * std::mem::size_of::<T>());
        check(
            unsafe { T::gather(table.ptr(), idx_dev.ptr() as _, out.ptr(), n_idx as i64, vocab as i64, self.embed_dim as i64) },
            "lhip_q8_0_gather",
        );
        self.staged = Some(idx_dev);
        vec![Tensor::new(out)]
    }
}

/// Host `Vec<f32>` -> device buffer of `T` (crates/luminal_cuda/src/prim.rs:26-62 for this backend).  A tensor that
/// already is a HIP buffer passes through.
#[derive(Clone, Debug, Default)]
pub struct HipCopyToDevice<T>(PhantomData<T>);

impl<T: HipFloat> Operator for HipCopyToDevice<T> {
    fn process(&mut self, mut inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        if inp[0].0.borrowed().is::<HipData>() {
            return vec![inp.pop().unwrap().0.cloned()];
        }
        let any = inp[0].0.borrowed();
        let host = any.downcast_ref::<Vec<f32>>().expect("HipCopyToDevice takes a host Vec<f32>");
        let converted: Vec<T> = host.iter().copied().map(T::from_f32).collect();
        vec![Tensor::new(HipData::from_host(&converted))]
    }
}

/// Device buffer of `T` -> host `Vec<f32>` (crates/luminal_cuda/src/prim.rs:64-96).  The copy is queued behind
/// the kernels that produce the buffer and returns when it has landed: this is where the host waits.
#[derive(Clone, Debug, Default)]
pub struct HipCopyFromDevice<T>(PhantomData<T>);

impl<T: HipFloat> Operator for HipCopyFromDevice<T> {
    fn process(&mut self, mut inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        if inp[0].0.borrowed().is::<Vec<f32>>() {
            return vec![inp.pop().unwrap().0.cloned()];
        }
        let dev = device(&inp[0].0, "HipCopyFromDevice input");
        let host: Vec<f32> = dev.to_host::<T>().into_iter().map(T::to_f32).collect();
        vec![Tensor::new(host)]
    }
}

/// Rewrites the consumers of the given Q8_0 weight nodes into the HIP quantized operators, and puts copy nodes
/// between them and the host operators around them.
///
/// Stands in for crates/luminal_cuda/src/quantized.rs:238-275.  That pass runs behind the dense CUDA backend and
/// swaps `Matmul<T>` / `CudaGather<T>` nodes; this one runs on the primitive graph, where
///   * a matmul (src/hl_ops/matmul.rs:4-33) is Mul -> SumReduce(r - 1) over activations [.., M, N(fake), K] and the
///     weight [..(fake), M(fake), N, K], the weight storage being (N, K) row-major;
///   * a gather (src/hl_ops/other.rs:114-123) is Mul -> SumReduce(1) over a one-hot mask [B, V, D(fake)] and the
///     table [B(fake), V, D]; the indices are found above the mask as the operand that is not built from constants
///     and was expanded over the vocabulary, [B, V(fake)].
/// The panics for a weight in the wrong slot, or feeding anything else, carry the CUDA pass's wording.
#[derive(Debug, Default)]
pub struct HipQuantizedCompiler<T> {
    weights: Vec<NodeIndex>,
    _t: PhantomData<T>,
}

impl<T> HipQuantizedCompiler<T> {
    pub fn new<W: ToIds>(weights: W) -> Self {
        Self { weights: weights.to_ids(), _t: PhantomData }
    }
}

/// Data edges leaving `node`: (edge, target, input slot, shape on the edge).
fn data_uses(graph: &Graph, node: NodeIndex) -> Vec<(petgraph::graph::EdgeIndex, NodeIndex, u8, ShapeTracker)> {
    graph
        .edges_directed(node, Direction::Outgoing)
        .filter_map(|e| e.weight().as_data().map(|(slot, _, shape)| (e.id(), e.target(), slot, shape)))
        .collect()
}

fn on_device<T: HipFloat>(graph: &Graph, node: NodeIndex) -> bool {
    graph.check_node_type::<QuantizedMatmul<T>>(node)
        || graph.check_node_type::<QuantizedGather<T>>(node)
        || graph.check_node_type::<HipCopyToDevice<T>>(node)
}

/// True when `node` is computed from constants alone (the arange of the one-hot mask: a constant and a cumulative
/// sum, src/hl_ops/other.rs:63-71).  Graph inputs (`Function`) are not constants.
fn constant_only(graph: &Graph, node: NodeIndex) -> bool {
    if graph.check_node_type::<Constant>(node) {
        return true;
    }
    let sources = graph.get_sources(node);
    !sources.is_empty() && sources.iter().all(|(src, _, _)| constant_only(graph, *src))
}

/// Above the one-hot mask: the edge that carries the indices, expanded over the vocabulary as [B, V(fake)].
fn find_indices(graph: &Graph, from: NodeIndex, batch: Expression, vocab: Expression) -> Option<(NodeIndex, u8, ShapeTracker)> {
    let (mut stack, mut seen) = (vec![from], FxHashSet::default());
    let mut found: Option<(NodeIndex, u8, ShapeTracker)> = None;
    while let Some(node) = stack.pop() {
        if !seen.insert(node) {
            continue;
        }
        for (src, out, shape) in graph.get_sources(node) {
            if constant_only(graph, src) {
                continue;
            }
            let dims = shape.dims();
            if dims.len() == 2 && dims[0] == batch && dims[1] == vocab && is_fake(&shape, 1) && !is_fake(&shape, 0) {
                if found.is_some_and(|(prev, _, _)| prev != src) {
                    return None; // two candidates: not the gather pattern
                }
                found = Some((src, out, shape));
            } else {
                stack.push(src);
            }
        }
    }
    found
}

/// Removes nodes that have lost their last consumer (the one-hot subgraph of a gather), walking upwards.
fn prune_dead(graph: &mut Graph, node: NodeIndex) {
    if graph.node_weight(node).is_none()
        || graph.edges_directed(node, Direction::Outgoing).next().is_some()
        || graph.to_retrieve.contains_key(&node)
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

impl<T: HipFloat> HipQuantizedCompiler<T> {
    /// The Mul that consumes a weight, with the SumReduce behind it, as a matmul or a gather: the new node, or
    /// None when the shapes spell neither.
    fn rewrite_mul<To: ToIdsMut>(graph: &mut Graph, ids: &mut To, weight: NodeIndex, w_out: u8, mul: NodeIndex, w: ShapeTracker) -> Option<NodeIndex> {
        let outs = data_uses(graph, mul);
        if outs.len() != 1 {
            return None;
        }
        let red = outs[0].1;
        let reduce_dim = graph.try_get_op::<SumReduce>(red)?.0;
        let sources = graph.get_sources(mul);
        if sources.len() != 2 {
            return None;
        }
        let (a_src, a_out, a) = sources[0];
        let r = w.len();
        if a.len() != r || a.dims() != w.dims() || r < 3 {
            return None;
        }
        let w_lead_fake = (0..r - 2).all(|i| is_fake(&w, i));
        let a_lead_real = (0..r - 2).all(|i| !is_fake(&a, i));
        let made = if reduce_dim == r - 1
            && w_lead_fake
            && a_lead_real
            && is_fake(&a, r - 2)
            && !is_fake(&a, r - 1)
            && !is_fake(&w, r - 2)
            && !is_fake(&w, r - 1)
        {
            // as crates/luminal_cpu/src/matmul.rs:37-41: drop the fake dimensions, swap the weight's last two
            let (mut a_view, mut w_view) = (a, w);
            a_view.remove_dim(r - 2);
            for _ in 0..r - 2 {
                w_view.remove_dim(0);
            }
            w_view.permute(&[1, 0]);
            graph.add_op(QuantizedMatmul::<T>::default()).input(a_src, a_out, a_view).input(weight, w_out, w_view).finish()
        } else if r == 3
            && reduce_dim == 1
            && is_fake(&w, 0)
            && !is_fake(&w, 1)
            && !is_fake(&w, 2)
            && is_fake(&a, 2)
            && !is_fake(&a, 0)
            && !is_fake(&a, 1)
        {
            let dims = w.dims();
            let (idx_src, idx_out, mut idx_view) = find_indices(graph, a_src, dims[0], dims[1])?;
            idx_view.remove_dim(1);
            let mut table_view = w;
            table_view.remove_dim(0);
            let embed_dim = dims[2].to_usize().expect("the embedding width is a known number");
            graph.add_op(QuantizedGather::<T>::new(embed_dim)).input(idx_src, idx_out, idx_view).input(weight, w_out, table_view).finish()
        } else {
            return None;
        };
        // the consumers of the SumReduce now read the new node; Mul and SumReduce go, and what only fed them with it
        move_outgoing_edge(red, made, &mut graph.graph);
        remap(red, made, &mut *ids, graph);
        graph.graph.remove_node(red);
        graph.graph.remove_node(mul);
        prune_dead(graph, a_src);
        Some(made)
    }

    /// Copy nodes around a quantized node: a host producer of a matmul's activations is read through a
    /// HipCopyToDevice; every consumer that is not itself a device node reads through one HipCopyFromDevice, and a
    /// retrieved result is retrieved from that copy (as crates/luminal_cuda/src/prim.rs:687-767 does around host
    /// Function nodes).
    fn insert_copies<To: ToIdsMut>(graph: &mut Graph, ids: &mut To, q: NodeIndex) {
        if graph.check_node_type::<QuantizedMatmul<T>>(q) {
            let (act_src, act_out, act_shape) = graph.get_sources(q)[0];
            if !on_device::<T>(graph, act_src) {
                // the copy takes the producer's whole result; the view stays on the edge into the matmul
                let up = graph.add_op(HipCopyToDevice::<T>::default()).input(act_src, act_out, ShapeTracker::new(())).finish();
                let old = graph
                    .edges_directed(q, Direction::Incoming)
                    .find(|e| e.weight().as_data().is_some_and(|(slot, _, _)| slot == 0))
                    .map(|e| e.id())
                    .unwrap();
                graph.remove_edge(old);
                graph.add_edge(up, q, Dependency::Data { input_order: 0, output_order: 0, shape: act_shape });
            }
        }
        let host_uses: Vec<_> = data_uses(graph, q)
            .into_iter()
            .filter(|(_, dst, _, _)| !on_device::<T>(graph, *dst) && !graph.check_node_type::<HipCopyFromDevice<T>>(*dst))
            .collect();
        let retrieved = graph.to_retrieve.get(&q).copied();
        if host_uses.is_empty() && retrieved.is_none() {
            return;
        }
        let down = graph.add_op(HipCopyFromDevice::<T>::default()).input(q, 0, ShapeTracker::new(())).finish();
        for (edge, dst, slot, shape) in host_uses {
            graph.remove_edge(edge);
            graph.add_edge(down, dst, Dependency::Data { input_order: slot, output_order: 0, shape });
        }
        if retrieved.is_some() {
            // to_retrieve, no_delete and the caller's handles move from the device node to the host copy
            remap(q, down, &mut *ids, graph);
        }
    }
}

impl<T: HipFloat> Compiler for HipQuantizedCompiler<T> {
    type Output = ();
    fn compile<To: ToIdsMut>(&self, graph: &mut Graph, mut ids: To) {
        check(unsafe { ffi::lhip_init(0) }, "lhip_init");
        let mut quantized = vec![];
        for weight in downstream(&self.weights, graph) {
            for (_, target, slot, shape) in data_uses(graph, weight) {
                let w_out = graph
                    .edges_connecting(weight, target)
                    .find_map(|e| e.weight().as_data().filter(|(s, _, _)| *s == slot).map(|(_, out, _)| out))
                    .unwrap();
                assert_eq!(slot, 1, "Quantized weight {target:?} is the wrong input!");
                let made = if graph.check_node_type::<Mul>(target) {
                    Self::rewrite_mul(graph, &mut ids, weight, w_out, target, shape)
                } else {
                    None
                };
                match made {
                    Some(node) => quantized.push(node),
                    None => {
                        let op = graph.node_weight(target).unwrap();
                        panic!("Quantized weight {target:?} is an input to a node that isn't a matmul or gather ({op:?})");
                    }
                }
            }
        }
        for q in quantized {
            Self::insert_copies(graph, &mut ids, q);
        }
    }
}
