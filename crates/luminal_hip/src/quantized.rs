//! Operators and compiler pass over the C ABI.
//!
//! Differences from the CUDA backend this stands in for: kernels are precompiled in the shared
//! library (nothing is compiled per weight node), Q8_0 weights live on the device in the planar form
//! produced once by `lhip_q8_0_repack`, and gather indices are uploaded by this wrapper because the
//! C entry point reads them from device memory.
use std::{any::Any, ffi::c_void, marker::PhantomData, ptr::null_mut};

use luminal::{
    op::{InputTensor, Operator},
    prelude::*,
};
use petgraph::{visit::EdgeRef, Direction};

use crate::ffi::{self, check};

/// Owned device allocation; the `Data` a tensor carries between HIP operators.
#[derive(Debug)]
pub struct HipData {
    pub ptr: *mut c_void,
    pub bytes: usize,
}

impl HipData {
    pub fn alloc(bytes: usize) -> Self {
        let mut ptr = null_mut();
        check(unsafe { ffi::lhip_malloc(&mut ptr, bytes.max(1)) }, "lhip_malloc");
        Self { ptr, bytes }
    }
    pub fn from_host<T: Copy>(host: &[T]) -> Self {
        let out = Self::alloc(std::mem::size_of_val(host));
        check(unsafe { ffi::lhip_memcpy_h2d(out.ptr, host.as_ptr() as _, out.bytes, null_mut()) }, "lhip_memcpy_h2d");
        out
    }
    pub fn to_host_f32(&self) -> Vec<f32> {
        let mut v = vec![0f32; self.bytes / 4];
        check(unsafe { ffi::lhip_memcpy_d2h(v.as_mut_ptr() as _, self.ptr, self.bytes, null_mut()) }, "lhip_memcpy_d2h");
        v
    }
    /// Raw GGUF Q8_0 blocks of an (n, k) weight -> planar device buffer.
    pub fn q8_0_from_raw(raw_blocks: &[u8], n: usize, k: usize) -> Self {
        assert_eq!(raw_blocks.len(), unsafe { ffi::lhip_q8_0_raw_nbytes(n as i64, k as i64) }, "Q8_0 size law n + n/16");
        let staged = Self::from_host(raw_blocks);
        let planar = Self::alloc(unsafe { ffi::lhip_q8_0_planar_nbytes(n as i64, k as i64) });
        check(unsafe { ffi::lhip_q8_0_repack(staged.ptr, planar.ptr, n as i64, k as i64, null_mut()) }, "lhip_q8_0_repack");
        check(unsafe { ffi::lhip_stream_sync(null_mut()) }, "lhip_stream_sync");
        planar
    }
}

impl Drop for HipData {
    fn drop(&mut self) {
        unsafe { ffi::lhip_free(self.ptr) };
    }
}

impl Data for HipData {
    fn as_any(&self) -> &dyn Any { self }
    fn as_any_mut(&mut self) -> &mut dyn Any { self }
}

fn device_ptr(t: &InputTensor) -> *mut c_void {
    t.borrowed().downcast_ref::<HipData>().expect("operand is not a HIP buffer").ptr
}

fn usize_dims(s: &ShapeTracker) -> Vec<usize> {
    s.dims().into_iter().map(|d| d.to_usize().unwrap()).collect()
}

/// (B, M, K) f32 x Q8_0 (N, K) -> (B, M, N) f32.
#[derive(Clone, Debug, Default)]
pub struct QuantizedMatmul<T>(PhantomData<T>);

impl Operator for QuantizedMatmul<f32> {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        assert!(!inp[1].1.is_contiguous(), "Weight matrix must be column-major");
        let (a, b) = (usize_dims(&inp[0].1), usize_dims(&inp[1].1));
        let rows: usize = a[..a.len() - 1].iter().product::<usize>().max(1); // batch * m
        let (k, n) = (b[b.len() - 2], b[b.len() - 1]);
        let out = HipData::alloc(rows * n * 4);
        check(
            unsafe {
                ffi::lhip_q8_0_matmul_f32(device_ptr(&inp[1].0), device_ptr(&inp[0].0) as _, out.ptr as _, rows as i64,
                                          n as i64, k as i64, null_mut())
            },
            "lhip_q8_0_matmul_f32",
        );
        vec![Tensor::new(out)]
    }
}

/// Row gather from a Q8_0 embedding table; indices arrive as host f32 like in the other backends.
#[derive(Clone, Debug)]
pub struct QuantizedGather<T> {
    pub embed_dim: usize,
    pub vocab: usize,
    _t: PhantomData<T>,
}

impl Operator for QuantizedGather<f32> {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        let idx = inp[0].0.borrowed().downcast_ref::<Vec<f32>>().expect("gather indices are host f32");
        let idx_dev = HipData::from_host(idx);
        let out = HipData::alloc(idx.len() * self.embed_dim * 4);
        check(
            unsafe {
                ffi::lhip_q8_0_gather_f32(device_ptr(&inp[1].0), idx_dev.ptr as _, out.ptr as _, idx.len() as i64,
                                          self.vocab as i64, self.embed_dim as i64, null_mut())
            },
            "lhip_q8_0_gather_f32",
        );
        check(unsafe { ffi::lhip_stream_sync(null_mut()) }, "lhip_stream_sync"); // idx_dev is freed on return
        vec![Tensor::new(out)]
    }
}

/// Rewrites the consumers of the given Q8_0 weight nodes into HIP quantized operators.
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

impl Compiler for HipQuantizedCompiler<f32> {
    type Output = ();
    fn compile<To: ToIdsMut>(&self, graph: &mut Graph, _ids: To) {
        check(unsafe { ffi::lhip_init(0) }, "lhip_init");
        for weight in downstream(&self.weights, graph) {
            let uses: Vec<_> = graph
                .edges_directed(weight, Direction::Outgoing)
                .filter_map(|e| e.weight().as_data().map(|(slot, _, _)| (e.target(), slot)))
                .collect();
            for (consumer, slot) in uses {
                assert_eq!(slot, 1, "Quantized weight {consumer:?} is the wrong input!");
                // With only GenericCompiler in front, the consumer is still the primitive Mul feeding a
                // SumReduce(2) (the pattern crates/luminal_cpu/src/matmul.rs matches) or the one-hot gather
                // pattern; `fuse_into` replaces that pair by one node and returns it.
                match crate::quantized::patterns::classify(graph, consumer) {
                    patterns::Use::Matmul(node) => *graph.node_weight_mut(node).unwrap() = Box::new(QuantizedMatmul::<f32>::default()),
                    patterns::Use::Gather { node, embed_dim, vocab } => {
                        *graph.node_weight_mut(node).unwrap() = Box::new(QuantizedGather::<f32> { embed_dim, vocab, _t: PhantomData })
                    }
                    patterns::Use::Other(op) => panic!("Quantized weight {consumer:?} feeds a node that is neither a matmul nor a gather ({op})"),
                }
            }
        }
    }
}

/// Pattern recognition the pass needs when no dense HIP compiler ran before it.
pub(crate) mod patterns {
    use luminal::{op::{Mul, SumReduce}, prelude::*};
    use petgraph::{visit::EdgeRef, Direction};

    pub enum Use {
        Matmul(NodeIndex),
        Gather { node: NodeIndex, embed_dim: usize, vocab: usize },
        Other(String),
    }

    /// `consumer` is the node that reads the weight.  A matmul is `Mul` whose only reader is `SumReduce` over the
    /// last axis; the pair is collapsed onto the `SumReduce` node, which keeps its outgoing edges.
    pub fn classify(graph: &mut Graph, consumer: NodeIndex) -> Use {
        let is_mul = graph.node_weight(consumer).map(|o| o.as_any().is::<Mul>()).unwrap_or(false);
        if is_mul {
            let readers: Vec<_> = graph.edges_directed(consumer, Direction::Outgoing).map(|e| e.target()).collect();
            if let [reduce] = readers[..] {
                let over_last = graph.node_weight(reduce).and_then(|o| o.as_any().downcast_ref::<SumReduce>().map(|s| s.0));
                if let Some(axis) = over_last {
                    let srcs = graph.get_sources(consumer);
                    if axis + 1 == srcs[0].2.len() {
                        // Re-point the Mul's inputs at the SumReduce node with the un-expanded shapes, then drop the Mul.
                        let (mut a, mut b) = (srcs[0].2, srcs[1].2);
                        a.remove_dim(a.len() - 2);
                        b.remove_dim(0);
                        b.permute(&[1, 0]);
                        graph.graph.remove_node(consumer);
                        graph.graph.add_edge(srcs[0].0, reduce, Dependency::Data { input_order: 0, output_order: srcs[0].1, shape: a });
                        graph.graph.add_edge(srcs[1].0, reduce, Dependency::Data { input_order: 1, output_order: srcs[1].1, shape: b });
                        return Use::Matmul(reduce);
                    }
                }
            }
        }
        let name = format!("{:?}", graph.node_weight(consumer));
        Use::Other(name)
    }
}
