//! Operators and compiler pass over the C ABI.
//!
//! Differences from the CUDA backend this stands in for: kernels are precompiled in the shared
//! library (nothing is compiled per weight node), Q8_0 weights live on the device in the planar form
//! produced once by `lhip_q8_0_repack`, and gather indices are uploaded by this wrapper because the
//! C entry point reads them from device memory.
use std::{any::Any, ffi::c_void, marker::PhantomData, ptr::null_mut};

use half::f16;

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

/// Activation operand: already on the device, or a host vector that is uploaded for this call.
enum Activation<'a> {
    Device(&'a HipData),
    Staged(HipData),
}

impl Activation<'_> {
    fn of(t: &InputTensor) -> Activation<'_> {
        let any = t.borrowed();
        if let Some(d) = any.downcast_ref::<HipData>() {
            Activation::Device(d)
        } else {
            Activation::Staged(HipData::from_host(any.downcast_ref::<Vec<f32>>().expect("activation is neither HipData nor Vec<f32>")))
        }
    }
    fn ptr(&self) -> *const f32 {
        (match self { Activation::Device(d) => d.ptr, Activation::Staged(d) => d.ptr }) as _
    }
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
        let x = Activation::of(&inp[0].0);
        check(
            unsafe {
                ffi::lhip_q8_0_matmul_f32(device_ptr(&inp[1].0), x.ptr(), out.ptr as _, rows as i64, n as i64, k as i64, null_mut())
            },
            "lhip_q8_0_matmul_f32",
        );
        check(unsafe { ffi::lhip_stream_sync(null_mut()) }, "lhip_stream_sync"); // a staged activation is freed on return
        vec![Tensor::new(out)]
    }
}

/// T = f16 (the type luminal's llama example runs in on CUDA): the activation is a device buffer of f16 — there is
/// no host f16 producer in this pipeline — and the output is f16; sums are f32 inside the kernel.
impl Operator for QuantizedMatmul<f16> {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        assert!(!inp[1].1.is_contiguous(), "Weight matrix must be column-major");
        let (a, b) = (usize_dims(&inp[0].1), usize_dims(&inp[1].1));
        let rows: usize = a[..a.len() - 1].iter().product::<usize>().max(1);
        let (k, n) = (b[b.len() - 2], b[b.len() - 1]);
        let out = HipData::alloc(rows * n * 2);
        check(
            unsafe {
                ffi::lhip_q8_0_matmul_f16(device_ptr(&inp[1].0), device_ptr(&inp[0].0), out.ptr, rows as i64, n as i64, k as i64, null_mut())
            },
            "lhip_q8_0_matmul_f16",
        );
        vec![Tensor::new(out)]
    }
}

/// Row gather from a Q8_0 embedding table; indices arrive as host f32 like in the other backends.
#[derive(Clone, Debug)]
pub struct QuantizedGather<T> {
    pub embed_dim: usize,
    _t: PhantomData<T>,
}

impl Operator for QuantizedGather<f32> {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        let idx = inp[0].0.borrowed().downcast_ref::<Vec<f32>>().expect("gather indices are host f32");
        let vocab = inp[1].1.dims().into_iter().map(|d| d.to_usize().unwrap()).product::<usize>() / self.embed_dim;
        let idx_dev = HipData::from_host(idx);
        let out = HipData::alloc(idx.len() * self.embed_dim * 4);
        check(
            unsafe {
                ffi::lhip_q8_0_gather_f32(device_ptr(&inp[1].0), idx_dev.ptr as _, out.ptr as _, idx.len() as i64,
                                          vocab as i64, self.embed_dim as i64, null_mut())
            },
            "lhip_q8_0_gather_f32",
        );
        check(unsafe { ffi::lhip_stream_sync(null_mut()) }, "lhip_stream_sync"); // idx_dev is freed on return
        vec![Tensor::new(out)]
    }
}

impl Operator for QuantizedGather<f16> {
    fn process(&mut self, inp: Vec<(InputTensor, ShapeTracker)>) -> Vec<Tensor> {
        let idx = inp[0].0.borrowed().downcast_ref::<Vec<f32>>().expect("gather indices are host f32");
        let vocab = inp[1].1.dims().into_iter().map(|d| d.to_usize().unwrap()).product::<usize>() / self.embed_dim;
        let idx_dev = HipData::from_host(idx);
        let out = HipData::alloc(idx.len() * self.embed_dim * 2);
        check(
            unsafe {
                ffi::lhip_q8_0_gather_f16(device_ptr(&inp[1].0), idx_dev.ptr as _, out.ptr, idx.len() as i64,
                                          vocab as i64, self.embed_dim as i64, null_mut())
            },
            "lhip_q8_0_gather_f16",
        );
        check(unsafe { ffi::lhip_stream_sync(null_mut()) }, "lhip_stream_sync"); // idx_dev is freed on return
        vec![Tensor::new(out)]
    }
}

/// Rewrites the consumers of the given Q8_0 weight nodes into HIP quantized operators.
///
/// Runs after the CPU backend's pattern passes (`luminal_cpu::MatMulCompiler`, `GatherCompiler`), which turn
/// Mul -> SumReduce and the one-hot lookup into `MatMul2D` / `BatchedMatMul2D` / `Gather` nodes; those are the nodes
/// replaced here, as the CUDA pass replaces `Matmul<T>` / `CudaGather<T>` (crates/luminal_cuda/src/quantized.rs:244-272).
/// Activations entering and leaving the quantized nodes are host `Vec<f32>` in that pipeline, so the operators below
/// accept either a `HipData` or a host vector as the activation operand and always return `HipData`; a graph that
/// keeps activations on the device needs `HipData`-aware neighbours (copy nodes or dense HIP operators).
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

/// The activation types the pass can emit operators for.
pub trait HipActivation: 'static + Sized {
    fn matmul() -> Box<dyn Operator>;
    fn gather(embed_dim: usize) -> Box<dyn Operator>;
}
impl HipActivation for f32 {
    fn matmul() -> Box<dyn Operator> { Box::new(QuantizedMatmul::<f32>::default()) }
    fn gather(embed_dim: usize) -> Box<dyn Operator> { Box::new(QuantizedGather::<f32> { embed_dim, _t: PhantomData }) }
}
impl HipActivation for f16 {
    fn matmul() -> Box<dyn Operator> { Box::new(QuantizedMatmul::<f16>::default()) }
    fn gather(embed_dim: usize) -> Box<dyn Operator> { Box::new(QuantizedGather::<f16> { embed_dim, _t: PhantomData }) }
}

impl<T: HipActivation> Compiler for HipQuantizedCompiler<T> {
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
                let op = graph.node_weight_mut(consumer).unwrap();
                if let Some(g) = op.as_any().downcast_ref::<luminal_cpu::Gather>() {
                    *op = T::gather(g.embed_dim);
                } else if op.as_any().is::<luminal_cpu::MatMul2D>() || op.as_any().is::<luminal_cpu::BatchedMatMul2D>() {
                    *op = T::matmul();
                } else {
                    panic!("Quantized weight {consumer:?} is an input to a node that isn't a matmul or gather ({op:?})");
                }
            }
        }
    }
}
