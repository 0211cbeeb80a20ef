//! luminal_hip: HIP quantized-matmul backend for Luminal on MI355X.
//!
//! Usage, in place of `CudaQuantizedCompiler` (examples/llama/src/main.rs:75-97):
//! ```ignore
//! let q_weights = loader::q8_load_hip("model.gguf", &model, &mut cx);   // uploads + repacks each Q8_0 tensor
//! cx.compile((GenericCompiler::default(), HipQuantizedCompiler::<f32>::new(q_weights)), (&mut logits, &mut cache));
//! ```
//! This crate cannot be compiled where the backend was developed (no Rust toolchain); it is the
//! maintainer-side half of the boundary declared in include/luminal_hip.h.
pub mod ffi;
mod quantized;

pub use quantized::{HipData, HipQuantizedCompiler, QuantizedGather, QuantizedMatmul};
