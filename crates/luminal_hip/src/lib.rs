//! luminal_hip: HIP quantized-matmul backend for Luminal on MI355X.
//!
//! Usage, in place of `CudaQuantizedCompiler` (examples/llama/src/main.rs:75-97) and with no dense backend in
//! front of it:
//! ```ignore
//! let q_weights = luminal_hip::q8_load_hip("model.gguf", &model, &mut cx);   // uploads + repacks each Q8_0 tensor
//! cx.compile(
//!     (GenericCompiler::default(), HipQuantizedCompiler::<f32>::new(q_weights)),
//!     (&mut logits, &mut cache),
//! );
//! ```
//! Behind `GenericCompiler` the graph still holds luminal's primitive operators, which run on host `Vec<f32>`
//! (src/op.rs).  The pass therefore recognises the matmul and the gather as those primitives spell them
//! (Mul -> SumReduce over fake-expanded operands, src/hl_ops/matmul.rs:4-33 and src/hl_ops/other.rs:114-123),
//! replaces them by `QuantizedMatmul` / `QuantizedGather`, and puts `HipCopyToDevice` / `HipCopyFromDevice` nodes
//! around them so that every other node keeps seeing host vectors.  It names no type of any other backend crate.
//! A third pass, `HipFusedMatvecCompiler` (f32, one activation row: batch-1 decode), folds sibling projections, the
//! RMS norm in front of them and the residual add or SwiGLU behind them into single `FusedMatvec` launches.
//!
//! This crate has not met a compiler: there is no Rust toolchain where the backend was developed.  Its logic is
//! the one of the C++ restatement `luminal_amd/host/luminal_hip.hpp`, which is compiled and tested on the GPU
//! (tests/cpp/host_mirror_test.cpp); the C ABI it binds is include/luminal_hip.h.
pub mod ffi;
mod fusion;
mod loader;
mod quantized;

pub use fusion::{Epilogue, FusedMatvec, HipFusedMatvecCompiler, Q8InterleaveRows};
pub use loader::q8_load_hip;
pub use quantized::{HipCopyFromDevice, HipCopyToDevice, HipData, HipQuantizedCompiler, QuantizedGather, QuantizedMatmul};
