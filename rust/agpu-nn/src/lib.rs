//! agpu-nn: the `nn` surface of async_gpu (crates/core/gpu-host/src/nn) on MI355X, as safe wrappers over the C ABI
//! of libagpu_hip.so (`agpu-sys`).  Names, argument meaning and error behaviour follow the reference, so the
//! quantized GPT-2 example (examples/std/gpt2-inference/src/main.rs:22-107) builds against this crate unchanged
//! apart from its `use` lines:
//!
//! | here | reference |
//! |---|---|
//! | `NnError`, `Result` | nn/error.rs:7-29 |
//! | `KernelRegistry` | nn/registry.rs:26-144 |
//! | `GpuTensor` | nn/tensor.rs:45-282 |
//! | `GpuArray`, `Residency` | gpu_array.rs:42-385 |
//! | `ops::*` | nn/ops/{gemm,norm,activation,reshape,attention,quantize}.rs |
//! | `Int4Linear`, `LayerNorm`, `Embedding`, `Module` | nn/layers/*.rs |
//! | `Gpt2Config`, `Int4Gpt2Model` | nn/models/gpt2.rs:20-93, 712-783, 1341-1580 |
pub mod error;
pub mod gpt2;
pub mod gpu_array;
pub mod layers;
pub mod ops;
pub mod registry;
pub mod tensor;

pub use error::{NnError, Result};
pub use gpt2::{Gpt2Config, Int4Gpt2Model};
pub use gpu_array::{GpuArray, Residency};
pub use layers::{Embedding, Int4Linear, LayerNorm, Module};
pub use registry::KernelRegistry;
pub use tensor::GpuTensor;
