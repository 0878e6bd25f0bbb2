//! NnError (nn/error.rs:7-29): the C ABI's int32 return codes mapped back onto the reference's variants.
use std::fmt;

#[derive(Debug, Clone, PartialEq)]
pub enum NnError {
    /// code -1
    ShapeMismatch { expected: String, actual: String },
    /// code -2
    DimOutOfRange { dim: usize, ndim: usize },
    /// code -3
    KernelNotFound { name: String },
    /// a positive code: the hipError_t of a failed runtime call (the reference's `Cuda(DriverError)`)
    Hip { code: i32, message: String },
    /// the library's other negative codes: null pointer, unsupported shape, scratch too small, a wait inside a
    /// kernel that gave up, a second thread on one context
    Library { code: i32, message: String },
}

pub type Result<T> = std::result::Result<T, NnError>;

impl fmt::Display for NnError {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        match self {
            NnError::ShapeMismatch { expected, actual } => write!(f, "shape mismatch: expected {expected}, got {actual}"),
            NnError::DimOutOfRange { dim, ndim } => write!(f, "dimension {dim} out of range for tensor with {ndim} dims"),
            NnError::KernelNotFound { name } => write!(f, "kernel not found in registry: {name}"),
            NnError::Hip { code, message } => write!(f, "HIP error {code}: {message}"),
            NnError::Library { code, message } => write!(f, "agpu error {code}: {message}"),
        }
    }
}

impl std::error::Error for NnError {}

impl NnError {
    /// The error for a non-zero return code, with the context's message.
    pub fn from_code(code: i32, message: String) -> NnError {
        match code {
            agpu_sys::AGPU_ERR_SHAPE_MISMATCH => NnError::ShapeMismatch { expected: message, actual: String::new() },
            agpu_sys::AGPU_ERR_DIM_OUT_OF_RANGE => NnError::Library { code, message },
            agpu_sys::AGPU_ERR_KERNEL_NOT_FOUND => NnError::KernelNotFound { name: message },
            c if c > 0 => NnError::Hip { code: c, message },
            c => NnError::Library { code: c, message },
        }
    }
}
