//! Error type of the crate (replaces cuda/src/error.rs:7-42: `Cuda(u32)`, `Cublas(u32)` and
//! `Cudnn(u32)` collapse into `Hip(u32)`, since GEMM and softmax are this library's own kernels).
use crate::ffi;
use std::ffi::CStr;
use std::fmt::{Display, Formatter};

#[derive(Debug)]
pub enum Error {
    NonContiguousMemory(String),
    InvalidArguments(String),
    Internal(String),
    /// A kernel exists for neither this element type nor this shape ("unsupported data type").
    Unsupported(String),
    /// A `hipError_t` reported by the HIP runtime.
    Hip(u32),
}

impl Display for Error {
    fn fmt(&self, f: &mut Formatter<'_>) -> std::fmt::Result {
        write!(f, "{:?}", self)
    }
}

impl std::error::Error for Error {}

pub type Result<T> = std::result::Result<T, Error>;

/// Status of a `rmlk_hip_*` call: 0 is success, positive values are `hipError_t`, negative values
/// the library's own argument errors (`rmlk_status`).
pub fn check(status: i32, what: &str) -> Result<()> {
    if status == ffi::RMLK_OK {
        return Ok(());
    }
    if status > 0 {
        return Err(Error::Hip(status as u32));
    }
    let name = unsafe { CStr::from_ptr(ffi::rmlk_hip_status_string(status)) }
        .to_string_lossy()
        .into_owned();
    let msg = format!("{what}: {name}");
    Err(match status {
        ffi::RMLK_ERR_UNSUPPORTED => Error::Unsupported(msg),
        ffi::RMLK_ERR_WORKSPACE | ffi::RMLK_ERR_SCRATCH_LIMIT => Error::Internal(msg),
        _ => Error::InvalidArguments(msg),
    })
}
