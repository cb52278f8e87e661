//! Element types the kernels know, by the numbers of `rmlk_dtype` (replaces cuda/src/params.rs:4-36,
//! where the trait maps Rust types to cuBLAS enums).
use crate::ffi;

pub trait HipType: Copy + 'static {
    const DTYPE: i32;
}

macro_rules! hip_type {
    ($($t:ty => $d:expr),* $(,)?) => { $(impl HipType for $t { const DTYPE: i32 = $d; })* };
}

hip_type! {
    f32 => ffi::RMLK_FLOAT,
    f64 => ffi::RMLK_DOUBLE,
    half::f16 => ffi::RMLK_FLOAT16,
    i8 => ffi::RMLK_INT8,
    i16 => ffi::RMLK_INT16,
    i32 => ffi::RMLK_INT32,
    i64 => ffi::RMLK_INT64,
    u8 => ffi::RMLK_UINT8,
    u16 => ffi::RMLK_UINT16,
    u32 => ffi::RMLK_UINT32,
    u64 => ffi::RMLK_UINT64,
}

/// ONNX bool tensors: one byte per element.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(transparent)]
pub struct Bool(pub u8);

impl HipType for Bool {
    const DTYPE: i32 = ffi::RMLK_BOOL;
}
