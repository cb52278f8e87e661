//! Contiguous unary maps (replaces cuda/src/kernels/unary.rs:10-42).
use crate::device::{DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(i32)]
pub enum UnaryOp {
    Sqrt = ffi::RMLK_SQRT,
    Neg = ffi::RMLK_NEG,
    Sin = ffi::RMLK_SIN,
    Cos = ffi::RMLK_COS,
    Sigmoid = ffi::RMLK_SIGMOID,
}

pub fn compute<T: HipType>(
    stream: &HipStream,
    op: UnaryOp,
    input: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    if input.len() != output.len() {
        return Err(Error::InvalidArguments("unary: input and output differ in length".into()));
    }
    check(
        unsafe {
            ffi::rmlk_hip_unary(stream.raw(), op as i32, T::DTYPE, input.len() as i64, input.as_ptr(), output.as_mut_ptr())
        },
        "unary",
    )
}
