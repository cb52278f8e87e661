//! Broadcast of a tensor to a larger shape (replaces cuda/src/kernels/expand.rs:78-248).
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

/// `in_shape` is given at the rank of `out_shape` (leading 1s added by the caller, as the
/// reference's backend does); every dim is equal to the output's or 1.
pub fn compute<T: HipType>(
    stream: &HipStream,
    in_shape: &[usize],
    out_shape: &[usize],
    input: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    if output.len() != out_shape.iter().product::<usize>() {
        return Err(Error::InvalidArguments("expand: output length does not match its shape".into()));
    }
    let (is, os) = (dims(in_shape)?, dims(out_shape)?);
    check(
        unsafe { ffi::rmlk_hip_expand(stream.raw(), T::DTYPE, &is, &os, input.as_ptr(), output.as_mut_ptr()) },
        "expand",
    )
}
