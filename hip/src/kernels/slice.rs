//! Strided slices (replaces cuda/src/kernels/slice.rs:61-122). The bounds are the ones the
//! reference's backend has already resolved on the host (backend/slice.rs:357-463): a start and a
//! non-zero step per dim of the input, and the output shape they give.
use crate::device::{dims, dims_i64, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

pub fn compute<T: HipType>(
    stream: &HipStream,
    in_shape: &[usize],
    starts: &[i64],
    steps: &[i64],
    out_shape: &[usize],
    input: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    let rank = in_shape.len();
    if starts.len() != rank || steps.len() != rank || out_shape.len() != rank {
        return Err(Error::InvalidArguments("slice: starts, steps and shapes differ in rank".into()));
    }
    if output.len() != out_shape.iter().product::<usize>() {
        return Err(Error::InvalidArguments("slice: output length does not match its shape".into()));
    }
    let (is, st, sp, os) = (dims(in_shape)?, dims_i64(starts)?, dims_i64(steps)?, dims(out_shape)?);
    check(
        unsafe { ffi::rmlk_hip_slice(stream.raw(), T::DTYPE, &is, &st, &sp, &os, input.as_ptr(), output.as_mut_ptr()) },
        "slice",
    )
}
