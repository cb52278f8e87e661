//! Concat along one axis: all inputs in one call (one launch for up to 8; the reference's backend copies slice
//! by slice from the host, runtime/src/providers/cuda/backend/concat.rs:28-76).
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;
use std::os::raw::c_void;

pub fn compute<T: HipType>(
    stream: &HipStream,
    in_shapes: &[&[usize]],
    inputs: &[&DeviceBuffer<T>],
    out_shape: &[usize],
    axis: usize,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    if in_shapes.len() != inputs.len() || inputs.is_empty() {
        return Err(Error::InvalidArguments("concat: one shape per input".into()));
    }
    if axis >= out_shape.len() || output.len() != out_shape.iter().product::<usize>() {
        return Err(Error::InvalidArguments("concat: axis or output length does not match the shape".into()));
    }
    let shapes: Vec<ffi::rmlk_dims> = in_shapes.iter().map(|s| dims(s)).collect::<Result<_>>()?;
    let ptrs: Vec<*const c_void> = inputs.iter().map(|b| b.as_ptr()).collect();
    let os = dims(out_shape)?;
    check(
        unsafe {
            ffi::rmlk_hip_concat_many(
                stream.raw(),
                T::DTYPE,
                inputs.len() as i32,
                shapes.as_ptr(),
                ptrs.as_ptr(),
                &os,
                axis as i32,
                output.as_mut_ptr(),
            )
        },
        "concat",
    )
}

/// One input written into its place along `axis` of the output, `axis_offset` elements in: the
/// per-input step of runtime/src/providers/cuda/backend/concat.rs:28-76 for callers that hold their
/// inputs one at a time.
pub fn compute_one<T: HipType>(
    stream: &HipStream,
    in_shape: &[usize],
    input: &DeviceBuffer<T>,
    out_shape: &[usize],
    axis: usize,
    axis_offset: usize,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    if axis >= out_shape.len() || in_shape.len() != out_shape.len() {
        return Err(Error::InvalidArguments("concat: axis or rank does not match the output".into()));
    }
    if input.len() != in_shape.iter().product::<usize>() || output.len() != out_shape.iter().product::<usize>() {
        return Err(Error::InvalidArguments("concat: buffer lengths do not match the shapes".into()));
    }
    let (is, os) = (dims(in_shape)?, dims(out_shape)?);
    check(
        unsafe {
            ffi::rmlk_hip_concat(
                stream.raw(),
                T::DTYPE,
                &is,
                &os,
                axis as i32,
                axis_offset as i64,
                input.as_ptr(),
                output.as_mut_ptr(),
            )
        },
        "concat",
    )
}
