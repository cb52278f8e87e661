//! Mean over a set of axes (replaces cuda/src/kernels/reduce_mean.rs:31-267; keepdims is a matter
//! of the output's shape only and stays with the caller).
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

pub fn compute<T: HipType>(
    stream: &HipStream,
    in_shape: &[usize],
    axes: &[usize],
    input: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    if axes.iter().any(|&a| a >= in_shape.len()) {
        return Err(Error::InvalidArguments("reduce_mean: axis out of range".into()));
    }
    let kept: usize =
        in_shape.iter().enumerate().filter(|(d, _)| !axes.contains(d)).map(|(_, &n)| n).product();
    if output.len() != kept {
        return Err(Error::InvalidArguments("reduce_mean: output length does not match the kept dims".into()));
    }
    let shape = dims(in_shape)?;
    let axes64: Vec<i64> = axes.iter().map(|&a| a as i64).collect();
    check(
        unsafe {
            ffi::rmlk_hip_reduce_mean(
                stream.raw(),
                T::DTYPE,
                &shape,
                axes64.as_ptr(),
                axes64.len() as i32,
                input.as_ptr(),
                output.as_mut_ptr(),
            )
        },
        "reduce_mean",
    )
}
