//! Permutation of dims (replaces cuda/src/kernels/transpose.rs:38-80).
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

/// `out.shape[d] = in_shape[perm[d]]`.
pub fn compute<T: HipType>(
    stream: &HipStream,
    in_shape: &[usize],
    perm: &[usize],
    input: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    if perm.len() != in_shape.len() {
        return Err(Error::InvalidArguments("transpose: perm and shape differ in rank".into()));
    }
    if input.len() != output.len() {
        return Err(Error::InvalidArguments("transpose: input and output differ in length".into()));
    }
    let shape = dims(in_shape)?;
    let perm64: Vec<i64> = perm.iter().map(|&p| p as i64).collect();
    check(
        unsafe {
            ffi::rmlk_hip_transpose(stream.raw(), T::DTYPE, &shape, perm64.as_ptr(), input.as_ptr(), output.as_mut_ptr())
        },
        "transpose",
    )
}
