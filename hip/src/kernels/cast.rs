//! Element type conversion (replaces cuda/src/kernels/cast.rs: one entry point instead of a kernel
//! name per (source, destination) pair).
use crate::device::{DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

pub fn compute<S: HipType, D: HipType>(
    stream: &HipStream,
    input: &DeviceBuffer<S>,
    output: &mut DeviceBuffer<D>,
) -> Result<()> {
    if input.len() != output.len() {
        return Err(Error::InvalidArguments("cast: input and output differ in length".into()));
    }
    check(
        unsafe {
            ffi::rmlk_hip_cast(stream.raw(), S::DTYPE, D::DTYPE, input.len() as i64, input.as_ptr(), output.as_mut_ptr())
        },
        "cast",
    )
}
