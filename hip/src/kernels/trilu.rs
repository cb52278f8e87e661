//! Upper / lower triangle of the last two dims (replaces cuda/src/kernels/trilu.rs:80-197; the
//! output needs no zero fill beforehand).
use crate::device::{DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

pub fn compute<T: HipType>(
    stream: &HipStream,
    shape: &[usize],
    upper: bool,
    k: i64,
    input: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
) -> Result<()> {
    if shape.len() < 2 {
        return Err(Error::InvalidArguments("trilu: rank below 2".into()));
    }
    let (rows, cols) = (shape[shape.len() - 2], shape[shape.len() - 1]);
    let batch: usize = shape[..shape.len() - 2].iter().product();
    if input.len() != batch * rows * cols || output.len() != input.len() {
        return Err(Error::InvalidArguments("trilu: buffer lengths do not match the shape".into()));
    }
    check(
        unsafe {
            ffi::rmlk_hip_trilu(
                stream.raw(),
                T::DTYPE,
                batch as i64,
                rows as i64,
                cols as i64,
                upper as i32,
                k,
                input.as_ptr(),
                output.as_mut_ptr(),
            )
        },
        "trilu",
    )
}
