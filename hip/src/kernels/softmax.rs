//! Softmax over one axis (replaces cuda/src/kernels/softmax.rs:5-37, cudnnSoftmaxForward in
//! accurate mode: the maximum is subtracted first).
use crate::device::{DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

/// `x_shape` is split at `axis` the way the reference's backend builds its 4-D descriptor:
/// `outer` = product of the dims before it, `inner` = product of the dims after it.
pub fn compute<T: HipType>(
    stream: &HipStream,
    x_data: &DeviceBuffer<T>,
    x_shape: &[usize],
    axis: usize,
    y_data: &mut DeviceBuffer<T>,
) -> Result<()> {
    if axis >= x_shape.len() {
        return Err(Error::InvalidArguments("softmax: axis out of range".into()));
    }
    let outer: usize = x_shape[..axis].iter().product();
    let inner: usize = x_shape[axis + 1..].iter().product();
    if x_data.len() != outer * x_shape[axis] * inner || y_data.len() != x_data.len() {
        return Err(Error::InvalidArguments("softmax: buffer lengths do not match the shape".into()));
    }
    check(
        unsafe {
            ffi::rmlk_hip_softmax(
                stream.raw(),
                T::DTYPE,
                outer as i64,
                x_shape[axis] as i64,
                inner as i64,
                x_data.as_ptr(),
                y_data.as_mut_ptr(),
            )
        },
        "softmax",
    )
}
