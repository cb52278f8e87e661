//! Gather along one axis in one launch (the reference's backend loops over `memcpy_dtod` on the
//! host, runtime/src/providers/cuda/backend/gather.rs:199-258). Negative indices count from the
//! end; an index out of range sets `*err_flag` on the device.
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

pub fn compute<T: HipType, I: HipType>(
    stream: &HipStream,
    data_shape: &[usize],
    axis: usize,
    data: &DeviceBuffer<T>,
    indices: &DeviceBuffer<I>,
    output: &mut DeviceBuffer<T>,
    err_flag: &mut DeviceBuffer<i32>,
) -> Result<()> {
    if axis >= data_shape.len() {
        return Err(Error::InvalidArguments("gather: axis out of range".into()));
    }
    let shape = dims(data_shape)?;
    check(
        unsafe {
            ffi::rmlk_hip_gather(
                stream.raw(),
                T::DTYPE,
                I::DTYPE,
                &shape,
                axis as i32,
                indices.len() as i64,
                data.as_ptr(),
                indices.as_ptr(),
                output.as_mut_ptr(),
                err_flag.as_mut_ptr().cast(),
            )
        },
        "gather",
    )
}
