//! Where with three-way broadcasting (replaces cuda/src/kernels/whereop.rs:57-101).
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::{Bool, HipType};

/// `out[i] = cond[ic] ? x[ix] : y[iy]`; strides are element strides per output dim, 0 on
/// broadcast dims.
pub fn compute<T: HipType>(
    stream: &HipStream,
    out_shape: &[usize],
    x_stride: &[usize],
    y_stride: &[usize],
    cond_stride: &[usize],
    x: &DeviceBuffer<T>,
    y: &DeviceBuffer<T>,
    cond: &DeviceBuffer<Bool>,
    out: &mut DeviceBuffer<T>,
) -> Result<()> {
    let rank = out_shape.len();
    if x_stride.len() != rank || y_stride.len() != rank || cond_stride.len() != rank {
        return Err(Error::InvalidArguments("where: shape and strides differ in rank".into()));
    }
    if out.len() != out_shape.iter().product::<usize>() {
        return Err(Error::InvalidArguments("where: output length does not match its shape".into()));
    }
    let (shape, sx, sy, sc) = (dims(out_shape)?, dims(x_stride)?, dims(y_stride)?, dims(cond_stride)?);
    check(
        unsafe {
            ffi::rmlk_hip_where(
                stream.raw(),
                T::DTYPE,
                &shape,
                &sx,
                &sy,
                &sc,
                x.as_ptr(),
                y.as_ptr(),
                cond.as_ptr(),
                out.as_mut_ptr(),
            )
        },
        "where",
    )
}
