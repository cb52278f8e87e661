//! Constant fill and arithmetic sequences written on the device. The reference's ConstantOfShape and
//! Range backends build a host vector and upload it
//! (runtime/src/providers/cuda/backend/constant_of_shape.rs:59-62, range.rs:103-109,140-151); here the
//! scalars travel as kernel arguments.
use crate::device::{DeviceBuffer, HipStream};
use crate::error::{check, Result};
use crate::ffi;
use crate::params::HipType;

/// Every element of `output` becomes `value`.
pub fn fill<T: HipType>(stream: &HipStream, value: T, output: &mut DeviceBuffer<T>) -> Result<()> {
    check(
        unsafe {
            ffi::rmlk_hip_fill(
                stream.raw(),
                T::DTYPE,
                output.len() as i64,
                (&value as *const T).cast(),
                output.as_mut_ptr(),
            )
        },
        "fill",
    )
}

/// `output[i] = start + i * delta` (f32, f64, i32, i64).
pub fn range<T: HipType>(stream: &HipStream, start: T, delta: T, output: &mut DeviceBuffer<T>) -> Result<()> {
    check(
        unsafe {
            ffi::rmlk_hip_range(
                stream.raw(),
                T::DTYPE,
                output.len() as i64,
                (&start as *const T).cast(),
                (&delta as *const T).cast(),
                output.as_mut_ptr(),
            )
        },
        "range",
    )
}

/// Up to 256 bytes of host values written to the start of `output` as kernel arguments (the host
/// vector + upload of runtime/src/providers/cuda/backend/shape.rs:67-72 for tiny tensors).
pub fn write_small<T: HipType>(stream: &HipStream, values: &[T], output: &mut DeviceBuffer<T>) -> Result<()> {
    let bytes = std::mem::size_of_val(values);
    if values.len() > output.len() || bytes > 256 {
        return Err(crate::Error::InvalidArguments("write_small: at most 256 bytes, within the output".into()));
    }
    check(
        unsafe { ffi::rmlk_hip_write_small(stream.raw(), output.as_mut_ptr(), values.as_ptr().cast(), bytes) },
        "write_small",
    )
}
