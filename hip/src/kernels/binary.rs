//! Broadcasting binary operators (replaces cuda/src/kernels/binary.rs:58-100 and the `info` buffer
//! of binary.rs:165-174: shape and strides travel by value, nothing is uploaded per call).
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(i32)]
pub enum BinaryOp {
    Add = ffi::RMLK_ADD,
    Sub = ffi::RMLK_SUB,
    Mul = ffi::RMLK_MUL,
    Div = ffi::RMLK_DIV,
    Pow = ffi::RMLK_POW,
    Equal = ffi::RMLK_EQUAL,
    Greater = ffi::RMLK_GREATER,
}

/// `c[i] = op(a[ia], b[ib])` over `c_shape`; `a_stride` / `b_stride` are element strides per
/// output dim, 0 on broadcast dims (what the reference packs into its info buffer).
pub fn compute_with_types<X: HipType, Y: HipType, O: HipType>(
    stream: &HipStream,
    op: BinaryOp,
    c_shape: &[usize],
    a_stride: &[usize],
    b_stride: &[usize],
    a: &DeviceBuffer<X>,
    b: &DeviceBuffer<Y>,
    c: &mut DeviceBuffer<O>,
) -> Result<()> {
    if c_shape.len() != a_stride.len() || c_shape.len() != b_stride.len() {
        return Err(Error::InvalidArguments("binary: shape and strides differ in rank".into()));
    }
    if c.len() != c_shape.iter().product::<usize>() {
        return Err(Error::InvalidArguments("binary: output length does not match its shape".into()));
    }
    let (shape, sa, sb) = (dims(c_shape)?, dims(a_stride)?, dims(b_stride)?);
    check(
        unsafe {
            ffi::rmlk_hip_binary(
                stream.raw(),
                op as i32,
                X::DTYPE,
                Y::DTYPE,
                &shape,
                &sa,
                &sb,
                a.as_ptr(),
                b.as_ptr(),
                c.as_mut_ptr(),
            )
        },
        "binary",
    )
}

/// Both operands and the result of one type (Add, Sub, Mul, Div).
pub fn compute<T: HipType>(
    stream: &HipStream,
    op: BinaryOp,
    c_shape: &[usize],
    a_stride: &[usize],
    b_stride: &[usize],
    a: &DeviceBuffer<T>,
    b: &DeviceBuffer<T>,
    c: &mut DeviceBuffer<T>,
) -> Result<()> {
    compute_with_types::<T, T, T>(stream, op, c_shape, a_stride, b_stride, a, b, c)
}
