//! Mul with broadcasting (replaces cuda/src/kernels/mul.rs: `load_kernel` is gone, `compute` stays).
use super::binary::{self, BinaryOp};
use crate::device::{DeviceBuffer, HipStream};
use crate::error::Result;
use crate::params::HipType;

pub fn compute<T: HipType>(
    stream: &HipStream,
    c_shape: &[usize],
    a_stride: &[usize],
    b_stride: &[usize],
    a: &DeviceBuffer<T>,
    b: &DeviceBuffer<T>,
    c: &mut DeviceBuffer<T>,
) -> Result<()> {
    binary::compute(stream, BinaryOp::Mul, c_shape, a_stride, b_stride, a, b, c)
}
