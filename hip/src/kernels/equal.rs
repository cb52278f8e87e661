//! Equal: a bool per element (replaces cuda/src/kernels/equal.rs).
use super::binary::{self, BinaryOp};
use crate::device::{DeviceBuffer, HipStream};
use crate::error::Result;
use crate::params::{Bool, HipType};

pub fn compute<T: HipType>(
    stream: &HipStream,
    c_shape: &[usize],
    a_stride: &[usize],
    b_stride: &[usize],
    a: &DeviceBuffer<T>,
    b: &DeviceBuffer<T>,
    c: &mut DeviceBuffer<Bool>,
) -> Result<()> {
    binary::compute_with_types::<T, T, Bool>(stream, BinaryOp::Equal, c_shape, a_stride, b_stride, a, b, c)
}
