//! Pow with its own exponent type (replaces cuda/src/kernels/pow.rs: base in {f32, f64, i32, i64},
//! exponent in any of those; the result has the base's type).
use super::binary::{self, BinaryOp};
use crate::device::{DeviceBuffer, HipStream};
use crate::error::Result;
use crate::params::HipType;

pub fn compute<B: HipType, E: HipType>(
    stream: &HipStream,
    c_shape: &[usize],
    a_stride: &[usize],
    b_stride: &[usize],
    base: &DeviceBuffer<B>,
    exponent: &DeviceBuffer<E>,
    out: &mut DeviceBuffer<B>,
) -> Result<()> {
    binary::compute_with_types::<B, E, B>(stream, BinaryOp::Pow, c_shape, a_stride, b_stride, base, exponent, out)
}
