//! Sigmoid (replaces cuda/src/kernels/sigmoid.rs).
use super::unary::{self, UnaryOp};
use crate::device::{DeviceBuffer, HipStream};
use crate::error::Result;
use crate::params::HipType;

pub fn compute<T: HipType>(stream: &HipStream, input: &DeviceBuffer<T>, output: &mut DeviceBuffer<T>) -> Result<()> {
    unary::compute(stream, UnaryOp::Sigmoid, input, output)
}
