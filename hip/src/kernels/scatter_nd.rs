//! ScatterND (replaces cuda/src/kernels/scatter_nd.rs:91-210). `output` already holds a copy of the
//! data tensor (`compute`), or receives it in the same pass (`compute_with_copy`). An index outside
//! the data tensor sets `*err_flag` on the device instead of faulting; the caller reads the flag
//! when it chooses (the reference checks indices on the host, backend/scatter_nd.rs:198-203).
use crate::device::{dims, DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(i32)]
pub enum Reduction {
    None = ffi::RMLK_SCATTER_NONE,
    Add = ffi::RMLK_SCATTER_ADD,
    Mul = ffi::RMLK_SCATTER_MUL,
    Max = ffi::RMLK_SCATTER_MAX,
    Min = ffi::RMLK_SCATTER_MIN,
}

fn tuples(indices_len: usize, tuple_size: usize, data_rank: usize) -> Result<usize> {
    if tuple_size == 0 || tuple_size > data_rank || indices_len % tuple_size != 0 {
        return Err(Error::InvalidArguments("scatter_nd: bad index tuple size".into()));
    }
    Ok(indices_len / tuple_size)
}

pub fn compute<T: HipType>(
    stream: &HipStream,
    reduction: Reduction,
    data_shape: &[usize],
    tuple_size: usize,
    indices: &DeviceBuffer<i64>,
    updates: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
    err_flag: &mut DeviceBuffer<i32>,
) -> Result<()> {
    let n_tuples = tuples(indices.len(), tuple_size, data_shape.len())?;
    let shape = dims(data_shape)?;
    check(
        unsafe {
            ffi::rmlk_hip_scatter_nd(
                stream.raw(),
                reduction as i32,
                T::DTYPE,
                &shape,
                n_tuples as i64,
                tuple_size as i32,
                indices.as_ptr().cast(),
                updates.as_ptr(),
                output.as_mut_ptr(),
                err_flag.as_mut_ptr().cast(),
            )
        },
        "scatter_nd",
    )
}

/// Plain assignment into a fresh output: the copy of `data` and the scattered slices in one pass.
pub fn compute_with_copy<T: HipType>(
    stream: &HipStream,
    data_shape: &[usize],
    tuple_size: usize,
    indices: &DeviceBuffer<i64>,
    updates: &DeviceBuffer<T>,
    data: &DeviceBuffer<T>,
    output: &mut DeviceBuffer<T>,
    err_flag: &mut DeviceBuffer<i32>,
) -> Result<()> {
    let n_tuples = tuples(indices.len(), tuple_size, data_shape.len())?;
    if data.len() != output.len() {
        return Err(Error::InvalidArguments("scatter_nd: data and output differ in length".into()));
    }
    let shape = dims(data_shape)?;
    check(
        unsafe {
            ffi::rmlk_hip_scatter_nd_copy(
                stream.raw(),
                T::DTYPE,
                &shape,
                n_tuples as i64,
                tuple_size as i32,
                indices.as_ptr().cast(),
                updates.as_ptr(),
                data.as_ptr(),
                output.as_mut_ptr(),
                err_flag.as_mut_ptr().cast(),
            )
        },
        "scatter_nd (with copy)",
    )
}
