//! Batched matrix products (replaces cuda/src/kernels/gemm.rs:9-136, cublasGemmStridedBatchedEx).
//! `gemm_params` keeps the reference's meaning: row-major operands, a logical transpose is a swap
//! of the last two strides, `b` products that differ by a batch stride (0 for a shared operand,
//! which the reference has to copy first).
use crate::device::{DeviceBuffer, HipStream};
use crate::error::{check, Error, Result};
use crate::ffi;
use crate::params::HipType;

#[derive(Clone, Debug)]
pub struct GemmParams {
    pub b: usize,
    pub m: usize,
    pub n: usize,
    pub k: usize,
    pub trans_a: bool,
    pub trans_b: bool,
    /// Elements from one row of A (of B, of the output) to the next.
    pub lda: usize,
    pub ldb: usize,
    pub ldc: usize,
    /// Elements from one matrix of the batch to the next; 0: every product reads the same matrix.
    pub stride_a: usize,
    pub stride_b: usize,
    pub stride_c: usize,
}

/// Dense row-major operands `a_shape = [.., m, k]` (or `[.., k, m]` with `trans_a`) and likewise
/// for `b`; `batch_a` / `batch_b`: whether the operand has its own matrix per product.
pub fn gemm_params(
    a_shape: &[usize],
    b_shape: &[usize],
    trans_a: bool,
    trans_b: bool,
    b: usize,
    batch_a: bool,
    batch_b: bool,
) -> Result<GemmParams> {
    if a_shape.len() < 2 || b_shape.len() < 2 {
        return Err(Error::InvalidArguments("gemm: operands need at least two dims".into()));
    }
    let (a_rows, a_cols) = (a_shape[a_shape.len() - 2], a_shape[a_shape.len() - 1]);
    let (b_rows, b_cols) = (b_shape[b_shape.len() - 2], b_shape[b_shape.len() - 1]);
    let (m, k) = if trans_a { (a_cols, a_rows) } else { (a_rows, a_cols) };
    let (kb, n) = if trans_b { (b_cols, b_rows) } else { (b_rows, b_cols) };
    if k != kb {
        return Err(Error::InvalidArguments(format!("gemm: inner dims differ ({k} and {kb})")));
    }
    Ok(GemmParams {
        b,
        m,
        n,
        k,
        trans_a,
        trans_b,
        lda: a_cols,
        ldb: b_cols,
        ldc: n,
        stride_a: if batch_a { a_rows * a_cols } else { 0 },
        stride_b: if batch_b { b_rows * b_cols } else { 0 },
        stride_c: m * n,
    })
}

/// Bytes of workspace `compute` needs for these sizes (split-K partial sums); may be 0.
pub fn workspace_size<T: HipType>(p: &GemmParams) -> usize {
    unsafe { ffi::rmlk_hip_matmul_workspace_size(T::DTYPE, p.b as i64, p.m as i64, p.n as i64, p.k as i64) }
}

/// `y[i] = a[i] . b[i]` for the `p.b` products. `workspace`: at least `workspace_size` bytes.
pub fn compute<T: HipType>(
    stream: &HipStream,
    a_data: &DeviceBuffer<T>,
    b_data: &DeviceBuffer<T>,
    y_data: &mut DeviceBuffer<T>,
    p: &GemmParams,
    workspace: Option<&mut DeviceBuffer<u8>>,
) -> Result<()> {
    if y_data.len() < p.b * p.m * p.n {
        return Err(Error::InvalidArguments("gemm: output shorter than b * m * n".into()));
    }
    let (ws_ptr, ws_bytes) = match workspace {
        Some(ws) => (ws.as_mut_ptr(), ws.len()),
        None => (std::ptr::null_mut(), 0),
    };
    check(
        unsafe {
            ffi::rmlk_hip_matmul(
                stream.raw(),
                T::DTYPE,
                p.b as i64,
                p.m as i64,
                p.n as i64,
                p.k as i64,
                a_data.as_ptr(),
                p.lda as i64,
                p.stride_a as i64,
                p.trans_a as i32,
                b_data.as_ptr(),
                p.ldb as i64,
                p.stride_b as i64,
                p.trans_b as i32,
                y_data.as_mut_ptr(),
                p.ldc as i64,
                p.stride_c as i64,
                ws_ptr,
                ws_bytes,
            )
        },
        "gemm",
    )
}

/// The same for callers that may not allocate (HIP graph capture, serving loops): the partial
/// sums go to a fixed array inside the library; `Error::Internal` when the problem needs more
/// than `RMLK_HIP_MATMUL_NOALLOC_SCRATCH_BYTES`. Calls on one GPU share that array.
pub fn compute_noalloc<T: HipType>(
    stream: &HipStream,
    a_data: &DeviceBuffer<T>,
    b_data: &DeviceBuffer<T>,
    y_data: &mut DeviceBuffer<T>,
    p: &GemmParams,
) -> Result<()> {
    if y_data.len() < p.b * p.m * p.n {
        return Err(Error::InvalidArguments("gemm: output shorter than b * m * n".into()));
    }
    check(
        unsafe {
            ffi::rmlk_hip_matmul_noalloc(
                stream.raw(),
                T::DTYPE,
                p.b as i64,
                p.m as i64,
                p.n as i64,
                p.k as i64,
                a_data.as_ptr(),
                p.lda as i64,
                p.stride_a as i64,
                p.trans_a as i32,
                b_data.as_ptr(),
                p.ldb as i64,
                p.stride_b as i64,
                p.trans_b as i32,
                y_data.as_mut_ptr(),
                p.ldc as i64,
                p.stride_c as i64,
            )
        },
        "gemm (no allocation)",
    )
}
