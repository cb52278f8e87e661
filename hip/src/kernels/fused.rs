//! Chains of a decoder layer as single launches. None of them has a counterpart in the reference's
//! kernel crate: a backend ported one to one never calls them; the session runtime of this
//! repository (`include/rmlk_runtime.h`) forms them from the operator graph. Operands are raw
//! device pointers here, since most of them are views into larger tensors (a KV cache, a row of a
//! joint projection).
use crate::device::{dims, HipStream};
use crate::error::{check, Result};
use crate::ffi;
use std::os::raw::c_void;

/// `out = x / sqrt(mean(x^2) + eps) * gamma` per row (`reciprocal_form`: `x * (1 / sqrt(..))`,
/// the rounding of a graph that spells the norm with a Reciprocal-like Div).
pub unsafe fn rmsnorm(
    stream: &HipStream,
    rows: usize,
    cols: usize,
    x: *const c_void,
    gamma: *const c_void,
    eps: f32,
    reciprocal_form: bool,
    out: *mut c_void,
) -> Result<()> {
    check(
        ffi::rmlk_hip_rmsnorm(
            stream.raw(),
            ffi::RMLK_FLOAT,
            rows as i64,
            cols as i64,
            x,
            gamma,
            eps,
            reciprocal_form as i32,
            out,
        ),
        "rmsnorm",
    )
}

/// `sum_out = a + b`, `out = rmsnorm(sum_out)`.
pub unsafe fn add_rmsnorm(
    stream: &HipStream,
    rows: usize,
    cols: usize,
    a: *const c_void,
    b: *const c_void,
    gamma: *const c_void,
    eps: f32,
    reciprocal_form: bool,
    sum_out: *mut c_void,
    out: *mut c_void,
) -> Result<()> {
    check(
        ffi::rmlk_hip_add_rmsnorm(
            stream.raw(),
            ffi::RMLK_FLOAT,
            rows as i64,
            cols as i64,
            a,
            b,
            gamma,
            eps,
            reciprocal_form as i32,
            sum_out,
            out,
        ),
        "add_rmsnorm",
    )
}

/// `out = gate * sigmoid(gate) * up`.
pub unsafe fn swiglu(stream: &HipStream, n: usize, gate: *const c_void, up: *const c_void, out: *mut c_void) -> Result<()> {
    check(ffi::rmlk_hip_swiglu(stream.raw(), ffi::RMLK_FLOAT, n as i64, gate, up, out), "swiglu")
}

/// How constant weights are held in device memory; the arithmetic is fp32 in every case.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum WeightStorage {
    F32,
    F16,
    BF16,
}

impl WeightStorage {
    pub fn dtype(self) -> i32 {
        match self {
            WeightStorage::F32 => ffi::RMLK_FLOAT,
            WeightStorage::F16 => ffi::RMLK_FLOAT16,
            WeightStorage::BF16 => ffi::RMLK_BFLOAT16,
        }
    }
}

/// `dst[i] = src[i]` rounded to nearest even in a 16-bit storage type.
pub unsafe fn store_weights(
    stream: &HipStream,
    storage: WeightStorage,
    n: usize,
    src: *const c_void,
    dst: *mut c_void,
) -> Result<()> {
    check(ffi::rmlk_hip_store_weights(stream.raw(), storage.dtype(), n as i64, src, dst), "store_weights")
}

/// One-row product over K-contiguous weights: `y[n] = sum_k x[k] * wt[n][k]`.
pub unsafe fn gemv_kmajor(
    stream: &HipStream,
    n: usize,
    k: usize,
    x: *const c_void,
    storage: WeightStorage,
    wt: *const c_void,
    ldw: usize,
    y: *mut c_void,
) -> Result<()> {
    check(
        ffi::rmlk_hip_gemv_kmajor(
            stream.raw(),
            ffi::RMLK_FLOAT,
            n as i64,
            k as i64,
            x,
            storage.dtype(),
            wt,
            ldw as i64,
            y,
        ),
        "gemv_kmajor",
    )
}

/// `gemv_kmajor` with a residual row added to the outputs (the Add behind an output projection).
pub unsafe fn gemv_kmajor_add(
    stream: &HipStream,
    n: usize,
    k: usize,
    x: *const c_void,
    storage: WeightStorage,
    wt: *const c_void,
    ldw: usize,
    residual: *const c_void,
    y: *mut c_void,
) -> Result<()> {
    check(
        ffi::rmlk_hip_gemv_kmajor_add(
            stream.raw(),
            ffi::RMLK_FLOAT,
            n as i64,
            k as i64,
            x,
            storage.dtype(),
            wt,
            ldw as i64,
            residual,
            y,
        ),
        "gemv_kmajor_add",
    )
}

/// RMSNorm parameters of the products that normalise their input row themselves.
#[derive(Clone, Copy, Debug)]
pub struct RowNorm {
    pub gamma: *const c_void,
    pub eps: f32,
    /// `x * (1 / rms)` instead of `x / rms` (the two decompositions exported graphs use).
    pub reciprocal_form: bool,
}

/// `gemv_kmajor` over `RMSNorm(x) * gamma`, the norm formed by the kernel (the bits of the norm kernel
/// followed by the product).
pub unsafe fn gemv_kmajor_normed(
    stream: &HipStream,
    n: usize,
    k: usize,
    x: *const c_void,
    norm: &RowNorm,
    storage: WeightStorage,
    wt: *const c_void,
    ldw: usize,
    y: *mut c_void,
) -> Result<()> {
    check(
        ffi::rmlk_hip_gemv_kmajor_normed(
            stream.raw(),
            ffi::RMLK_FLOAT,
            n as i64,
            k as i64,
            x,
            norm.gamma,
            norm.eps,
            norm.reciprocal_form as i32,
            storage.dtype(),
            wt,
            ldw as i64,
            y,
        ),
        "gemv_kmajor_normed",
    )
}

/// `y[i] = silu(wt[gate_row + i] . x) * (wt[up_row + i] . x)` over a joint [gate | up] matrix; with
/// `norm` the input row is normalised first.
pub unsafe fn gemv_kmajor_swiglu(
    stream: &HipStream,
    n: usize,
    k: usize,
    x: *const c_void,
    norm: Option<&RowNorm>,
    storage: WeightStorage,
    wt: *const c_void,
    ldw: usize,
    gate_row: usize,
    up_row: usize,
    y: *mut c_void,
) -> Result<()> {
    match norm {
        Some(nm) => check(
            ffi::rmlk_hip_gemv_kmajor_swiglu_normed(
                stream.raw(),
                ffi::RMLK_FLOAT,
                n as i64,
                k as i64,
                x,
                nm.gamma,
                nm.eps,
                nm.reciprocal_form as i32,
                storage.dtype(),
                wt,
                ldw as i64,
                gate_row as i64,
                up_row as i64,
                y,
            ),
            "gemv_kmajor_swiglu_normed",
        ),
        None => check(
            ffi::rmlk_hip_gemv_kmajor_swiglu(
                stream.raw(),
                ffi::RMLK_FLOAT,
                n as i64,
                k as i64,
                x,
                storage.dtype(),
                wt,
                ldw as i64,
                gate_row as i64,
                up_row as i64,
                y,
            ),
            "gemv_kmajor_swiglu",
        ),
    }
}

/// Sets `*fits` (device memory, 1 before the call) to 0 when one of the `n` floats at `src` would not
/// survive storage as `storage`.
pub unsafe fn weights_fit(
    stream: &HipStream,
    storage: WeightStorage,
    n: usize,
    src: *const c_void,
    fits: *mut i32,
) -> Result<()> {
    check(ffi::rmlk_hip_weights_fit(stream.raw(), storage.dtype(), n as i64, src, fits), "weights_fit")
}

/// Rotary embedding of `x` read through strides: `out = x * cos + rotate_half(x) * sin`.
pub unsafe fn rotary(
    stream: &HipStream,
    shape: &[usize],
    x_stride: &[usize],
    cos_stride: &[usize],
    sin_stride: &[usize],
    x: *const c_void,
    cos: *const c_void,
    sin: *const c_void,
    out: *mut c_void,
) -> Result<()> {
    let (sh, xs, cs, ss) = (dims(shape)?, dims(x_stride)?, dims(cos_stride)?, dims(sin_stride)?);
    check(
        ffi::rmlk_hip_rotary(stream.raw(), ffi::RMLK_FLOAT, &sh, &xs, &cs, &ss, x, cos, sin, out),
        "rotary",
    )
}

/// `Softmax(x (*|/) scale + mask)` along the last axis in one pass.
pub unsafe fn scale_mask_softmax(
    stream: &HipStream,
    shape: &[usize],
    mask_stride: &[usize],
    scale_is_mul: bool,
    scale: f32,
    x: *const c_void,
    mask: *const c_void,
    out: *mut c_void,
) -> Result<()> {
    let (sh, ms) = (dims(shape)?, dims(mask_stride)?);
    check(
        ffi::rmlk_hip_scale_mask_softmax(stream.raw(), ffi::RMLK_FLOAT, &sh, &ms, scale_is_mul as i32, scale, x, mask, out),
        "scale_mask_softmax",
    )
}

/// Bytes that the three bfloat16 pieces of a dense float matrix `[m, k]` take (`bf16x3_split`).
pub fn bf16x3_pieces_size(m: usize, k: usize) -> usize {
    unsafe { ffi::rmlk_hip_bf16x3_pieces_size(m as i64, k as i64) }
}

/// Splits the float matrix `a` `[m, k]` into three bfloat16 pieces whose sum it is exactly, as
/// the planes `[3][m rounded up to 128][k]` that `matmul_bf16x3` reads.
pub unsafe fn bf16x3_split(
    stream: &HipStream,
    m: usize,
    k: usize,
    a: *const c_void,
    lda: usize,
    pieces: *mut c_void,
) -> Result<()> {
    check(ffi::rmlk_hip_bf16x3_split(stream.raw(), m as i64, k as i64, a, lda as i64, pieces), "bf16x3_split")
}

/// RMSNorm (over `partials[0] + .. + partials[splits-1]`, plus `b` when given, the formed rows then
/// also stored to `sum_out`) whose result goes to `out` and, as by `bf16x3_split`, to `pieces`.
pub unsafe fn rmsnorm_pieces(
    stream: &HipStream,
    rows: usize,
    cols: usize,
    partials: *const c_void,
    splits: usize,
    slab: usize,
    b: *const c_void,
    gamma: *const c_void,
    eps: f32,
    reciprocal_form: bool,
    sum_out: *mut c_void,
    out: *mut c_void,
    pieces: *mut c_void,
) -> Result<()> {
    check(
        ffi::rmlk_hip_rmsnorm_pieces(
            stream.raw(),
            rows as i64,
            cols as i64,
            partials,
            splits as i32,
            slab as i64,
            b,
            gamma,
            eps,
            reciprocal_form as i32,
            sum_out,
            out,
            pieces,
        ),
        "rmsnorm_pieces",
    )
}

/// Slabs of K with which `matmul_bf16x3` fills the GPU for a size; `None`: a size it does not take.
pub fn bf16x3_splits(m: usize, n: usize, k: usize) -> Option<usize> {
    match unsafe { ffi::rmlk_hip_bf16x3_splits(m as i64, n as i64, k as i64) } {
        s if s > 0 => Some(s as usize),
        _ => None,
    }
}

/// `c[m, n] = a . wt^T` over the pieces of `a` and bfloat16 weights `wt` `[n, k]` on the bf16
/// matrix cores, fp32 results. `splits > 1`: one partial product per slab of K, `slab` elements
/// apart, for a reader that adds them up.
pub unsafe fn matmul_bf16x3(
    stream: &HipStream,
    m: usize,
    n: usize,
    k: usize,
    pieces: *const c_void,
    wt: *const c_void,
    ldw: usize,
    splits: usize,
    c: *mut c_void,
    ldc: usize,
    slab: usize,
) -> Result<()> {
    check(
        ffi::rmlk_hip_matmul_bf16x3(
            stream.raw(),
            m as i64,
            n as i64,
            k as i64,
            pieces,
            wt,
            ldw as i64,
            splits as i32,
            c,
            ldc as i64,
            slab as i64,
        ),
        "matmul_bf16x3",
    )
}

/// `outs[i]` (dense `[m, widths[i]]`) `= a . (the next widths[i] rows of wt)^T` over the pieces of
/// `a`, one launch over the joint matrix. At most 4 members, widths multiples of 32.
pub unsafe fn matmul_bf16x3_grouped(
    stream: &HipStream,
    m: usize,
    k: usize,
    pieces: *const c_void,
    wt: *const c_void,
    ldw: usize,
    widths: &[i64],
    outs: &[*mut c_void],
) -> Result<()> {
    assert_eq!(widths.len(), outs.len());
    check(
        ffi::rmlk_hip_matmul_bf16x3_grouped(
            stream.raw(),
            m as i64,
            k as i64,
            pieces,
            wt,
            ldw as i64,
            widths.len() as i32,
            widths.as_ptr(),
            outs.as_ptr(),
        ),
        "matmul_bf16x3_grouped",
    )
}

/// `out[m, n] = swiglu(a . wt[gate_row..+n]^T, a . wt[up_row..+n]^T)` over the pieces of `a`;
/// `out_pieces` (null: not wanted): where the same launch also stores the pieces of `out`.
pub unsafe fn matmul_bf16x3_swiglu(
    stream: &HipStream,
    m: usize,
    n: usize,
    k: usize,
    pieces: *const c_void,
    wt: *const c_void,
    ldw: usize,
    gate_row: usize,
    up_row: usize,
    out: *mut c_void,
    ldc: usize,
    out_pieces: *mut c_void,
) -> Result<()> {
    check(
        ffi::rmlk_hip_matmul_bf16x3_swiglu(
            stream.raw(),
            m as i64,
            n as i64,
            k as i64,
            pieces,
            wt,
            ldw as i64,
            gate_row as i64,
            up_row as i64,
            out,
            ldc as i64,
            out_pieces,
        ),
        "matmul_bf16x3_swiglu",
    )
}

/// Shape of a grouped-query attention call.
#[derive(Clone, Copy, Debug)]
pub struct AttentionShape {
    pub batch: usize,
    pub kv_heads: usize,
    /// Query heads per KV head.
    pub rep: usize,
    pub q_len: usize,
    pub kv_len: usize,
    pub head_dim: usize,
}

/// Bytes of workspace with which `attention` skips the key chunks a query tile cannot see
/// (0: skipping does not apply to this shape and no workspace is needed).
pub fn attention_workspace_size(shape: &AttentionShape, mask_stride: &[usize; 4]) -> Result<usize> {
    let ms = dims(mask_stride)?;
    Ok(unsafe {
        ffi::rmlk_hip_attention_workspace_size(
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
            &ms,
        )
    })
}

/// `Softmax(q . k^T (*|/) scale + mask) . v` over many query rows in one kernel; `workspace` may be
/// null with 0 bytes.
pub unsafe fn attention(
    stream: &HipStream,
    shape: &AttentionShape,
    q: *const c_void,
    k: *const c_void,
    v: *const c_void,
    mask: *const c_void,
    mask_stride: &[usize; 4],
    scale_is_mul: bool,
    scale: f32,
    out_seq_major: bool,
    workspace: *mut c_void,
    workspace_bytes: usize,
    out: *mut c_void,
) -> Result<()> {
    let ms = dims(mask_stride)?;
    check(
        ffi::rmlk_hip_attention_ws(
            stream.raw(),
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
            q,
            k,
            v,
            mask,
            &ms,
            scale_is_mul as i32,
            scale,
            out_seq_major as i32,
            workspace,
            workspace_bytes,
            out,
        ),
        "attention",
    )
}

/// Bytes of workspace of `attention_few_rows` (0: more than 16 query rows per KV head, not its case).
pub fn attention_few_rows_workspace_size(shape: &AttentionShape) -> usize {
    unsafe {
        ffi::rmlk_hip_attention_few_rows_workspace_size(
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
        )
    }
}

/// The attention of a decode step (at most 16 query rows per KV head): the keys split over blocks,
/// the chunks merged by the block that finishes a KV head last when `counters` (one `i32` per
/// batch x KV head, zero before the first call and left zero) is given, by a second launch otherwise.
pub unsafe fn attention_few_rows(
    stream: &HipStream,
    shape: &AttentionShape,
    q: *const c_void,
    k: *const c_void,
    v: *const c_void,
    mask: *const c_void,
    mask_stride: &[usize; 4],
    scale_is_mul: bool,
    scale: f32,
    out_seq_major: bool,
    workspace: *mut c_void,
    workspace_bytes: usize,
    counters: Option<*mut i32>,
    out: *mut c_void,
) -> Result<()> {
    let ms = dims(mask_stride)?;
    match counters {
        Some(cnt) => check(
            ffi::rmlk_hip_attention_few_rows_one_launch(
                stream.raw(),
                ffi::RMLK_FLOAT,
                shape.batch as i64,
                shape.kv_heads as i64,
                shape.rep as i64,
                shape.q_len as i64,
                shape.kv_len as i64,
                shape.head_dim as i64,
                q,
                k,
                v,
                mask,
                &ms,
                scale_is_mul as i32,
                scale,
                out_seq_major as i32,
                workspace,
                workspace_bytes,
                cnt,
                out,
            ),
            "attention_few_rows_one_launch",
        ),
        None => check(
            ffi::rmlk_hip_attention_few_rows(
                stream.raw(),
                ffi::RMLK_FLOAT,
                shape.batch as i64,
                shape.kv_heads as i64,
                shape.rep as i64,
                shape.q_len as i64,
                shape.kv_len as i64,
                shape.head_dim as i64,
                q,
                k,
                v,
                mask,
                &ms,
                scale_is_mul as i32,
                scale,
                out_seq_major as i32,
                workspace,
                workspace_bytes,
                out,
            ),
            "attention_few_rows",
        ),
    }
}

/// Bytes of a map of the mask's visible (query tile, key chunk) pairs that several `attention_mapped`
/// calls over one mask share (0: skipping does not apply to this shape).
pub fn attention_map_size(shape: &AttentionShape, mask_stride: &[usize; 4]) -> Result<usize> {
    let ms = dims(mask_stride)?;
    Ok(unsafe {
        ffi::rmlk_hip_attention_map_size(
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
            &ms,
        )
    })
}

/// Makes the map of `mask` in `map` (`attention_map_size` bytes, 16-byte aligned), once for all the
/// layers that read the mask.
pub unsafe fn attention_map(
    stream: &HipStream,
    shape: &AttentionShape,
    mask: *const c_void,
    mask_stride: &[usize; 4],
    map: *mut c_void,
    map_bytes: usize,
) -> Result<()> {
    let ms = dims(mask_stride)?;
    check(
        ffi::rmlk_hip_attention_map(
            stream.raw(),
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
            mask,
            &ms,
            map,
            map_bytes,
        ),
        "attention_map",
    )
}

/// `attention` over a map made by `attention_map` for this mask and these sizes (same bits).
pub unsafe fn attention_mapped(
    stream: &HipStream,
    shape: &AttentionShape,
    q: *const c_void,
    k: *const c_void,
    v: *const c_void,
    mask: *const c_void,
    mask_stride: &[usize; 4],
    scale_is_mul: bool,
    scale: f32,
    out_seq_major: bool,
    map: *const c_void,
    map_bytes: usize,
    out: *mut c_void,
) -> Result<()> {
    let ms = dims(mask_stride)?;
    check(
        ffi::rmlk_hip_attention_mapped(
            stream.raw(),
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
            q,
            k,
            v,
            mask,
            &ms,
            scale_is_mul as i32,
            scale,
            out_seq_major as i32,
            map,
            map_bytes,
            out,
        ),
        "attention_mapped",
    )
}

/// `attention_mapped` with the `[batch, q_len, heads, head_dim]` result also stored as the three
/// bfloat16 pieces `bf16x3_split` would make of it (`out_pieces`).
pub unsafe fn attention_mapped_with_pieces(
    stream: &HipStream,
    shape: &AttentionShape,
    q: *const c_void,
    k: *const c_void,
    v: *const c_void,
    mask: *const c_void,
    mask_stride: &[usize; 4],
    scale_is_mul: bool,
    scale: f32,
    map: *const c_void,
    map_bytes: usize,
    out: *mut c_void,
    out_pieces: *mut c_void,
) -> Result<()> {
    let ms = dims(mask_stride)?;
    check(
        ffi::rmlk_hip_attention_mapped_pieces(
            stream.raw(),
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
            q,
            k,
            v,
            mask,
            &ms,
            scale_is_mul as i32,
            scale,
            map,
            map_bytes,
            out,
            out_pieces,
        ),
        "attention_mapped_with_pieces",
    )
}

/// `attention` with a `[batch, q_len, heads, head_dim]` result that is also stored as the three
/// bfloat16 pieces `bf16x3_split` would make of it (`out_pieces`), for an output projection over them.
pub unsafe fn attention_with_pieces(
    stream: &HipStream,
    shape: &AttentionShape,
    q: *const c_void,
    k: *const c_void,
    v: *const c_void,
    mask: *const c_void,
    mask_stride: &[usize; 4],
    scale_is_mul: bool,
    scale: f32,
    workspace: *mut c_void,
    workspace_bytes: usize,
    out: *mut c_void,
    out_pieces: *mut c_void,
) -> Result<()> {
    let ms = dims(mask_stride)?;
    check(
        ffi::rmlk_hip_attention_ws_pieces(
            stream.raw(),
            ffi::RMLK_FLOAT,
            shape.batch as i64,
            shape.kv_heads as i64,
            shape.rep as i64,
            shape.q_len as i64,
            shape.kv_len as i64,
            shape.head_dim as i64,
            q,
            k,
            v,
            mask,
            &ms,
            scale_is_mul as i32,
            scale,
            workspace,
            workspace_bytes,
            out,
            out_pieces,
        ),
        "attention_with_pieces",
    )
}

/// While a value of this type lives, operators over tiny tensors issued on `stream` through this
/// crate are recorded and go out as one launch, in call order (`rmlk_hip_batch_begin` / `_end`).
/// Work put on the stream by other means must be preceded by `flush`.
pub struct CollectedLaunches<'a> {
    stream: &'a HipStream,
}

impl<'a> CollectedLaunches<'a> {
    pub fn begin(stream: &'a HipStream) -> Result<Self> {
        check(unsafe { ffi::rmlk_hip_batch_begin(stream.raw()) }, "batch_begin")?;
        Ok(CollectedLaunches { stream })
    }

    pub fn flush(&self) -> Result<()> {
        check(unsafe { ffi::rmlk_hip_batch_flush(self.stream.raw()) }, "batch_flush")
    }

    /// Sends the recorded calls out and reports the status of the launches the batch made.
    pub fn end(self) -> Result<()> {
        let status = unsafe { ffi::rmlk_hip_batch_end(self.stream.raw()) };
        std::mem::forget(self);
        check(status, "batch_end")
    }
}

impl Drop for CollectedLaunches<'_> {
    fn drop(&mut self) {
        let _ = unsafe { ffi::rmlk_hip_batch_end(self.stream.raw()) };
    }
}
