//! The little of cudarc the provider used directly: a stream and typed device memory
//! (runtime/src/providers/cuda/allocator.rs:96-139, data.rs:24-25, store.rs:385-416 of the reference).
use crate::error::{check, Result};
use crate::ffi;
use std::marker::PhantomData;
use std::os::raw::c_void;

/// A HIP stream handle owned elsewhere (null: the default stream). Streams keep their default
/// priority.
#[derive(Clone, Copy, Debug)]
pub struct HipStream(ffi::rmlk_stream_t);

unsafe impl Send for HipStream {}

impl HipStream {
    pub const DEFAULT: HipStream = HipStream(std::ptr::null_mut());

    /// # Safety
    /// `raw` is a valid `hipStream_t` (or null) for as long as the value is used.
    pub unsafe fn from_raw(raw: *mut c_void) -> Self {
        HipStream(raw)
    }

    pub fn raw(&self) -> ffi::rmlk_stream_t {
        self.0
    }

    pub fn synchronize(&self) -> Result<()> {
        check(unsafe { ffi::rmlk_hip_stream_sync(self.0) }, "stream_sync")
    }
}

/// `len` elements of `T` in device memory, freed on drop.
pub struct DeviceBuffer<T> {
    ptr: *mut c_void,
    len: usize,
    _elem: PhantomData<T>,
}

unsafe impl<T: Send> Send for DeviceBuffer<T> {}

impl<T: Copy> DeviceBuffer<T> {
    pub fn alloc(len: usize) -> Result<Self> {
        let mut ptr: *mut c_void = std::ptr::null_mut();
        let bytes = len.max(1) * std::mem::size_of::<T>();
        check(unsafe { ffi::rmlk_hip_malloc(&mut ptr, bytes) }, "malloc")?;
        Ok(DeviceBuffer { ptr, len, _elem: PhantomData })
    }

    pub fn from_host(stream: &HipStream, host: &[T]) -> Result<Self> {
        let buf = Self::alloc(host.len())?;
        if !host.is_empty() {
            check(
                unsafe {
                    ffi::rmlk_hip_memcpy_htod(stream.raw(), buf.ptr, host.as_ptr().cast(), std::mem::size_of_val(host))
                },
                "memcpy_htod",
            )?;
        }
        Ok(buf)
    }

    /// Copies to the host and waits for the copy.
    pub fn to_host(&self, stream: &HipStream) -> Result<Vec<T>>
    where
        T: Default,
    {
        let mut host = vec![T::default(); self.len];
        if self.len > 0 {
            check(
                unsafe {
                    ffi::rmlk_hip_memcpy_dtoh(
                        stream.raw(),
                        host.as_mut_ptr().cast(),
                        self.ptr,
                        self.len * std::mem::size_of::<T>(),
                    )
                },
                "memcpy_dtoh",
            )?;
            stream.synchronize()?;
        }
        Ok(host)
    }

    /// Device-to-device copy of `src` into this buffer (what Reshape and Unsqueeze do in the
    /// reference, runtime/src/providers/cuda/backend/reshape.rs:46), ordered on `stream`.
    pub fn copy_from_device(&mut self, stream: &HipStream, src: &DeviceBuffer<T>) -> Result<()> {
        if src.len != self.len {
            return Err(crate::Error::InvalidArguments("copy_from_device: lengths differ".into()));
        }
        check(
            unsafe { ffi::rmlk_hip_memcpy_dtod(stream.raw(), self.ptr, src.ptr, self.len * std::mem::size_of::<T>()) },
            "memcpy_dtod",
        )
    }

    /// Every byte of the buffer becomes `byte` (a fill kernel: safe to record into a HIP graph).
    pub fn memset(&mut self, stream: &HipStream, byte: u8) -> Result<()> {
        check(
            unsafe { ffi::rmlk_hip_memset(stream.raw(), self.ptr, byte as i32, self.len * std::mem::size_of::<T>()) },
            "memset",
        )
    }

    pub fn len(&self) -> usize {
        self.len
    }

    pub fn is_empty(&self) -> bool {
        self.len == 0
    }

    pub fn as_ptr(&self) -> *const c_void {
        self.ptr
    }

    pub fn as_mut_ptr(&mut self) -> *mut c_void {
        self.ptr
    }
}

impl<T> Drop for DeviceBuffer<T> {
    fn drop(&mut self) {
        if !self.ptr.is_null() {
            unsafe { ffi::rmlk_hip_free(self.ptr) };
        }
    }
}

/// Name, architecture, compute units, wavefront size, LDS per block, clock and memory of a GPU.
pub fn device_info(device: i32) -> Result<ffi::rmlk_device_info> {
    let mut info = std::mem::MaybeUninit::<ffi::rmlk_device_info>::zeroed();
    check(unsafe { ffi::rmlk_hip_device_info(device, info.as_mut_ptr()) }, "device_info")?;
    Ok(unsafe { info.assume_init() })
}

/// A shape or stride vector as the kernels take it (by value, at most 8 dims).
pub fn dims(values: &[usize]) -> Result<ffi::rmlk_dims> {
    if values.len() > ffi::RMLK_MAX_RANK {
        return Err(crate::Error::InvalidArguments(format!("rank {} above 8", values.len())));
    }
    let mut d = ffi::rmlk_dims { rank: values.len() as i32, v: [0; ffi::RMLK_MAX_RANK] };
    for (slot, &value) in d.v.iter_mut().zip(values) {
        *slot = value as i64;
    }
    Ok(d)
}

/// The same for signed values (slice starts and steps).
pub fn dims_i64(values: &[i64]) -> Result<ffi::rmlk_dims> {
    if values.len() > ffi::RMLK_MAX_RANK {
        return Err(crate::Error::InvalidArguments(format!("rank {} above 8", values.len())));
    }
    let mut d = ffi::rmlk_dims { rank: values.len() as i32, v: [0; ffi::RMLK_MAX_RANK] };
    d.v[..values.len()].copy_from_slice(values);
    Ok(d)
}
