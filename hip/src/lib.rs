//! MI355X kernels behind the module layout of the reference's `rmlk-cuda` crate
//! (cuda/src/lib.rs:6-12): `kernels::<op>::compute`, an `Error` type, and the few device helpers
//! the provider took from cudarc. Every function is a thin, checked call into the C ABI of
//! `include/rmlk_hip.h`; nothing is loaded at run time (the reference's `load_kernel` functions
//! have no counterpart: the code objects are linked into librmlk_hip.so).
#![allow(clippy::too_many_arguments)]
#![allow(clippy::missing_safety_doc)]

pub mod device;
mod error;
pub mod ffi;
pub mod kernels;
pub mod params;

pub use device::{DeviceBuffer, HipStream};
pub use error::{check, Error, Result};
