//! One module per operator, as in cuda/src/kernels/mod.rs:1-29 of the reference. The operators of
//! the decoder path are here; conv, max_pool, global_average_pool and relu (cuDNN wrappers in the
//! reference) have no HIP counterpart in this library.
pub mod add;
pub mod binary;
pub mod cast;
pub mod concat;
pub mod cos;
pub mod div;
pub mod equal;
pub mod expand;
pub mod fill;
pub mod fused;
pub mod gather;
pub mod gemm;
pub mod greater;
pub mod mul;
pub mod neg;
pub mod pow;
pub mod reduce_mean;
pub mod scatter_nd;
pub mod sigmoid;
pub mod sin;
pub mod slice;
pub mod softmax;
pub mod sqrt;
pub mod sub;
pub mod transpose;
pub mod trilu;
pub mod unary;
pub mod whereop;
