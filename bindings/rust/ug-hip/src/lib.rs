//! MI355X (gfx950) backend for ug: `ug::Device` / `ug::Slice` over the C ABI of `libughip.so`.
//!
//! The counterpart of `ug-cuda/src/lib.rs`; everything with behaviour lives behind `ffi`.
pub mod ffi;
pub mod runtime;

pub use runtime::{Device, Func, Slice};
