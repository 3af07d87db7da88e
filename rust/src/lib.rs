//! Rust host side of the MI355X quantized-linear kernels.
//!
//! * `sys`     — the raw `extern "C"` declarations, generated from `include/gpu_api.h`;
//! * `ffi`     — dtype / prologue codes and the checked-call macro `k!`, with the names the reference's model code
//!               uses (its src/ffi.rs:8-29,336-351), so that `k!(gpu_quant_rows(...))` call sites compile unchanged;
//! * `hip`     — the runtime layer that takes the place of the reference's src/cuda.rs: device setup, streams,
//!               events, device and pinned buffers, copies;
//! * `qlinear` — the call pattern of one quantized linear (quantize rows, then the fused int8 GEMM).
//!
//! The image this repository is built in has no Rust toolchain: this crate has never been compiled.  The C ABI it
//! binds is exercised through ctypes by the Python tests; `tests/test_host_boundary.py` checks that `sys.rs` declares
//! exactly what the headers declare.
pub mod ffi;
pub mod hip;
pub mod qlinear;
pub mod sys;
