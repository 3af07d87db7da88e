//! Codes of the C ABI and checked calls into it.
use crate::hip::{self, Stream};
use anyhow::{bail, Result};

pub use crate::sys::*;

// dtype codes, include/gpu_api.h (the reference's src/ffi.rs:11-13)
pub const DT_F32: i32 = 0;
pub const DT_F16: i32 = 1;
pub const DT_BF16: i32 = 2;

// row prologue ids, include/gpu_api.h (the reference's src/ffi.rs:15-29)
pub const PRO_PLAIN: i32 = 0;
pub const PRO_RMS: i32 = 1;
pub const PRO_GATE: i32 = 2;
pub const PRO_SWIGLU: i32 = 3;
pub const PRO_LAYERNORM: i32 = 4;
pub const PRO_SILU: i32 = 5;
pub const PRO_GELU: i32 = 6;
pub const PRO_ADALN: i32 = 7;
pub const PRO_SITU: i32 = 8;
pub const PRO_LN_MOD: i32 = 9;
pub const PRO_LN_AFFINE: i32 = 10;
pub const PRO_GELU_TANH: i32 = 11;
pub const PRO_LN_AFFINE_SILU: i32 = 12;
/// accepted by `gpu_quant_rows` only; this library evaluates it with `PRO_SITU`'s accurate expression
pub const PRO_SITU_FAST: i32 = 13;

/// Size in bytes of one element of a dtype code.
pub fn dt_size(dt: i32) -> usize {
    if dt == DT_F32 { 4 } else { 2 }
}

/// Turns a kernel launcher's return value into a `Result`: 0 is success, a positive value is a `hipError_t` from
/// the launch, a negative one is the launcher refusing its arguments (the codes are listed at the top of
/// include/gpu_api.h).
pub fn ok(code: i32, what: &str) -> Result<()> {
    if code == 0 {
        return Ok(());
    }
    if code > 0 {
        bail!("{what}: HIP error {code} ({})", hip::err_str(code));
    }
    bail!("{what}: arguments refused with code {code}");
}

/// `k!(gpu_int8_gemm(a, w, ...))`: the unsafe call and the check of its return code in one expression.  Exported at
/// the crate root (`gpu_kernels_hip::k!`, `crate::k!` inside the crate).
#[macro_export]
macro_rules! k {
    ($f:ident ( $($a:expr),* $(,)? )) => {
        $crate::ffi::ok(unsafe { $crate::ffi::$f($($a),*) }, stringify!($f))
    };
}

/// The stream argument every entry point takes last.
pub fn s(st: &Stream) -> PM {
    st.raw()
}

pub fn null() -> P {
    std::ptr::null()
}

pub fn null_mut() -> PM {
    std::ptr::null_mut()
}
