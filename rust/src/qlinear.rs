//! One quantized linear as the model code issues it (the reference's src/dit.rs:550-555, src/unet.rs:436-456,
//! src/h3.rs:1208-1251): quantize the activation rows, then the int8 GEMM with the fused dequantizing epilogue.
//! Everything here is two or three checked calls; the buffers are the caller's.
use crate::ffi::{self, P, PM};
use crate::hip::Stream;
use crate::k;
use anyhow::{ensure, Result};

/// A W8A8 weight resident on the device: int8 [n, k] row-major, one f32 scale per output channel, optional bias in
/// the output dtype.  `rotate` is the Hadamard block the weight was rotated with when it was quantized (0 = none).
pub struct W8Linear {
    pub w: P,
    pub ws: P,
    pub bias: P,
    pub n: i64,
    pub k: i64,
    pub rotate: i32,
}

/// Scratch for one call: int8 codes [m, k] and f32 row scales [m].
pub struct QuantScratch {
    pub q: PM,
    pub scales: PM,
}

impl W8Linear {
    /// d[m, n] (`out_dt`) = dequant(quant(x) . w^T) + bias, for x: T[m, x_stride] with T = `in_dt` (bf16 or f32).
    pub fn forward(&self, in_dt: i32, x: P, x_stride: i64, m: i64, scratch: &QuantScratch, d: PM, out_dt: i32,
        st: &Stream) -> Result<()> {
        ensure!(m <= i32::MAX as i64 && self.k <= 32768, "shape outside the quantizer's range");
        k!(gpu_quant_rows(in_dt, ffi::PRO_PLAIN, x, x_stride, ffi::null(), 0, 0, ffi::null(), 0.0, ffi::null(),
            ffi::null(), scratch.q, scratch.scales, m as i32, self.k as i32, self.rotate, ffi::s(st)))?;
        k!(gpu_int8_gemm(scratch.q as P, self.w, scratch.scales as P, self.ws, self.bias, d, m, self.n, self.k,
            out_dt, ffi::s(st)))
    }

    /// The same with the residual epilogue: d = resid + rscale[n] * round_to_out_dt(linear(x)); `d` may be `resid`.
    pub fn forward_residual(&self, in_dt: i32, x: P, x_stride: i64, m: i64, scratch: &QuantScratch, rscale: P, resid: P,
        d: PM, out_dt: i32, st: &Stream) -> Result<()> {
        ensure!(m <= i32::MAX as i64 && self.k <= 32768, "shape outside the quantizer's range");
        k!(gpu_quant_rows(in_dt, ffi::PRO_PLAIN, x, x_stride, ffi::null(), 0, 0, ffi::null(), 0.0, ffi::null(),
            ffi::null(), scratch.q, scratch.scales, m as i32, self.k as i32, self.rotate, ffi::s(st)))?;
        k!(gpu_int8_gemm_residual(scratch.q as P, self.w, scratch.scales as P, self.ws, self.bias, rscale, resid, d, m,
            self.n, self.k, out_dt, ffi::s(st)))
    }

    /// For callers that may not allocate (graph capture, serving loops): the same result through
    /// `gpu_int8_gemm_static`, which refuses (-200 / -210) what would need scratch beyond the library's own.
    pub fn forward_no_alloc(&self, in_dt: i32, x: P, x_stride: i64, m: i64, scratch: &QuantScratch, d: PM, out_dt: i32,
        st: &Stream) -> Result<()> {
        ensure!(m <= i32::MAX as i64 && self.k <= 32768, "shape outside the quantizer's range");
        k!(gpu_quant_rows(in_dt, ffi::PRO_PLAIN, x, x_stride, ffi::null(), 0, 0, ffi::null(), 0.0, ffi::null(),
            ffi::null(), scratch.q, scratch.scales, m as i32, self.k as i32, self.rotate, ffi::s(st)))?;
        k!(gpu_int8_gemm_static(scratch.q as P, self.w, scratch.scales as P, self.ws, self.bias, d, m, self.n, self.k,
            out_dt, ffi::s(st)))
    }
}

/// A W6A8 weight with group scales: 24-bit words of four 6-bit codes [n, 3k/4], f32 scales [n, k/128].
pub struct W6GroupLinear {
    pub packed: P,
    pub sw: P,
    pub bias: P,
    pub n: i64,
    pub k: i64,
    pub rotate: i32,
}

impl W6GroupLinear {
    pub fn forward(&self, in_dt: i32, x: P, x_stride: i64, m: i64, scratch: &QuantScratch, d: PM, out_dt: i32,
        st: &Stream) -> Result<()> {
        ensure!(m <= i32::MAX as i64 && self.k <= 32768 && self.k % 128 == 0, "shape outside the kernels' range");
        k!(gpu_quant_rows(in_dt, ffi::PRO_PLAIN, x, x_stride, ffi::null(), 0, 0, ffi::null(), 0.0, ffi::null(),
            ffi::null(), scratch.q, scratch.scales, m as i32, self.k as i32, self.rotate, ffi::s(st)))?;
        k!(gpu_w6a8_group_gemm(scratch.q as P, self.packed, scratch.scales as P, self.sw, self.bias, d,
            ffi::null_mut(), m, self.n, self.k, out_dt, ffi::s(st)))
    }
}
