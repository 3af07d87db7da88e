// Shared device helpers for the gfx950 quantized-linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/gpu_api.h"

#define GPU_API extern "C" __attribute__((visibility("default")))

// Launch check in the reference's convention (csrc/common.cuh:128): a positive hipError_t on failure.
#define KCHECK()                                   \
    do {                                           \
        hipError_t e__ = hipGetLastError();        \
        if (e__ != hipSuccess) return (int)e__;    \
    } while (0)

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// bf16 / f16 <-> f32; the narrowing conversions round to nearest even (v_cvt_pk_bf16_f32 / v_cvt_f16_f32).
__device__ __forceinline__ float bf16_to_f(uint16_t b) { return u2f((uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f_to_bf16(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
__device__ __forceinline__ float f16_to_f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
// The empty asm keeps the compiler from folding a preceding fp32 fma into v_fma_mixlo_f16, which rounds the exact
// fma result to f16 once; the reference rounds to fp32 first and converts afterwards, and ties differ between the two.
__device__ __forceinline__ uint16_t f_to_f16(float v) {
    asm("" : "+v"(v));
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}

// Two floats -> packed bf16 pair (a in the low half), one v_cvt_pk_bf16_f32.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}

// Round a float to the precision of the dtype code and widen back (rnd<T>, csrc/common.cuh:25-28).
template <int DT> __device__ __forceinline__ float rnd_dt(float v) {
    if (DT == DT_BF16) return bf16_to_f(f_to_bf16(v));
    if (DT == DT_F16) return f16_to_f(f_to_f16(v));
    return v;
}
template <int DT> __device__ __forceinline__ float ld_dt(const void* p, int64_t i) {
    if (DT == DT_BF16) return bf16_to_f(((const uint16_t*)p)[i]);
    if (DT == DT_F16) return f16_to_f(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}
template <int DT> __device__ __forceinline__ void st_dt(void* p, int64_t i, float v) {
    if (DT == DT_BF16) ((uint16_t*)p)[i] = f_to_bf16(v);
    else if (DT == DT_F16) ((uint16_t*)p)[i] = f_to_f16(v);
    else ((float*)p)[i] = v;
}
template <int DT> struct dt_size { static constexpr int value = DT == DT_F32 ? 4 : 2; };
