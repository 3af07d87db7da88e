// The activation functions of the row prologues (csrc/common.cuh:71-95), shared by the prologue kernels and the quantizer.
// exp, expm1, erf and tanh are evaluated in fp64 and rounded to fp32, i.e. correctly rounded fp32 functions: the
// reference calls CUDA's expf / erff / tanhf, 1-2 ulp routines whose bits only a run could show.
#pragma once
#include "common.hpp"

// Kept out of line: the fp64 routines are long, and the callers evaluate them 16 times per lane in many kernel variants.
static __device__ __attribute__((noinline)) float exp_cr(float x) { return (float)exp((double)x); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.f + exp_cr(-x)); }          // csrc/common.cuh:71
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + exp_cr(-x)); }     // :72
static __device__ __attribute__((noinline)) float stable_tanh(float x) {                                      // :74-77
    const float t = (float)expm1((double)(-2.f * fabsf(x)));
    return copysignf(-t / (t + 2.f), x);
}
static __device__ __attribute__((noinline)) float gelu_f(float x) { return 0.5f * x * (1.f + (float)erf((double)(x * 0.70710678118654752f))); }  // :91
static __device__ __attribute__((noinline)) float gelu_tanh_f(float x) {                                      // :92-95
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    return 0.5f * x * (1.f + (float)tanh((double)(k0 * __builtin_fmaf(k1 * x * x, x, x))));
}

// MOSS Image's soft-capped gated activation as one float expression, csrc/common.cuh:80-82:
//   4.f * stable_tanh(gate / 4.f) / (1.f + expf(-gate)) * (25.f * stable_tanh(hidden / 25.f))
// evaluated left to right: (gate factor) * (hidden factor), each an fp32 value of one argument.
__device__ __forceinline__ float situ_gate_f(float gate) { return 4.f * stable_tanh(gate / 4.f) / (1.f + exp_cr(-gate)); }
__device__ __forceinline__ float situ_hidden_f(float hidden) { return 25.f * stable_tanh(hidden / 25.f); }
__device__ __forceinline__ float situ_f(float hidden, float gate) { return situ_gate_f(gate) * situ_hidden_f(hidden); }
