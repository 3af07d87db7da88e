// Lookup tables of the prologue activations over all 65536 values of a 16-bit row dtype.  A 16-bit input has only that
// many values, so R(f(x)) -- f evaluated in fp64 and rounded as the prologue rounds it -- is read from a 128 KB table
// instead of being evaluated per element; the entries are filled on the device by the same routines the element-wise
// path uses, so both give the same bits.  Built once per device, by gpu_act_tables_init() or at the first prologue call
// (two device allocations that live until the process ends, and one synchronisation); a call made while its stream
// is being captured does not build them and evaluates per element.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

struct ActTables {
    // bf16 input bits -> bf16 bits of rnd(f(x))
    const uint16_t* sigmoid_bf16;
    const uint16_t* silu_bf16;
    const uint16_t* gelu_bf16;
    const uint16_t* gelu_tanh_bf16;
    // bf16 input bits -> fp32 factors of situ_f: 4 tanh(g/4) / (1 + exp(-g)) and 25 tanh(h/25)
    const float* situ_gate_bf16;
    const float* situ_hidden_bf16;
    // f16 input bits -> f16 bits of rnd(gelu(x))
    const uint16_t* gelu_f16;
};

// Tables of the current device, or nullptr if they are not built and cannot be built now (`stream` is being captured,
// or an allocation failed: callers then evaluate per element, and a later call tries again).
const ActTables* act_tables(hipStream_t stream);
