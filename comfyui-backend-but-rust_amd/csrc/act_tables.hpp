// Lookup tables of the prologue activations over all 65536 values of a 16-bit row dtype.  A 16-bit input has only that
// many values, so R(f(x)) -- f evaluated in fp64 and rounded as the prologue rounds it -- is read from a 128 KB table
// instead of being evaluated per element; the entries are filled on the device by the same routines the element-wise
// path uses, so both give the same bits.  Built once per device at first use (a device allocation and one
// synchronisation: the first call with a prologue must not happen under graph capture).
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

// Tables of the current device, or nullptr if they could not be built (callers then evaluate per element).
const ActTables* act_tables();
