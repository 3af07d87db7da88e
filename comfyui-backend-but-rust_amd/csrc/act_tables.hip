#include "act_tables.hpp"

#include <mutex>

#include "common.hpp"
#include "rowmath.hpp"

namespace {

enum { T_SIGMOID, T_SILU, T_GELU, T_GELU_TANH, T_SITU_GATE, T_SITU_HIDDEN, T_GELU_F16, T_COUNT };

__global__ void __launch_bounds__(256) fill_tables_kernel(uint16_t* h16, float* f32) {
    const uint32_t bits = blockIdx.x * 256 + threadIdx.x;     // 0..65535
    const float b = bf16_to_f((uint16_t)bits), h = f16_to_f((uint16_t)bits);
    h16[0 * 65536 + bits] = f_to_bf16(sigmoid_f(b));
    h16[1 * 65536 + bits] = f_to_bf16(silu_f(b));
    h16[2 * 65536 + bits] = f_to_bf16(gelu_f(b));
    h16[3 * 65536 + bits] = f_to_bf16(gelu_tanh_f(b));
    h16[4 * 65536 + bits] = f_to_f16(gelu_f(h));
    f32[0 * 65536 + bits] = situ_gate_f(b);
    f32[1 * 65536 + bits] = situ_hidden_f(b);
}

constexpr int kMaxDevices = 16;
std::mutex g_mu;
ActTables g_tables[kMaxDevices];
int g_state[kMaxDevices];   // 0 not built (yet), 1 built

}  // namespace

const ActTables* act_tables(hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> hold(g_mu);
    if (g_state[dev] == 1) return &g_tables[dev];
    // Building allocates, launches on the null stream and synchronizes, none of which a stream capture survives: a
    // call made while `stream` is being captured evaluates per element instead, and a later call builds the tables.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (stream && (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone)) return nullptr;
    // A failure (a transient out-of-memory, say) leaves the state at "not built", so that the next call tries again.
    uint16_t* h16 = nullptr;
    float* f32 = nullptr;
    if (hipMalloc(&h16, 5 * 65536 * sizeof(uint16_t)) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    if (hipMalloc(&f32, 2 * 65536 * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(h16);
        return nullptr;
    }
    hipLaunchKernelGGL(fill_tables_kernel, dim3(256), dim3(256), 0, 0, h16, f32);
    if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
        (void)hipFree(h16);
        (void)hipFree(f32);
        return nullptr;
    }
    g_tables[dev] = ActTables{h16, h16 + 65536, h16 + 2 * 65536, h16 + 3 * 65536, f32, f32 + 65536, h16 + 4 * 65536};
    g_state[dev] = 1;
    return &g_tables[dev];
}

// Explicit warm-up for callers that capture graphs or want the first prologue call to be asynchronous like the rest.
GPU_API int gpu_act_tables_init(void) { return act_tables(nullptr) ? 0 : -1; }
