#include "act_tables.hpp"

#include <atomic>
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
std::atomic<int> g_state[kMaxDevices];   // 0 not built (yet), 1 built; read without the lock, written under it

}  // namespace

const ActTables* act_tables(hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    if (g_state[dev].load(std::memory_order_acquire) == 1) return &g_tables[dev];
    // Building allocates and waits for a fill kernel, which a capture of `stream` does not survive: a call made while
    // `stream` is being captured evaluates per element instead, and a later call builds the tables.  A capture on another
    // stream (in the global mode every thread's allocations are illegal while it runs) is kept intact by switching this
    // thread to the relaxed capture mode for the length of the build.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (stream && (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone)) return nullptr;
    std::lock_guard<std::mutex> hold(g_mu);
    if (g_state[dev].load(std::memory_order_acquire) == 1) return &g_tables[dev];
    struct RelaxedCapture {   // calls that are unsafe under another stream's capture become legal for this thread
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        bool swapped;
        RelaxedCapture() { swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess; }
        ~RelaxedCapture() { if (swapped) (void)hipThreadExchangeStreamCaptureMode(&mode); }
    } relaxed;
    // A failure (a transient out-of-memory, say) leaves the state at "not built", so that the next call tries again.
    uint16_t* h16 = nullptr;
    float* f32 = nullptr;
    if (hipMalloc(&h16, 5 * 65536 * sizeof(uint16_t)) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    if (hipMalloc(&f32, 2 * 65536 * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(h16);
        return nullptr;
    }
    // filled on a stream of its own that does not synchronize with the null stream, so that the work of other streams
    // (one of which may be capturing) is neither waited for nor disturbed
    hipStream_t fill = nullptr;
    bool ok = hipStreamCreateWithFlags(&fill, hipStreamNonBlocking) == hipSuccess;
    if (ok) {
        hipLaunchKernelGGL(fill_tables_kernel, dim3(256), dim3(256), 0, fill, h16, f32);
        ok = hipGetLastError() == hipSuccess && hipStreamSynchronize(fill) == hipSuccess;
        (void)hipStreamDestroy(fill);
    }
    if (!ok) {
        (void)hipGetLastError();
        (void)hipFree(h16);
        (void)hipFree(f32);
        return nullptr;
    }
    g_tables[dev] = ActTables{h16, h16 + 65536, h16 + 2 * 65536, h16 + 3 * 65536, f32, f32 + 65536, h16 + 4 * 65536};
    g_state[dev].store(1, std::memory_order_release);
    return &g_tables[dev];
}

// Explicit warm-up for callers that capture graphs or want the first prologue call to be asynchronous like the rest.
GPU_API int gpu_act_tables_init(void) { return act_tables(nullptr) ? 0 : -1; }
