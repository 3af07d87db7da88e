// 6-bit weight formats of the W6A8 linears.
//
// gpu_w6_decode restates csrc/h3.cu:11-46: a row of K codes is a nibble plane of K/2 bytes followed by a K/4-byte plane
// of the top two bits, with one fp8-e4m3 scale per G columns; it expands to the int8 grid round((c - 32) * s), clamped
// to +-127, that the int8 GEMM reads.
#include "common.hpp"

namespace {

// fp8 e4m3 (1-4-3, bias 7, no infinities, S.1111.111 = NaN) -> float, exact.
__device__ __forceinline__ float e4m3_to_f(uint32_t v) {
    const uint32_t s = (v & 0x80u) << 24, e = (v >> 3) & 0xfu, m = v & 7u;
    float f;
    if (e == 0) f = (float)m * 0.001953125f;                     // m/8 * 2^-6
    else if (e == 15 && m == 7) f = u2f(0x7fc00000u);
    else f = u2f(((e + 120u) << 23) | (m << 20));
    return u2f(f2u(f) | s);
}

__device__ __forceinline__ int w6_grid(uint32_t c, float s) {
    return (int)fminf(127.f, fmaxf(-127.f, nearbyintf(((float)c - 32.f) * s)));
}

// One thread expands 16 consecutive codes: 8 nibble bytes + 4 top-bit bytes -> 16 int8.
__global__ void __launch_bounds__(256) w6_decode_kernel(const uint8_t* q, const uint8_t* s_rel, int8_t* out, int64_t N, int K, int G) {
    const int64_t per = K / 16;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N * per) return;
    const int64_t n = i / per;
    const int c = (int)(i - n * per);
    const uint8_t* row = q + n * (int64_t)(K / 4 * 3);
    const uint2 lo = *reinterpret_cast<const uint2*>(row + c * 8);
    const uint32_t hi = *reinterpret_cast<const uint32_t*>(row + K / 2 + c * 4);
    const float s = e4m3_to_f(s_rel[n * (K / G) + c * 16 / G]);
    const uint32_t words[2] = {lo.x, lo.y};
    uint32_t o[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const uint32_t nib = (words[e >> 3] >> (4 * (e & 7))) & 0xfu;
        const uint32_t top = (hi >> (2 * e)) & 3u;
        o[e >> 2] |= ((uint32_t)w6_grid(nib | (top << 4), s) & 0xffu) << (8 * (e & 3));
    }
    *reinterpret_cast<uint4*>(out + n * (int64_t)K + c * 16) = make_uint4(o[0], o[1], o[2], o[3]);
}

}  // namespace

GPU_API int gpu_w6_decode(const void* q, const void* s_rel, void* out, int64_t N, int K, int G, void* stream) {
    if (K % 32 || G % 16) return -1;  // csrc/h3.cu:41
    if (N <= 0 || K <= 0) return 0;
    const int64_t n = N * (K / 16);
    hipLaunchKernelGGL(w6_decode_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)q, (const uint8_t*)s_rel, (int8_t*)out, N, K, G);
    KCHECK();
    return 0;
}

// The W6A8 linear as the reference's model code issues it (src/h3.rs:1208-1216,1251): expand the packed weights to the
// int8 grid, then the ordinary int8 GEMM with the per-row s_channel as the weight scale.  The expanded weights live in
// a stream-ordered scratch allocation that is released on the same stream.
GPU_API int gpu_w6a8_gemm(const int8_t* A, const void* wq, const void* s_rel, int G, const float* xs, const float* s_channel,
                          const void* bias, void* D, int64_t M, int64_t N, int64_t K, int out_dt, void* stream) {
    if (K % 32 || G % 16 || K > 0x7fffffff) return -1;
    if (M == 0 || N == 0 || K == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    int8_t* w8 = nullptr;
    hipError_t e = hipMallocAsync((void**)&w8, (size_t)N * (size_t)K, st);
    if (e != hipSuccess) return (int)e;
    int rc = gpu_w6_decode(wq, s_rel, w8, N, (int)K, G, stream);
    if (rc == 0) rc = gpu_int8_gemm(A, w8, xs, s_channel, bias, D, M, N, K, out_dt, stream);
    e = hipFreeAsync(w8, st);
    if (rc == 0 && e != hipSuccess) rc = (int)e;
    return rc;
}

GPU_API const char* gpu_kernels_build_info(void) { return "gpu_kernels gfx950 quantized-linear " __DATE__; }
