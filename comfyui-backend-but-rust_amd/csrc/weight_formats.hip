// Weight-side kernels around the int8 formats: int8 rows back to floats, with and without the ConvRot rotation
// (H256 is its own inverse, so rotating q * s gives the weight in its original basis).
#include "common.hpp"
#include "convrot.hpp"

namespace {
using namespace convrot;

enum { OUT_F32 = 0, OUT_BF16 = 1, OUT_F32_OF_BF16 = 2 };

// One wave per (row, 1024-value chunk): out = H256(q * s[row]).
template <int OUT>
__global__ void __launch_bounds__(256) convrot_dequant_kernel(const int8_t* q, const float* s, void* out, int64_t N, int K, int cpr) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float* wl = lds + wave * kLdsPerWave;
    const int64_t gid = (int64_t)blockIdx.x * 4 + wave;
    const int64_t m = gid / cpr;
    const int e0 = (int)(gid % cpr) * kChunk + lane * 16;
    const bool act = m < N && e0 < K;     // a wave past the last row still runs the (barrier-free) rotation on zeros
    float v[16];
    if (act) {
        const float sc = s[m];
        const uint4 u = *reinterpret_cast<const uint4*>(q + m * K + e0);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = (float)(int8_t)(w[i >> 2] >> (8 * (i & 3))) * sc;   // csrc/kernels.cu:1350
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = 0.f;
    }
    rotate_chunk<256>(v, wl, lane);
    if (!act) return;
    if (OUT == OUT_BF16) {
        uint32_t w[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) w[i] = (uint32_t)f_to_bf16(v[2 * i]) | ((uint32_t)f_to_bf16(v[2 * i + 1]) << 16);
        uint4* o = reinterpret_cast<uint4*>((uint16_t*)out + m * K + e0);
        o[0] = make_uint4(w[0], w[1], w[2], w[3]);
        o[1] = make_uint4(w[4], w[5], w[6], w[7]);
    } else {
        float4* o = reinterpret_cast<float4*>((float*)out + m * K + e0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float4 f = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
            if (OUT == OUT_F32_OF_BF16) {   // the table's original dtype was bf16, csrc/kernels.cu:629-630
                f.x = rnd_dt<DT_BF16>(f.x); f.y = rnd_dt<DT_BF16>(f.y); f.z = rnd_dt<DT_BF16>(f.z); f.w = rnd_dt<DT_BF16>(f.w);
            }
            o[i] = f;
        }
    }
}

template <int OUT>
int launch_dequant(const void* q, const void* s, void* out, int64_t N, int K, hipStream_t st) {
    if (K <= 0 || (K % 256) != 0) return -1;
    if (N <= 0) return 0;
    const int cpr = (K + kChunk - 1) / kChunk;
    const int64_t waves = N * cpr;
    const int64_t grid = (waves + 3) / 4;
    if (grid > 0x7fffffff) return -2;
    hipLaunchKernelGGL(convrot_dequant_kernel<OUT>, dim3((unsigned)grid), dim3(256), 4 * kLdsPerWave * sizeof(float), st,
                       (const int8_t*)q, (const float*)s, out, N, K, cpr);
    KCHECK();
    return 0;
}

// int8 [N, K] * s[row] -> fp32, 16 values per thread (4 when the row length is not a multiple of 16)
template <int V>
__global__ void __launch_bounds__(256) dequant_i8_kernel(const int8_t* q, const float* s, float* out, int64_t total, int64_t K) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= total) return;
    const float sc = s[i / K];
    if (V == 16) {
        const uint4 u = *reinterpret_cast<const uint4*>(q + i);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            reinterpret_cast<float4*>(out + i)[j] =
                make_float4((float)(int8_t)w[j] * sc, (float)(int8_t)(w[j] >> 8) * sc, (float)(int8_t)(w[j] >> 16) * sc,
                            (float)(int8_t)(w[j] >> 24) * sc);
    } else {
        const uint32_t w = *reinterpret_cast<const uint32_t*>(q + i);
        *reinterpret_cast<float4*>(out + i) = make_float4((float)(int8_t)w * sc, (float)(int8_t)(w >> 8) * sc,
                                                          (float)(int8_t)(w >> 16) * sc, (float)(int8_t)(w >> 24) * sc);
    }
}

}  // namespace

// Replaces gpu_dequant_i8, csrc/kernels.cu:329-343.
GPU_API int gpu_dequant_i8(const int8_t* q, const float* s, float* out, int64_t N, int64_t K, void* stream) {
    if (K <= 0 || K % 4) return -1;
    if (N <= 0) return 0;
    const int64_t total = N * K;
    const int v = K % 16 == 0 ? 16 : 4;
    const int64_t grid = (total / v + 255) / 256;
    if (grid > 0x7fffffff) return -2;
    if (v == 16) hipLaunchKernelGGL(dequant_i8_kernel<16>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, q, s, out, total, K);
    else hipLaunchKernelGGL(dequant_i8_kernel<4>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, q, s, out, total, K);
    KCHECK();
    return 0;
}

// Replaces gpu_embed_dequant, csrc/kernels.cu:620-639: rows of a ConvRot int8 embedding table -> fp32 rows holding bf16
// values.  rotate == 0 is refused as there; K must be a multiple of 256 (the reference assumes it).
GPU_API int gpu_embed_dequant(const int8_t* q, const float* s, float* out, int M, int K, int rotate, void* stream) {
    if (!rotate) return -1;
    return launch_dequant<OUT_F32_OF_BF16>(q, s, out, M, K, (hipStream_t)stream);
}

// Replaces gpu_convrot_dequant, csrc/kernels.cu:1345-1407: the weight in its original basis, fp32 or (any other dtype
// code, as there) bf16.
GPU_API int gpu_convrot_dequant(int dtype, const void* q, const void* s, void* out, int64_t N, int K, void* stream) {
    return dtype == DT_F32 ? launch_dequant<OUT_F32>(q, s, out, N, K, (hipStream_t)stream)
                           : launch_dequant<OUT_BF16>(q, s, out, N, K, (hipStream_t)stream);
}
