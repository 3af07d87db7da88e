// W6 requantizer for the reference's two-plane format: a bf16 weight in its original basis -> ConvRot256 -> 6-bit codes
// (nibble plane, then 2-bit plane), one fp8-e4m3 relative scale per 32 columns, one fp32 scale per row.  Replaces
// gpu_w6_requant, csrc/vendor/w6a8_requant.cu: same steps and float expressions (cited by line), one workgroup per row.
// A load-time / LoRA-bake kernel: 1.5 B read + 0.78 B written per weight, bound by its arithmetic, not by HBM.
#include "common.hpp"
#include "convrot.hpp"

namespace {

constexpr int kG = 32;   // columns per relative scale

__device__ __forceinline__ uint32_t pcg(uint32_t x) {                            // :21-25
    x = x * 747796405u + 2891336453u;
    const uint32_t w = ((x >> ((x >> 28u) + 4u)) ^ x) * 277803737u;
    return (w >> 22u) ^ w;
}
__device__ __forceinline__ float uniform01(int64_t idx, uint64_t seed) {          // :27-31
    return (float)(pcg((uint32_t)idx ^ (uint32_t)seed ^ (uint32_t)(seed >> 32)) >> 8) * (1.0f / 16777216.0f);
}
// float -> fp8 e4m3 bits, round to nearest even, saturating at 448 (finite inputs)
__device__ __forceinline__ uint32_t f_to_e4m3(float x) {
    const uint32_t sgn = (f2u(x) >> 31) << 7;
    const float a = fabsf(x);
    if (a != a) return sgn | 0x7f;
    if (a > 448.f) return sgn | 0x7e;
    if (a < 0.015625f) return sgn | (uint32_t)nearbyintf(a * 512.f);
    const uint32_t u = f2u(a);
    int e = (int)(u >> 23) - 127;
    const float frac = u2f((u & 0x007fffffu) | 0x3f800000u);                     // in [1, 2)
    int m = (int)nearbyintf((frac - 1.f) * 8.f);
    if (m == 8) { m = 0; ++e; }
    const uint32_t code = ((uint32_t)(e + 7) << 3) | (uint32_t)m;
    return sgn | (code > 0x7e ? 0x7e : code);
}
__device__ __forceinline__ float e4m3_to_f(uint32_t v) {
    const uint32_t e = (v >> 3) & 0xf, m = v & 7;
    const float f = e == 0 ? (float)m * 0.001953125f : (e == 15 && m == 7) ? __builtin_nanf("") : u2f(((e + 120) << 23) | (m << 20));
    return (v & 0x80) ? -f : f;
}
__device__ __forceinline__ float level(int i, float s) {                          // :59-61
    return fminf(127.0f, fmaxf(-127.0f, nearbyintf((float)(i - 31) * s)));
}
__device__ __forceinline__ int lower_bound(float t, float s, float inv_s) {       // :63-69
    const float est = nearbyintf((ceilf(t) - 0.5f) * inv_s);
    int i = (est > 2.0e9f ? 2000000000 : est < -2.0e9f ? -2000000000 : (int)est) + 31;
    i = min(max(i, 0), 63);
    while (i > 0 && level(i - 1, s) >= t) --i;
    while (i < 63 && level(i, s) < t) ++i;
    return i;
}
__global__ void __launch_bounds__(256) w6_requant_kernel(const uint16_t* w, uint8_t* packed, uint8_t* s_rel, float* s_channel, int K,
                                                        uint64_t seed) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    __shared__ float red[4];
    float* row = smem;                                  // [K]
    float* gscale = smem + K;                           // [K / 32]
    float* tiles = smem + K + K / kG;                   // four wave-private rotation tiles, 16-byte aligned (K % 256 == 0)
    const int64_t n = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // ConvRot256 (:174-206) as the row quantizer does it: a wave per chunk of 1024 values, 16 consecutive values per
    // lane, strides 1 and 4 inside the lane and one trip through the wave's LDS tile for strides 16 and 64; the
    // rotated row is kept in the weight dtype (:209-217).
    for (int c = wave; c * convrot::kChunk < K; c += 4) {
        const int e0 = c * convrot::kChunk + lane * 16;
        float v[16];
        if (e0 < K) {                                   // K % 256 == 0: a lane's 16 values are all in or all out
            const uint4* src = reinterpret_cast<const uint4*>(w + n * K + e0);
            const uint4 a = src[0], b = src[1];
            const uint32_t ww[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[2 * i] = u2f(ww[i] << 16);
                v[2 * i + 1] = u2f(ww[i] & 0xffff0000u);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = 0.f;
        }
        convrot::rotate_chunk<256>(v, tiles + wave * convrot::kLdsPerWave, lane);
        if (e0 < K) {
#pragma unroll
            for (int i = 0; i < 16; i += 4)
                *reinterpret_cast<float4*>(row + e0 + i) = make_float4(rnd_dt<DT_BF16>(v[i]), rnd_dt<DT_BF16>(v[i + 1]),
                                                                       rnd_dt<DT_BF16>(v[i + 2]), rnd_dt<DT_BF16>(v[i + 3]));
        }
    }
    __syncthreads();

    // phase 1: per-group step by two alternating-least-squares rounds; row maximum of the decoded weight, :94-120
    const int groups = K / kG;
    float amax_t = 0.f;
    for (int g = tid; g < groups; g += 256) {
        const float* x = row + g * kG;
        float amax = 0.f;
        for (int i = 0; i < kG; ++i) amax = fmaxf(amax, fabsf(x[i]));
        float gs = fmaxf(amax / 31.0f, 1e-8f), inv = 1.0f / gs;
        for (int it = 0; it < 2; ++it) {
            float num = 0.f, den = 0.f;
            for (int i = 0; i < kG; ++i) {
                const float q = fminf(31.0f, fmaxf(-31.0f, nearbyintf(x[i] * inv)));
                num = __builtin_fmaf(x[i], q, num);
                den = __builtin_fmaf(q, q, den);
            }
            gs = fmaxf(num / fmaxf(den, 1e-8f), 1e-8f);
            inv = 1.0f / gs;
        }
        gscale[g] = gs;
        for (int i = 0; i < kG; ++i) amax_t = fmaxf(amax_t, fabsf(fminf(31.0f, fmaxf(-31.0f, nearbyintf(x[i] * inv))) * gs));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax_t = fmaxf(amax_t, __shfl_xor(amax_t, o, 64));
    if ((tid & 63) == 0) red[tid >> 6] = amax_t;
    __syncthreads();
    const float sc = fmaxf(fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) / 127.0f, 1e-8f);   // :121
    const float inv_sc = 1.0f / sc;
    if (tid == 0) s_channel[n] = sc;

    // phase 2: e4m3 relative scale, stochastic assignment between the two bracketing levels, code = level + 1, pack: :126-151
    uint8_t* lo_plane = packed + n * (int64_t)(K * 3 / 4);
    uint8_t* hi_plane = lo_plane + K / 2;
    for (int g = tid; g < groups; g += 256) {
        const uint32_t bits = f_to_e4m3(gscale[g] / sc);
        s_rel[n * groups + g] = (uint8_t)bits;
        const float sr = e4m3_to_f(bits), inv_sr = 1.0f / fmaxf(sr, 1e-30f);
        const int base = g * kG;
#pragma unroll 1
        for (int p4 = 0; p4 < kG / 4; ++p4) {
            uint32_t u[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = base + 4 * p4 + j;
                const float t = row[e] * inv_sc;
                const int pos = lower_bound(t, sr, inv_sr);
                const int l = min(max(pos - 1, 0), 61);                           // :75-80
                const float l0 = level(l, sr);
                const float thr = __builtin_fmaf(uniform01(n * K + e, seed), level(l + 1, sr) - l0, l0);
                u[j] = (uint32_t)min(l + (t > thr ? 1 : 0), 62) + 1u;
            }
            lo_plane[g * (kG / 2) + 2 * p4] = (uint8_t)((u[0] & 0xF) | ((u[1] & 0xF) << 4));
            lo_plane[g * (kG / 2) + 2 * p4 + 1] = (uint8_t)((u[2] & 0xF) | ((u[3] & 0xF) << 4));
            hi_plane[g * (kG / 4) + p4] = (uint8_t)((u[0] >> 4) | ((u[1] >> 4) << 2) | ((u[2] >> 4) << 4) | ((u[3] >> 4) << 6));
        }
    }
}

}  // namespace

// weight bf16 [N, K] -> packed [N, 3K/4], s_rel e4m3 [N, K/32], s_channel f32 [N].  Rounding is always stochastic, keyed by
// element index and seed, as in the reference's launcher (csrc/vendor/w6a8_requant.cu:242-251).
GPU_API int gpu_w6_requant(const void* weight, void* packed, void* s_rel, void* s_channel, int64_t N, int K, uint64_t seed,
                           void* stream) {
    if (K <= 0 || K % 256) return -1;
    const size_t smem = (size_t)(K + K / kG + 4 * convrot::kLdsPerWave) * sizeof(float);
    constexpr size_t kMaxDynamic = 160 * 1024 - 256;   // the kernel also has a few bytes of static LDS
    if (smem > kMaxDynamic || N > 0x7fffffff) return -2;
    if (N <= 0) return 0;
    static PerDeviceOnce once;
    if (const int e = allow_dynamic_lds((const void*)w6_requant_kernel, (int)kMaxDynamic, once)) return e;
    hipLaunchKernelGGL(w6_requant_kernel, dim3((unsigned)N), dim3(256), smem, (hipStream_t)stream, (const uint16_t*)weight,
                       (uint8_t*)packed, (uint8_t*)s_rel, (float*)s_channel, K, seed);
    KCHECK();
    return 0;
}
