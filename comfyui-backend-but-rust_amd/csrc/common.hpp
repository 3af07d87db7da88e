// Shared device helpers for the gfx950 quantized-linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/gpu_api.h"

#define GPU_API extern "C" __attribute__((visibility("default")))

// Launch check in the reference's convention (csrc/common.cuh:128): a positive hipError_t on failure.
#define KCHECK()                                   \
    do {                                           \
        hipError_t e__ = hipGetLastError();        \
        if (e__ != hipSuccess) return (int)e__;    \
    } while (0)

// "Done once per device" flags for host-side set-up (a kernel's dynamic LDS limit, a memory pool attribute): one bit per
// device ordinal, set after the call has succeeded on that device.  Two threads that race both make the call, which is
// idempotent.  Devices past 63 are not remembered and make the call every time.
struct PerDeviceOnce {
    std::atomic<uint64_t> done{0};
    static int current() {
        int dev = 0;
        return hipGetDevice(&dev) == hipSuccess ? dev : -1;
    }
    bool is_done(int dev) const { return dev >= 0 && dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1u); }
    void mark(int dev) { if (dev >= 0 && dev < 64) done.fetch_or((uint64_t)1 << dev, std::memory_order_release); }
};
// Raises a kernel's dynamic LDS limit on the current device, the first time it is asked for there.  0 or a hipError_t.
inline int allow_dynamic_lds(const void* kern, int bytes, PerDeviceOnce& once) {
    const int dev = PerDeviceOnce::current();
    if (once.is_done(dev)) return 0;
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return (int)e;
    once.mark(dev);
    return 0;
}

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

// Workgroup -> tile.  Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so first renumber them
// XCD-contiguously, then walk tiles in panels of 4 tile rows so that the 32 workgroups an XCD runs at once cover a
// 4 x 8 patch of tiles and share A rows / W rows in that XCD's L2.
// A persistent kernel calls this three times per tile (two operand streams and the epilogue), and two integer divisions
// are about a hundred dependent scalar instructions each time, so the divisions are multiplications: `magic` =
// panel_magic(tiles_m, tiles_n) from the host turns lin / (4 * tiles_n) into a multiply-high, and the rows of a panel
// are 4, or 1..3 in the last one.  magic == 0 (shapes beyond the multiply's exact range) divides.
__host__ __device__ inline uint32_t panel_magic(int tiles_m, int tiles_n) {
    // floor(n / d) == (n * ceil(2^32 / d)) >> 32 for n, d <= 65536
    const int64_t per_panel = 4 * (int64_t)tiles_n, ntiles = (int64_t)tiles_m * tiles_n;
    if (per_panel > 65536 || ntiles > 65536) return 0;
    return (uint32_t)(((1ull << 32) + (uint64_t)per_panel - 1) / (uint64_t)per_panel);
}
__device__ __forceinline__ void tile_of_block(int b, int nblocks, int tiles_m, int tiles_n, int& tm, int& tn, uint32_t magic = 0) {
    const int base = nblocks >> 3, rem = nblocks & 7;
    const int xcd = b & 7, idx = b >> 3;
    const int lin = xcd * base + (xcd < rem ? xcd : rem) + idx;
    constexpr int GM = 4;
    const int per_panel = GM * tiles_n;
    const int panel = magic ? (int)__umulhi((uint32_t)lin, magic) : lin / per_panel;
    const int first_m = panel * GM;
    const int rows = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int in_panel = lin - panel * per_panel;
    int q;   // in_panel / rows
    if (rows == 4) q = in_panel >> 2;
    else if (rows == 2) q = in_panel >> 1;
    else if (rows == 1) q = in_panel;
    else if (magic) q = (int)__umulhi((uint32_t)in_panel, 0x55555556u);   // rows == 3, in_panel < 65536
    else q = in_panel / rows;
    tm = first_m + in_panel - q * rows;
    tn = q;
}


// Four consecutive elements of a dtype-coded array <-> four floats (8- or 16-byte vector access).
template <int OUT_DT> __device__ __forceinline__ void load4(const void* p, int64_t i, float* v) {
    if (OUT_DT == DT_F32) {
        const float4 f = *reinterpret_cast<const float4*>((const float*)p + i);
        v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
    } else {
        const uint2 u = *reinterpret_cast<const uint2*>((const uint16_t*)p + i);
        if (OUT_DT == DT_BF16) {
            v[0] = u2f(u.x << 16); v[1] = u2f(u.x & 0xffff0000u); v[2] = u2f(u.y << 16); v[3] = u2f(u.y & 0xffff0000u);
        } else {
            v[0] = f16_to_f((uint16_t)(u.x & 0xffffu)); v[1] = f16_to_f((uint16_t)(u.x >> 16));
            v[2] = f16_to_f((uint16_t)(u.y & 0xffffu)); v[3] = f16_to_f((uint16_t)(u.y >> 16));
        }
    }
}
template <int OUT_DT> __device__ __forceinline__ void store4(void* p, int64_t i, const float* v) {
    if (OUT_DT == DT_F32) {
        *reinterpret_cast<float4*>((float*)p + i) = make_float4(v[0], v[1], v[2], v[3]);
    } else if (OUT_DT == DT_BF16) {
        uint2 u;
        u.x = pack_bf16x2(v[0], v[1]);
        u.y = pack_bf16x2(v[2], v[3]);
        *reinterpret_cast<uint2*>((uint16_t*)p + i) = u;
    } else {
        uint2 u;
        u.x = (uint32_t)f_to_f16(v[0]) | ((uint32_t)f_to_f16(v[1]) << 16);
        u.y = (uint32_t)f_to_f16(v[2]) | ((uint32_t)f_to_f16(v[3]) << 16);
        *reinterpret_cast<uint2*>((uint16_t*)p + i) = u;
    }
}

