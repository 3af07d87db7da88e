// The ConvRot group rotation of one 1024-value chunk held by a wave, 16 consecutive values per lane: the staged radix-4
// butterflies of csrc/common.cuh:99-126 (left-to-right adds, x0.5 per stage).  Strides 1 and 4 run inside a lane; for the
// wider strides the chunk makes one trip through a wave-private LDS tile so that those butterflies are lane-local too.
#pragma once
#include "common.hpp"

namespace convrot {

constexpr int kChunk = 1024;           // values per wave-chunk (64 lanes x 16)
constexpr int kLdsPerWave = 1024 + 64; // floats: one chunk plus 16 pad floats per 256

// LDS position of chunk element e.  Each lane's 16 consecutive values are four 16-byte vectors; vector i of lane L is
// rotated to slot (i + L/2) & 3 so that 8 neighbouring lanes cover all 32 banks in a 128-bit access, and every 256
// elements are padded by 16 floats so that the stride-16 accesses of the second phase spread over both bank halves.
__device__ __forceinline__ int lds_pos(int e) {
    const int L = e >> 4, i = (e >> 2) & 3, j = e & 3;
    return (L << 4) + (((i + (L >> 1)) & 3) << 2) + j + ((e >> 8) << 4);
}

// h4_row x 4 outputs with the reference's left-to-right adds, scaled by 0.5 (csrc/common.cuh:99-106,119-122).
// HALVE = false leaves the scaling out: the 128-wide transform, which is this library's own definition, applies its three
// halvings together with the closing 1/sqrt(2), in one multiplication per output (bit-identical to halving per stage
// while every intermediate stays in the normal range, and four instructions per butterfly shorter).
template <bool HALVE = true> __device__ __forceinline__ void bfly4(float& a, float& b, float& c, float& d) {
    const float x0 = a, x1 = b, x2 = c, x3 = d;
    const float h = HALVE ? 0.5f : 1.0f;
    a = h * (x0 + x1 + x2 - x3);
    b = h * (x0 + x1 - x2 + x3);
    c = h * (x0 - x1 + x2 + x3);
    d = h * (-x0 + x1 + x2 + x3);
}

// Rotate one chunk held as v[16] per lane (element 16*lane + i).  wl is the wave's LDS tile.
// The LDS tile is private to the wave and the LDS unit executes one wave's accesses in program order, so between the
// phases of rotate_chunk it is enough to stop the compiler from reordering them: no workgroup barrier is needed.
#define LDS_WAVE_ORDER() asm volatile("" ::: "memory")

template <int G> __device__ __forceinline__ void rotate_chunk(float* v, float* wl, int lane) {
    // strides 1 and 4: inside the lane
    constexpr bool HV = G != 128;
#pragma unroll
    for (int i = 0; i < 4; ++i) bfly4<HV>(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
#pragma unroll
    for (int j = 0; j < 4; ++j) bfly4<HV>(v[j], v[j + 4], v[j + 8], v[j + 12]);
    // to LDS in row order
#pragma unroll
    for (int i = 0; i < 4; ++i)
        *reinterpret_cast<float4*>(wl + lds_pos(16 * lane + 4 * i)) = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    LDS_WAVE_ORDER();
    if (G == 256) {
        // lane (R = lane/16, b = lane%16) takes elements R*256 + a*16 + b, a = 0..15: strides 16 and 64 are lane-local
        const int base = (lane >> 4) * 256 + (lane & 15);
        float w[16];
#pragma unroll
        for (int a = 0; a < 16; ++a) w[a] = wl[lds_pos(base + a * 16)];
#pragma unroll
        for (int i = 0; i < 4; ++i) bfly4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
#pragma unroll
        for (int j = 0; j < 4; ++j) bfly4(w[j], w[j + 4], w[j + 8], w[j + 12]);
#pragma unroll
        for (int a = 0; a < 16; ++a) wl[lds_pos(base + a * 16)] = w[a];
    } else if (G == 64) {
        // lane (Q = lane/4, p = lane%4) takes elements Q*64 + d*16 + 4p + j: stride 16 is lane-local
        const int base = (lane >> 2) * 64 + (lane & 3) * 4;
        float4 w[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) w[d] = *reinterpret_cast<float4*>(wl + lds_pos(base + d * 16));
        bfly4(w[0].x, w[1].x, w[2].x, w[3].x);
        bfly4(w[0].y, w[1].y, w[2].y, w[3].y);
        bfly4(w[0].z, w[1].z, w[2].z, w[3].z);
        bfly4(w[0].w, w[1].w, w[2].w, w[3].w);
#pragma unroll
        for (int d = 0; d < 4; ++d) *reinterpret_cast<float4*>(wl + lds_pos(base + d * 16)) = w[d];
    } else {
        // G == 128: lane (O = lane/8, p = lane%8) takes O*128 + t*64 + d*16 + 2p + j: stride 16 (radix 4) and the
        // closing radix-2 stage at stride 64; every output is then scaled once, by fl(1/sqrt(2)) / 8
        const int base = (lane >> 3) * 128 + (lane & 7) * 2;
        float2 w[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int d = 0; d < 4; ++d) w[t][d] = *reinterpret_cast<float2*>(wl + lds_pos(base + t * 64 + d * 16));
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            bfly4<false>(w[t][0].x, w[t][1].x, w[t][2].x, w[t][3].x);
            bfly4<false>(w[t][0].y, w[t][1].y, w[t][2].y, w[t][3].y);
        }
        const float c = 0.70710678118654752f * 0.125f;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const float ax = w[0][d].x, bx = w[1][d].x, ay = w[0][d].y, by = w[1][d].y;
            w[0][d].x = (ax + bx) * c; w[1][d].x = (ax - bx) * c;
            w[0][d].y = (ay + by) * c; w[1][d].y = (ay - by) * c;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int d = 0; d < 4; ++d) *reinterpret_cast<float2*>(wl + lds_pos(base + t * 64 + d * 16)) = w[t][d];
    }
    LDS_WAVE_ORDER();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float4 f = *reinterpret_cast<float4*>(wl + lds_pos(16 * lane + 4 * i));
        v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
    }
    LDS_WAVE_ORDER();
}

}  // namespace convrot
