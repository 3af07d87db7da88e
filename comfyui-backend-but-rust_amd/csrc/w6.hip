// 6-bit weight formats of the W6A8 linears.
//
// gpu_w6_decode computes what csrc/h3.cu:11-46 computes: a row of K codes is a nibble plane of K/2 bytes followed by a K/4-byte plane
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

// Expansion of one row is a pure stream: 0.75 B in and 1 B out per weight, so the kernel is arranged around memory
// access width and a short instruction count per code.
//  * A wave owns 2048 consecutive codes of a row; lane l takes codes 32l..32l+31: one 16-byte load from the nibble plane,
//    one 8-byte load from the top-bit plane, two 16-byte stores.  Workgroups walk (row, chunk) pairs grid-stride.
//  * The two-bit fields are spread by table: a top-bit byte covers four codes, and a 256-entry LDS table returns its
//    four fields already sitting at bits 4..5 of the bytes they belong to (even codes in the low half, odd codes in
//    the high half, matching the split of the nibble words into even and odd nibbles).
//  * A code dword then holds four 6-bit codes in its bytes.  Per code: byte -> float (v_cvt_f32_ubyteN), one fma
//    c*s + (128 - 32 s), one median against [1, 255], and v_cvt_pk_u8_f32, which rounds to nearest even and drops the
//    byte into place; a final xor 0x80 per dword turns the biased bytes into two's complement.
// Arithmetic: s = e4m3 has 4 significant bits and |c - 32| <= 32, so (c - 32) * s is exact in fp32, the reference's
// product rounds nothing, and c*s + (128 - 32 s) is the same number plus 128, also exact (23 bits).  Rounding to
// nearest even and clamping to integers commute, and a NaN scale (0x7f / 0xff) takes the median's minimum, 1, which is
// -127 after the xor: what fminf(127, fmaxf(-127, NaN)) gives in the reference (csrc/h3.cu:29-33).
constexpr int kCodesPerLane = 32, kCodesPerWave = 64 * kCodesPerLane;

__device__ __forceinline__ uint32_t w6_four(uint32_t codes, float s, float bias128) {
    uint32_t o = 0;
    o = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(__builtin_fmaf((float)(codes & 0xffu), s, bias128), 1.f, 255.f), 0, o);
    o = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(__builtin_fmaf((float)((codes >> 8) & 0xffu), s, bias128), 1.f, 255.f), 1, o);
    o = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(__builtin_fmaf((float)((codes >> 16) & 0xffu), s, bias128), 1.f, 255.f), 2, o);
    o = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(__builtin_fmaf((float)(codes >> 24), s, bias128), 1.f, 255.f), 3, o);
    return o ^ 0x80808080u;
}

__global__ void __launch_bounds__(256) w6_decode_kernel(const uint8_t* __restrict__ q, const uint8_t* __restrict__ s_rel,
                                                        int8_t* __restrict__ out, int64_t N, int K, int G) {
    __shared__ uint32_t spread[256];
    {   // entry t: fields 0 and 2 of t at bits 4..5 and 12..13, fields 1 and 3 at bits 20..21 and 28..29
        const uint32_t t = threadIdx.x;
        spread[t] = ((t & 3u) << 4) | (((t >> 4) & 3u) << 12) | (((t >> 2) & 3u) << 20) | (((t >> 6) & 3u) << 28);
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int chunks = (K + kCodesPerWave - 1) / kCodesPerWave;
    const int64_t units = N * chunks, stride = (int64_t)gridDim.x * 4;
    const int64_t row_bytes = (int64_t)(K / 4) * 3;
    const int gpr = K / G;
    for (int64_t u = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); u < units; u += stride) {
        const int64_t n = u / chunks;
        const int k0 = (int)(u - n * chunks) * kCodesPerWave + lane * kCodesPerLane;
        if (k0 >= K) continue;                                   // K % 32 == 0: a lane's 32 codes are all in or all out
        const uint8_t* row = q + n * row_bytes;
        const uint4 lo = *reinterpret_cast<const uint4*>(row + (k0 >> 1));
        const uint2 hi = *reinterpret_cast<const uint2*>(row + (K >> 1) + (k0 >> 2));
        // G % 16 == 0: codes k0..k0+15 share a scale and so do k0+16..k0+31
        const float s0 = e4m3_to_f(s_rel[n * gpr + k0 / G]), s1 = e4m3_to_f(s_rel[n * gpr + (k0 + 16) / G]);
        const float b0 = __builtin_fmaf(-32.f, s0, 128.f), b1 = __builtin_fmaf(-32.f, s1, 128.f);   // exact
        const uint32_t lw[4] = {lo.x, lo.y, lo.z, lo.w}, hw[2] = {hi.x, hi.y};
        uint32_t o[8];
#pragma unroll
        for (int w = 0; w < 4; ++w) {                            // nibble word w: codes 8w..8w+7, top bits in 16 bits of hw
            const uint32_t even = lw[w] & 0x0f0f0f0fu, odd = (lw[w] >> 4) & 0x0f0f0f0fu;   // codes 0,2,4,6 / 1,3,5,7 of the word
            const uint32_t t16 = hw[w >> 1] >> (16 * (w & 1));
            const uint32_t l0 = spread[t16 & 0xffu], l1 = spread[(t16 >> 8) & 0xffu];      // codes 0..3 / 4..7
            const uint32_t ce = even | (l0 & 0xffffu) | (l1 << 16);
            const uint32_t co = odd | (l0 >> 16) | (l1 & 0xffff0000u);
            // output dwords hold codes in order: (e0 o0 e1 o1), (e2 o2 e3 o3)
            const uint32_t c0 = __builtin_amdgcn_perm(co, ce, 0x05010400u), c1 = __builtin_amdgcn_perm(co, ce, 0x07030602u);
            const float s = w < 2 ? s0 : s1, b = w < 2 ? b0 : b1;
            o[2 * w] = w6_four(c0, s, b);
            o[2 * w + 1] = w6_four(c1, s, b);
        }
        uint4* dst = reinterpret_cast<uint4*>(out + n * (int64_t)K + k0);
        dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
        dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
    }
}

}  // namespace

GPU_API int gpu_w6_decode(const void* q, const void* s_rel, void* out, int64_t N, int K, int G, void* stream) {
    if (K % 32 || G % 16) return -1;  // csrc/h3.cu:41
    if (N <= 0 || K <= 0) return 0;
    const int64_t waves = N * ((K + kCodesPerWave - 1) / kCodesPerWave);
    const int64_t want = (waves + 3) / 4;
    const unsigned grid = (unsigned)(want < 256 * 16 ? want : 256 * 16);   // grid-stride beyond 16 workgroups per CU
    hipLaunchKernelGGL(w6_decode_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
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
