// W6A8 linear with 6-bit weights packed four codes to three bytes and fp32 scales per group of 128 along K: the
// unpack to int8 happens in LDS, ahead of the MFMA, inside the GEMM kernel.  The format is this library's own (the
// reference's W6 layout is the two-plane one of csrc/h3.cu:8-37, served by gpu_w6_decode / gpu_w6a8_gemm):
//
//   Wp  uint8 [N, 3K/4]   codes u = q + 32, q in [-32, 31]; every 3 bytes are the little-endian 24-bit word
//                         u0 | u1 << 6 | u2 << 12 | u3 << 18 of four consecutive k
//   sw  f32   [N, K/128]  one scale per output channel and group
//   D[m,n] = Out(fma(accf, xs[m], bias[n])),  accf = fma(float(p_g), sw[n,g], accf) for g = 0, 1, ... from accf = 0,
//   p_g = sum over the 128 k of group g of A[m,k] * q[n,k], an exact int32.
//
// One K tile of the kernel is one group, so every group's int32 partial is a fresh MFMA accumulation (first MFMA with
// C = 0) that is folded into the fp32 accumulators while the next partials are being multiplied.  Per iteration:
//   * LDS-DMA brings A(g+1) (256 x 128 int8), the packed weights of group g+2 (128 rows x 96 bytes) and the 128 scales
//     of group g+1 straight into LDS;
//   * every thread expands four 12-byte pieces of the packed weights of group g+1 into 16 int8 each and writes them
//     in the swizzled fragment layout (conflict-free both ways);
//   * each wave (2 x 2 grid, 128 x 64 outputs, 8 MFMA tiles) multiplies group g in four pairs of tiles; the
//     fp32 scaling of a pair rides between the MFMAs of the next pair.
// The scaling costs two VALU operations per output and group and the unpack about ten per four codes, together more
// issue slots than the MFMAs themselves: the kernel is bound by VALU issue, not by the matrix pipe.
#include "common.hpp"

#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

namespace {

struct W6Args {
    const int8_t* A;
    const uint8_t* Wp;
    const float* xs;
    const float* sw;
    const void* bias;
    void* D;
    int32_t* partials;
    int M, N, K, ng;
    int tiles_m, tiles_n;
};

constexpr int BM = 256, BN = 128, BK = 128, RAW_ROW = 96;
constexpr int A_STAGE = BM * BK, U_STAGE = BN * BK, R_STAGE = BN * RAW_ROW, S_STAGE = BN * 4;
constexpr int U_BASE = 2 * A_STAGE, R_BASE = U_BASE + 2 * U_STAGE, S_BASE = R_BASE + 2 * R_STAGE;
constexpr int SMEM = S_BASE + 2 * S_STAGE;
constexpr int TM = 4, TN = 2;   // 32x32 MFMA tiles of one wave: 128 rows (m) x 64 columns (n)

// Four 6-bit fields of a 24-bit word (bits above 23 are ignored) -> four int8 q = u - 32, one per byte.
__device__ __forceinline__ int spread6(uint32_t w) {
    const uint32_t x = (w & 0x00000fffu) | ((w << 4) & ~0x00000fffu);     // fields 0,1 | 2,3 on 16-bit lanes
    const uint32_t y = (x & 0x003f003fu) | ((x << 2) & ~0x003f003fu);     // one field per byte, junk in bits 6-7
    const uint32_t z = (y & 0x3f3f3f3fu) | 0x80808080u;                   // u | 0x80: no borrow between bytes below
    return (int)((z - 0x20202020u) ^ 0x80808080u);                        // (u + 0x60) ^ 0x80 = u - 32 mod 256
}

__device__ __forceinline__ void dma16(uint32_t lds_dst, uint32_t lane_off, const void* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_dst), "v"(lane_off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void dma4(uint32_t lds_dst, uint32_t lane_off, const void* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_dst), "v"(lane_off), "s"(base) : "memory", "m0");
}

template <int OUT_DT, bool DUMP>
__global__ void __launch_bounds__(256, 1) w6a8_group_gemm_kernel(W6Args p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    int tm, tn;
    tile_of_block((int)blockIdx.x, (int)gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN, ng = p.ng;
    const uint32_t lds_base = (uint32_t)(uintptr_t)smem;

    // DMA sources: 32-bit lane offsets from a per-group scalar base.  Rows past the edge re-read the last valid row;
    // what they produce is never stored.
    const int lrow = lane >> 3, lch = ((lane & 7) ^ lrow) * 16;   // swizzle applied on the global side
    uint32_t ga[8], gr[3], gs;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int row = (wave + 4 * j) * 8 + lrow;
        const int r = m0 + row < p.M ? m0 + row : p.M - 1;
        ga[j] = (uint32_t)r * (uint32_t)p.K + lch;
    }
    const uint32_t wrow = (uint32_t)p.K / 4 * 3;                   // bytes per packed weight row
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int c = (wave + 4 * j) * 64 + lane;                  // 16-byte chunk of the raw tile: row c/6, part c%6
        const int row = c / 6, part = c - row * 6;
        const int r = n0 + row < p.N ? n0 + row : p.N - 1;
        gr[j] = (uint32_t)r * wrow + part * 16;
    }
    {
        const int row = 32 * wave + (lane & 31);
        const int r = n0 + row < p.N ? n0 + row : p.N - 1;
        gs = (uint32_t)r * (uint32_t)ng * 4u;
    }
    auto fetch_a = [&](int g, int stage) {
        const int8_t* base = p.A + (int64_t)(g < ng ? g : ng - 1) * BK;
#pragma unroll
        for (int j = 0; j < 8; ++j) dma16(lds_base + stage * A_STAGE + (wave + 4 * j) * 1024, ga[j], base);
    };
    auto fetch_raw = [&](int g, int stage) {
        const uint8_t* base = p.Wp + (int64_t)(g < ng ? g : ng - 1) * RAW_ROW;
#pragma unroll
        for (int j = 0; j < 3; ++j) dma16(lds_base + R_BASE + stage * R_STAGE + (wave + 4 * j) * 1024, gr[j], base);
    };
    auto fetch_scales = [&](int g, int stage) {
        const float* base = p.sw + (g < ng ? g : ng - 1);
        if (lane < 32) dma4(lds_base + S_BASE + stage * S_STAGE + wave * 128, gs, base);
    };
    // Piece e of the raw tile is bytes [12e, 12e+12): row e/8, codes 16*(e%8) .. +15 -> one 16-byte chunk.
    auto unpack = [&](int rstage, int ustage, int i) {
        const int e = tid + 256 * i;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(smem + R_BASE + rstage * R_STAGE + 12 * e);
        const uint32_t d0 = src[0], d1 = src[1], d2 = src[2];
        const v4i out = v4i{spread6(d0), spread6(__builtin_amdgcn_alignbit(d1, d0, 24)),
                            spread6(__builtin_amdgcn_alignbit(d2, d1, 16)), spread6(d2 >> 8)};
        const int r = e >> 3, pc = e & 7;
        *reinterpret_cast<v4i*>(smem + U_BASE + ustage * U_STAGE + r * BK + ((pc ^ (r & 7)) << 4)) = out;
    };

    // fragment addresses inside a stage: row r at r*128, chunk c at slot c ^ (r&7); K sub-step kk flips bits 5 and 6
    const int frow = lane & 31, fhalf = lane >> 5;
    const int fsw = (fhalf ^ (frow & 7)) << 4;
    int aoff[4], woff[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        aoff[kk] = ((wm * 128 + frow) * BK + fsw) ^ (kk << 5);
        woff[kk] = ((wn * 64 + frow) * BK + fsw) ^ (kk << 5);
    }

    v16i part[TN][TM];      // int32 partial of the current group
    float accf[TN][TM][16]; // fp32 accumulators
#pragma unroll
    for (int in = 0; in < TN; ++in)
#pragma unroll
        for (int im = 0; im < TM; ++im)
#pragma unroll
            for (int r = 0; r < 16; ++r) accf[in][im][r] = 0.f;

    // prologue: A(0), raw(0), raw(1), scales(0) land; raw(0) is unpacked
    fetch_a(0, 0);
    fetch_raw(0, 0);
    fetch_raw(1, 1);
    fetch_scales(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) unpack(0, 0, i);
    __syncthreads();

    for (int g = 0; g < ng; ++g) {
        const int s = g & 1;
        const uint8_t* sa = smem + s * A_STAGE;
        const uint8_t* su = smem + U_BASE + s * U_STAGE;
        const float* sc = reinterpret_cast<const float*>(smem + S_BASE + s * S_STAGE);
        // All of these targets were last read during iteration g-1, which every wave has left.
        fetch_a(g + 1, s ^ 1);
        fetch_raw(g + 2, s);
        fetch_scales(g + 1, s ^ 1);
        SCHED_FENCE();

        v4i fa[2][4], fw[4], na[2][4], nw[4];
        auto load_a = [&](v4i (&dst)[2][4], int imb) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) dst[t][kk] = *reinterpret_cast<const v4i*>(sa + aoff[kk] + (imb + t) * 32 * BK);
        };
        auto load_w = [&](v4i (&dst)[4], int in) {
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) dst[kk] = *reinterpret_cast<const v4i*>(su + woff[kk] + in * 32 * BK);
        };
        // fp32 fold of register group q of both tiles of a pair: accf += float(part) * sw[n, g]
        auto fold = [&](int in, int imb, int q) {
            const float4 s4 = *reinterpret_cast<const float4*>(sc + wn * 64 + in * 32 + 8 * q + 4 * fhalf);
            const float sv[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    accf[in][imb + t][4 * q + c] = __builtin_fmaf((float)part[in][imb + t][4 * q + c], sv[c], accf[in][imb + t][4 * q + c]);
        };
        // Eight MFMAs of the pair (in; imb, imb+1), the two accumulation chains interleaved; between(i) is issued
        // after the i-th of them.
        auto mma_pair = [&](int in, int imb, v4i (&a)[2][4], v4i (&w)[4], auto&& between) {
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    if (kk == 0) {
                        v16i zero;
#pragma unroll
                        for (int r = 0; r < 16; ++r) zero[r] = 0;
                        part[in][imb + t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[kk], a[t][kk], zero, 0, 0, 0);
                    } else {
                        part[in][imb + t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[kk], a[t][kk], part[in][imb + t], 0, 0, 0);
                    }
                    SCHED_FENCE();
                    between(kk * 2 + t);
                    SCHED_FENCE();
                }
        };

        load_w(fw, 0);
        load_a(fa, 0);
        mma_pair(0, 0, fa, fw, [&](int i) {
            if (i == 0) load_a(na, 2);
            if (i == 4) unpack(s ^ 1, s ^ 1, 0);
        });
        mma_pair(0, 2, na, fw, [&](int i) {
            if (i < 4) fold(0, 0, i);
            if (i == 4) { load_w(nw, 1); load_a(fa, 0); }
            if (i == 6) unpack(s ^ 1, s ^ 1, 1);
        });
        mma_pair(1, 0, fa, nw, [&](int i) {
            if (i < 4) fold(0, 2, i);
            if (i == 4) load_a(na, 2);
            if (i == 6) unpack(s ^ 1, s ^ 1, 2);
        });
        mma_pair(1, 2, na, nw, [&](int i) {
            if (i < 4) fold(1, 0, i);
            if (i == 5) unpack(s ^ 1, s ^ 1, 3);
        });
#pragma unroll
        for (int q = 0; q < 4; ++q) fold(1, 2, q);

        if (DUMP) {   // test hook: the exact int32 partials, [M, N, ng]
#pragma unroll
            for (int in = 0; in < TN; ++in)
#pragma unroll
                for (int im = 0; im < TM; ++im)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int m = m0 + wm * 128 + im * 32 + frow;
                        const int n = n0 + wn * 64 + in * 32 + 8 * (r >> 2) + 4 * fhalf + (r & 3);
                        if (m < p.M && n < p.N) p.partials[((int64_t)m * p.N + n) * ng + g] = part[in][im][r];
                    }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the DMA of this iteration has landed
        __syncthreads();                                    // ... for every wave, and the unpacked tile is written
    }

    // epilogue: four consecutive n per lane and register group, straight from the accumulators
    const bool vec_ok = (p.N & 3) == 0 && ((uintptr_t)p.D & (4 * dt_size<OUT_DT>::value - 1)) == 0 &&
                        ((uintptr_t)p.bias & (4 * dt_size<OUT_DT>::value - 1)) == 0;
#pragma unroll
    for (int im = 0; im < TM; ++im) {
        const int m = m0 + wm * 128 + im * 32 + frow;
        if (m >= p.M) continue;
        const float xs = p.xs[m];
#pragma unroll
        for (int in = 0; in < TN; ++in)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * 64 + in * 32 + 8 * q + 4 * fhalf;
                if (n >= p.N) continue;
                const int64_t o = (int64_t)m * p.N + n;
                float b[4] = {0.f, 0.f, 0.f, 0.f}, out[4];
                if (vec_ok) {
                    if (p.bias) load4<OUT_DT>(p.bias, n, b);
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) if (p.bias && n + c < p.N) b[c] = ld_dt<OUT_DT>(p.bias, n + c);
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) out[c] = __builtin_fmaf(accf[in][im][4 * q + c], xs, b[c]);
                if (vec_ok) {
                    store4<OUT_DT>(p.D, o, out);
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) if (n + c < p.N) st_dt<OUT_DT>(p.D, o + c, out[c]);
                }
            }
    }
}

template <int OUT_DT, bool DUMP>
int launch(W6Args a, hipStream_t st) {
    auto kern = w6a8_group_gemm_kernel<OUT_DT, DUMP>;
    static bool once = false;  // benign race: the attribute is idempotent
    if (!once) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
        if (e != hipSuccess) return (int)e;
        once = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(a.tiles_m * a.tiles_n)), dim3(256), SMEM, st, a);
    KCHECK();
    return 0;
}

template <int OUT_DT>
int launch_dt(const W6Args& a, hipStream_t st) {
    return a.partials ? launch<OUT_DT, true>(a, st) : launch<OUT_DT, false>(a, st);
}

}  // namespace

GPU_API int gpu_w6a8_group_gemm(const int8_t* A, const void* Wp, const float* xs, const float* sw, const void* bias,
                                void* D, int32_t* partials, int64_t M, int64_t N, int64_t K, int out_dt, void* stream) {
    if (K < 0 || (K % 128) != 0) return -1;
    if (out_dt < DT_F32 || out_dt > DT_BF16 || M < 0 || N < 0) return -200;
    if (M == 0 || N == 0) return 0;
    // 32-bit DMA lane offsets and tile counts
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff || M * K >= ((int64_t)1 << 32) || N * (K / 4 * 3) >= ((int64_t)1 << 32) ||
        N * (K / 128) * 4 >= ((int64_t)1 << 32))
        return -200;
    W6Args a{A, (const uint8_t*)Wp, xs, sw, bias, D, partials, (int)M, (int)N, (int)K, (int)(K / 128), 0, 0};
    a.tiles_m = (int)((M + BM - 1) / BM);
    a.tiles_n = (int)((N + BN - 1) / BN);
    if ((int64_t)a.tiles_m * a.tiles_n > 0x7fffffff || K == 0) return -200;
    hipStream_t st = (hipStream_t)stream;
    switch (out_dt) {
        case DT_F32: return launch_dt<DT_F32>(a, st);
        case DT_F16: return launch_dt<DT_F16>(a, st);
        default: return launch_dt<DT_BF16>(a, st);
    }
}
