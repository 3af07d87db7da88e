// Per-row absmax int8 quantization with the optional ConvRot group rotation, for gfx950 (wave64).
//
// Arithmetic follows the reference's quantizers exactly (csrc/kernels.cu:184-258 for bf16/f32 rows,
// csrc/sd.cu:578-598 for fp16 rows, csrc/common.cuh:99-126 for the staged radix-4 Hadamard butterflies): same
// float operation order, same rounding points.  The structure does not: a row is cut into chunks of 1024 values, one
// wave per chunk, each lane holding 16 consecutive values in registers.  Radix-4 stages with strides 1 and 4 run inside
// a lane; for the wider strides the chunk makes one trip through a wave-private LDS tile so that those butterflies are
// again lane-local, then returns to row order for the 16-byte code stores.
#include "common.hpp"
#include "convrot.hpp"
#include "rowmath.hpp"
#include "act_tables.hpp"

namespace {
using namespace convrot;

enum { MODE_BF16 = 0, MODE_F32 = 1, MODE_SD_F16 = 2, MODE_ROT_F32 = 3 };

struct QuantArgs {
    const void* x;
    int64_t x_stride;  // elements between rows
    int8_t* q;         // [M, K]
    float* scales;     // [M]
    float* out_f;      // MODE_ROT_F32: rotated rows [M, K]
    int M, K;
    int wpr;           // waves per row
    int rpb;           // rows per block
    uint64_t seed;     // nonzero: stochastic rounding keyed by element index + seed (gpu_convrot_requant)
    // row prologue (csrc/kernels.cu:21-37), PRO kernels only
    int pro;
    const void* g;          // GATE: logits [M, g_stride]
    int64_t g_stride;
    int64_t up_offset;      // SWIGLU, SITU: column of the second half inside the x row
    const float* norm_w;    // RMS, LAYERNORM, LN_AFFINE
    const float* norm_b;    // LN_AFFINE
    float eps;
    const void* mod_scale;  // [K] in the row dtype
    const void* mod_shift;
    int d, dp;              // PRO_SD_UNPAD: heads of d values, each stored dp wide
    int per;                // PRO_SD_GN: channels per group; g holds the (mean, rstd) pairs, g_stride the pixels per image
    ActTables tab;          // activation tables for 16-bit rows (null members: evaluate per element)
};

// Sources of the SD UNet's fused quantizers (csrc/sd.cu:611-663), fp16 rows only.  Its LayerNorm source is PRO_LN_AFFINE.
enum { PRO_SD_GEGLU = 101, PRO_SD_UNPAD = 102, PRO_SD_GN = 103 };

// csrc/kernels.cu:1355-1359
__device__ __forceinline__ uint32_t pcg_hash(uint32_t x) {
    const uint32_t state = x * 747796405u + 2891336453u;
    const uint32_t word = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
    return (word >> 22u) ^ word;
}
// a + b of two bf16 values rounded once to bf16, what the bf16 add instruction behind __hadd gives
// (csrc/kernels.cu:1341-1343): the exact sum fits a double, which is then cut to 8 significant bits, ties to even.
__device__ __forceinline__ float bf16_add_once(float a, float b) {
    const double s = (double)a + (double)b;
    uint64_t u = __builtin_bit_cast(uint64_t, s);
    const uint64_t rem = u & ((1ull << 45) - 1), half = 1ull << 44;
    u >>= 45;
    if (rem > half || (rem == half && (u & 1))) ++u;
    return (float)__builtin_bit_cast(double, u << 45);
}

template <int MODE> __device__ __forceinline__ void load16(const void* x, int64_t off, float* v) {
    if (MODE == MODE_BF16) {
        const uint4* p = reinterpret_cast<const uint4*>((const uint16_t*)x + off);
        const uint4 a = p[0], b = p[1];
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[2 * i] = u2f(w[i] << 16);
            v[2 * i + 1] = u2f(w[i] & 0xffff0000u);
        }
    } else if (MODE == MODE_SD_F16) {
        const uint4* p = reinterpret_cast<const uint4*>((const uint16_t*)x + off);
        const uint4 a = p[0], b = p[1];
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[2 * i] = f16_to_f((uint16_t)(w[i] & 0xffffu));
            v[2 * i + 1] = f16_to_f((uint16_t)(w[i] >> 16));
        }
    } else {
        const float4* p = reinterpret_cast<const float4*>((const float*)x + off);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 f = p[i];
            v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
        }
    }
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Sum over the waves of one row in fp64, rounded to fp32 once (every wave of the block calls it).
__device__ __forceinline__ float row_sum_f64(double v, double* red, int wave, int lane, int wpr, int rloc) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < wpr; ++i) t += red[rloc * wpr + i];
    return (float)t;
}

// PRO: the row prologue (csrc/kernels.cu:88-182) runs on the values as they are loaded, with the reference's rounding
// points; p.pro selects it at run time.  Row sums are fp64, rounded once; the activation functions are correctly rounded.
// SR: stochastic rounding keyed by element index + p.seed (gpu_convrot_requant); a kernel variant of its own, so that the
// plain quantizer carries neither the hash nor a branch per element.
template <int MODE, int G, int C, bool PRO, bool SR = false>
__global__ void __launch_bounds__(512) quant_rows_kernel(QuantArgs p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ float red[8];
    __shared__ double dred[8];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rloc = wave / p.wpr, wr = wave - rloc * p.wpr;
    const int64_t m = (int64_t)blockIdx.x * p.rpb + rloc;
    const bool row_ok = m < p.M;
    float* wl = lds + wave * kLdsPerWave;
    // the row dtype T of the prologue's roundings, and how a T vector is loaded
    constexpr int TD = MODE == MODE_BF16 ? DT_BF16 : MODE == MODE_SD_F16 ? DT_F16 : DT_F32;
    constexpr int TMODE = MODE == MODE_BF16 ? MODE_BF16 : MODE == MODE_SD_F16 ? MODE_SD_F16 : MODE_F32;
    auto R = [](float x) { return rnd_dt<TD>(x); };
    // dst[i] = rnd(f(src[i])) for the 16 values of a lane: through a table of all 65536 bf16 inputs when it is there (one
    // test for the 16 lookups, which then issue as a batch), else evaluated
    auto map16 = [](const uint16_t* tab, const float* src, float* dst, auto f) {
        if (MODE == MODE_BF16 && tab) {
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[i] = bf16_to_f(tab[f2u(src[i]) >> 16]);
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[i] = rnd_dt<TD>(f(src[i]));
        }
    };

    float v[C][16];
    float amax = 0.f;
    const int pro = PRO ? p.pro : PRO_PLAIN;
    const bool ln = pro == PRO_LAYERNORM || pro == PRO_LN_MOD || pro == PRO_LN_AFFINE;
    const bool norm = ln || pro == PRO_RMS || pro == PRO_ADALN;
    double part = 0.0;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int e0 = (wr + c * p.wpr) * kChunk + lane * 16;
        const bool act = row_ok && e0 < p.K;
        if (PRO && MODE == MODE_SD_F16 && pro == PRO_SD_UNPAD) {                     // csrc/sd.cu:650-652
            const uint16_t* r = (const uint16_t*)p.x + m * p.x_stride;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int k = e0 + i;
                v[c][i] = act ? f16_to_f(r[(k / p.d) * p.dp + k % p.d]) : 0.f;
            }
        } else if (act) {
            load16<MODE>(p.x, m * p.x_stride + e0, v[c]);
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) v[c][i] = 0.f;
        }
        if (PRO && act) {
            if (MODE == MODE_SD_F16) {
                if (pro == PRO_SD_GEGLU) {                                           // :642-649, row = [value | gate]
                    float gg[16];
                    load16<TMODE>(p.x, m * p.x_stride + p.up_offset + e0, gg);
                    if (p.tab.gelu_f16) {
#pragma unroll
                        for (int i = 0; i < 16; ++i) gg[i] = f16_to_f(p.tab.gelu_f16[f_to_f16(gg[i])]);
                    } else {
#pragma unroll
                        for (int i = 0; i < 16; ++i) gg[i] = R(gelu_f(gg[i]));
                    }
#pragma unroll
                    for (int i = 0; i < 16; ++i) v[c][i] = R(v[c][i] * gg[i]);
                } else if (pro == PRO_SD_GN) {                                       // :653-662
                    const float2* stats = (const float2*)p.g + (m / p.g_stride) * (int64_t)(p.K / p.per) * 2;
                    float nw[16], nb[16];
                    load16<MODE_F32>(p.norm_w, e0, nw);
                    load16<MODE_F32>(p.norm_b, e0, nb);
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const float2 st = stats[((e0 + i) / p.per) * 2];
                        v[c][i] = R(__builtin_fmaf((v[c][i] - st.x) * st.y, nw[i], nb[i]));
                    }
                } else if (ln) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) part += (double)v[c][i];
                }
            } else if (pro == PRO_GATE) {                                            // csrc/kernels.cu:95-100
                float gg[16];
                load16<TMODE>(p.g, m * p.g_stride + e0, gg);
                map16(p.tab.sigmoid_bf16, gg, gg, [](float x) { return sigmoid_f(x); });
#pragma unroll
                for (int i = 0; i < 16; ++i) v[c][i] = R(v[c][i] * gg[i]);
            } else if (pro == PRO_SWIGLU || pro == PRO_SITU || pro == PRO_SITU_FAST) {  // :101-112
                float u[16];
                load16<TMODE>(p.x, m * p.x_stride + p.up_offset + e0, u);
                if (pro == PRO_SWIGLU) {
                    map16(p.tab.silu_bf16, v[c], v[c], [](float x) { return silu_f(x); });
#pragma unroll
                    for (int i = 0; i < 16; ++i) v[c][i] = R(v[c][i] * u[i]);
                } else if (MODE == MODE_BF16 && p.tab.situ_gate_bf16) {
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        v[c][i] = p.tab.situ_gate_bf16[f2u(u[i]) >> 16] * p.tab.situ_hidden_bf16[f2u(v[c][i]) >> 16];
                } else {   // one float expression, not rounded to T; the lossy id runs the same accurate form
#pragma unroll
                    for (int i = 0; i < 16; ++i) v[c][i] = situ_f(v[c][i], u[i]);
                }
            } else if (pro == PRO_SILU) {
                map16(p.tab.silu_bf16, v[c], v[c], [](float x) { return silu_f(x); });
            } else if (pro == PRO_GELU) {
                map16(p.tab.gelu_bf16, v[c], v[c], [](float x) { return gelu_f(x); });
            } else if (pro == PRO_GELU_TANH) {
                map16(p.tab.gelu_tanh_bf16, v[c], v[c], [](float x) { return gelu_tanh_f(x); });
            } else if (ln) {
#pragma unroll
                for (int i = 0; i < 16; ++i) part += (double)v[c][i];
            } else if (norm) {
#pragma unroll
                for (int i = 0; i < 16; ++i) part += (double)v[c][i] * (double)v[c][i];
            }
        }
    }
    if (PRO && norm) {   // uniform over the block
        if (ln) {        // :133-145
            const float mean = row_sum_f64(part, dred, wave, lane, p.wpr, rloc) / (float)p.K;
            part = 0.0;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const int e0 = (wr + c * p.wpr) * kChunk + lane * 16;
                if (!(row_ok && e0 < p.K)) continue;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    v[c][i] -= mean;
                    part += (double)v[c][i] * (double)v[c][i];
                }
            }
        }
        const float ss = row_sum_f64(part, dred, wave, lane, p.wpr, rloc);
        const float rstd = (float)(1.0 / sqrt((double)(ss / (float)p.K + p.eps)));   // :148
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int e0 = (wr + c * p.wpr) * kChunk + lane * 16;
            if (!(row_ok && e0 < p.K)) continue;
            float msv[16], shv[16], nw[16], nb[16];
            const bool mod = p.mod_scale != nullptr;
            if (mod) {
                load16<TMODE>(p.mod_scale, e0, msv);
                load16<TMODE>(p.mod_shift, e0, shv);
            }
            if (p.norm_w && (pro == PRO_RMS || pro == PRO_LAYERNORM || pro == PRO_LN_AFFINE)) load16<MODE_F32>(p.norm_w, e0, nw);
            if (pro == PRO_LN_AFFINE) load16<MODE_F32>(p.norm_b, e0, nb);
            // the form is chosen once per 16 values, not per value
            if (pro == PRO_ADALN) {                                                  // :163-166, one rounding
#pragma unroll
                for (int i = 0; i < 16; ++i) v[c][i] = R(__builtin_fmaf(v[c][i] * rstd, 1.f + (mod ? msv[i] : 0.f), mod ? shv[i] : 0.f));
            } else if (pro == PRO_LN_MOD) {                                          // ln_finish, :40-46
#pragma unroll
                for (int i = 0; i < 16; ++i) v[c][i] = R(__builtin_fmaf(R(v[c][i] * rstd), R(1.f + (mod ? msv[i] : 0.f)), mod ? shv[i] : 0.f));
            } else if (pro == PRO_LN_AFFINE) {
#pragma unroll
                for (int i = 0; i < 16; ++i) v[c][i] = R(__builtin_fmaf(v[c][i] * rstd, nw[i], nb[i]));
            } else {                                                                 // RMS, LAYERNORM: :171-179
                if (p.norm_w) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) v[c][i] = R(v[c][i] * rstd * nw[i]);
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i) v[c][i] = R(v[c][i] * rstd);
                }
                if (mod) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const float aa = R(1.f + msv[i]);
                        v[c][i] = R(R(aa * v[c][i]) + shv[i]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int e0 = (wr + c * p.wpr) * kChunk + lane * 16;
        const bool act = row_ok && e0 < p.K;
        if (G != 0) rotate_chunk<G>(v[c], wl, lane);
        if (MODE == MODE_ROT_F32) {
            if (act) {
                float4* o = reinterpret_cast<float4*>(p.out_f + m * (int64_t)p.K + e0);
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = make_float4(v[c][4 * i], v[c][4 * i + 1], v[c][4 * i + 2], v[c][4 * i + 3]);
            }
        } else if (MODE == MODE_SD_F16) {
            // the maximum is taken over the half-rounded row (csrc/sd.cu:587)
#pragma unroll
            for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(rnd_dt<DT_F16>(v[c][i])));
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[c][i]));
        }
    }
    if (MODE == MODE_ROT_F32) return;

    amax = wave_max(amax);
    if (p.wpr > 1) {  // uniform over the block
        if (lane == 0) red[wave] = amax;
        __syncthreads();
        amax = 0.f;
        for (int i = 0; i < p.wpr; ++i) amax = fmaxf(amax, red[rloc * p.wpr + i]);
    }

    float scale, st, rinv = 0.f;
    if (MODE == MODE_SD_F16) {
        scale = fmaxf(amax, 1e-30f) / 127.f;                       // csrc/sd.cu:589
        const float sh = rnd_dt<DT_F16>(scale);
        st = sh > 0.f ? sh : scale;                                // :593
    } else if (MODE == MODE_BF16) {
        scale = fmaxf(fminf(amax, 3.38953139e38f) * (1.f / 127.f), 1.0e-30f);  // csrc/kernels.cu:241
        st = rnd_dt<DT_BF16>(scale);
        rinv = __builtin_amdgcn_rcpf(st);
    } else {
        scale = fmaxf(fminf(amax, 3.402823466e+38f) * (1.f / 127.f), 1.0e-30f);
        st = scale;
    }
    if (row_ok && wr == 0 && lane == 0) p.scales[m] = scale;

#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int e0 = (wr + c * p.wpr) * kChunk + lane * 16;
        if (!(row_ok && e0 < p.K)) continue;
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t acc = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float x = v[c][4 * i + j];
                float t;
                if (MODE == MODE_BF16) {
                    // Both operands carry 8 significant bits, so their exact quotient is never closer than 2^-17
                    // (relative) to a bf16 rounding boundary: a 1-ulp reciprocal times the numerator rounds to the
                    // same bf16 value as the IEEE quotient does.
                    t = rnd_dt<DT_BF16>(rnd_dt<DT_BF16>(x) * rinv);
                } else if (MODE == MODE_SD_F16) {
                    t = rnd_dt<DT_F16>(rnd_dt<DT_F16>(x) / st);
                } else {
                    t = x / st;
                }
                if (SR && (MODE == MODE_BF16 || MODE == MODE_F32)) {   // csrc/kernels.cu:1385-1388
                    const uint64_t key = (uint64_t)(m * (int64_t)p.K + e0 + 4 * i + j) + p.seed;
                    const float noise = (float)(pcg_hash((uint32_t)key ^ (uint32_t)(key >> 32)) >> 8) * 0x1.0p-24f;
                    const float r = floorf(MODE == MODE_F32 ? t + noise : bf16_add_once(t, rnd_dt<DT_BF16>(noise)));
                    const int qi = (int)fminf(127.f, fmaxf(-128.f, r));
                    acc |= ((uint32_t)qi & 0xffu) << (8 * j);
                } else if (MODE == MODE_F32) {
                    const int qi = (int)fminf(127.f, fmaxf(-128.f, nearbyintf(t)));
                    acc |= ((uint32_t)qi & 0xffu) << (8 * j);
                } else {
                    // clamp(rint(t), -128, 127) + 128 as one instruction: t is a 16-bit float, so t + 128 is exact
                    // wherever t has a bit at 2^-16 or above set, and below that both t and t + 128 round to the
                    // same integer; v_cvt_pk_u8_f32 rounds to nearest even, saturates to 0..255 (NaN to 0, which is
                    // the -128 that fminf(127, fmaxf(-128, NaN)) gives) and drops the byte into place.
                    acc = __builtin_amdgcn_cvt_pk_u8_f32(t + 128.f, j, acc);
                }
            }
            w[i] = (!SR && MODE != MODE_F32) ? acc ^ 0x80808080u : acc;
        }
        *reinterpret_cast<uint4*>(p.q + m * (int64_t)p.K + e0) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

template <int MODE, int G, int C>
int launch(const QuantArgs& a, int nw, hipStream_t st) {
    const int grid = (a.M + a.rpb - 1) / a.rpb;
    const size_t smem = G ? (size_t)nw * kLdsPerWave * sizeof(float) : 0;
    constexpr bool CAN_PRO = true;
    constexpr bool CAN_SR = (MODE == MODE_BF16 || MODE == MODE_F32) && G == 256;
    if (CAN_SR && a.seed != 0 && a.pro == PRO_PLAIN)
        hipLaunchKernelGGL((quant_rows_kernel<MODE, G, C, false, CAN_SR>), dim3(grid), dim3(nw * 64), smem, st, a);
    else if (CAN_PRO && a.pro != PRO_PLAIN)
        hipLaunchKernelGGL((quant_rows_kernel<MODE, G, C, CAN_PRO>), dim3(grid), dim3(nw * 64), smem, st, a);
    else
        hipLaunchKernelGGL((quant_rows_kernel<MODE, G, C, false>), dim3(grid), dim3(nw * 64), smem, st, a);
    KCHECK();
    return 0;
}

template <int MODE, int G>
int launch_c(const QuantArgs& a, int nw, int C, hipStream_t st) {
    switch (C) {
        case 1: return launch<MODE, G, 1>(a, nw, st);
        case 2: return launch<MODE, G, 2>(a, nw, st);
        case 3: return launch<MODE, G, 3>(a, nw, st);
        default: return launch<MODE, G, 4>(a, nw, st);
    }
}

// g: rotation group width (0, 64, 128, 256).  Picks waves per row so that a wave holds at most 4 chunks.
template <int MODE>
int run_quant(QuantArgs a, int g, hipStream_t st) {
    if (a.M <= 0) return 0;
    const int nchunks = (a.K + kChunk - 1) / kChunk;
    int wpr = 1;
    while ((nchunks + wpr - 1) / wpr > 4) wpr *= 2;
    if (wpr > 8) return -2;
    // few rows: more waves per row (down to one chunk per wave) so that the launch has enough waves to hide latency
    while (wpr < 8 && wpr < nchunks && (int64_t)a.M * wpr < 2048) wpr *= 2;
    const int C = (nchunks + wpr - 1) / wpr;
    const int nw = wpr < 2 ? 2 : wpr;   // two rows per workgroup at least: small workgroups spread evenly over the CUs
    a.wpr = wpr;
    a.rpb = nw / wpr;
    switch (g) {
        case 0: return launch_c<MODE, 0>(a, nw, C, st);
        case 64: return launch_c<MODE, 64>(a, nw, C, st);
        case 128: if (MODE == MODE_SD_F16 || MODE == MODE_ROT_F32) return -1; return launch_c<MODE == MODE_F32 || MODE == MODE_BF16 ? MODE : MODE_BF16, 128>(a, nw, C, st);
        default: return launch_c<MODE, 256>(a, nw, C, st);
    }
}

// The activation tables, for the prologues that evaluate exp / erf / tanh on a 16-bit row.
void attach_tables(QuantArgs& a, hipStream_t st) {
    const int p = a.pro;
    if (p == PRO_GATE || p == PRO_SWIGLU || p == PRO_SITU || p == PRO_SITU_FAST || p == PRO_SILU || p == PRO_GELU || p == PRO_GELU_TANH ||
        p == PRO_SD_GEGLU)
        if (const ActTables* t = act_tables(st)) a.tab = *t;
}

int rotate_group(int rotate) { return rotate == 0 ? 0 : (rotate == 64 || rotate == 128) ? rotate : 256; }

bool known_prologue(int p) { return p >= PRO_PLAIN && p <= PRO_SITU_FAST && p != PRO_LN_AFFINE_SILU; }

}  // namespace

GPU_API int gpu_quant_rows(int dtype, int prologue, const void* x, int64_t x_stride, const void* g, int64_t g_stride,
                           int64_t up_offset, const float* norm_w, float eps, const void* mod_scale,
                           const void* mod_shift, int8_t* q, float* scales, int M, int K, int rotate, void* stream) {
    const int grp = rotate_group(rotate);
    const int need = grp == 0 ? 64 : grp;
    if (K <= 0 || (K % need) != 0) return -1;
    if (dtype != DT_BF16 && dtype != DT_F32) return -4;
    if (!known_prologue(prologue)) return -3;   // the id list of csrc/kernels.cu:280-292
    if (K > 32768) return -2;
    QuantArgs a{x, x_stride, q, scales, nullptr, M, K, 1, 1, 0, prologue, g, g_stride, up_offset, norm_w, nullptr, eps, mod_scale,
                mod_shift};
    if (dtype == DT_BF16 && M > 0) attach_tables(a, (hipStream_t)stream);
    return dtype == DT_BF16 ? run_quant<MODE_BF16>(a, grp, (hipStream_t)stream) : run_quant<MODE_F32>(a, grp, (hipStream_t)stream);
}

GPU_API int gpu_quant_rows_b(int dtype, int prologue, const void* x, int64_t x_stride, const float* norm_w,
                             const float* norm_b, float eps, const void* mod_scale, const void* mod_shift, int8_t* q,
                             float* scales, int M, int K, int rotate, void* stream) {
    if ((K % 256) != 0) return -1;
    if (dtype != DT_BF16) return -4;
    if (prologue != PRO_LN_MOD && prologue != PRO_LN_AFFINE) return -3;
    if (K <= 0) return -1;
    if (K > 32768) return -2;
    QuantArgs a{x, x_stride, q, scales, nullptr, M, K, 1, 1, 0, prologue, nullptr, 0, 0, norm_w, norm_b, eps, mod_scale, mod_shift};
    return run_quant<MODE_BF16>(a, rotate_group(rotate), (hipStream_t)stream);
}

GPU_API int gpu_rotate_rows_f32(int prologue, const float* x, int64_t x_stride, int64_t up_offset, const float* norm_w,
                                float eps, float* out, int M, int K, void* stream) {
    if (K <= 0 || (K % 256) != 0) return -1;
    if (prologue != PRO_PLAIN && prologue != PRO_RMS && prologue != PRO_SWIGLU) return -3;
    if (K > 32768) return -2;
    QuantArgs a{x, x_stride, nullptr, nullptr, out, M, K, 1, 1, 0, prologue, nullptr, 0, up_offset, norm_w, nullptr, eps, nullptr,
                nullptr};
    return run_quant<MODE_ROT_F32>(a, 256, (hipStream_t)stream);
}

GPU_API int gpu_sd_quant_rows(const void* x, int64_t x_stride, int8_t* q, float* scales, int M, int K, int rotate,
                              void* stream) {
    if ((rotate != 0 && rotate != 64 && rotate != 256) || (rotate && K % rotate)) return -1;
    if (K <= 0 || (K % 16) != 0) return -1;   // 16 values per lane
    if (K > 32768) return -2;
    QuantArgs a{x, x_stride, q, scales, nullptr, M, K, 1, 1};
    return run_quant<MODE_SD_F16>(a, rotate, (hipStream_t)stream);
}

// The SD UNet's fused quantizers (csrc/sd.cu:608-724): the half row of LayerNorm / GEGLU / head un-padding / GroupNorm,
// computed on the values as the fp16 quantizer loads them; it is rounded to half there as in the reference.
extern "C" int gpu_internal_sd_group_stats(const void* x, void* stats, int n_images, int64_t P, int C, int G, float eps,
                                           void* stream);
namespace {
int sd_fused(QuantArgs a, int rotate, hipStream_t st) {
    if ((rotate != 0 && rotate != 64 && rotate != 256) || (rotate && a.K % rotate)) return -1;   // csrc/sd.cu:682
    if (a.K <= 0 || (a.K % 16) != 0) return -1;
    if (a.K > 32768) return -2;
    if (a.M <= 0) return 0;
    attach_tables(a, st);
    return run_quant<MODE_SD_F16>(a, rotate, st);
}
}  // namespace

GPU_API int gpu_sd_ln_quant_rows(const void* x, int64_t x_stride, const float* w, const float* b, float eps, int8_t* q,
                                 float* scales, int M, int K, int rotate, void* stream) {
    QuantArgs a{x, x_stride, q, scales, nullptr, M, K, 1, 1, 0, PRO_LN_AFFINE, nullptr, 0, 0, w, b, eps, nullptr, nullptr};
    return sd_fused(a, rotate, (hipStream_t)stream);
}
GPU_API int gpu_sd_geglu_quant_rows(const void* in, int8_t* q, float* scales, int M, int I, int rotate, void* stream) {
    QuantArgs a{in, 2 * (int64_t)I, q, scales, nullptr, M, I, 1, 1, 0, PRO_SD_GEGLU, nullptr, 0, I, nullptr, nullptr, 0.f, nullptr,
                nullptr};
    return sd_fused(a, rotate, (hipStream_t)stream);
}
GPU_API int gpu_sd_unpad_quant_rows(const void* src, int8_t* q, float* scales, int M, int H, int d, int dp, int rotate,
                                    void* stream) {
    if (H <= 0 || d <= 0 || dp < d) return -1;
    QuantArgs a{src, (int64_t)H * dp, q, scales, nullptr, M, H * d, 1, 1, 0, PRO_SD_UNPAD, nullptr, 0, 0, nullptr, nullptr, 0.f,
                nullptr, nullptr, d, dp};
    return sd_fused(a, rotate, (hipStream_t)stream);
}
GPU_API int gpu_sd_group_norm_quant_rows(const void* x, const float* w, const float* b, void* sums, int N, int64_t P, int C, int G,
                                         float eps, int8_t* q, float* scales, int rotate, void* stream) {
    if (G <= 0 || C % G) return -1;                                                             // csrc/sd.cu:713
    if ((rotate != 0 && rotate != 64 && rotate != 256) || (rotate && C % rotate) || C <= 0 || C % 16) return -1;
    if (N <= 0 || P <= 0) return 0;
    const int rc = gpu_internal_sd_group_stats(x, sums, N, P, C, G, eps, stream);
    if (rc) return rc;
    QuantArgs a{x, C, q, scales, nullptr, (int)(N * P), C, 1, 1, 0, PRO_SD_GN, sums, P, 0, w, b, eps, nullptr, nullptr, 0, 0, C / G};
    return sd_fused(a, rotate, (hipStream_t)stream);
}

// x [N, K] in its original basis -> rotated int8 rows + row scales: the 256-wide quantizer with rounding to nearest
// (seed 0) or stochastic rounding keyed by element index + seed.  Replaces gpu_convrot_requant, csrc/kernels.cu:1361-1420;
// as there, any dtype other than DT_F32 is read as bf16.
GPU_API int gpu_convrot_requant(int dtype, const void* x, void* q, void* s, int64_t N, int K, uint64_t seed, void* stream) {
    if (K <= 0 || (K % 256) != 0) return -1;
    if (K > 32768 || N > 0x7fffffff) return -2;
    QuantArgs a{x, K, (int8_t*)q, (float*)s, nullptr, (int)N, K, 1, 1, seed};
    return dtype == DT_F32 ? run_quant<MODE_F32>(a, 256, (hipStream_t)stream) : run_quant<MODE_BF16>(a, 256, (hipStream_t)stream);
}
