// Row prologues of the quantizer (csrc/kernels.cu:88-182 inside quant_rows_kernel, :348-474 as prologue_rows_kernel):
// RMSNorm / LayerNorm with modulation, gates, SwiGLU, activations.  Every prologue ends on a rounding to the row dtype
// T.  This file writes that row (gpu_prologue_rows[_b], which the reference exports for its bf16/f32 GEMMs); the
// quantizer entry points apply the same expressions inside their own kernel (quant_rows.hip).
//
// Arithmetic: the reference's expressions and rounding points (rnd<T> after the same operations), with two choices
// where its result depends on things a port cannot copy:
//   * row sums (mean, sum of squares) are accumulated in fp64 and rounded to fp32 once, so they do not depend on how
//     a row is spread over lanes (the reference adds fp32 partials in the order of its own thread layout);
//   * exp, expm1, erf, tanh and 1/sqrt are evaluated in fp64 and rounded to fp32, i.e. correctly rounded fp32 functions
//     (the reference calls CUDA's expf/erff/tanhf/rsqrtf, 1-2 ulp routines whose bits only a run could show).
//   * a*b + c written as one expression is contracted to an fma, as nvcc does by default.
// One workgroup per row.
#include "common.hpp"
#include "rowmath.hpp"
#include "act_tables.hpp"

namespace {

struct ProArgs {
    const void* x;
    int64_t x_stride;
    const void* g;
    int64_t g_stride;
    int64_t up_offset;
    const float* norm_w;
    const float* norm_b;
    float eps;
    const void* mod_scale;
    const void* mod_shift;
    void* out;
    int64_t out_stride;
    int K;
    ActTables tab;   // activation tables for bf16 rows (null members: evaluate per element)
};

template <int PRO> __device__ __forceinline__ constexpr bool is_ln() {
    return PRO == PRO_LAYERNORM || PRO == PRO_LN_MOD || PRO == PRO_LN_AFFINE || PRO == PRO_LN_AFFINE_SILU;
}

// Sum over the workgroup in fp64, rounded to fp32 once.
__device__ __forceinline__ float block_sum_f64(double v, double* red) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) red[wid] = v;
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < nw; ++i) t += red[i];
    return (float)t;
}

template <int DT, int PRO>
__global__ void __launch_bounds__(256) prologue_rows_kernel(ProArgs p) {
    __shared__ double red[4];
    const int K = p.K;
    const int64_t m = blockIdx.x;
    constexpr int SZ = dt_size<DT>::value;
    const uint8_t* x = (const uint8_t*)p.x + m * p.x_stride * SZ;
    uint8_t* o = (uint8_t*)p.out + m * p.out_stride * SZ;
    auto R = [](float v) { return rnd_dt<DT>(v); };
    // rnd(f(x)) of a bf16 value through the table of all 65536 inputs, when it is there
    auto via = [](const uint16_t* tab, float v, auto f) {
        if (DT == DT_BF16 && tab) return bf16_to_f(tab[f2u(v) >> 16]);
        return rnd_dt<DT>(f(v));
    };
    if (PRO == PRO_RMS || is_ln<PRO>() || PRO == PRO_ADALN) {
        float mean = 0.f;
        if (is_ln<PRO>()) {
            double s = 0.0;
            for (int k = threadIdx.x; k < K; k += blockDim.x) s += (double)ld_dt<DT>(x, k);
            mean = block_sum_f64(s, red) / (float)K;
        }
        double s2 = 0.0;
        for (int k = threadIdx.x; k < K; k += blockDim.x) {
            const float v = ld_dt<DT>(x, k) - mean;
            s2 += (double)v * (double)v;
        }
        const float ss = block_sum_f64(s2, red);
        const float rstd = (float)(1.0 / sqrt((double)(ss / (float)K + p.eps)));
        const void* ms = p.mod_scale;
        const void* sh = p.mod_shift;
        for (int k = threadIdx.x; k < K; k += blockDim.x) {
            float n = (ld_dt<DT>(x, k) - mean) * rstd;
            const float msv = ms ? ld_dt<DT>(ms, k) : 0.f, shv = ms ? ld_dt<DT>(sh, k) : 0.f;
            if (PRO == PRO_ADALN) {                                       // csrc/kernels.cu:163-166: one rounding
                st_dt<DT>(o, k, __builtin_fmaf(n, 1.f + msv, shv));
            } else if (PRO == PRO_LN_MOD) {                               // ln_finish, :40-46
                st_dt<DT>(o, k, __builtin_fmaf(R(n), R(1.f + msv), shv));
            } else if (PRO == PRO_LN_AFFINE) {
                st_dt<DT>(o, k, __builtin_fmaf(n, p.norm_w[k], p.norm_b[k]));
            } else if (PRO == PRO_LN_AFFINE_SILU) {
                st_dt<DT>(o, k, silu_f(R(__builtin_fmaf(n, p.norm_w[k], p.norm_b[k]))));
            } else {                                                      // RMS, LAYERNORM: :171-179
                if (p.norm_w) n *= p.norm_w[k];
                n = R(n);
                if (ms) {
                    const float a = R(1.f + msv);
                    n = R(a * n);
                    n = R(n + shv);
                }
                st_dt<DT>(o, k, n);
            }
        }
    } else if (PRO == PRO_GATE) {                                         // :108-113
        const uint8_t* g = (const uint8_t*)p.g + m * p.g_stride * SZ;
        for (int k = threadIdx.x; k < K; k += blockDim.x) st_dt<DT>(o, k, ld_dt<DT>(x, k) * via(p.tab.sigmoid_bf16, ld_dt<DT>(g, k), [](float t) { return sigmoid_f(t); }));
    } else if (PRO == PRO_SWIGLU) {                                       // :114-119
        for (int k = threadIdx.x; k < K; k += blockDim.x)
            st_dt<DT>(o, k, via(p.tab.silu_bf16, ld_dt<DT>(x, k), [](float t) { return silu_f(t); }) * ld_dt<DT>(x, p.up_offset + k));
    } else if (PRO == PRO_SILU) {
        for (int k = threadIdx.x; k < K; k += blockDim.x) st_dt<DT>(o, k, via(p.tab.silu_bf16, ld_dt<DT>(x, k), [](float t) { return silu_f(t); }));
    } else if (PRO == PRO_GELU) {
        for (int k = threadIdx.x; k < K; k += blockDim.x) st_dt<DT>(o, k, via(p.tab.gelu_bf16, ld_dt<DT>(x, k), [](float t) { return gelu_f(t); }));
    } else if (PRO == PRO_GELU_TANH) {
        for (int k = threadIdx.x; k < K; k += blockDim.x) st_dt<DT>(o, k, via(p.tab.gelu_tanh_bf16, ld_dt<DT>(x, k), [](float t) { return gelu_tanh_f(t); }));
    } else if (PRO == PRO_SITU) {                                         // csrc/kernels.cu:409-417, the eager chain
        for (int k = threadIdx.x; k < K; k += blockDim.x) {
            const float hidden = ld_dt<DT>(x, k), gate = ld_dt<DT>(x, p.up_offset + k);
            const float capped = R(4.f * R(stable_tanh(R(gate / 4.f))));
            const float g = R(capped * R(sigmoid_f(gate)));
            const float h = R(25.f * R(stable_tanh(R(hidden / 25.f))));
            st_dt<DT>(o, k, g * h);
        }
    } else {
        for (int k = threadIdx.x; k < K; k += blockDim.x) st_dt<DT>(o, k, ld_dt<DT>(x, k));
    }
}

// GroupNorm statistics of fp16 x [N, P, C]: one workgroup per (image, group).  Sums in fp64, then csrc/sd.cu:203-207:
// mean = s / cnt, var = max(ss / cnt - mean^2, 0), rstd = 1 / sqrt(var + eps), both narrowed to fp32.
__global__ void __launch_bounds__(256) sd_group_stats_kernel(const uint16_t* x, float2* stats, int64_t P, int C, int G, float eps) {
    __shared__ double red[4];
    __shared__ double keep;
    const int ng = blockIdx.x, n = ng / G, g = ng % G, per = C / G;
    const uint16_t* base = x + (int64_t)n * P * C + g * per;
    const int64_t count = P * per;
    double s = 0.0, ss = 0.0;
    for (int64_t i = threadIdx.x; i < count; i += blockDim.x) {
        const double v = (double)f16_to_f(base[(i / per) * C + (i % per)]);
        s += v;
        ss += v * v;
    }
    // block_sum_f64 narrows to fp32; these sums stay in fp64
    for (int o = 32; o > 0; o >>= 1) { s += __shfl_xor(s, o); ss += __shfl_xor(ss, o); }
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    if (lane == 0) red[wid] = s;
    __syncthreads();
    if (threadIdx.x == 0) keep = red[0] + red[1] + red[2] + red[3];
    __syncthreads();
    if (lane == 0) red[wid] = ss;
    __syncthreads();
    if (threadIdx.x == 0) {
        const double cnt = (double)count, mean = keep / cnt;
        const double var = fmax((red[0] + red[1] + red[2] + red[3]) / cnt - mean * mean, 0.0);
        stats[ng * 2] = make_float2((float)mean, (float)(1.0 / sqrt(var + (double)eps)));
    }
}

template <int DT, int PRO>
int launch(const ProArgs& p, int M, hipStream_t st) {
    if (M <= 0) return 0;
    hipLaunchKernelGGL((prologue_rows_kernel<DT, PRO>), dim3((unsigned)M), dim3(256), 0, st, p);
    KCHECK();
    return 0;
}

template <int DT>
int dispatch(int prologue, ProArgs p, int M, hipStream_t st, bool b_variant) {
    if (DT == DT_BF16 && M > 0 &&
        (prologue == PRO_GATE || prologue == PRO_SWIGLU || prologue == PRO_SILU || prologue == PRO_GELU || prologue == PRO_GELU_TANH))
        if (const ActTables* t = act_tables(st)) p.tab = *t;
    switch (prologue) {
        case PRO_PLAIN: return launch<DT, PRO_PLAIN>(p, M, st);
        case PRO_RMS: return b_variant ? -3 : launch<DT, PRO_RMS>(p, M, st);
        case PRO_GATE: return b_variant ? -3 : launch<DT, PRO_GATE>(p, M, st);
        case PRO_SWIGLU: return b_variant ? -3 : launch<DT, PRO_SWIGLU>(p, M, st);
        case PRO_LAYERNORM: return launch<DT, PRO_LAYERNORM>(p, M, st);
        case PRO_SILU: return launch<DT, PRO_SILU>(p, M, st);
        case PRO_GELU: return launch<DT, PRO_GELU>(p, M, st);
        case PRO_ADALN: return b_variant ? -3 : launch<DT, PRO_ADALN>(p, M, st);
        case PRO_SITU: return b_variant ? -3 : launch<DT, PRO_SITU>(p, M, st);
        case PRO_LN_MOD: return b_variant ? launch<DT, PRO_LN_MOD>(p, M, st) : -3;
        case PRO_LN_AFFINE: return b_variant ? launch<DT, PRO_LN_AFFINE>(p, M, st) : -3;
        case PRO_LN_AFFINE_SILU: return b_variant ? launch<DT, PRO_LN_AFFINE_SILU>(p, M, st) : -3;
        case PRO_GELU_TANH: return b_variant ? launch<DT, PRO_GELU_TANH>(p, M, st) : -3;
        default: return -3;
    }
}

}  // namespace

// Replaces gpu_prologue_rows, csrc/kernels.cu:420-446 (dtype bf16 or f32; the id list of :429-439).
GPU_API int gpu_prologue_rows(int dtype, int prologue, const void* x, int64_t x_stride, const void* g, int64_t g_stride,
                              int64_t up_offset, const float* norm_w, float eps, const void* mod_scale,
                              const void* mod_shift, void* out, int64_t out_stride, int M, int K, void* stream) {
    ProArgs p{x, x_stride, g, g_stride, up_offset, norm_w, nullptr, eps, mod_scale, mod_shift, out, out_stride, K};
    if (dtype == DT_BF16) return dispatch<DT_BF16>(prologue, p, M, (hipStream_t)stream, false);
    if (dtype == DT_F32) return dispatch<DT_F32>(prologue, p, M, (hipStream_t)stream, false);
    return -4;
}

// Replaces gpu_prologue_rows_b, csrc/kernels.cu:449-474 (bf16, f16 or f32; LayerNorm variants with a bias, activations).
GPU_API int gpu_prologue_rows_b(int dtype, int prologue, const void* x, int64_t x_stride, const float* norm_w,
                                const float* norm_b, float eps, const void* mod_scale, const void* mod_shift, void* out,
                                int64_t out_stride, int M, int K, void* stream) {
    ProArgs p{x, x_stride, nullptr, 0, 0, norm_w, norm_b, eps, mod_scale, mod_shift, out, out_stride, K};
    if (dtype == DT_BF16) return dispatch<DT_BF16>(prologue, p, M, (hipStream_t)stream, true);
    if (dtype == DT_F16) return dispatch<DT_F16>(prologue, p, M, (hipStream_t)stream, true);
    if (dtype == DT_F32) return dispatch<DT_F32>(prologue, p, M, (hipStream_t)stream, true);
    return -4;
}

// GroupNorm statistics for gpu_sd_group_norm_quant_rows: (mean, rstd) of group ng as two floats at stats + 16 * ng bytes,
// the layout csrc/sd.cu:203-207 leaves.
extern "C" int gpu_internal_sd_group_stats(const void* x, void* stats, int n_images, int64_t P, int C, int G, float eps,
                                           void* stream) {
    hipLaunchKernelGGL(sd_group_stats_kernel, dim3((unsigned)(n_images * G)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t*)x, (float2*)stats, P, C, G, eps);
    KCHECK();
    return 0;
}
