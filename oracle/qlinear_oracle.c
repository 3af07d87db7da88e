/*
 * CPU oracle for the quantized-linear hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the arithmetic of the reference's W8A8 / W6A8 linear, written from its
 * source text.  It exists so that the HIP kernels can be checked bit-for-bit on the same inputs.  Nothing in the
 * product (the HIP library, its host wrappers) may call, link or import it: only the tests, the smoke check and
 * the bench's CPU-baseline leg do, and only as the checker / the reported CPU number.
 *
 * Every function cites the reference lines it follows (paths relative to the reference checkout).
 * Build with -ffp-contract=off: an FMA appears only where `fmaf` is written.
 *
 * Parity status of each function (what pins it, see tests/test_oracle_*.py):
 *   orc_bf16_round / orc_f16_round     pinned: exhaustive/sampled against torch.bfloat16 / numpy.float16 casts
 *   orc_fht                            g=64,256 pinned: dense Kronecker matrix, H=H^T, H.H=I, exact on small integers;
 *                                      g=128 is this build's own definition (the reference has no 128 transform)
 *   orc_quant_rows / orc_sd_quant_rows pinned: torch bf16/f16 tensor arithmetic (divide, round, clamp), closed-form
 *                                      special rows (zero row, single outlier, +-127.5 ties, inf, NaN)
 *   orc_int8_gemm_acc                  pinned: numpy int64 matmul, torch._int_mm
 *   orc_epilogue[_residual]            pinned for the non-fused form: numpy float32 ops; the fused form against exact
 *                                      rational arithmetic.  Which of the two the reference's CUTLASS/nvcc build
 *                                      produces is PARITY UNPINNED (only a run of the reference could tell); both
 *                                      are provided and differ by at most one ulp of the output type.
 *   orc_e4m3_to_f32 / orc_w6_decode    pinned: exhaustive 256 bytes against torch.float8_e4m3fn; exhaustive
 *                                      64 codes x 256 scales against the definition; pack/unpack round trip
 *   orc_f32_to_e4m3 / orc_w6_requant   encoder pinned exhaustively against torch.float8_e4m3fn casts; the requantizer by
 *                                      its invariants (decoded weight within half a grid step of the rotated input in
 *                                      expectation, codes 1..63, scales reproduce the least-squares steps in numpy) --
 *                                      the fma contractions are assumptions about nvcc's default: PARITY UNPINNED
 *   orc_w6a8_group_gemm                this build's own format (no reference counterpart); integer partials pinned by
 *                                      numpy int64
 *   orc_quant_rows_wide                pinned: equals orc_quant_rows for f32, torch bf16 arithmetic on fp32 values
 *   orc_convrot_requant                seed 0 equals orc_quant_rows(rotate 256); the stochastic form against exact
 *                                      rational arithmetic on the same hash values, unbiasedness, hash known answers
 *   orc_convrot_dequant, orc_dequant_i8  numpy products and the dense Kronecker matrix
 *   orc_sd_source_rows                 LN / GEGLU / GroupNorm against torch float64 layer_norm, gelu, group_norm rounded to
 *                                      half; un-padding against a numpy gather.  Last bit vs the reference unpinned, as below
 *   orc_prologue_rows, orc_situ_rows_wide  structure and rounding points pinned: torch float64 / bf16 tensor arithmetic
 *                                      (normalizations, gates, activations from torch.nn.functional) to one ulp of T,
 *                                      closed-form rows.  PARITY UNPINNED against the reference in the last bit: its
 *                                      row sums are fp32 in the order of its thread layout and its expf / erff /
 *                                      tanhf / rsqrtf are CUDA's 1-2 ulp routines; here sums are fp64 rounded once and
 *                                      the functions are correctly rounded (fp64 libm rounded to fp32).
 *   orc_attn_rot128                    pinned: dense Sylvester-Hadamard matrix (scipy) with the sign diagonal, unit columns exact
 *   orc_attn_quant_qk / orc_attn_quant_v  structure pinned: half-step bound of every code against the rotated row with the
 *                                      scale of the group the layout names, V scales against the numpy expression, anchor on
 *                                      for offset keys only; the anchor detector's fma is an assumption about nvcc
 *   orc_attn_int8                      pinned as attention: exact fp64 softmax attention of the same inputs, one-key case.
 *                                      PARITY UNPINNED against a run of the reference (its exp2 / reciprocal are PTX
 *                                      approximations and its build may use fast math): see the section's own header
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2 }; /* csrc/common.cuh:15 */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---------------------------------------------------------------------------------------------
 * Rounding helpers: rnd<T> of csrc/common.cuh:25-28 (round to T with RNE, widen back to float).
 * ------------------------------------------------------------------------------------------- */
ORC_API uint16_t orc_f32_to_bf16(float v) {
    uint32_t u = f2u(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    /* integer form used by tests/sparse_attn_match_comfy.rs:20-23 */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
ORC_API float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
ORC_API float orc_bf16_round(float v) { return orc_bf16_to_f32(orc_f32_to_bf16(v)); }

ORC_API uint16_t orc_f32_to_f16(float v) {
    const uint32_t u = f2u(v);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);          /* NaN */
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);         /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return sign;                                 /* <= 2^-25 rounds to 0 (tie to even) */
    int e = (int)(a >> 23) - 127;
    uint32_t man = (a & 0x7fffffu) | 0x800000u;                       /* 24-bit significand */
    int shift;                                                        /* bits dropped from `man` */
    uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }                /* half subnormal */
    else { shift = 13; base = (uint32_t)(e + 15) << 10; man &= 0x7fffffu; }
    uint32_t keep = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (keep & 1u))) ++keep;           /* RNE; a carry ripples into the exponent */
    return (uint16_t)(sign | (base + keep));
}
ORC_API float orc_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const int e = (h >> 10) & 0x1f;
    const uint32_t m = h & 0x3ffu;
    if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
    if (e == 0) {
        const float f = ldexpf((float)m, -24);
        return (h & 0x8000u) ? -f : f;
    }
    return u2f(sign | ((uint32_t)(e + 112) << 23) | (m << 13));
}
ORC_API float orc_f16_round(float v) { return orc_f16_to_f32(orc_f32_to_f16(v)); }

static inline float rnd_t(int dt, float v) {
    return dt == ORC_BF16 ? orc_bf16_round(v) : dt == ORC_F16 ? orc_f16_round(v) : v;
}
static inline float ld_t(int dt, const void* p, int64_t i) {
    return dt == ORC_BF16 ? orc_bf16_to_f32(((const uint16_t*)p)[i])
         : dt == ORC_F16  ? orc_f16_to_f32(((const uint16_t*)p)[i])
                          : ((const float*)p)[i];
}
static inline void st_t(int dt, void* p, int64_t i, float v) {
    if (dt == ORC_BF16) ((uint16_t*)p)[i] = orc_f32_to_bf16(v);
    else if (dt == ORC_F16) ((uint16_t*)p)[i] = orc_f32_to_f16(v);
    else ((float*)p)[i] = v;
}
/* fmaxf/fminf as the device code uses them: a NaN operand is dropped (csrc/kernels.cu:224,255). */
static inline float fmax_dev(float a, float b) { return isnan(a) ? b : isnan(b) ? a : (a > b ? a : b); }
static inline float fmin_dev(float a, float b) { return isnan(a) ? b : isnan(b) ? a : (a < b ? a : b); }

/* ---------------------------------------------------------------------------------------------
 * ConvRot group transform.  h4_row: csrc/common.cuh:99-106 (left-to-right adds).  Staged order:
 * fht256_rows_smem csrc/common.cuh:110-126 (4 radix-4 stages, strides 1,4,16,64, each scaled by 0.5) and
 * fht64_rows_smem csrc/sd.cu:560-576 (3 stages).  g = 128 has no reference form: it is defined here as the three
 * radix-4 stages of each 64-block WITHOUT their halvings, then one radix-2 stage at stride 64, then one scaling of
 * every output by fl(1/sqrt(2)) / 8 (the three halvings and the 1/sqrt(2) in one exactly representable constant).
 * A halving is exact in fp32, so this equals "halve after every stage, scale the last by fl(1/sqrt(2))" bit for bit
 * as long as no intermediate leaves the normal range; where they differ, this definition overflows to infinity once
 * partial sums pass 3.4e38 (inputs beyond about 5e36 in a group of like signs; the halved form would hold out to
 * 3.4e38) and keeps the low bits of results below 1.2e-38 that the halved form would round away.
 * ------------------------------------------------------------------------------------------- */
static inline float h4_row(int d, float x0, float x1, float x2, float x3) {
    switch (d) {
        case 0: return x0 + x1 + x2 - x3;
        case 1: return x0 + x1 - x2 + x3;
        case 2: return x0 - x1 + x2 + x3;
        default: return -x0 + x1 + x2 + x3;
    }
}
ORC_API int orc_fht(float* row, int K, int g) {
    if (g != 64 && g != 128 && g != 256) return -1;
    if (K % g) return -1;
    const int blk = g == 256 ? 256 : 64;          /* width the radix-4 stages span */
    const int nstage = g == 256 ? 4 : 3;
    for (int stage = 0; stage < nstage; ++stage) {
        const int s = 1 << (2 * stage);
        for (int b = 0; b < K / 4; ++b) {
            const int grp = b / (blk / 4), r = b % (blk / 4);
            const int i0 = grp * blk + (r / s) * (4 * s) + (r % s);
            const float x0 = row[i0], x1 = row[i0 + s], x2 = row[i0 + 2 * s], x3 = row[i0 + 3 * s];
            const float half = g == 128 ? 1.0f : 0.5f;
            row[i0] = half * h4_row(0, x0, x1, x2, x3);
            row[i0 + s] = half * h4_row(1, x0, x1, x2, x3);
            row[i0 + 2 * s] = half * h4_row(2, x0, x1, x2, x3);
            row[i0 + 3 * s] = half * h4_row(3, x0, x1, x2, x3);
        }
    }
    if (g == 128) {
        const float c = 0.70710678118654752f * 0.125f;
        for (int base = 0; base < K; base += 128)
            for (int i = 0; i < 64; ++i) {
                const float a = row[base + i], b = row[base + 64 + i];
                row[base + i] = (a + b) * c;
                row[base + 64 + i] = (a - b) * c;
            }
    }
    return 0;
}

/* `rotate` argument of the drop-in boundary: 0 none; 1 or 256 -> 256 (the reference's flag, csrc/kernels.cu:193);
 * 64 and 128 are this build's extension. */
static int rotate_group(int rotate) {
    if (rotate == 0) return 0;
    if (rotate == 64 || rotate == 128) return rotate;
    return 256;
}

/* ---------------------------------------------------------------------------------------------
 * gpu_quant_rows, PRO_PLAIN: csrc/kernels.cu:271-298 (argument checks), :184-258 (rotation, amax, scale, codes).
 * x is T[M, x_stride], T = bf16 or f32.  The K % 256 check of the reference is relaxed to K % 64 when no 256-wide
 * rotation is asked for (the reference returns -1 there; every reference-valid call behaves identically).
 * ------------------------------------------------------------------------------------------- */
static int quant_check(int dtype, int K, int rotate) {
    const int g = rotate_group(rotate);
    const int need = (g == 256 || g == 0) ? (g == 0 ? 64 : 256) : g;
    if (K <= 0 || (K % need) != 0) return -1;
    if (dtype != ORC_BF16 && dtype != ORC_F32) return -4;
    if (K > 32768) return -2; /* more than 32 warps of 4 groups, csrc/kernels.cu:263-265 */
    return 0;
}
/* ld: the type the row is stored in; rd: the type T whose rounding the quantizer applies.  They differ only for the
 * fused PRO_SITU prologue of a bf16 row, which hands unrounded fp32 values to the quantizer (csrc/kernels.cu:107-112). */
/* csrc/kernels.cu:1355-1359 */
static inline uint32_t pcg_hash(uint32_t x) {
    const uint32_t state = x * 747796405u + 2891336453u;
    const uint32_t word = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
    return (word >> 22u) ^ word;
}
/* bf16 + bf16 rounded once to bf16 (the add instruction behind __hadd, csrc/kernels.cu:1341-1343): the sum is exact in
 * long double / double for the magnitudes here and is rounded by the integer form on the double's bits. */
ORC_API float orc_bf16_add_once(float a, float b);
static inline float bf16_add_once(float a, float b) {
    const double sum = (double)a + (double)b;
    uint64_t u; memcpy(&u, &sum, 8);
    const uint64_t rem = u & ((1ull << 45) - 1), half = 1ull << 44;
    u >>= 45;
    if (rem > half || (rem == half && (u & 1))) ++u;
    u <<= 45;
    double r; memcpy(&r, &u, 8);
    return (float)r;
}
ORC_API float orc_bf16_add_once(float a, float b) { return bf16_add_once(a, b); }
/* seed != 0: the stochastic rounding of gpu_convrot_requant, csrc/kernels.cu:1379-1389. */
static int quant_rows_impl(int ld, int rd, const void* x, int64_t x_stride, int8_t* q, float* scales, int M, int K,
                           int rotate, uint64_t seed) {
    const int rc = quant_check(rd, K, rotate);
    if (rc) return rc;
    const int g = rotate_group(rotate);
    const float tmax = rd == ORC_BF16 ? 3.38953139e38f : 3.402823466e+38f; /* csrc/kernels.cu:48-50 */
#pragma omp parallel
    {
        float* v = (float*)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (int m = 0; m < M; ++m) {
            for (int k = 0; k < K; ++k) v[k] = ld_t(ld, x, (int64_t)m * x_stride + k);
            if (g) orc_fht(v, K, g);
            float amax = 0.f;
            for (int k = 0; k < K; ++k) amax = fmax_dev(amax, fabsf(v[k]));
            const float scale = fmax_dev(fmin_dev(amax, tmax) * (1.f / 127.f), 1.0e-30f); /* :241 */
            scales[m] = scale;
            const float st = rnd_t(rd, scale);                                              /* :243 */
            for (int k = 0; k < K; ++k) {
                const float t = rnd_t(rd, rnd_t(rd, v[k]) / st);                            /* :254 */
                float r = nearbyintf(t);
                if (seed) {
                    const uint64_t key = (uint64_t)((int64_t)m * K + k) + seed;
                    const float noise = (float)(pcg_hash((uint32_t)key ^ (uint32_t)(key >> 32)) >> 8) * 0x1.0p-24f;
                    r = floorf(rd == ORC_F32 ? t + noise : bf16_add_once(t, orc_bf16_round(noise)));
                }
                q[(int64_t)m * K + k] = (int8_t)fmin_dev(127.f, fmax_dev(-128.f, r));
            }
        }
        free(v);
    }
    return 0;
}
ORC_API int orc_quant_rows(int dtype, const void* x, int64_t x_stride, int8_t* q, float* scales, int M, int K,
                           int rotate) {
    return quant_rows_impl(dtype, dtype, x, x_stride, q, scales, M, K, rotate, 0);
}
/* fp32 values quantized with T = rd's rounding. */
ORC_API int orc_quant_rows_wide(int rd, const float* x, int64_t x_stride, int8_t* q, float* scales, int M, int K,
                                int rotate) {
    return quant_rows_impl(ORC_F32, rd, x, x_stride, q, scales, M, K, rotate, 0);
}
/* gpu_convrot_requant, csrc/kernels.cu:1361-1420: weight rows [N, K] (f32, else bf16) -> rotated codes + row scales. */
ORC_API int orc_convrot_requant(int dtype, const void* x, int8_t* q, float* scales, int N, int K, uint64_t seed) {
    const int dt = dtype == ORC_F32 ? ORC_F32 : ORC_BF16;
    return quant_rows_impl(dt, dt, x, K, q, scales, N, K, 1, seed);
}
/* gpu_convrot_dequant (csrc/kernels.cu:1345-1353, out f32 or bf16 bits) and gpu_embed_dequant (:620-631, mode 2: f32
 * holding bf16 values): out = H256(q * s[row]). */
ORC_API int orc_convrot_dequant(int mode, const int8_t* q, const float* s, void* out, int64_t N, int K) {
    if (K <= 0 || K % 256) return -1;
    float* row = (float*)malloc(sizeof(float) * (size_t)K);
    for (int64_t m = 0; m < N; ++m) {
        for (int k = 0; k < K; ++k) row[k] = (float)q[m * K + k] * s[m];
        orc_fht(row, K, 256);
        for (int k = 0; k < K; ++k) {
            if (mode == 1) ((uint16_t*)out)[m * K + k] = orc_f32_to_bf16(row[k]);
            else ((float*)out)[m * K + k] = mode == 2 ? orc_bf16_round(row[k]) : row[k];
        }
    }
    free(row);
    return 0;
}
/* gpu_dequant_i8, csrc/kernels.cu:329-343 */
ORC_API int orc_dequant_i8(const int8_t* q, const float* s, float* out, int64_t N, int64_t K) {
    if (K % 4) return -1;
    for (int64_t i = 0; i < N * K; ++i) out[i] = (float)q[i] * s[i / K];
    return 0;
}

/* gpu_rotate_rows_f32, PRO_PLAIN: csrc/kernels.cu:316-327 with :227-238 (rotation always on, f32 in, f32 out). */
ORC_API int orc_rotate_rows_f32(const float* x, int64_t x_stride, float* out, int M, int K) {
    if (K <= 0 || (K % 256) != 0) return -1;
    if (K > 32768) return -2;
    for (int m = 0; m < M; ++m) {
        float* o = out + (int64_t)m * K;
        for (int k = 0; k < K; ++k) o[k] = x[(int64_t)m * x_stride + k];
        orc_fht(o, K, 256);
    }
    return 0;
}

/* gpu_sd_quant_rows: csrc/sd.cu:578-606 (fp16 rows; rotate in {0,64,256}). */
ORC_API int orc_sd_quant_rows(const uint16_t* x, int64_t x_stride, int8_t* q, float* scales, int M, int K,
                              int rotate) {
    if ((rotate != 0 && rotate != 64 && rotate != 256) || (rotate && K % rotate)) return -1; /* :600 */
#pragma omp parallel
    {
        float* row = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
#pragma omp for schedule(static)
        for (int m = 0; m < M; ++m) {
            for (int k = 0; k < K; ++k) row[k] = orc_f16_to_f32(x[(int64_t)m * x_stride + k]);
            if (rotate) orc_fht(row, K, rotate);
            float mx = 0.f;
            for (int k = 0; k < K; ++k) mx = fmax_dev(mx, fabsf(orc_f16_round(row[k])));     /* :587 */
            const float scale = fmax_dev(mx, 1e-30f) / 127.f;                                /* :589 */
            scales[m] = scale;
            const float sh = orc_f16_round(scale);
            const float st = sh > 0.f ? sh : scale;                                          /* :593 */
            for (int k = 0; k < K; ++k) {
                const float t = orc_f16_round(orc_f16_round(row[k]) / st);
                q[(int64_t)m * K + k] = (int8_t)fmin_dev(127.f, fmax_dev(-128.f, nearbyintf(t)));
            }
        }
        free(row);
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * int8 x int8 -> int32 GEMM, A[M,K] . W[N,K]^T: csrc/vendor/cutlass_gemm_int8.cu:70-75,105 (exact for K <= 13824).
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_int8_gemm_acc(const int8_t* A, const int8_t* W, int32_t* acc, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            const int8_t* a = A + m * K;
            const int8_t* w = W + n * K;
            int32_t s = 0;
            for (int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)w[k];
            acc[m * N + n] = s;
        }
}

/* Dequant epilogue: csrc/vendor/cutlass_gemm_int8.cu:84-95.  t0 = float(acc)*xs[m]; t1 = t0*ws[n];
 * t2 = t1 + float(bias[n]) (bias read in the output type, null = 0); D = Out(t2).  `fma` selects the contracted form
 * fmaf(t0, ws, bias) that nvcc may emit for the last two nodes. */
static inline float epi_plain(int32_t acc, float xs, float ws, float b, int fma) {
    const float t0 = (float)acc * xs;
    return fma ? fmaf(t0, ws, b) : (t0 * ws) + b;
}
ORC_API void orc_epilogue(const int32_t* acc, const float* xs, const float* ws, const void* bias, void* D, int64_t M,
                          int64_t N, int out_dt, int fma) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            const float b = bias ? ld_t(out_dt, bias, n) : 0.f;
            st_t(out_dt, D, m * N + n, epi_plain(acc[m * N + n], xs[m], ws[n], b, fma));
        }
}
/* Residual epilogue: csrc/vendor/cutlass_gemm_int8.cu:149-161.  z = Out(plain epilogue);
 * D = Out(float(z)*float(rscale[n]) + float(resid[m,n])).  D may alias resid (csrc/gemm.cu:131). */
ORC_API void orc_epilogue_residual(const int32_t* acc, const float* xs, const float* ws, const void* bias,
                                   const void* rscale, const void* resid, void* D, int64_t M, int64_t N, int out_dt,
                                   int fma) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            const float b = bias ? ld_t(out_dt, bias, n) : 0.f;
            const float z = rnd_t(out_dt, epi_plain(acc[m * N + n], xs[m], ws[n], b, fma));
            const float rs = ld_t(out_dt, rscale, n), r = ld_t(out_dt, resid, m * N + n);
            st_t(out_dt, D, m * N + n, fma ? fmaf(z, rs, r) : (z * rs) + r);
        }
}

/* gpu_int8_gemm: csrc/gemm.cu:124-129 -> launch_cutlass_int8_dequant csrc/vendor/cutlass_gemm_int8.cu:373-388.
 * Returns 0, or -200 for an unknown output type.  M, N or K == 0 returns 0 and writes nothing (:377). */
ORC_API int orc_int8_gemm(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias, void* D,
                          int64_t M, int64_t N, int64_t K, int out_dt, int fma) {
    if (M == 0 || N == 0 || K == 0) return 0;
    if (out_dt < 0 || out_dt > 2) return -200;
    int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M * N));
    orc_int8_gemm_acc(A, W, acc, M, N, K);
    orc_epilogue(acc, xs, ws, bias, D, M, N, out_dt, fma);
    free(acc);
    return 0;
}
/* gpu_int8_gemm_residual: csrc/gemm.cu:132-140 -> launch_cutlass_int8_dequant_residual
 * csrc/vendor/cutlass_gemm_int8.cu:348-371: M or N == 0 -> ok; K == 0 or a null rscale/resid -> refused (-201). */
ORC_API int orc_int8_gemm_residual(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias,
                                   const void* rscale, const void* resid, void* D, int64_t M, int64_t N, int64_t K,
                                   int out_dt, int fma) {
    if (M == 0 || N == 0) return 0;
    if (K == 0 || !rscale || !resid) return -201;
    if (out_dt < 0 || out_dt > 2) return -201;
    int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M * N));
    orc_int8_gemm_acc(A, W, acc, M, N, K);
    orc_epilogue_residual(acc, xs, ws, bias, rscale, resid, D, M, N, out_dt, fma);
    free(acc);
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * W6 decode, reference format: csrc/h3.cu:5 (e4m3), :11-46.  Row n = K/2 nibble bytes then K/4 top-bit bytes;
 * s_rel is fp8-e4m3 [N, K/G]; out = clamp(rint((c-32)*s), -127, 127).
 * ------------------------------------------------------------------------------------------- */
ORC_API float orc_e4m3_to_f32(uint8_t v) {
    const int s = v >> 7, e = (v >> 3) & 0xf, m = v & 7;
    float f;
    if (e == 15 && m == 7) f = NAN;                         /* S.1111.111 is the only NaN; there is no infinity */
    else if (e == 0) f = ldexpf((float)m, -9);              /* subnormal: m/8 * 2^-6 */
    else f = ldexpf((float)(8 + m), e - 10);                /* (1 + m/8) * 2^(e-7) */
    return s ? -f : f;
}
ORC_API int orc_w6_decode(const uint8_t* q, const uint8_t* s_rel, int8_t* out, int64_t N, int K, int G) {
    if (K % 32 || G % 16) return -1; /* csrc/h3.cu:41 */
    for (int64_t n = 0; n < N; ++n) {
        const uint8_t* lo = q + n * (K * 3 / 4);
        const uint8_t* hi = lo + K / 2;
        for (int e = 0; e < K; ++e) {
            const unsigned nib = (lo[e / 2] >> (4 * (e & 1))) & 0xFu;
            const unsigned top = (hi[e / 4] >> (2 * (e & 3))) & 3u;
            const unsigned c = nib | (top << 4);
            const float s = orc_e4m3_to_f32(s_rel[n * (K / G) + e / G]);
            out[n * K + e] = (int8_t)fmin_dev(127.f, fmax_dev(-127.f, nearbyintf(((float)c - 32.f) * s)));
        }
    }
    return 0;
}
/* Packer for the reference two-plane layout (the inverse of the unpack above; layout from
 * csrc/vendor/w6a8_requant.cu:138-150).  codes[N,K] hold c = q+32 in 0..63. */
ORC_API void orc_w6_pack_planes(const uint8_t* codes, uint8_t* q, int64_t N, int K) {
    for (int64_t n = 0; n < N; ++n) {
        uint8_t* lo = q + n * (K * 3 / 4);
        uint8_t* hi = lo + K / 2;
        memset(lo, 0, (size_t)(K * 3 / 4));
        for (int e = 0; e < K; ++e) {
            const unsigned c = codes[n * K + e] & 63u;
            lo[e / 2] |= (uint8_t)((c & 0xFu) << (4 * (e & 1)));
            hi[e / 4] |= (uint8_t)((c >> 4) << (2 * (e & 3)));
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * W6 requantizer, reference format: csrc/vendor/w6a8_requant.cu (one launch: bf16 weight in its original basis ->
 * ConvRot256 -> two-plane 6-bit codes + e4m3 s_rel per 32 + f32 s_channel).  Cited by line below.  Expressions of the
 * form a*b + c are contracted to an fma where nvcc's default would (num += w*q, den += q*q, lo + u*(hi - lo)).
 * ------------------------------------------------------------------------------------------- */
/* __nv_cvt_float_to_fp8(x, __NV_SATFINITE, __NV_E4M3) for finite x: round to nearest even, saturate at 448. */
ORC_API uint8_t orc_f32_to_e4m3(float x) {
    const uint8_t sgn = (uint8_t)((f2u(x) >> 31) << 7);
    const float a = fabsf(x);
    if (a != a) return (uint8_t)(sgn | 0x7f);
    if (a > 448.f) return (uint8_t)(sgn | 0x7e);
    if (a < 0.015625f) return (uint8_t)(sgn | (uint8_t)nearbyintf(a * 512.f));   /* subnormals: multiples of 2^-9 */
    int ex;
    const float f = frexpf(a, &ex);                                               /* a = f * 2^ex, f in [0.5, 1) */
    int m = (int)nearbyintf((2.f * f - 1.f) * 8.f), e = ex - 1;
    if (m == 8) { m = 0; ++e; }
    const int code = ((e + 7) << 3) | m;
    return (uint8_t)(sgn | (code > 0x7e ? 0x7e : code));
}
static inline float w6_level(int i, float s) {                                    /* :59-61 */
    return fmin_dev(127.f, fmax_dev(-127.f, nearbyintf((float)(i - 31) * s)));
}
static inline int w6_lower_bound(float t, float s, float inv_s) {                 /* :63-69 */
    const float est = nearbyintf((ceilf(t) - 0.5f) * inv_s);                      /* __float2int_rn saturates */
    int i = (est > 2.0e9f ? 2000000000 : est < -2.0e9f ? -2000000000 : (int)est) + 31;
    i = i < 0 ? 0 : i > 63 ? 63 : i;
    while (i > 0 && w6_level(i - 1, s) >= t) --i;
    while (i < 63 && w6_level(i, s) < t) ++i;
    return i;
}
static inline float rq_uniform(int64_t idx, uint64_t seed) {                      /* :27-31 */
    const uint32_t h = pcg_hash((uint32_t)idx ^ (uint32_t)seed ^ (uint32_t)(seed >> 32));
    return (float)(h >> 8) * (1.0f / 16777216.0f);
}
ORC_API int orc_w6_requant(const uint16_t* w, uint8_t* packed, uint8_t* s_rel, float* s_channel, int64_t N, int K,
                           uint64_t seed) {
    if (K % 256) return -1;                                                        /* :243 */
    enum { G = 32 };
    float* row = (float*)malloc(sizeof(float) * (size_t)K);
    float* gscale = (float*)malloc(sizeof(float) * (size_t)(K / G));
    for (int64_t n = 0; n < N; ++n) {
        /* rotation, the result rounded to the weight dtype: :174-218 (the butterflies of orc_fht, group 256) */
        for (int k = 0; k < K; ++k) row[k] = orc_bf16_to_f32(w[n * K + k]);
        orc_fht(row, K, 256);
        for (int k = 0; k < K; ++k) row[k] = orc_bf16_round(row[k]);
        /* phase 1: per-group step, two alternating-least-squares rounds; row amax of the decoded weight (:94-120) */
        float row_amax = 0.f;
        for (int g = 0; g < K / G; ++g) {
            const float* x = row + g * G;
            float amax = 0.f;
            for (int i = 0; i < G; ++i) amax = fmax_dev(amax, fabsf(x[i]));
            float gs = fmax_dev(amax / 31.0f, 1e-8f), inv = 1.0f / gs;
            for (int it = 0; it < 2; ++it) {
                float num = 0.f, den = 0.f;
                for (int i = 0; i < G; ++i) {
                    const float q = fmin_dev(31.0f, fmax_dev(-31.0f, nearbyintf(x[i] * inv)));
                    num = fmaf(x[i], q, num);
                    den = fmaf(q, q, den);
                }
                gs = fmax_dev(num / fmax_dev(den, 1e-8f), 1e-8f);
                inv = 1.0f / gs;
            }
            gscale[g] = gs;
            for (int i = 0; i < G; ++i)
                row_amax = fmax_dev(row_amax, fabsf(fmin_dev(31.0f, fmax_dev(-31.0f, nearbyintf(x[i] * inv))) * gs));
        }
        const float sc = fmax_dev(row_amax / 127.0f, 1e-8f), inv_sc = 1.0f / sc;    /* :121-123 */
        s_channel[n] = sc;
        /* phase 2: e4m3 s_rel, stochastic grid assignment (the launcher always passes stochastic = true, :249),
         * code = level index + 1 = q + 32, two-plane pack (:126-151) */
        uint8_t* lo = packed + n * (K * 3 / 4);
        uint8_t* hi = lo + K / 2;
        memset(lo, 0, (size_t)(K * 3 / 4));
        for (int g = 0; g < K / G; ++g) {
            const uint8_t bits = orc_f32_to_e4m3(gscale[g] / sc);
            s_rel[n * (K / G) + g] = bits;
            const float sr = orc_e4m3_to_f32(bits), inv_sr = 1.0f / fmax_dev(sr, 1e-30f);
            for (int i = 0; i < G; ++i) {
                const int e = g * G + i;
                const float t = row[e] * inv_sc;
                const int pos = w6_lower_bound(t, sr, inv_sr);
                int l = pos - 1;                                                  /* :75-80 */
                l = l < 0 ? 0 : l > 61 ? 61 : l;
                const float level_lo = w6_level(l, sr);
                const float thr = fmaf(rq_uniform(n * K + e, seed), w6_level(l + 1, sr) - level_lo, level_lo);
                int lev = l + (t > thr ? 1 : 0);
                lev = lev > 62 ? 62 : lev;
                const unsigned c = (unsigned)(lev + 1);
                lo[e / 2] |= (uint8_t)((c & 0xFu) << (4 * (e & 1)));
                hi[e / 4] |= (uint8_t)((c >> 4) << (2 * (e & 3)));
            }
        }
    }
    free(row);
    free(gscale);
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * W6A8 with per-group weight scales: this build's own format (the reference has none like it).
 * Weights: 4 codes per 3 bytes along K, 24-bit little-endian word u0 | u1<<6 | u2<<12 | u3<<18 with u = q + 32,
 * q in [-31,31]; sw f32 [N, K/128].  For each output: p_g = sum over group g of A*q (int32, exact);
 * accf = fmaf((float)p_g, sw[n,g], accf) for g ascending from accf = 0; y = Out(fmaf(accf, xs[m], bias[n])).
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_w6_pack_words(const int8_t* qv, uint8_t* packed, int64_t N, int K) {
    for (int64_t n = 0; n < N; ++n)
        for (int k = 0; k < K; k += 4) {
            uint32_t w = 0;
            for (int j = 0; j < 4; ++j) w |= (uint32_t)((qv[n * K + k + j] + 32) & 63) << (6 * j);
            uint8_t* p = packed + n * (K * 3 / 4) + (k / 4) * 3;
            p[0] = (uint8_t)w; p[1] = (uint8_t)(w >> 8); p[2] = (uint8_t)(w >> 16);
        }
}
ORC_API void orc_w6_unpack_words(const uint8_t* packed, int8_t* qv, int64_t N, int K) {
    for (int64_t n = 0; n < N; ++n)
        for (int k = 0; k < K; k += 4) {
            const uint8_t* p = packed + n * (K * 3 / 4) + (k / 4) * 3;
            const uint32_t w = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
            for (int j = 0; j < 4; ++j) qv[n * K + k + j] = (int8_t)((int)((w >> (6 * j)) & 63u) - 32);
        }
}
ORC_API int orc_w6a8_group_gemm(const int8_t* A, const uint8_t* packed, const float* xs, const float* sw,
                                const void* bias, void* D, int32_t* partials, int64_t M, int64_t N, int64_t K,
                                int out_dt) {
    if (K % 128) return -1;
    if (out_dt < 0 || out_dt > 2) return -200;
    if (M == 0 || N == 0) return 0;
    const int64_t ng = K / 128;
    int8_t* w = (int8_t*)malloc((size_t)(N * K));
    orc_w6_unpack_words(packed, w, N, (int)K);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float accf = 0.f;
            for (int64_t g = 0; g < ng; ++g) {
                int32_t p = 0;
                for (int64_t k = g * 128; k < (g + 1) * 128; ++k) p += (int32_t)A[m * K + k] * (int32_t)w[n * K + k];
                if (partials) partials[(m * N + n) * ng + g] = p;
                accf = fmaf((float)p, sw[n * ng + g], accf);
            }
            const float b = bias ? ld_t(out_dt, bias, n) : 0.f;
            st_t(out_dt, D, m * N + n, fmaf(accf, xs[m], b));
        }
    free(w);
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Row prologues: csrc/kernels.cu:88-182 (inside quant_rows_kernel) and :348-418 (prologue_rows_kernel), helpers
 * csrc/common.cuh:71-95, ln_finish csrc/kernels.cu:40-46.  Writes the T row the quantizer would consume.
 * prologue ids: csrc/kernels.cu:13-15.  SITU is the eager chain of :409-417.
 * ------------------------------------------------------------------------------------------- */
enum { OP_PLAIN = 0, OP_RMS = 1, OP_GATE = 2, OP_SWIGLU = 3, OP_LAYERNORM = 4, OP_SILU = 5, OP_GELU = 6, OP_ADALN = 7,
       OP_SITU = 8, OP_LN_MOD = 9, OP_LN_AFFINE = 10, OP_GELU_TANH = 11, OP_LN_AFFINE_SILU = 12 };
static inline float exp_cr(float x) { return (float)exp((double)x); }
static inline float silu_o(float x) { return x / (1.f + exp_cr(-x)); }
static inline float sigmoid_o(float x) { return 1.f / (1.f + exp_cr(-x)); }
static inline float stable_tanh_o(float x) {
    const float t = (float)expm1((double)(-2.f * fabsf(x)));
    return copysignf(-t / (t + 2.f), x);
}
static inline float gelu_o(float x) { return 0.5f * x * (1.f + (float)erf((double)(x * 0.70710678118654752f))); }
static inline float gelu_tanh_o(float x) {
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    return 0.5f * x * (1.f + (float)tanh((double)(k0 * fmaf(k1 * x * x, x, x))));
}
/* situ_f, csrc/common.cuh:80-82: one float expression; the fused PRO_SITU of the quantizer (csrc/kernels.cu:107-112)
 * hands its unrounded value on.  out: fp32 [M, K]. */
ORC_API int orc_situ_rows_wide(int dt, const void* x, int64_t x_stride, int64_t up_offset, float* out, int M, int K) {
    if (dt < 0 || dt > 2) return -4;
    for (int64_t m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            const float hidden = ld_t(dt, x, m * x_stride + k), gate = ld_t(dt, x, m * x_stride + up_offset + k);
            out[m * K + k] = 4.f * stable_tanh_o(gate / 4.f) / (1.f + exp_cr(-gate)) * (25.f * stable_tanh_o(hidden / 25.f));
        }
    return 0;
}
ORC_API int orc_prologue_rows(int dt, int pro, const void* x, int64_t x_stride, const void* g, int64_t g_stride,
                              int64_t up_offset, const float* norm_w, const float* norm_b, float eps, const void* ms,
                              const void* sh, void* out, int64_t out_stride, int M, int K) {
    if (dt < 0 || dt > 2) return -4;
    if (pro < OP_PLAIN || pro > OP_LN_AFFINE_SILU) return -3;
    for (int64_t m = 0; m < M; ++m) {
        const int64_t xb = m * x_stride, ob = m * out_stride;
#define X(k) ld_t(dt, x, xb + (k))
#define R(v) rnd_t(dt, (v))
        if (pro == OP_RMS || pro == OP_ADALN || pro == OP_LAYERNORM || pro >= OP_LN_MOD && pro != OP_GELU_TANH) {
            const int ln = pro != OP_RMS && pro != OP_ADALN;
            float mean = 0.f;
            if (ln) {
                double s = 0.0;
                for (int k = 0; k < K; ++k) s += (double)X(k);
                mean = (float)s / (float)K;
            }
            double s2 = 0.0;
            for (int k = 0; k < K; ++k) { const float v = X(k) - mean; s2 += (double)v * (double)v; }
            const float ss = (float)s2;
            const float rstd = (float)(1.0 / sqrt((double)(ss / (float)K + eps)));
            for (int k = 0; k < K; ++k) {
                float n = (X(k) - mean) * rstd;
                const float msv = ms ? ld_t(dt, ms, k) : 0.f, shv = ms ? ld_t(dt, sh, k) : 0.f;
                float r;
                if (pro == OP_ADALN) r = fmaf(n, 1.f + msv, shv);
                else if (pro == OP_LN_MOD) r = fmaf(R(n), R(1.f + msv), shv);
                else if (pro == OP_LN_AFFINE) r = fmaf(n, norm_w[k], norm_b[k]);
                else if (pro == OP_LN_AFFINE_SILU) r = silu_o(R(fmaf(n, norm_w[k], norm_b[k])));
                else {
                    if (norm_w) n *= norm_w[k];
                    n = R(n);
                    if (ms) { const float a = R(1.f + msv); n = R(a * n); n = R(n + shv); }
                    r = n;
                }
                st_t(dt, out, ob + k, r);
            }
        } else if (pro == OP_GATE) {
            for (int k = 0; k < K; ++k) st_t(dt, out, ob + k, X(k) * R(sigmoid_o(ld_t(dt, g, m * g_stride + k))));
        } else if (pro == OP_SWIGLU) {
            for (int k = 0; k < K; ++k) st_t(dt, out, ob + k, R(silu_o(X(k))) * X(up_offset + k));
        } else if (pro == OP_SILU) {
            for (int k = 0; k < K; ++k) st_t(dt, out, ob + k, silu_o(X(k)));
        } else if (pro == OP_GELU) {
            for (int k = 0; k < K; ++k) st_t(dt, out, ob + k, gelu_o(X(k)));
        } else if (pro == OP_GELU_TANH) {
            for (int k = 0; k < K; ++k) st_t(dt, out, ob + k, gelu_tanh_o(X(k)));
        } else if (pro == OP_SITU) {
            for (int k = 0; k < K; ++k) {
                const float hidden = X(k), gate = X(up_offset + k);
                const float capped = R(4.f * R(stable_tanh_o(R(gate / 4.f))));
                const float gg = R(capped * R(sigmoid_o(gate)));
                const float h = R(25.f * R(stable_tanh_o(R(hidden / 25.f))));
                st_t(dt, out, ob + k, gg * h);
            }
        } else {
            for (int k = 0; k < K; ++k) st_t(dt, out, ob + k, X(k));
        }
#undef X
#undef R
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * The SD UNet's fused quantizer sources, csrc/sd.cu:611-663: the half row that LayerNorm (:629-641), GEGLU (:642-649),
 * head un-padding (:650-652) or GroupNorm without SiLU (:653-662, statistics :203-207) would have written; the fp16
 * quantizer (orc_sd_quant_rows) then reads it.  Sums in fp64 rounded once, 1/sqrt correctly rounded, as in the prologues.
 * mode: 1 LN, 2 GEGLU, 3 UNPAD, 4 GN.  out: half bits [M, K].
 * ------------------------------------------------------------------------------------------- */
ORC_API int orc_sd_source_rows(int mode, const uint16_t* x, int64_t x_stride, const float* w, const float* b, float eps,
                               int heads, int d, int dp, int groups, int64_t P, uint16_t* out, int M, int K) {
    if (mode < 1 || mode > 4) return -3;
    if (mode == 4 && (groups <= 0 || K % groups)) return -1;
    for (int64_t m = 0; m < M; ++m) {
        uint16_t* o = out + m * K;
        if (mode == 1) {
            const uint16_t* r = x + m * x_stride;
            double s = 0.0;
            for (int k = 0; k < K; ++k) s += (double)orc_f16_to_f32(r[k]);
            const float mean = (float)s / (float)K;
            double s2 = 0.0;
            for (int k = 0; k < K; ++k) { const float dd = orc_f16_to_f32(r[k]) - mean; s2 += (double)dd * (double)dd; }
            const float rstd = (float)(1.0 / sqrt((double)((float)s2 / (float)K + eps)));
            for (int k = 0; k < K; ++k) o[k] = orc_f32_to_f16(fmaf((orc_f16_to_f32(r[k]) - mean) * rstd, w[k], b[k]));
        } else if (mode == 2) {
            const uint16_t* r = x + m * 2 * K;
            for (int k = 0; k < K; ++k)
                o[k] = orc_f32_to_f16(orc_f16_to_f32(r[k]) * orc_f16_round(gelu_o(orc_f16_to_f32(r[K + k]))));
        } else if (mode == 3) {
            const uint16_t* r = x + m * heads * dp;
            for (int k = 0; k < K; ++k) o[k] = r[(k / d) * dp + k % d];
        } else {
            const int per = K / groups;
            const int64_t n = m / P;
            const uint16_t* img = x + n * P * K;
            for (int g = 0; g < groups; ++g) {
                /* statistics of (image n, group g); recomputed per row for simplicity, rows of one image agree */
                double s = 0.0, ss = 0.0;
                for (int64_t pp = 0; pp < P; ++pp)
                    for (int c = 0; c < per; ++c) { const double v = (double)orc_f16_to_f32(img[pp * K + g * per + c]); s += v; ss += v * v; }
                const double cnt = (double)P * per, mean = s / cnt;
                const double var = fmax(ss / cnt - mean * mean, 0.0);
                const float mf = (float)mean, rf = (float)(1.0 / sqrt(var + (double)eps));
                for (int c = g * per; c < (g + 1) * per; ++c)
                    o[c] = orc_f32_to_f16(fmaf((orc_f16_to_f32(x[m * K + c]) - mf) * rf, w[c], b[c]));
            }
        }
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * The whole linear on the CPU (quantize -> GEMM -> epilogue), for the bench's CPU-baseline leg.  Row-parallel with
 * OpenMP; returns the thread count it ran with through *threads.
 * ------------------------------------------------------------------------------------------- */
#ifdef _OPENMP
#include <omp.h>
#endif
ORC_API int orc_linear_w8a8(int dtype, const void* x, int64_t x_stride, int rotate, const int8_t* W, const float* ws,
                            const void* bias, void* D, int M, int N, int K, int out_dt, int fma, int* threads) {
    int8_t* q = (int8_t*)malloc((size_t)M * (size_t)K);
    float* xs = (float*)malloc(sizeof(float) * (size_t)M);
    int rc = orc_quant_rows(dtype, x, x_stride, q, xs, M, K, rotate);
    if (!rc) rc = orc_int8_gemm(q, W, xs, ws, bias, D, M, N, K, out_dt, fma);
    free(q);
    free(xs);
    if (threads) {
#ifdef _OPENMP
        *threads = omp_get_max_threads();
#else
        *threads = 1;
#endif
    }
    return rc;
}
ORC_API void orc_set_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n > 0 ? n : 1);
#else
    (void)n;
#endif
}

/* ---------------------------------------------------------------------------------------------
 * INT8 attention, head dim 128 (csrc/attn_int8.cu:118-160 chains the three stages below).
 *
 * PARITY UNPINNED against a run of the reference: its exp2 and reciprocal are PTX approximations
 * (csrc/vendor/sage/math.cuh:54-58,111-115), and its build compiles the sage units (quant_qk_int8.cu, quant_v_int8.cu,
 * sage_attn_launcher.cu with the attention kernel) with --use_fast_math (build.rs:84-86,139-141): approximate division,
 * reciprocal and rsqrt, denormals flushed, so the scales mx / 127 + 1e-7 and 1 / scale can differ from IEEE in the last
 * bit and a code that sits on a rounding boundary with them.  Here exp2 is fp64 libm rounded to fp32 and divisions are
 * IEEE.  (The linear path's units -- kernels.cu, gemm.cu, sd.cu, h3.cu, cutlass_gemm_int8.cu -- are built without fast
 * math, build.rs:69-81.)  The structure (rotation, scale groups, anchor, tile maxima, u8
 * probabilities, integer P.V partials folded with fmaf) is pinned by the tests against a dense Hadamard matrix, the
 * quantizer's half-step bound and exact fp64 softmax attention.
 * ------------------------------------------------------------------------------------------- */
#define ATTN_DMAX 256   /* head dims 64, 128, 256 (csrc/attn_int8.cu:42-45) */
#define ATTN_U8_OFFSET 7.9943534f   /* csrc/vendor/sage/attn_utils.cuh:40 */

/* Sign diagonal, then a normalized Walsh-Hadamard transform over 128 channels: H4 on each run of four channels, then
 * radix-2 butterflies over channel bits 2..6, then one scaling (csrc/vendor/sage/quant_qk_int8.cu:72-109,136-157). */
/* The normalized H4 on each run of four adjacent channels (convrot4, quant_qk_int8.cu:72-85). */
static void attn_h4(float* v, int n) {
    for (int g = 0; g < n; g += 4) {
        const float a0 = v[g] + v[g + 1], a1 = v[g] - v[g + 1], a2 = v[g + 2] + v[g + 3], a3 = v[g + 2] - v[g + 3];
        v[g] = (a0 + a2) * 0.5f;
        v[g + 1] = (a1 + a3) * 0.5f;
        v[g + 2] = (a0 - a2) * 0.5f;
        v[g + 3] = (a1 - a3) * 0.5f;
    }
}
/* Walsh-Hadamard over n = 64 or 128 channels without the sign diagonal: H4, then radix-2 butterflies over the lane
 * bits (channel bits 2 and up) in ascending order, then one scaling (convrot64 :111-133, convrot128_plain :136-157). */
static void attn_h_plain(float* v, int n, float scale) {
    attn_h4(v, n);
    for (int bit = 1; bit < n / 4; bit <<= 1)
        for (int lane = 0; lane < n / 4; ++lane) {
            if (lane & bit) continue;
            for (int c = 0; c < 4; ++c) {
                const float lo = v[lane * 4 + c], hi = v[(lane | bit) * 4 + c];
                v[lane * 4 + c] = lo + hi;
                v[(lane | bit) * 4 + c] = lo - hi;
            }
        }
    for (int ch = 0; ch < n; ++ch) v[ch] *= scale;
}
ORC_API void orc_attn_rot128(float* v) {
    static const uint32_t signs[4] = {0x1035997bu, 0x8087f5eeu, 0xee2e4e1au, 0x71132418u};
    for (int ch = 0; ch < 128; ++ch) {
        const int lane = ch >> 2, c = ch & 3;
        const uint32_t flip = ((signs[lane >> 3] >> ((lane & 7) * 4 + c)) & 1u) ^ 1u;
        v[ch] = u2f(f2u(v[ch]) ^ (flip << 31));
    }
    attn_h_plain(v, 128, 0.1767766952966369f);
}

/* The rotation the quantizers apply, chosen by head dim and key count (quant_qk_int8.cu:1150-1195): sequences of at most
 * 256 keys take only the H4 blocks (ROTATION 4); longer ones H64 at head dim 64, the sign diagonal and H128 at 128, and
 * the plain H128 on each half at 256 (ROTATION 64, 128, 129). */
ORC_API void orc_attn_rotate_d(float* v, int D, int lk) {
    if (lk <= 256) attn_h4(v, D);
    else if (D == 64) attn_h_plain(v, 64, 0.25f);
    else if (D == 128) orc_attn_rot128(v);
    else {
        attn_h_plain(v, 128, 0.1767766952966369f);
        attn_h_plain(v + 128, 128, 0.1767766952966369f);
    }
}
ORC_API void orc_attn_rotate(float* v, int lk) { orc_attn_rotate_d(v, 128, lk); }

static inline int8_t attn_rn_s8(float v) {                       /* cvt.rni.sat.s8.f32, float_utils.cuh:39-45 */
    if (isnan(v)) return 0;
    const float r = rintf(v);
    return (int8_t)(r > 127.f ? 127.f : r < -128.f ? -128.f : r);
}

/* The 32-lane shfl_down tree as lane 0 sees it (quant_qk_int8.cu:664-674). */
static float attn_tree_sum32(const float* x) {
    float t[32];
    memcpy(t, x, sizeof t);
    for (int off = 16; off > 0; off >>= 1)
        for (int i = 0; i < off; ++i) t[i] += t[i + off];
    return t[0];
}

/* Per-head RMSNorm, weight and RoPE of a 128-channel row ahead of the quantizers: gpu_qk_norm_rope (csrc/kernels.cu:482-540)
 * as the INT8 attention applies it in its quantizers (csrc/vendor/sage/quant_qk_int8.cu:160-291), bf16 rows.
 * v = bf16((v * rstd) * w), rstd = 1/sqrt(mean(v^2) + eps); rope_mode 1 turns the pairs (2p, 2p+1), 2 the pairs
 * (j, j+64), by (cos, sin) = rope_row[2p], rope_row[2p+1]; the result is rounded to bf16 again.
 * The sum of squares follows the reference's lane order.  Where the reference depends on its machine this build
 * defines: a correctly rounded 1/sqrt (CUDA's rsqrtf is an approximation, up to 2 ulp) and c*a - s*b / s*a + c*b
 * contracted to one fma on their first product.  Against a run of the reference: parity unpinned for those two. */
typedef struct { const float* w; const float* rope; float eps; int mode; int on; } attn_norm_t;

/* Sum of squares of a 128-channel row in the order of the reference's warp: lane l accumulates its four channels by fma
 * in order (nvcc contracts ss += v * v), then warp_sum adds lanes at distances 16, 8, 4, 2, 1 (csrc/common.cuh:30-34).
 * Lane l owns channels 4l..4l+3, or with rope_mode 2 (split, with or without a table) 2l, 2l+1, 64+2l, 65+2l
 * (csrc/kernels.cu:497-505). */
ORC_API float orc_attn_sumsq128(const float* v, int split) {
    float lane[32];
    for (int l = 0; l < 32; ++l) {
        const int i0 = split ? 2 * l : 4 * l, i2 = split ? 64 + 2 * l : 4 * l + 2;
        float t = fmaf(v[i0], v[i0], 0.f);
        t = fmaf(v[i0 + 1], v[i0 + 1], t);
        t = fmaf(v[i2], v[i2], t);
        lane[l] = fmaf(v[i2 + 1], v[i2 + 1], t);
    }
    for (int o = 16; o > 0; o >>= 1) {
        float nx[32];
        for (int l = 0; l < 32; ++l) nx[l] = lane[l] + lane[l ^ o];
        memcpy(lane, nx, sizeof nx);
    }
    return lane[0];
}

static void attn_norm_rope_row(float* v, const attn_norm_t* nm, int row) {
    const int D = 128;   /* the fused norm exists for head dim 128 only (csrc/attn_int8.cu:135) */
    const float rstd = (float)(1.0 / sqrt((double)(orc_attn_sumsq128(v, nm->mode == 2) / 128.f + nm->eps)));
    for (int c = 0; c < D; ++c) v[c] = rnd_t(ORC_BF16, v[c] * rstd * (nm->w ? nm->w[c] : 1.f));
    if (!nm->rope || nm->mode == 0) return;
    const float* r = nm->rope + (int64_t)row * D;
    if (nm->mode == 1) {
        for (int p = 0; p < 64; ++p) {
            const float c = r[2 * p], s = r[2 * p + 1], a = v[2 * p], b = v[2 * p + 1];
            v[2 * p] = rnd_t(ORC_BF16, fmaf(c, a, -(s * b)));
            v[2 * p + 1] = rnd_t(ORC_BF16, fmaf(s, a, c * b));
        }
    } else {
        for (int j = 0; j < 64; ++j) {
            const float c = r[2 * j], s = r[2 * j + 1], a = v[j], b = v[j + 64];
            v[j] = rnd_t(ORC_BF16, fmaf(a, c, -(b * s)));
            v[j + 64] = rnd_t(ORC_BF16, fmaf(b, c, a * s));
        }
    }
}

/* One row of q or k as the quantizer sees it. */
static void attn_load_row(int dt, const void* x, int64_t base, int64_t stride_n, int row, const attn_norm_t* nm, int D, float* out) {
    for (int c = 0; c < D; ++c) out[c] = ld_t(dt, x, base + (int64_t)row * stride_n + c);
    if (nm && nm->on) attn_norm_rope_row(out, nm, row);
}

/* K anchor for one (batch, head): nine evenly spaced keys, the one closest to their mean, kept only when it lowers
 * the sampled energy without raising the sampled abs-max by more than 12.5 % (quant_qk_int8.cu:591-756).  The
 * reference's block has 128 threads in four warps; thread t walks channels t and t + 128 (head dim 256) with one set of
 * accumulators, threads past the head dim (64) hold zeros; warps add by a shuffle-down tree, then the four warps in
 * order.  The distance 9*s - sum is taken as one fma, nvcc's default contraction. */
static int attn_detect_anchor(int dt, const void* k, int64_t base, int64_t stride_n, int Lk, const attn_norm_t* nm, int D) {
    float s[9][ATTN_DMAX];
    for (int i = 0; i < 9; ++i) attn_load_row(dt, k, base, stride_n, (int)((int64_t)i * (Lk - 1) / 8), nm, D, s[i]);
    float energy[128], dist[9][128], amax = 0.f;
    for (int t = 0; t < 128; ++t) {
        float e = 0.f, d9[9] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int c = t; c < D; c += 128) {
            float sum = 0.f;
            for (int i = 0; i < 9; ++i) {
                e = fmaf(s[i][c], s[i][c], e);
                amax = fmax_dev(amax, fabsf(s[i][c]));
                sum += s[i][c];
            }
            for (int i = 0; i < 9; ++i) {
                const float d = fmaf(9.f, s[i][c], -sum);
                d9[i] = fmaf(d, d, d9[i]);
            }
        }
        energy[t] = e;
        for (int i = 0; i < 9; ++i) dist[i][t] = d9[i];
    }
    int best = 0;
    float best_d = 3.402823466e+38F;
    for (int i = 0; i < 9; ++i) {
        float d = 0.f;
        for (int w = 0; w < 4; ++w) d += attn_tree_sum32(&dist[i][w * 32]);
        if (d < best_d) { best = i; best_d = d; }
    }
    float e0 = 0.f, e1 = 0.f, m1 = 0.f;
    float be[128];
    for (int t = 0; t < 128; ++t) {
        float e = 0.f;
        for (int c = t; c < D; c += 128)
            for (int i = 0; i < 9; ++i) {
                const float r = s[i][c] - s[best][c];
                e = fmaf(r, r, e);
                m1 = fmax_dev(m1, fabsf(r));
            }
        be[t] = e;
    }
    for (int w = 0; w < 4; ++w) {
        e0 += attn_tree_sum32(&energy[w * 32]);
        e1 += attn_tree_sum32(&be[w * 32]);
    }
    return (e1 < e0 && m1 <= amax * 1.125f) ? (int)((int64_t)best * (Lk - 1) / 8) : -1;
}

/* One scale group: rows[0..n) (absolute row numbers, those >= L skipped) of one head, minus `bias` when given,
 * rotated, abs-max over the group, scale = max/127 + 1e-7, codes = rn(v * (1/scale))
 * (quant_qk_int8.cu:296-413 for Q, :422-575 for K). */
static void attn_quant_group(int dt, const void* x, int64_t base, int64_t stride_n, const int* rows, int n, int L,
                             const float* bias, const attn_norm_t* nm, int lk, int D, int8_t* out, float* scale) {
    float buf[32][ATTN_DMAX];
    float mx = 0.f;
    for (int i = 0; i < n; ++i) {
        if (rows[i] >= L) continue;
        attn_load_row(dt, x, base, stride_n, rows[i], nm, D, buf[i]);
        if (bias)
            for (int c = 0; c < D; ++c) buf[i][c] -= bias[c];
        orc_attn_rotate_d(buf[i], D, lk);
        for (int c = 0; c < D; ++c) mx = fmax_dev(mx, fabsf(buf[i][c]));
    }
    const float sc = mx / 127.f + 1e-7f, inv = 1.f / sc;
    *scale = sc;
    for (int i = 0; i < n; ++i) {
        if (rows[i] >= L) continue;
        for (int c = 0; c < D; ++c) out[(int64_t)rows[i] * D + c] = attn_rn_s8(buf[i][c] * inv);
    }
}

/* q [b, lq, h, D], k [b, lk, hk, D] through element strides (batch, row, head).  qi [b,h,lq,D];
 * qs [b,h,ceil(lq/128)*(128/WQ)*8]: eight groups per WQ rows, group g of a block holding rows g, g+8, .. of it, WQ = 32
 * rows (16 at head dim 256, csrc/attn_int8.cu:44); ki [b,hk,lk,D]; ks [b,hk,ceil(lk/ck)*4] (four groups per ck keys:
 * keys with (key % 8) / 2 equal); anchors [b,hk].
 * norm != 0 (head dim 128): q (always) and k (when kw is not null) go through attn_norm_rope_row first; rope may be null. */
ORC_API int orc_attn_quant_qk_d(int dt, const void* q, const void* k, int b, int lq, int lk, int h, int hk, int D, int64_t q_bs,
                                int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs, int ck, int use_anchor,
                                int8_t* qi, float* qs, int8_t* ki, float* ks, int32_t* anchors, int norm, const float* qw,
                                const float* kw, const float* rope, float eps, int rope_mode) {
    if (ck != 64 && ck != 128) return -1;
    if (D != 64 && D != 128 && D != 256) return -1;
    if (norm && (dt != ORC_BF16 || D != 128)) return -400;
    const attn_norm_t qn = {qw, rope, eps, rope_mode, norm ? 1 : 0}, kn = {kw, rope, eps, rope_mode, (norm && kw) ? 1 : 0};
    const int wq = D == 256 ? 16 : 32, nr = wq / 8;
    const int qg = (lq + 127) / 128 * (128 / wq), kb = (lk + ck - 1) / ck;
    for (int bi = 0; bi < b; ++bi)
        for (int hi = 0; hi < h; ++hi)
            for (int t = 0; t < qg; ++t)
                for (int g = 0; g < 8; ++g) {
                    int rows[4];
                    for (int j = 0; j < nr; ++j) rows[j] = t * wq + g + 8 * j;
                    const int64_t bh = (int64_t)bi * h + hi;
                    attn_quant_group(dt, q, bi * q_bs + hi * q_hs, q_rs, rows, nr, lq, NULL, &qn, lk, D, qi + bh * lq * D,
                                     &qs[(bh * qg + t) * 8 + g]);
                }
    for (int bi = 0; bi < b; ++bi)
        for (int hi = 0; hi < hk; ++hi) {
            const int64_t bh = (int64_t)bi * hk + hi, base = bi * k_bs + hi * k_hs;
            const int anchor = use_anchor ? attn_detect_anchor(dt, k, base, k_rs, lk, &kn, D) : -1;
            anchors[bh] = anchor;
            float bias[ATTN_DMAX];
            if (anchor >= 0) attn_load_row(dt, k, base, k_rs, anchor, &kn, D, bias);
            for (int t = 0; t < kb; ++t)
                for (int g = 0; g < 4; ++g) {
                    int rows[32];
                    const int n = ck / 4;
                    for (int i = 0; i < n; ++i) rows[i] = t * ck + (i / 2) * 8 + g * 2 + (i % 2);
                    attn_quant_group(dt, k, base, k_rs, rows, n, lk, anchor >= 0 ? bias : NULL, &kn, lk, D, ki + bh * lk * D,
                                     &ks[(bh * kb + t) * 4 + g]);
                }
        }
    return 0;
}

ORC_API int orc_attn_quant_qk_norm(int dt, const void* q, const void* k, int b, int lq, int lk, int h, int hk, int64_t q_bs,
                                   int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs, int ck, int use_anchor,
                                   int8_t* qi, float* qs, int8_t* ki, float* ks, int32_t* anchors, int norm, const float* qw,
                                   const float* kw, const float* rope, float eps, int rope_mode) {
    return orc_attn_quant_qk_d(dt, q, k, b, lq, lk, h, hk, 128, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, ck, use_anchor, qi, qs, ki, ks,
                               anchors, norm, qw, kw, rope, eps, rope_mode);
}

ORC_API int orc_attn_quant_qk(int dt, const void* q, const void* k, int b, int lq, int lk, int h, int hk, int64_t q_bs,
                              int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs, int ck, int use_anchor,
                              int8_t* qi, float* qs, int8_t* ki, float* ks, int32_t* anchors) {
    return orc_attn_quant_qk_d(dt, q, k, b, lq, lk, h, hk, 128, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, ck, use_anchor, qi, qs, ki, ks,
                               anchors, 0, NULL, NULL, NULL, 0.f, 0);
}

/* The row transform alone, for pins: v[128] float in place. */
ORC_API void orc_attn_norm_rope_row(float* v, const float* w, const float* rope_row, float eps, int rope_mode) {
    const attn_norm_t nm = {w, rope_row, eps, rope_mode, 1};
    attn_norm_rope_row(v, &nm, 0);
}

/* v [b, lk, hk, 128] -> vi [b,hk,lk,128] (plain order; the reference stores it transposed and permuted for its MMA,
 * quant_v_int8.cu:178-190), vs [b,hk,128]: scale = max(absmax/127 as a product with 1/127, 1e-12) (:163-168). */
ORC_API int orc_attn_quant_v_d(int dt, const void* v, int b, int lk, int hk, int D, int64_t v_bs, int64_t v_rs, int64_t v_hs,
                               int8_t* vi, float* vs) {
    for (int bi = 0; bi < b; ++bi)
        for (int hi = 0; hi < hk; ++hi) {
            const int64_t bh = (int64_t)bi * hk + hi, base = bi * v_bs + hi * v_hs;
            for (int c = 0; c < D; ++c) {
                float mx = 0.f;
                for (int n = 0; n < lk; ++n) mx = fmax_dev(mx, fabsf(ld_t(dt, v, base + (int64_t)n * v_rs + c)));
                const float sc = fmax_dev(mx * (1.f / 127.f), 1e-12f), inv = 1.f / sc;
                vs[bh * D + c] = sc;
                for (int n = 0; n < lk; ++n)
                    vi[(bh * lk + n) * D + c] = attn_rn_s8(ld_t(dt, v, base + (int64_t)n * v_rs + c) * inv);
            }
        }
    return 0;
}

ORC_API int orc_attn_quant_v(int dt, const void* v, int b, int lk, int hk, int64_t v_bs, int64_t v_rs, int64_t v_hs,
                             int8_t* vi, float* vs) {
    return orc_attn_quant_v_d(dt, v, b, lk, hk, 128, v_bs, v_rs, v_hs, vi, vs);
}

static inline float attn_exp2(float x) { return (float)exp2((double)x); }

/* The attention proper over the quantized tensors (csrc/vendor/sage/qk_int_sv_i8_cuda.cuh, mask none).  Per query row
 * and tile of ck keys: integer scores; per key group the maximum score times that group's scale, minus the u8 offset
 * (attn_utils.cuh:719-741; the last tile takes the float path with its -50000 floor, :569-596); probabilities
 * exp2(fma(score, scale, -tile_max)) rounded to u8 (:700-717, mma.cuh:793-804); denominators and outputs rescaled by
 * exp2(-|m_prev - tile_max|) on whichever side is smaller (:742-756); outputs += float(sum p*v) * tile_scale by fmaf
 * (:1254-1258); O = RO / d * v_scale (:1130-1146, qk_int_sv_i8_cuda.cuh:1056-1072).  The denominator is summed here
 * per row in key order; the reference keeps four per-thread partials.
 * The last tile always takes the reference's unfused form (qk_int_sv_i8_cuda.cuh:956-1000: maximum from a raw score
 * of -50000, keys past lk at -1e30 raw, the denominator summing the UNROUNDED probabilities in the four per-thread
 * partials of a row, attn_utils.cuh:922-940, :1113-1122).  unfused: every tile takes it, which is what the reference's
 * build does for f16 outputs and at most 512 keys (sage_attn_launcher.cu:187-191, qk_int_sv_i8_cuda.cuh:132-139). */
ORC_API int orc_attn_int8_d(int out_dt, const int8_t* qi, const int8_t* ki, const int8_t* vi, const float* qs,
                            const float* ks, const float* vs, int b, int lq, int lk, int h, int hk, int D, int ck, float scale,
                            float sink, void* o, int64_t o_bs, int64_t o_rs, int64_t o_hs, int unfused) {
    if ((ck != 64 && ck != 128) || hk <= 0 || h % hk != 0 || (D != 64 && D != 128 && D != 256)) return -1;
    const int wq = D == 256 ? 16 : 32;
    const int qg = (lq + 127) / 128 * (128 / wq), kb = (lk + ck - 1) / ck, rep = h / hk;
    const float sm = scale * 1.44269504088896340736f;
    #pragma omp parallel for collapse(2) schedule(dynamic, 8)
    for (int bh = 0; bh < b * h; ++bh)
        for (int r = 0; r < lq; ++r) {
            const int bi = bh / h, hi = bh % h;
            const int64_t kvh = (int64_t)bi * hk + hi / rep;
            const int8_t* qrow = qi + ((int64_t)bh * lq + r) * D;
            const float q_scale = qs[((int64_t)bh * qg + r / wq) * 8 + r % 8];
            float m = -50000.f, d = 1.f, ro[ATTN_DMAX], d4[4] = {0.f, 0.f, 0.f, 0.f}, pf[128];
            for (int c = 0; c < D; ++c) ro[c] = 0.f;
            int32_t s[128];
            for (int t = 0; t < kb; ++t) {
                const int n = lk - t * ck < ck ? lk - t * ck : ck;
                const int last = t == kb - 1;
                float gs[4], tile_m = 0.f;
                for (int g = 0; g < 4; ++g) gs[g] = sm * (q_scale * ks[(kvh * kb + t) * 4 + g]);
                for (int j = 0; j < n; ++j) {
                    const int8_t* krow = ki + ((int64_t)kvh * lk + t * ck + j) * D;
                    int32_t acc = 0;
                    for (int c = 0; c < D; ++c) acc += (int32_t)qrow[c] * (int32_t)krow[c];
                    s[j] = acc;
                }
                for (int g = 0; g < 4; ++g) {
                    float mg = (last || unfused) ? -50000.f : -3.0e38f;
                    int any = 0;
                    for (int j = 0; j < n; ++j)
                        if ((j % 8) / 2 == g) { mg = fmax_dev(mg, (float)s[j]); any = 1; }
                    if (!any && !last) continue;
                    const float cand = fmaf(mg, gs[g], -ATTN_U8_OFFSET);
                    tile_m = (g == 0 || cand > tile_m) ? cand : tile_m;
                }
                const float smaller = attn_exp2(-fabsf(m - tile_m));
                const float o_scale = m < tile_m ? smaller : 1.f, t_scale = tile_m < m ? smaller : 1.f;
                m = m > tile_m ? m : tile_m;
                int32_t pv[ATTN_DMAX];
                int32_t psum = 0;
                for (int c = 0; c < D; ++c) pv[c] = 0;
                for (int j = n; j < ck; ++j) pf[j] = 0.f;       /* keys past lk: -1e30 raw, probability zero */
                for (int j = 0; j < n; ++j) {
                    float p = attn_exp2(fmaf((float)s[j], gs[(j % 8) / 2], -tile_m));
                    pf[j] = p;
                    p = rintf(p > 255.f ? 255.f : p);
                    const int32_t pi = (int32_t)p;
                    psum += pi;
                    const int8_t* vrow = vi + ((int64_t)kvh * lk + t * ck + j) * D;
                    for (int c = 0; c < D; ++c) pv[c] += pi * (int32_t)vrow[c];
                }
                d *= o_scale;
                for (int l = 0; l < 4; ++l) d4[l] *= o_scale;
                if (unfused || last) {
                    /* the unrounded probabilities in the four per-thread partials of a row */
                    for (int fk = 0; fk < ck / 16; ++fk)
                        for (int l = 0; l < 4; ++l) {
                            const float* q4 = pf + fk * 16;
                            d4[l] += ((q4[2 * l] + q4[2 * l + 1]) + (q4[8 + 2 * l] + q4[8 + 2 * l + 1])) * t_scale;
                        }
                } else {
                    d += (float)psum * t_scale;
                }
                for (int c = 0; c < D; ++c) ro[c] = fmaf((float)pv[c], t_scale, ro[c] * o_scale);
            }
            /* `sink` more keys of score zero and value zero: each adds exp2(0 - m) to the denominator and nothing to
             * the output (attn_utils.cuh:1122-1130, csrc/attn_int8.cu:193-197) */
            d += (d4[0] + d4[1]) + (d4[2] + d4[3]);
            if (sink != 0.f) d = fmaf(sink, attn_exp2(-m), d);
            const float rcp = 1.f / d;
            for (int c = 0; c < D; ++c)
                st_t(out_dt, o, bi * o_bs + (int64_t)r * o_rs + hi * o_hs + c, ro[c] * rcp * vs[kvh * D + c]);
        }
    return 0;
}

ORC_API int orc_attn_int8(int out_dt, const int8_t* qi, const int8_t* ki, const int8_t* vi, const float* qs,
                          const float* ks, const float* vs, int b, int lq, int lk, int h, int hk, int ck, float scale,
                          float sink, void* o, int64_t o_bs, int64_t o_rs, int64_t o_hs, int unfused) {
    return orc_attn_int8_d(out_dt, qi, ki, vi, qs, ks, vs, b, lq, lk, h, hk, 128, ck, scale, sink, o, o_bs, o_rs, o_hs, unfused);
}

/* The same attention with an additive bias per key on the logits (gpu_int8_attn_key_bias, csrc/attn_int8.cu:204-223):
 * bias f32 [lk], one row for every batch item, head and query.  The reference takes two routes by key tile length.
 *
 * ck = 64 (lk <= 1024), sage's per-key mask (mask mode kCustomKey: qk_int_sv_i8_cuda.cuh:637-700, attn_utils.cuh:466-515,
 * 569-650, 862-880, 922-940): scores are scaled first, rs = float(S) * (sm * q_scale * k_scale); a key that is kept
 * (inside lk, finite bias) becomes rs + bias * log2e (an fma with 1.0), any other -50000; the tile maximum starts at
 * -50000 and has the u8 offset subtracted; probabilities exp2(rs - tile_max) are packed to u8 for P.V, but the
 * DENOMINATOR sums the unrounded float probabilities: each of the four threads of a row keeps its own partial, adding per
 * 16 keys ((p[2l] + p[2l+1]) + (p[8+2l] + p[8+2l+1])) * tile_scale, and the four are added pairwise at the end
 * (attn_utils.cuh:1113-1122).  A row with no kept key at all gives zeros (qk_int_sv_i8_cuda.cuh:1031-1051).
 *
 * ck = 128 (lk > 1024), sage's prepared key mask (sage_attn_launcher.cu:343-391: non-finite biases and the padding past
 * lk become -inf; a tile of 128 keys whose biases are all equal is marked with that value): a tile with a finite
 * constant bias that is not the last takes the integer route with the bias added to the maximum and folded into the
 * exponent's constant (attn_utils.cuh:719-790 with add_bias, qk_int_sv_i8_cuda.cuh:613-620); any other tile takes the
 * float route, scores fma(float(S), scale, bias * log2e), maximum from -50000, probabilities exp2(score - tile_max)
 * (:799-856).  Both sum the ROUNDED u8 probabilities into the denominator.  A tile whose biases are all -inf is skipped
 * by the reference; the float route leaves m, d and the output as they were for it, so it is not special here.
 * PARITY UNPINNED against a run of the reference for the same reasons as orc_attn_int8. */
ORC_API int orc_attn_int8_bias(int out_dt, const int8_t* qi, const int8_t* ki, const int8_t* vi, const float* qs,
                               const float* ks, const float* vs, int b, int lq, int lk, int h, int hk, int ck, float scale,
                               const float* bias, void* o, int64_t o_bs, int64_t o_rs, int64_t o_hs) {
    if ((ck != 64 && ck != 128) || hk <= 0 || h % hk != 0 || !bias) return -1;
    const int D = 128;   /* the key-bias entry point exists for head dim 128 only (csrc/attn_int8.cu:191) */
    const int qg = (lq + 127) / 128 * 4, kb = (lk + ck - 1) / ck, rep = h / hk;
    const float log2e = 1.44269504088896340736f;
    const float sm = scale * log2e;
    /* prepared biases: bias * log2e, -inf for non-finite ones and for the padding */
    float* bl = (float*)malloc(sizeof(float) * (size_t)kb * ck);
    float* tb = (float*)malloc(sizeof(float) * (size_t)kb);
    for (int j = 0; j < kb * ck; ++j) bl[j] = (j < lk && isfinite(bias[j])) ? bias[j] * log2e : -INFINITY;
    for (int t = 0; t < kb; ++t) {
        float lo = INFINITY, hi = -INFINITY;
        for (int j = 0; j < ck; ++j) {
            const int key = t * ck + j;
            const float v = (key < lk && isfinite(bias[key])) ? bias[key] : -INFINITY;
            lo = v < lo ? v : lo;
            hi = v > hi ? v : hi;
        }
        tb[t] = lo == hi ? hi : NAN;
    }
    #pragma omp parallel for collapse(2) schedule(dynamic, 8)
    for (int bh = 0; bh < b * h; ++bh)
        for (int r = 0; r < lq; ++r) {
            const int bi = bh / h, hi = bh % h;
            const int64_t kvh = (int64_t)bi * hk + hi / rep;
            const int8_t* qrow = qi + ((int64_t)bh * lq + r) * D;
            const float q_scale = qs[((int64_t)bh * qg + r / 32) * 8 + r % 8];
            float m = -50000.f, ro[ATTN_DMAX], d4[4] = {1.f, 1.f, 1.f, 1.f}, d = 1.f;
            int valid = 0;
            for (int c = 0; c < D; ++c) ro[c] = 0.f;
            int32_t s[128];
            float f[128], pf[128];
            for (int t = 0; t < kb; ++t) {
                const int n = lk - t * ck < ck ? lk - t * ck : ck;
                const int last = t == kb - 1;
                float gs[4];
                for (int g = 0; g < 4; ++g) gs[g] = sm * (q_scale * ks[(kvh * kb + t) * 4 + g]);
                for (int j = 0; j < ck; ++j) {
                    s[j] = 0;
                    if (j >= n) continue;
                    const int8_t* krow = ki + ((int64_t)kvh * lk + t * ck + j) * D;
                    int32_t acc = 0;
                    for (int c = 0; c < D; ++c) acc += (int32_t)qrow[c] * (int32_t)krow[c];
                    s[j] = acc;
                }
                float tile_m, neg_m = 0.f;
                int route;   /* 0: per-key mask (ck 64), 1: prepared, constant tile, 2: prepared, float route */
                if (ck == 64) {
                    route = 0;
                    float mx = -50000.f;
                    for (int j = 0; j < ck; ++j) {
                        const float bj = bl[t * ck + j];
                        const int keep = j < n && bj != -INFINITY;
                        valid |= keep;
                        const float rs = (float)s[j] * gs[(j % 8) / 2];
                        f[j] = keep ? fmaf(rs, 1.0f, bj) : -50000.f;
                        mx = f[j] > mx ? f[j] : mx;
                    }
                    tile_m = mx - ATTN_U8_OFFSET;
                } else if (!last && isfinite(tb[t])) {
                    route = 1;
                    const float tbl = tb[t] * log2e;
                    tile_m = -INFINITY;
                    for (int g = 0; g < 4; ++g) {
                        int32_t mg = INT32_MIN;
                        for (int j = 0; j < ck; ++j)
                            if ((j % 8) / 2 == g) mg = s[j] > mg ? s[j] : mg;
                        const float cand = fmaf((float)mg, gs[g], -ATTN_U8_OFFSET) + tbl;
                        tile_m = cand > tile_m ? cand : tile_m;
                    }
                    neg_m = tbl - tile_m;
                } else {
                    route = 2;
                    float mx = -50000.f;
                    for (int j = 0; j < ck; ++j) {
                        f[j] = fmaf((float)s[j], gs[(j % 8) / 2], bl[t * ck + j]);
                        mx = f[j] > mx ? f[j] : mx;
                    }
                    tile_m = mx - ATTN_U8_OFFSET;
                }
                const float smaller = attn_exp2(-fabsf(m - tile_m));
                const float o_scale = m < tile_m ? smaller : 1.f, t_scale = tile_m < m ? smaller : 1.f;
                m = m > tile_m ? m : tile_m;
                int32_t pv[ATTN_DMAX];
                int32_t psum = 0;
                for (int c = 0; c < D; ++c) pv[c] = 0;
                for (int j = 0; j < ck; ++j) {
                    float p = route == 1 ? attn_exp2(fmaf((float)s[j], gs[(j % 8) / 2], neg_m)) : attn_exp2(f[j] + (-tile_m));
                    pf[j] = p;
                    p = p != p ? 0.f : p;                       /* the clamp maps NaN to 0 (mma.cuh:790-800) */
                    p = rintf(p > 255.f ? 255.f : (p < 0.f ? 0.f : p));
                    const int32_t pi = (int32_t)p;
                    psum += pi;
                    if (j >= n || pi == 0) continue;
                    const int8_t* vrow = vi + ((int64_t)kvh * lk + t * ck + j) * D;
                    for (int c = 0; c < D; ++c) pv[c] += pi * (int32_t)vrow[c];
                }
                if (route == 0) {
                    for (int l = 0; l < 4; ++l) d4[l] *= o_scale;
                    for (int fk = 0; fk < ck / 16; ++fk)
                        for (int l = 0; l < 4; ++l) {
                            const float* q4 = pf + fk * 16;
                            const float tile_sum = (q4[2 * l] + q4[2 * l + 1]) + (q4[8 + 2 * l] + q4[8 + 2 * l + 1]);
                            d4[l] += tile_sum * t_scale;
                        }
                } else {
                    d *= o_scale;
                    d += (float)psum * t_scale;
                }
                for (int c = 0; c < D; ++c) ro[c] = fmaf((float)pv[c], t_scale, ro[c] * o_scale);
            }
            if (ck == 64) d = (d4[0] + d4[1]) + (d4[2] + d4[3]);
            const float rcp = 1.f / d;
            for (int c = 0; c < D; ++c) {
                float out = ro[c] * rcp;
                if (ck == 64 && !valid) out = 0.f;
                st_t(out_dt, o, bi * o_bs + (int64_t)r * o_rs + hi * o_hs + c, out * vs[kvh * D + c]);
            }
        }
    free(bl);
    free(tb);
    return 0;
}

/* csrc/attn_int8.cu:56 */
ORC_API int orc_attn_cta_k(int lk, int d) { return lk > 1024 && d != 64 ? 128 : 64; }
