// INT8 attention for head dim 128 on gfx950: Q and K rotated and quantized per scale group, V per channel, integer
// scores and integer P.V partials on v_mfma_i32_32x32x32_i8, softmax state in fp32.
//
// Semantics follow the reference's Sage-style path (csrc/attn_int8.cu:118-160 chains the stages;
// csrc/vendor/sage/quant_qk_int8.cu:72-157 rotation, :296-413 Q groups, :422-575 K groups, :591-756 K anchor;
// csrc/vendor/sage/quant_v_int8.cu:94-190 V; csrc/vendor/sage/qk_int_sv_i8_cuda.cuh + attn_utils.cuh:700-800 the tile
// update with u8 probabilities).  The design is for CDNA4:
//   * keys ride in src0 and queries in src1 of the score MFMA, so a lane ends up with one query row and 16 keys per
//     32-key block: row maxima and sums are in-lane plus one exchange with lane ^ 32;
//   * those 16 scores are, in order, exactly the 16 K-bytes that lane must supply as src1 of the P.V MFMA when V^T is
//     stored with the matching key order, so probabilities never cross lanes;
//   * the matrix cores multiply signed bytes only: probabilities 0..255 are fed as p - 128 and the accumulator starts
//     at 128 * (column sums of the V tile), which the V quantizer leaves in the workspace.  The integers are exact.
// The workspace layout is private to this file.
#include <climits>
#include <cstdio>
#include <type_traits>

#include "common.hpp"

namespace {

constexpr float kU8Offset = 7.9943534f;
// Head dims 64, 128 and 256 (csrc/attn_int8.cu:42-45).  A row's channels lie on D/16 consecutive lanes, sixteen channels
// each; the Q quantizer's row block is 32 rows, 16 at head dim 256.
constexpr int lanes_per_row(int D) { return D / 16; }
constexpr int q_block_rows(int D) { return D == 256 ? 16 : 32; }

struct AttnArgs {
    const void *q, *k, *v;
    void* o;
    int8_t *qi, *ki, *vt;
    float *qs, *ks, *vs;
    int* anchors;
    uint32_t* vmax;
    int* vsum;
    int b, lq, lk, h, hk, rep, qg, kb, ck, nblk;
    int64_t q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs, o_rs, o_hs;
    float sm, sink;
    int vec_ok, in_vec, v_vec, use_anchor;
    int rot4;   // lk <= 256: the rotation is only the H4 on runs of four channels, without the sign diagonal
    // per-head RMSNorm (+ weight) and RoPE ahead of the quantizers (csrc/kernels.cu:482-540 through
    // csrc/vendor/sage/quant_qk_int8.cu:160-291): q_norm / k_norm say which of Q and K take it
    const float *qw, *kw, *rope;   // [128] or null (ones); rope [L][64] x (cos, sin) or null
    float eps;
    int q_norm, k_norm, rope_mode;
    const float* bias;    // per-key logit bias of the caller, f32 [lk], or null
    float* kbias;         // prepared: bias * log2e per key of every tile (-inf: not kept / padding), then one value per tile
    float* tbias;         // per tile: the bias all its keys share (times log2e), NaN when they differ, -inf when none is kept
};

// fmaxf as the reference's device code uses it: a NaN operand is dropped.
__device__ __forceinline__ float fmax_nn(float a, float b) { return __builtin_fmaxf(a, b); }

__device__ __forceinline__ int8_t rn_s8(float v) {
    if (v != v) return 0;
    const float r = __builtin_rintf(v);
    return (int8_t)(r > 127.f ? 127.f : r < -128.f ? -128.f : r);
}

// Cross-lane moves inside a run of eight lanes, as data-parallel-primitive modifiers (no LDS traffic).
template <int CTRL> __device__ __forceinline__ float dpp_mov(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_xor1(float x) { return dpp_mov<0xB1>(x); }                   // quad_perm [1,0,3,2]
__device__ __forceinline__ float lane_xor2(float x) { return dpp_mov<0x4E>(x); }                   // quad_perm [2,3,0,1]
__device__ __forceinline__ float lane_xor4(float x) { return dpp_mov<0x1B>(dpp_mov<0x141>(x)); }   // half-row mirror (xor 7), then quad reverse (xor 3)

__device__ __forceinline__ float lane_xor8(float x) { return dpp_mov<0x128>(x); }                  // row_ror:8 within a row of 16 lanes

// Normalized Walsh-Hadamard over the 16 << LB channels of one row held by 1 << LB consecutive lanes, sixteen adjacent
// channels per lane (ol = lane within the run), after the sign diagonal when SIGN (head dim 128 only).  Same operation
// order as the oracle: H4 on runs of four channels, radix-2 butterflies over the higher channel bits in ascending order
// (two in the lane, LB across lanes), one scaling.  LB = 3: H128 (the reference's convrot128 / convrot128_plain), LB = 2:
// H64 (convrot64).
template <int LB, bool SIGN> __device__ __forceinline__ void rot_wh(float (&v)[16], int ol) {
    if (SIGN) {
        const uint32_t word = (ol >> 1) == 0 ? 0x1035997bu : (ol >> 1) == 1 ? 0x8087f5eeu : (ol >> 1) == 2 ? 0xee2e4e1au : 0x71132418u;
        const uint32_t keep = word >> ((ol & 1) * 16);
#pragma unroll
        for (int e = 0; e < 16; ++e) v[e] = u2f(f2u(v[e]) ^ ((((keep >> e) & 1u) ^ 1u) << 31));
    }
#pragma unroll
    for (int g = 0; g < 16; g += 4) {
        const float a0 = v[g] + v[g + 1], a1 = v[g] - v[g + 1], a2 = v[g + 2] + v[g + 3], a3 = v[g + 2] - v[g + 3];
        v[g] = (a0 + a2) * 0.5f;
        v[g + 1] = (a1 + a3) * 0.5f;
        v[g + 2] = (a0 - a2) * 0.5f;
        v[g + 3] = (a1 - a3) * 0.5f;
    }
#pragma unroll
    for (int bit = 4; bit < 16; bit <<= 1)
#pragma unroll
        for (int e = 0; e < 16; ++e)
            if (!(e & bit)) {
                const float lo = v[e], hi = v[e | bit];
                v[e] = lo + hi;
                v[e | bit] = lo - hi;
            }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const float other = lane_xor1(v[e]);
        v[e] = (ol & 1) ? other - v[e] : v[e] + other;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const float other = lane_xor2(v[e]);
        v[e] = (ol & 2) ? other - v[e] : v[e] + other;
    }
    if (LB == 3) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float other = lane_xor4(v[e]);
            v[e] = (ol & 4) ? other - v[e] : v[e] + other;
        }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] *= LB == 3 ? 0.1767766952966369f : 0.25f;
}

// The rotation of sequences of at most 256 keys (csrc/vendor/sage/quant_qk_int8.cu:1160-1166, ROTATION 4): the
// normalized H4 on each run of four adjacent channels and nothing else.
__device__ __forceinline__ void rot4(float (&v)[16]) {
#pragma unroll
    for (int g = 0; g < 16; g += 4) {
        const float a0 = v[g] + v[g + 1], a1 = v[g] - v[g + 1], a2 = v[g + 2] + v[g + 3], a3 = v[g + 2] - v[g + 3];
        v[g] = (a0 + a2) * 0.5f;
        v[g + 1] = (a1 + a3) * 0.5f;
        v[g + 2] = (a0 - a2) * 0.5f;
        v[g + 3] = (a1 - a3) * 0.5f;
    }
}

// The rotation the quantizers apply to a row of head dim D (csrc/vendor/sage/quant_qk_int8.cu:1150-1195): the H4 blocks
// alone up to 256 keys, beyond that H64 at head dim 64, sign diagonal + H128 at 128, the plain H128 on each half at 256.
template <int D> __device__ __forceinline__ void rotate_row(float (&v)[16], int ol, bool h4_only) {
    if (h4_only) rot4(v);
    else if (D == 64) rot_wh<2, false>(v, ol);
    else if (D == 128) rot_wh<3, true>(v, ol);
    else rot_wh<3, false>(v, ol & 7);
}

// Maximum over the lanes of a row.
template <int D> __device__ __forceinline__ float max_row(float m) {
    m = fmax_nn(m, lane_xor1(m));
    m = fmax_nn(m, lane_xor2(m));
    if (D >= 128) m = fmax_nn(m, lane_xor4(m));
    if (D == 256) m = fmax_nn(m, lane_xor8(m));
    return m;
}

// Sum of squares of one 128-channel row in the order of the reference's warp of 32 lanes (csrc/kernels.cu:497-513,
// csrc/common.cuh:30-34): lane L accumulates its four channels by fma in index order, then the lanes add pairwise at
// distances 16, 8, 4, 2, 1.  Lane L owns channels 4L..4L+3, or, with split = rope_mode 2 (with or without a table),
// channels 2L, 2L+1, 64+2L, 65+2L.  Here eight lanes hold sixteen adjacent channels each (o8 = lane within the eight),
// so a lane carries four (eight, split) of the reference's lanes; all eight lanes get the sum.
__device__ __forceinline__ float sumsq128(const float (&v)[16], int o8, bool split) {
    if (!split) {
        float s[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            s[i] = v[4 * i] * v[4 * i];
            s[i] = __builtin_fmaf(v[4 * i + 1], v[4 * i + 1], s[i]);
            s[i] = __builtin_fmaf(v[4 * i + 2], v[4 * i + 2], s[i]);
            s[i] = __builtin_fmaf(v[4 * i + 3], v[4 * i + 3], s[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += lane_xor4(s[i]);   // distance 16
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += lane_xor2(s[i]);   // 8
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += lane_xor1(s[i]);   // 4
        return (s[0] + s[2]) + (s[1] + s[3]);                   // 2, then 1
    }
    // split: the lanes of the low half start each chain (channels 2L, 2L+1), the lanes of the high half finish it
    float s[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float p = __builtin_fmaf(v[2 * i + 1], v[2 * i + 1], v[2 * i] * v[2 * i]);
        const float q = lane_xor4(p);
        s[i] = __builtin_fmaf(v[2 * i + 1], v[2 * i + 1], __builtin_fmaf(v[2 * i], v[2 * i], q));   // meaningful where o8 >= 4
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] += lane_xor2(s[i]);       // distance 16
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] += lane_xor1(s[i]);       // 8
    const float t = ((s[0] + s[4]) + (s[2] + s[6])) + ((s[1] + s[5]) + (s[3] + s[7]));   // 4, 2, 1
    const float u = lane_xor4(t);
    return o8 >= 4 ? t : u;
}

// The same sum by one thread over a row in memory.
__device__ inline float sumsq128_serial(const float* x, bool split) {
    float s[32];
    for (int l = 0; l < 32; ++l) {
        const int i0 = split ? 2 * l : 4 * l, i2 = split ? 64 + 2 * l : 4 * l + 2;
        float t = x[i0] * x[i0];
        t = __builtin_fmaf(x[i0 + 1], x[i0 + 1], t);
        t = __builtin_fmaf(x[i2], x[i2], t);
        s[l] = __builtin_fmaf(x[i2 + 1], x[i2 + 1], t);
    }
    for (int o = 16; o > 0; o >>= 1)
        for (int l = 0; l < o; ++l) s[l] += s[l + o];
    return s[0];
}

// Per-head RMSNorm, weight and RoPE of one 128-channel row held by eight lanes (sixteen adjacent channels each), as the
// reference applies them to q and k ahead of the quantizer (csrc/kernels.cu:482-540, csrc/vendor/sage/quant_qk_int8.cu:
// 211-278): v = T((v * rstd) * w), rstd = 1/sqrt(mean(v^2) + eps) with the sum in the reference's order (sumsq128);
// rope mode 1 turns the pairs (2p, 2p+1), mode 2 the pairs (j, j + 64), with (cos, sin) = rope_row[2p], rope_row[2p+1];
// the result is rounded to bf16 again.  This build's definition of the two parts the reference leaves to its machine:
// 1/sqrt is correctly rounded (the reference's rsqrtf is an approximation of up to two units in the last place), and
// c*a - s*b, s*a + c*b contract to one fma each on their first product.  w == nullptr means ones; rope_row == nullptr
// means no rotation.  All eight lanes must call it.
__device__ __forceinline__ void norm_rope_row(float (&v)[16], int o8, const float* w, const float* rope_row, float eps, int mode) {
    const float ss = sumsq128(v, o8, mode == 2);
    const float rstd = (float)(1.0 / sqrt((double)(ss / 128.f + eps)));
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = rnd_dt<DT_BF16>(v[e] * rstd * (w ? w[o8 * 16 + e] : 1.f));
    if (!rope_row) return;
    if (mode == 1) {
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            const float c = rope_row[o8 * 16 + e], sn = rope_row[o8 * 16 + e + 1];
            const float a = v[e], b = v[e + 1];
            v[e] = rnd_dt<DT_BF16>(__builtin_fmaf(c, a, -(sn * b)));
            v[e + 1] = rnd_dt<DT_BF16>(__builtin_fmaf(sn, a, c * b));
        }
    } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int j = (o8 & 3) * 16 + e;
            const float c = rope_row[2 * j], sn = rope_row[2 * j + 1];
            const float other = lane_xor4(v[e]);
            v[e] = rnd_dt<DT_BF16>(o8 < 4 ? __builtin_fmaf(v[e], c, -(other * sn)) : __builtin_fmaf(v[e], c, other * sn));
        }
    }
}

__device__ __forceinline__ uint4 codes16(const float (&v)[16], float inv) {
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < 16; ++e) w[e / 4] |= (uint32_t)(uint8_t)rn_s8(v[e] * inv) << (8 * (e % 4));
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// Four consecutive elements: one 8-byte load when the caller's strides and base allow it.
template <int DT> __device__ __forceinline__ void ld4_dt(const void* p, int64_t i, bool vec, float (&v)[4]) {
    if (vec) {
        load4<DT>(p, i, v);
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = ld_dt<DT>(p, i + c);
    }
}

template <int DT> __device__ __forceinline__ void ld16_dt(const void* p, int64_t i, bool vec, float (&v)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        float x[4];
        ld4_dt<DT>(p, i + g * 4, vec, x);
#pragma unroll
        for (int c = 0; c < 4; ++c) v[g * 4 + c] = x[c];
    }
}

// The K anchor of one (kv head, batch).  The nine sampled keys go to LDS (a thread per channel); the sums then follow the
// reference's block of 128 threads in four warps: thread t walks channels t and t + 128 with one set of accumulators
// (head dim 256), threads past the head dim hold zeros (64), warps add by a shuffle-down tree and the four warps in
// order (csrc/vendor/sage/quant_qk_int8.cu:640-756).
template <int DT, int D>
__device__ __forceinline__ void anchor_body(const AttnArgs& a, const int hi, const int bi) {
    __shared__ float s[9][D];
    __shared__ float energy[128], best_energy[128], amax[128], bmax[128], dist[9][128];
    __shared__ int chosen;
    const int tid = threadIdx.x, c = tid & (D - 1);
    const int64_t base = bi * a.k_bs + hi * a.k_hs;
    if (tid < D) {   // the V quantizer's accumulators for this (kv head, batch) start at zero
        const int64_t bh = (int64_t)bi * a.hk + hi;
        a.vmax[bh * D + c] = 0u;
        for (int t = 0; t < a.kb; ++t) a.vsum[(bh * a.kb + t) * D + c] = 0;
    }
    bool normed = false;
    if constexpr (D == 128) {
        if (a.k_norm) {
            normed = true;
            // the nine sampled keys as the K quantizer will see them: norm_rope_row's arithmetic with a thread per channel
            __shared__ float rstd9[9];
            __shared__ float nrm[9][D];
#pragma unroll
            for (int i = 0; i < 9; ++i) {
                const int row = (int)((int64_t)i * (a.lk - 1) / 8);
                s[i][c] = ld_dt<DT>(a.k, base + (int64_t)row * a.k_rs + c);
            }
            __syncthreads();
            if (tid < 9) rstd9[tid] = (float)(1.0 / sqrt((double)(sumsq128_serial(s[tid], a.rope_mode == 2) / 128.f + a.eps)));
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 9; ++i) nrm[i][c] = rnd_dt<DT_BF16>(s[i][c] * rstd9[i] * (a.kw ? a.kw[c] : 1.f));
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 9; ++i) {
                float x = nrm[i][c];
                if (a.rope) {
                    const int row = (int)((int64_t)i * (a.lk - 1) / 8);
                    const float* r = a.rope + (int64_t)row * D;
                    if (a.rope_mode == 1) {
                        const float cs = r[c & ~1], sn = r[c | 1], other = nrm[i][c ^ 1];
                        x = rnd_dt<DT_BF16>((c & 1) ? __builtin_fmaf(sn, other, cs * x) : __builtin_fmaf(cs, x, -(sn * other)));
                    } else {
                        const int j = c & 63;
                        const float cs = r[2 * j], sn = r[2 * j + 1], other = nrm[i][c ^ 64];
                        x = rnd_dt<DT_BF16>(c < 64 ? __builtin_fmaf(x, cs, -(other * sn)) : __builtin_fmaf(x, cs, other * sn));
                    }
                }
                s[i][c] = x;
            }
        }
    }
    if (!normed && tid < D) {
#pragma unroll
        for (int i = 0; i < 9; ++i) {
            const int row = (int)((int64_t)i * (a.lk - 1) / 8);
            s[i][c] = ld_dt<DT>(a.k, base + (int64_t)row * a.k_rs + c);
        }
    }
    __syncthreads();
    if (tid < 128) {
        float e = 0.f, m = 0.f, d9[9];
#pragma unroll
        for (int i = 0; i < 9; ++i) d9[i] = 0.f;
        for (int ch = tid; ch < D; ch += 128) {
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 9; ++i) {
                const float x = s[i][ch];
                e = fmaf(x, x, e);
                m = fmax_nn(m, fabsf(x));
                sum += x;
            }
#pragma unroll
            for (int i = 0; i < 9; ++i) {
                const float d = fmaf(9.f, s[i][ch], -sum);
                d9[i] = fmaf(d, d, d9[i]);
            }
        }
        energy[tid] = e;
        amax[tid] = m;
#pragma unroll
        for (int i = 0; i < 9; ++i) dist[i][tid] = d9[i];
    }
    __syncthreads();
    auto tree = [](const float* x) {
        float t[32];
        for (int i = 0; i < 32; ++i) t[i] = x[i];
        for (int off = 16; off > 0; off >>= 1)
            for (int i = 0; i < off; ++i) t[i] += t[i + off];
        return t[0];
    };
    __shared__ float warp_sum[11][4];   // nine candidate distances, then the two energies
    if (tid < 36) warp_sum[tid / 4][tid % 4] = tree(&dist[tid / 4][(tid % 4) * 32]);
    else if (tid < 40) warp_sum[9][tid - 36] = tree(&energy[(tid - 36) * 32]);
    __syncthreads();
    if (tid == 0) {
        int best = 0;
        float best_d = 3.402823466e+38F;
        for (int i = 0; i < 9; ++i) {
            float d = 0.f;
            for (int w = 0; w < 4; ++w) d += warp_sum[i][w];
            if (d < best_d) { best = i; best_d = d; }
        }
        chosen = best;
    }
    __syncthreads();
    const int best = chosen;
    if (tid < 128) {
        float be = 0.f, bm = 0.f;
        for (int ch = tid; ch < D; ch += 128) {
#pragma unroll
            for (int i = 0; i < 9; ++i) {
                const float r = s[i][ch] - s[best][ch];
                be = fmaf(r, r, be);
                bm = fmax_nn(bm, fabsf(r));
            }
        }
        best_energy[tid] = be;
        bmax[tid] = bm;
    }
    __syncthreads();
    if (tid < 4) warp_sum[10][tid] = tree(&best_energy[tid * 32]);
    __syncthreads();
    if (tid == 0) {
        float e0 = 0.f, e1 = 0.f, m0 = 0.f, m1 = 0.f;
        for (int w = 0; w < 4; ++w) {
            e0 += warp_sum[9][w];
            e1 += warp_sum[10][w];
        }
        for (int i = 0; i < 128; ++i) {
            m0 = fmax_nn(m0, amax[i]);
            m1 = fmax_nn(m1, bmax[i]);
        }
        a.anchors[bi * a.hk + hi] = (a.use_anchor && e1 < e0 && m1 <= m0 * 1.125f) ? (int)((int64_t)best * (a.lk - 1) / 8) : -1;
    }
}

// Q: every run of D/16 lanes is one scale group (rows g, g+8, .. of a block of 32 rows, 16 at head dim 256), a lane
// holding 16 channels of each of the group's rows; a wave carries 64 / (D/16) groups, a workgroup four waves.
template <int DT, int D>
__device__ __forceinline__ void quant_q_body(const AttnArgs& a, const int hi, const int ty, const int bi) {
    constexpr int LPR = lanes_per_row(D), GPW = 64 / LPR, WQ = q_block_rows(D), NR = WQ / 8;
    const int lane = threadIdx.x & 63, ol = lane & (LPR - 1);
    const int gid = (ty * 4 + (threadIdx.x >> 6)) * GPW + lane / LPR;   // scale group of the head: block * 8 + g
    if (gid >= a.qg * 8) return;
    const int t = gid >> 3, g = gid & 7;
    const int64_t bh = (int64_t)bi * a.h + hi, base = bi * a.q_bs + hi * a.q_hs + ol * 16;
    float v[NR][16];
#pragma unroll
    for (int j = 0; j < NR; ++j) {
        const int row = t * WQ + g + 8 * j;
        const int rr = row < a.lq ? row : a.lq - 1;
        ld16_dt<DT>(a.q, base + (int64_t)rr * a.q_rs, a.in_vec, v[j]);
        if constexpr (D == 128) {
            if (a.q_norm) norm_rope_row(v[j], ol, a.qw, a.rope ? a.rope + (int64_t)rr * D : nullptr, a.eps, a.rope_mode);
        }
    }
    float mx = 0.f;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
        rotate_row<D>(v[j], ol, a.rot4);
        if (t * WQ + g + 8 * j < a.lq) {
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmax_nn(mx, fabsf(v[j][e]));
        }
    }
    mx = max_row<D>(mx);
    const float sc = mx / 127.f + 1e-7f, inv = 1.f / sc;
    if (ol == 0) a.qs[bh * a.qg * 8 + gid] = sc;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
        const int row = t * WQ + g + 8 * j;
        if (row < a.lq) *reinterpret_cast<uint4*>(a.qi + (bh * a.lq + row) * D + ol * 16) = codes16(v[j], inv);
    }
}

// K: one workgroup of 256 threads per tile of CK keys.  A scale group is the keys with (key % 8) / 2 == g; its CK/4 rows
// are shared out over the runs of D/16 lanes that serve the group, whose maxima meet in LDS.  The tile is assembled in
// LDS in fragment order, [32-key block][channel step of 32][half of 16 channels][key][16 bytes] (the 64 lanes of the
// attention kernel read one contiguous KB per load), and leaves as 16-byte stores over its contiguous CK * D bytes;
// keys past lk are zeros.
template <int DT, int CK, int D>
__device__ __forceinline__ void quant_k_body(const AttnArgs& a, const int hi, const int t, const int bi) {
    constexpr int LPR = lanes_per_row(D), RUNS = 256 / LPR, NSUB = RUNS / 4;
    constexpr int R = (CK / 4) / NSUB;   // rows per run
    static_assert(R >= 1 && R * NSUB * 4 == CK, "rows of a group divide over its runs");
    __shared__ float omax[RUNS];
    __shared__ __align__(16) uint8_t stage[CK * D];
    const int ol = threadIdx.x & (LPR - 1), run = threadIdx.x / LPR, g = run & 3, sub = run >> 2;
    const int64_t bh = (int64_t)bi * a.hk + hi, base = bi * a.k_bs + hi * a.k_hs + ol * 16;
    const int anchor = a.anchors[bh];
    float bias[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) bias[e] = 0.f;
    if (anchor >= 0) {
        ld16_dt<DT>(a.k, base + (int64_t)anchor * a.k_rs, a.in_vec, bias);
        if constexpr (D == 128) {
            if (a.k_norm) norm_rope_row(bias, ol, a.kw, a.rope ? a.rope + (int64_t)anchor * D : nullptr, a.eps, a.rope_mode);
        }
    }
    float v[R][16];
    int rt[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int i = sub * R + j;                  // index within the group
        rt[j] = (i / 2) * 8 + g * 2 + (i % 2);      // row within the tile
        const int row = t * CK + rt[j], rr = row < a.lk ? row : a.lk - 1;
        ld16_dt<DT>(a.k, base + (int64_t)rr * a.k_rs, a.in_vec, v[j]);
        if constexpr (D == 128) {
            if (a.k_norm) norm_rope_row(v[j], ol, a.kw, a.rope ? a.rope + (int64_t)rr * D : nullptr, a.eps, a.rope_mode);
        }
    }
    float mx = 0.f;
#pragma unroll
    for (int j = 0; j < R; ++j) {
#pragma unroll
        for (int e = 0; e < 16; ++e) v[j][e] -= bias[e];
        rotate_row<D>(v[j], ol, a.rot4);
        if (t * CK + rt[j] < a.lk) {
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmax_nn(mx, fabsf(v[j][e]));
        }
    }
    mx = max_row<D>(mx);
    if (ol == 0) omax[run] = mx;
    __syncthreads();
    mx = 0.f;
#pragma unroll
    for (int x = 0; x < NSUB; ++x) mx = fmax_nn(mx, omax[x * 4 + g]);
    const float sc = mx / 127.f + 1e-7f, inv = 1.f / sc;
    if (sub == 0 && ol == 0) a.ks[(bh * a.kb + t) * 4 + g] = sc;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        uint4 w = make_uint4(0u, 0u, 0u, 0u);
        if (t * CK + rt[j] < a.lk) w = codes16(v[j], inv);
        *reinterpret_cast<uint4*>(stage + (rt[j] / 32) * (32 * D) + (ol >> 1) * 1024 + (ol & 1) * 512 + (rt[j] % 32) * 16) = w;
    }
    __syncthreads();
    uint4* out = reinterpret_cast<uint4*>(a.ki + (bh * a.nblk + (int64_t)t * (CK / 32)) * (32 * D));
#pragma unroll
    for (int i = 0; i < CK * D / 16 / 256; ++i)
        out[i * 256 + threadIdx.x] = *reinterpret_cast<const uint4*>(stage + (i * 256 + threadIdx.x) * 16);
}

// V abs-max per channel: 256 threads take 128 rows of one (kv head, batch), four channels per thread; non-negative
// floats order as their bits, so the workgroups combine with an integer atomic max.
template <int DT, int D>
__device__ __forceinline__ void v_absmax_body(const AttnArgs& a, const int hi, const int chunk, const int bi) {
    constexpr int TPR = D / 4, RL = 256 / TPR;   // threads per row, rows per pass
    __shared__ float red[RL][D];
    const int c4 = threadIdx.x % TPR, rl = threadIdx.x / TPR;
    const int64_t base = bi * a.v_bs + hi * a.v_hs + c4 * 4;
    float mx[4] = {0.f, 0.f, 0.f, 0.f};
    const int r0 = chunk * 128;
#pragma unroll 4
    for (int i = 0; i < 128 / RL; ++i) {
        const int r = r0 + rl + RL * i;
        if (r < a.lk) {
            float x[4];
            ld4_dt<DT>(a.v, base + (int64_t)r * a.v_rs, a.v_vec, x);
#pragma unroll
            for (int c = 0; c < 4; ++c) mx[c] = fmax_nn(mx[c], fabsf(x[c]));
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) red[rl][c4 * 4 + c] = mx[c];
    __syncthreads();
    if (threadIdx.x < D) {
        float m = 0.f;
#pragma unroll
        for (int i = 0; i < RL; ++i) m = fmax_nn(m, red[i][threadIdx.x]);
        atomicMax(&a.vmax[((int64_t)bi * a.hk + hi) * D + threadIdx.x], f2u(m));
    }
}

// Two launches carry the four bodies above: work that does not depend on each other shares a launch, heads fastest so
// that neighbouring workgroups read neighbouring memory.  Stage 1: anchors (which also clear the V accumulators) and Q.
// Stage 2: K (needs the anchors) and the V abs-max (needs the cleared accumulators).
template <int DT, int D>
__global__ __launch_bounds__(256) void attn_stage1_kernel(AttnArgs a) {
    int id = blockIdx.x;
    const int n_anchor = a.hk * a.b;
    if (id < n_anchor) {
        anchor_body<DT, D>(a, id % a.hk, id / a.hk);
        return;
    }
    id -= n_anchor;
    constexpr int GPB = 4 * (64 / lanes_per_row(D));   // scale groups per workgroup
    const int ny = (a.qg * 8 + GPB - 1) / GPB;
    quant_q_body<DT, D>(a, id % a.h, (id / a.h) % ny, id / (a.h * ny));
}

template <int DT, int CK, int D>
__global__ __launch_bounds__(256) void attn_stage2_kernel(AttnArgs a) {
    int id = blockIdx.x;
    const int n_k = a.hk * a.kb * a.b;
    if (id < n_k) {
        quant_k_body<DT, CK, D>(a, id % a.hk, (id / a.hk) % a.kb, id / (a.hk * a.kb));
        return;
    }
    id -= n_k;
    const int nc = (a.lk + 127) / 128;
    v_absmax_body<DT, D>(a, id % a.hk, (id / a.hk) % nc, id / (a.hk * nc));
}

// V codes: one workgroup per block of 32 keys.  Rows are read as they lie (a thread takes 16 channels of one key),
// quantized and turned through LDS.  vt[(kv head, block)][d][32]: position h*16 + j of a row holds key
// (j/4)*8 + h*4 + j%4 of the block, which is the order a lane of the attention kernel holds its 16 scores in.  Keys past
// lk are zeros.  128 x the column sums go to vsum[(kv head, key tile)][d] by integer atomics.
template <int DT, int D>
__global__ __launch_bounds__(256) void attn_v_quant_kernel(AttnArgs a) {
    constexpr int LPR = lanes_per_row(D), KPP = 256 / LPR;   // keys per pass of the read phase
    __shared__ float inv_s[D];
    __shared__ __align__(16) int8_t tile[32][D];
    const int hi = blockIdx.x, s = blockIdx.y, bi = blockIdx.z;
    const int64_t bh = (int64_t)bi * a.hk + hi;
    if (threadIdx.x < D) {
        const float sc = fmax_nn(u2f(a.vmax[bh * D + threadIdx.x]) * (1.f / 127.f), 1e-12f);
        if (s == 0) a.vs[bh * D + threadIdx.x] = sc;
        inv_s[threadIdx.x] = 1.f / sc;
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < (32 + KPP - 1) / KPP; ++pass) {
        const int key = pass * KPP + threadIdx.x / LPR, seg = threadIdx.x % LPR;
        if (key >= 32) break;
        const int row = s * 32 + key;
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        if (row < a.lk) {
            const int64_t at = bi * a.v_bs + hi * a.v_hs + (int64_t)row * a.v_rs + seg * 16;
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                float x[4];
                ld4_dt<DT>(a.v, at + g4 * 4, a.v_vec, x);
#pragma unroll
                for (int c = 0; c < 4; ++c) w[g4] |= (uint32_t)(uint8_t)rn_s8(x[c] * inv_s[seg * 16 + g4 * 4 + c]) << (8 * c);
            }
        }
        *reinterpret_cast<uint4*>(&tile[key][seg * 16]) = make_uint4(w[0], w[1], w[2], w[3]);
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < (2 * D + 255) / 256; ++pass) {
        const int id = pass * 256 + threadIdx.x;
        if (id >= 2 * D) break;
        const int d = id % D, hh = id / D;
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        int sum = 0;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int q = tile[(j / 4) * 8 + hh * 4 + (j % 4)][d];
            sum += q;
            w[j / 4] |= (uint32_t)(uint8_t)q << (8 * (j % 4));
        }
        *reinterpret_cast<uint4*>(a.vt + ((bh * a.nblk + s) * D + d) * 32 + hh * 16) = make_uint4(w[0], w[1], w[2], w[3]);
        atomicAdd(&a.vsum[(bh * a.kb + s / (a.ck / 32)) * D + d], 128 * sum);
    }
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;

// The attention: a workgroup of four waves owns 128 query rows, a wave 32 of them.  The K tile, the V tile and the
// tile's 128 x column sums are contiguous in the workspace, in the order the fragment reads want them, so the four waves
// copy them global -> LDS with DMA loads (no registers) into one of two stages, a tile ahead; one barrier per tile.
// FD (no mask, 64-key tiles): the reference's unfused probability path in every tile, which its build takes for f16
// outputs and at most 512 keys (csrc/vendor/sage/sage_attn_launcher.cu:187-191, qk_int_sv_i8_cuda.cuh:132-139,637-700):
// every tile's maximum starts at a raw score of -50000 and the denominator sums the unrounded probabilities in
// per-thread partials (attn_utils.cuh:922-940).  Without FD only the last tile takes that form.
template <int OUT_DT, int CK, bool MASK = false, bool FD = false, int D = 128>
__global__ __launch_bounds__(256, D == 256 ? 1 : 2) void attn_int8_kernel(AttnArgs a) {
    constexpr int NB = CK / 32, NS = D / 32, KV = CK * D, STAGE = 2 * KV + D * 4, WQ = q_block_rows(D);
    static_assert(!MASK || D == 128, "the key-bias form exists for head dim 128 only");
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    const int hi = blockIdx.y, bi = blockIdx.z;
    const int row0 = blockIdx.x * 128 + wave * 32;
    const int64_t bh = (int64_t)bi * a.h + hi, kvh = (int64_t)bi * a.hk + hi / a.rep;
    // rows past lq are computed on a clamped row and never stored: every wave takes part in the copies and barriers
    const int r = row0 + l32, rc = r < a.lq ? r : a.lq - 1;

    auto fetch = [&](int t) {
        uint8_t* st = smem + (t & 1) * STAGE;
        const int64_t tile = (kvh * a.nblk + (int64_t)t * NB) * (32 * D) + lane * 16;
#pragma unroll
        for (int j = 0; j < KV / 4096; ++j) {
            const int c = wave + 4 * j;
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(a.ki + tile + c * 1024), (lds_ptr_t)(st + c * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(a.vt + tile + c * 1024), (lds_ptr_t)(st + KV + c * 1024), 16, 0, 0);
        }
        if (wave == 0 && lane < D / 4)
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(a.vsum + (kvh * a.kb + t) * D + lane * 4), (lds_ptr_t)(st + 2 * KV), 16, 0, 0);
    };
    fetch(0);

    v4i qf[NS];
    {
        const int8_t* qrow = a.qi + (bh * a.lq + rc) * D + hh * 16;
#pragma unroll
        for (int s = 0; s < NS; ++s) qf[s] = *reinterpret_cast<const v4i*>(qrow + s * 32);
    }
    const float q_scale = a.qs[(bh * a.qg + r / WQ) * 8 + (r & 7)];

    float ro[NS][16];
#pragma unroll
    for (int x = 0; x < NS; ++x)
#pragma unroll
        for (int i = 0; i < 16; ++i) ro[x][i] = 0.f;
    float m = -50000.f, dsum = 1.f;
    float dsum2 = 0.f;   // the unfused and per-key mask routes keep the reference's four partial denominators per row: two per lane
    bool kept = false;   // that route: some key of this lane was kept
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // One key tile.  The last tile (the only one that can hold keys past lk) is a separate instantiation, so that the
    // validity compares exist only there.
    auto tile = [&](const int t, auto last_tag) {
        constexpr bool last = decltype(last_tag)::value;
        const uint8_t* st = smem + (t & 1) * STAGE;
        const int key0 = t * CK;
        // Channel steps outside, key blocks inside: consecutive MFMAs write different accumulators, so none waits for
        // the one before it.
        v16i S[NB];
#pragma unroll
        for (int blk = 0; blk < NB; ++blk) S[blk] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int blk = 0; blk < NB; ++blk) {
                const v4i kf = *reinterpret_cast<const v4i*>(st + blk * (32 * D) + s * 1024 + lane * 16);
                S[blk] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[s], S[blk], 0, 0, 0);
            }
        if constexpr (!last) fetch(t + 1);   // the other stage: every wave left it at the barrier that ended the last tile
        const float* ksc = a.ks + (kvh * a.kb + t) * 4 + hh * 2;
        const float gs0 = a.sm * (q_scale * ksc[0]), gs1 = a.sm * (q_scale * ksc[1]);

        // Probabilities: v_cvt_pk_u8_f32 rounds to nearest even, saturates to 0..255 (NaN to 0) and writes one byte of a
        // dword, which is the reference's cvt.rni.sat.u8 plus the packing.  p - 128 as a signed byte is p ^ 0x80.
        v4i pf[NB];
        uint32_t psum = 0;
        float tile_m, o_scale, t_scale;
        auto rescale = [&]() {
            tile_m = fmax_nn(tile_m, __shfl_xor(tile_m, 32));
            const float smaller = __builtin_amdgcn_exp2f(-fabsf(m - tile_m));
            o_scale = m < tile_m ? smaller : 1.f;
            t_scale = tile_m < m ? smaller : 1.f;
            m = fmax_nn(m, tile_m);
        };
        // integer route: exp2(fma(score, group scale, negm)), the unmasked path and a tile with one bias for all its keys
        auto probabilities = [&](auto masked, const float negm) {
#pragma unroll
            for (int blk = 0; blk < NB; ++blk) {
                uint32_t w[4];
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    uint32_t packed = 0u;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float e = __builtin_amdgcn_exp2f(fmaf((float)S[blk][g4 * 4 + c], c < 2 ? gs0 : gs1, negm));
                        if constexpr (decltype(masked)::value) {
                            const int key = key0 + blk * 32 + g4 * 8 + hh * 4 + c;
                            e = key < a.lk ? e : 0.f;
                        }
                        packed = __builtin_amdgcn_cvt_pk_u8_f32(e, c, packed);
                    }
                    psum = __builtin_amdgcn_sad_u8(packed, 0u, psum);
                    w[g4] = packed ^ 0x80808080u;
                }
                pf[blk] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
                __builtin_amdgcn_sched_barrier(0);   // one block at a time: the converted scores die here
            }
        };
        auto int_maxima = [&](int& i0, int& i1) {
            i0 = i1 = INT_MIN;
#pragma unroll
            for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if ((i % 4) < 2) i0 = max(i0, S[blk][i]);
                    else i1 = max(i1, S[blk][i]);
                }
        };
        // float route of the masked forms: scores already carry scale and bias; exp2(score - tile_m)
        float fsc[MASK ? NB : 1][16];
        auto float_probabilities = [&](auto sum_floats) {
#pragma unroll
            for (int blk = 0; blk < NB; ++blk) {
                uint32_t w[4];
                float e[4][4];
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    uint32_t packed = 0u;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        e[g4][c] = __builtin_amdgcn_exp2f(fsc[MASK ? blk : 0][g4 * 4 + c] + (-tile_m));
                        packed = __builtin_amdgcn_cvt_pk_u8_f32(e[g4][c], c, packed);
                    }
                    psum = __builtin_amdgcn_sad_u8(packed, 0u, psum);
                    w[g4] = packed ^ 0x80808080u;
                }
                if constexpr (decltype(sum_floats)::value) {
                    // the reference's thread l of a row owns keys 2l, 2l+1, 8+2l, 9+2l of each 16: this lane carries
                    // threads 2hh (c = 0, 1) and 2hh + 1 (c = 2, 3); a 16-key group is two g4 steps
#pragma unroll
                    for (int fk = 0; fk < 2; ++fk) {
                        dsum += ((e[2 * fk][0] + e[2 * fk][1]) + (e[2 * fk + 1][0] + e[2 * fk + 1][1])) * t_scale;
                        dsum2 += ((e[2 * fk][2] + e[2 * fk][3]) + (e[2 * fk + 1][2] + e[2 * fk + 1][3])) * t_scale;
                    }
                }
                pf[blk] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        if constexpr (!MASK && (FD || last)) {
            // The unfused form: every tile with FD, and the last tile always (the reference's last iteration has no fused
            // variant, qk_int_sv_i8_cuda.cuh:956-1000).  Maxima start at a raw score of -50000, keys past lk drop out
            // (-1e30 raw), and the denominator takes the unrounded probabilities, in the two per-thread partials of the
            // reference that this lane carries (threads 2hh: c = 0, 1 and 2hh + 1: c = 2, 3 of each 16 keys).
            int i0 = -50000, i1 = -50000;
#pragma unroll
            for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    int sv = S[blk][i];
                    if constexpr (last) {
                        const int key = key0 + blk * 32 + (i / 4) * 8 + hh * 4 + (i % 4);
                        sv = key < a.lk ? sv : INT_MIN;
                    }
                    if ((i % 4) < 2) i0 = max(i0, sv);
                    else i1 = max(i1, sv);
                }
            tile_m = fmax_nn(fmaf((float)i0, gs0, -kU8Offset), fmaf((float)i1, gs1, -kU8Offset));
            rescale();
            dsum *= o_scale;
            dsum2 *= o_scale;
#pragma unroll
            for (int blk = 0; blk < NB; ++blk) {
                uint32_t w[4];
                float e[4][4];
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    uint32_t packed = 0u;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        e[g4][c] = __builtin_amdgcn_exp2f(fmaf((float)S[blk][g4 * 4 + c], c < 2 ? gs0 : gs1, -tile_m));
                        if constexpr (last) {
                            const int key = key0 + blk * 32 + g4 * 8 + hh * 4 + c;
                            e[g4][c] = key < a.lk ? e[g4][c] : 0.f;
                        }
                        packed = __builtin_amdgcn_cvt_pk_u8_f32(e[g4][c], c, packed);
                    }
                    w[g4] = packed ^ 0x80808080u;
                }
#pragma unroll
                for (int fk = 0; fk < 2; ++fk) {
                    dsum += ((e[2 * fk][0] + e[2 * fk][1]) + (e[2 * fk + 1][0] + e[2 * fk + 1][1])) * t_scale;
                    dsum2 += ((e[2 * fk][2] + e[2 * fk][3]) + (e[2 * fk + 1][2] + e[2 * fk + 1][3])) * t_scale;
                }
                pf[blk] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
                __builtin_amdgcn_sched_barrier(0);
            }
        } else if constexpr (!MASK) {
            // Group maxima on the integers (exact in fp32: |score| < 2^24).
            int i0, i1;
            int_maxima(i0, i1);
            tile_m = fmax_nn(fmaf((float)i0, gs0, -kU8Offset), fmaf((float)i1, gs1, -kU8Offset));
            rescale();
            dsum *= o_scale;
            probabilities(std::false_type{}, -tile_m);
            dsum += (float)psum * t_scale;
        } else {
            // this lane's prepared biases: four consecutive keys per (blk, g4)
            auto load_bias = [&](float (&bj)[NB][16]) {
#pragma unroll
                for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const float4 b4 = *reinterpret_cast<const float4*>(a.kbias + key0 + blk * 32 + g4 * 8 + hh * 4);
                        bj[blk][g4 * 4] = b4.x; bj[blk][g4 * 4 + 1] = b4.y; bj[blk][g4 * 4 + 2] = b4.z; bj[blk][g4 * 4 + 3] = b4.w;
                    }
            };
            if constexpr (CK == 64) {
                // per-key mask: scaled score, plus the bias where the key is kept, -50000 elsewhere; the denominator sums
                // the unrounded probabilities in the reference's per-thread partials
                float bj[NB][16];
                load_bias(bj);
                float mx = -50000.f;
#pragma unroll
                for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const bool keep = bj[blk][i] != -__builtin_inff();   // padding past lk is prepared as -inf too
                        kept = kept || keep;
                        const float rs = (float)S[blk][i] * ((i % 4) < 2 ? gs0 : gs1);
                        fsc[MASK ? blk : 0][i] = keep ? rs + bj[blk][i] : -50000.f;
                        mx = fmax_nn(mx, fsc[MASK ? blk : 0][i]);
                    }
                tile_m = mx - kU8Offset;
                rescale();
                dsum *= o_scale;
                dsum2 *= o_scale;
                float_probabilities(std::true_type{});
            } else {
                const float tb = a.tbias[t];   // uniform: a scalar branch
                if (!last && __builtin_isfinite(tb)) {
                    int i0, i1;
                    int_maxima(i0, i1);
                    tile_m = fmax_nn(fmaf((float)i0, gs0, -kU8Offset) + tb, fmaf((float)i1, gs1, -kU8Offset) + tb);
                    rescale();
                    probabilities(std::false_type{}, tb - tile_m);
                } else {
                    float bj[NB][16];
                    load_bias(bj);
                    float mx = -50000.f;
#pragma unroll
                    for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            fsc[MASK ? blk : 0][i] = fmaf((float)S[blk][i], (i % 4) < 2 ? gs0 : gs1, bj[blk][i]);
                            mx = fmax_nn(mx, fsc[MASK ? blk : 0][i]);
                        }
                    tile_m = mx - kU8Offset;
                    rescale();
                    float_probabilities(std::false_type{});
                }
                dsum *= o_scale;
                dsum += (float)psum * t_scale;
            }
        }

        // P.V: the 32-channel blocks of the output keep their own accumulators (the scores are dead by now), key blocks
        // outside, so that consecutive MFMAs are independent here too; four output blocks at a time.
#pragma unroll
        for (int x0 = 0; x0 < NS; x0 += 4) {
            constexpr int NX = NS < 4 ? NS : 4;
            v16i acc[NX];
#pragma unroll
            for (int x = 0; x < NX; ++x) {
                const int* vsp = reinterpret_cast<const int*>(st + 2 * KV) + (x0 + x) * 32 + hh * 4;
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const v4i c4 = *reinterpret_cast<const v4i*>(vsp + g4 * 8);
                    acc[x][g4 * 4 + 0] = c4[0];
                    acc[x][g4 * 4 + 1] = c4[1];
                    acc[x][g4 * 4 + 2] = c4[2];
                    acc[x][g4 * 4 + 3] = c4[3];
                }
            }
#pragma unroll
            for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                for (int x = 0; x < NX; ++x) {
                    const v4i vf = *reinterpret_cast<const v4i*>(st + KV + ((blk * D + (x0 + x) * 32 + l32) * 32 + hh * 16));
                    acc[x] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf, pf[blk], acc[x], 0, 0, 0);
                }
#pragma unroll
            for (int x = 0; x < NX; ++x)
#pragma unroll
                for (int i = 0; i < 16; ++i) ro[x0 + x][i] = fmaf((float)acc[x][i], t_scale, ro[x0 + x][i] * o_scale);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's share of the next tile has landed
        __syncthreads();
    };
    for (int t = 0; t + 1 < a.kb; ++t) tile(t, std::false_type{});
    tile(a.kb - 1, std::true_type{});

    dsum += dsum2;   // (d0 + d1) and (d2 + d3) of the reference's four threads
    float dtot = dsum + __shfl_xor(dsum, 32);
    bool row_kept = true;
    if constexpr (MASK && CK == 64) row_kept = (__shfl_xor((int)kept, 32) | (int)kept) != 0;   // a row with no kept key gives zeros
    // `sink` more keys of score zero and value zero: each adds exp2(0 - m) to the denominator, nothing to the output
    if (a.sink != 0.f) dtot = fmaf(a.sink, __builtin_amdgcn_exp2f(-m), dtot);
    const float rcp = 1.f / dtot;
    if (r < a.lq) {
        const int64_t ob = bi * a.o_bs + (int64_t)r * a.o_rs + hi * a.o_hs;
#pragma unroll
        for (int x = 0; x < NS; ++x)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int d0 = x * 32 + g4 * 8 + hh * 4;
                const float4 s4 = *reinterpret_cast<const float4*>(a.vs + kvh * D + d0);
                float out[4] = {ro[x][g4 * 4] * rcp * s4.x, ro[x][g4 * 4 + 1] * rcp * s4.y, ro[x][g4 * 4 + 2] * rcp * s4.z,
                                ro[x][g4 * 4 + 3] * rcp * s4.w};
                if constexpr (MASK && CK == 64) {
                    if (!row_kept) out[0] = out[1] = out[2] = out[3] = 0.f;
                }
                if (a.vec_ok) store4<OUT_DT>(a.o, ob + d0, out);
                else
#pragma unroll
                    for (int c = 0; c < 4; ++c) st_dt<OUT_DT>(a.o, ob + d0 + c, out[c]);
            }
    }
}

int cta_k_for(int lk, int d) { return lk > 1024 && d != 64 ? 128 : 64; }   // csrc/attn_int8.cu:56

// The caller's per-key bias, prepared once per call (csrc/vendor/sage/sage_attn_launcher.cu:343-391; attn_utils.cuh:
// 466-515 for the per-key form): bias * log2e per key of every tile, -inf where the bias is not finite and for the
// padding past lk; for 128-key tiles also the value all keys of a tile share (times log2e), NaN when they differ.
template <int CK>
__global__ __launch_bounds__(CK) void attn_key_bias_kernel(const float* bias, int lk, float* kbias, float* tbias) {
    __shared__ float lo_s[CK / 64], hi_s[CK / 64];
    const int tid = threadIdx.x, key = blockIdx.x * CK + tid;
    float raw = key < lk ? bias[key] : -__builtin_inff();
    if (!__builtin_isfinite(raw)) raw = -__builtin_inff();
    kbias[key] = raw * 1.44269504088896340736f;
    if constexpr (CK == 128) {
        float lo = raw, hi = raw;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            lo = fminf(lo, __shfl_xor(lo, o));
            hi = fmaxf(hi, __shfl_xor(hi, o));
        }
        if ((tid & 63) == 0) { lo_s[tid >> 6] = lo; hi_s[tid >> 6] = hi; }
        __syncthreads();
        if (tid == 0) {
            lo = fminf(lo_s[0], lo_s[1]);
            hi = fmaxf(hi_s[0], hi_s[1]);
            tbias[blockIdx.x] = lo == hi ? hi * 1.44269504088896340736f : __builtin_nanf("");
        }
    }
}

struct Plan {
    int64_t qi, ki, qs, ks, vt, vs, anchors, vmax, vsum, total;
    int ck, kb, qg, nblk;
};

Plan plan_for(int64_t b, int64_t h, int64_t hk, int64_t lq, int64_t lk, int D) {
    Plan p;
    p.ck = cta_k_for((int)lk, D);
    p.kb = (int)((lk + p.ck - 1) / p.ck);
    p.qg = (int)((lq + 127) / 128 * (128 / q_block_rows(D)));   // row blocks of the Q quantizer, eight scale groups each
    p.nblk = p.kb * (p.ck / 32);
    int64_t n = 0;
    auto add = [&](int64_t bytes) { const int64_t at = n; n += (bytes + 255) / 256 * 256; return at; };
    p.qi = add(b * h * lq * D);
    p.ki = add(b * hk * (int64_t)p.nblk * 32 * D);
    p.qs = add(b * h * p.qg * 8 * 4);
    p.ks = add(b * hk * p.kb * 4 * 4);
    p.vt = add(b * hk * (int64_t)p.nblk * D * 32);
    p.vs = add(b * hk * D * 4);
    p.anchors = add(b * hk * 4);
    p.vmax = add(b * hk * D * 4);
    p.vsum = add(b * hk * (int64_t)p.kb * D * 4);
    p.total = n;
    return p;
}

// More than 64 KB of dynamic LDS has to be allowed once per kernel and device.
template <class K> bool allow_lds(K kern, int bytes) {
    static PerDeviceOnce once;
    return allow_dynamic_lds(reinterpret_cast<const void*>(kern), bytes, once) == 0;
}

template <int DT, int CK, bool MASK, bool FD, int D>
int launch_attn(const AttnArgs& a, hipStream_t st) {
    constexpr int kLds = 2 * (2 * CK * D + D * 4);
    auto kern = attn_int8_kernel<DT, CK, MASK, FD, D>;
    if (kLds > 64 * 1024 && !allow_lds(kern, kLds)) return -401;
    kern<<<dim3((a.lq + 127) / 128, a.h, a.b), 256, kLds, st>>>(a);
    return hipGetLastError() == hipSuccess ? 0 : -401;
}

template <int DT, int D>
int run(AttnArgs a, hipStream_t st) {
    constexpr int GPB = 4 * (64 / lanes_per_row(D));   // scale groups per workgroup of the Q quantizer
    const int64_t n1 = (int64_t)a.hk * a.b + (int64_t)a.h * ((a.qg * 8 + GPB - 1) / GPB) * a.b;
    const int64_t n2 = (int64_t)a.hk * a.kb * a.b + (int64_t)a.hk * ((a.lk + 127) / 128) * a.b;
    if (n1 > 0x7fffffff || n2 > 0x7fffffff) return -400;
    attn_stage1_kernel<DT, D><<<dim3((unsigned)n1), 256, 0, st>>>(a);
    if (a.ck == 64) attn_stage2_kernel<DT, 64, D><<<dim3((unsigned)n2), 256, 0, st>>>(a);
    else if constexpr (D != 64) attn_stage2_kernel<DT, 128, D><<<dim3((unsigned)n2), 256, 0, st>>>(a);
    attn_v_quant_kernel<DT, D><<<dim3(a.hk, a.nblk, a.b), 256, 0, st>>>(a);
    if (hipGetLastError() != hipSuccess) return -401;
    if constexpr (D == 128) {
        if (a.bias) {
            if (a.ck == 64) {
                attn_key_bias_kernel<64><<<dim3(a.kb), 64, 0, st>>>(a.bias, a.lk, a.kbias, a.tbias);
                return launch_attn<DT, 64, true, false, D>(a, st);
            }
            attn_key_bias_kernel<128><<<dim3(a.kb), 128, 0, st>>>(a.bias, a.lk, a.kbias, a.tbias);
            return launch_attn<DT, 128, true, false, D>(a, st);
        }
    }
    // f16 outputs with at most 512 keys: the reference's build takes its unfused probability path in every tile
    if (DT == DT_F16 && a.lk <= 512 && a.ck == 64) return launch_attn<DT_F16, 64, false, true, D>(a, st);
    if (a.ck == 64) return launch_attn<DT, 64, false, false, D>(a, st);
    if constexpr (D != 64) return launch_attn<DT, 128, false, false, D>(a, st);
    return -400;
}

// Per-head RMSNorm and RoPE for q and k, applied on the way into the quantizer (csrc/attn_int8.cu:69-76).  A null kw
// takes K as it is (csrc/vendor/sage/quant_qk_int8.cu:1264-1268).
struct QkNorm {
    const float* qw;
    const float* kw;
    const float* rope;
    float eps;
    int rope_mode;
};

int int8_attn(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h, int hk, int Dh,
              int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs, int64_t v_bs, int64_t v_rs,
              int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale, int dt, void* stream, float sink = 0.f,
              const QkNorm* norm = nullptr, const float* bias = nullptr) {
    const char* why = nullptr;
    if (Dh != 64 && Dh != 128 && Dh != 256) why = "head dim must be 64, 128 or 256";
    else if ((norm || bias) && (dt != DT_BF16 || Dh != 128)) why = "fused q/k norm and key bias need bf16 head dim 128";   // csrc/attn_int8.cu:135
    else if (norm && (norm->rope_mode < 0 || norm->rope_mode > 2)) why = "rope_mode must be 0, 1 or 2";   // quant_qk_int8.cu:1279
    else if (!q || !k || !v || !o || !ws) why = "null pointer";
    else if (b <= 0 || lq <= 0 || lk <= 0 || h <= 0 || hk <= 0 || h % hk != 0) why = "bad sizes";
    else if (b > 65535 || h > 65535 || lq > (1 << 20) || lk > (1 << 20)) why = "batch, head count or length beyond the grid limits";
    else if (((uintptr_t)ws & 255) != 0) why = "workspace must be 256-byte aligned";
    if (why) {
        fprintf(stderr, "int8 attention: %s\n", why);
        return -400;
    }
    const Plan p = plan_for(b, h, hk, lq, lk, Dh);
    char* w = (char*)ws;
    AttnArgs a;
    a.q = q; a.k = k; a.v = v; a.o = o;
    a.qi = (int8_t*)(w + p.qi); a.ki = (int8_t*)(w + p.ki); a.vt = (int8_t*)(w + p.vt);
    a.qs = (float*)(w + p.qs); a.ks = (float*)(w + p.ks); a.vs = (float*)(w + p.vs);
    a.anchors = (int*)(w + p.anchors); a.vmax = (uint32_t*)(w + p.vmax); a.vsum = (int*)(w + p.vsum);
    a.b = b; a.lq = lq; a.lk = lk; a.h = h; a.hk = hk; a.rep = h / hk;
    a.qg = p.qg; a.kb = p.kb; a.ck = p.ck; a.nblk = p.nblk;
    a.q_bs = q_bs; a.q_rs = q_rs; a.q_hs = q_hs; a.k_bs = k_bs; a.k_rs = k_rs; a.k_hs = k_hs;
    a.v_bs = v_bs; a.v_rs = v_rs; a.v_hs = v_hs; a.o_bs = o_bs; a.o_rs = o_rs; a.o_hs = o_hs;
    a.sm = scale * 1.44269504088896340736f;
    a.rot4 = lk <= 256 ? 1 : 0;
    a.sink = sink;
    a.use_anchor = sink == 0.f ? 1 : 0;   // with a sink a zero key's score must stay zero: no shift (csrc/attn_int8.cu:134-141)
    a.vec_ok = ((o_bs | o_rs | o_hs) % 4 == 0 && ((uintptr_t)o & 7) == 0) ? 1 : 0;
    a.v_vec = ((v_bs | v_rs | v_hs) % 4 == 0 && ((uintptr_t)v & 7) == 0) ? 1 : 0;
    a.in_vec = ((q_bs | q_rs | q_hs | k_bs | k_rs | k_hs) % 4 == 0 && (((uintptr_t)q | (uintptr_t)k) & 7) == 0) ? 1 : 0;
    a.bias = bias;
    a.kbias = (float*)(w + p.total);   // the key-bias form's workspace is this much longer
    a.tbias = a.kbias + (int64_t)p.kb * p.ck;
    a.qw = a.kw = a.rope = nullptr;
    a.eps = 0.f;
    a.q_norm = a.k_norm = a.rope_mode = 0;
    if (norm) {
        a.qw = norm->qw;
        a.kw = norm->kw;
        a.rope = (norm->rope && norm->rope_mode != 0) ? norm->rope : nullptr;
        a.eps = norm->eps;
        a.rope_mode = norm->rope_mode;
        a.q_norm = 1;
        a.k_norm = norm->kw ? 1 : 0;
    }
    hipStream_t st = (hipStream_t)stream;
    if (Dh == 64) return dt == DT_F16 ? run<DT_F16, 64>(a, st) : run<DT_BF16, 64>(a, st);
    if (Dh == 256) return dt == DT_F16 ? run<DT_F16, 256>(a, st) : run<DT_BF16, 256>(a, st);
    return dt == DT_F16 ? run<DT_F16, 128>(a, st) : run<DT_BF16, 128>(a, st);
}

}  // namespace

GPU_API int64_t gpu_int8_attn_workspace_d(int b, int h, int hk, int lq, int lk, int head_dim) {
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return 0;
    if (b <= 0 || h <= 0 || hk <= 0 || lq <= 0 || lk <= 0) return 0;
    return plan_for(b, h, hk, lq, lk, head_dim).total;
}

GPU_API int64_t gpu_int8_attn_workspace(int b, int h, int hk, int lq, int lk) {
    return gpu_int8_attn_workspace_d(b, h, hk, lq, lk, 128);
}

GPU_API int gpu_int8_attn_d(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h,
                            int hk, int head_dim, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs,
                            int64_t k_hs, int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs,
                            float scale, void* stream) {
    return int8_attn(q, k, v, o, ws, b, lq, lk, h, hk, head_dim, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs,
                     o_rs, o_hs, scale, DT_BF16, stream);
}

GPU_API int gpu_int8_attn_f16(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h,
                              int hk, int head_dim, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs,
                              int64_t k_hs, int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs,
                              int64_t o_hs, float scale, void* stream) {
    return int8_attn(q, k, v, o, ws, b, lq, lk, h, hk, head_dim, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs,
                     o_rs, o_hs, scale, DT_F16, stream);
}

GPU_API int gpu_int8_attn(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h,
                          int hk, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs,
                          int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale,
                          void* stream) {
    return int8_attn(q, k, v, o, ws, b, lq, lk, h, hk, 128, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs, o_rs,
                     o_hs, scale, DT_BF16, stream);
}

GPU_API int gpu_int8_attn_sink(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h,
                               int hk, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs,
                               int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale,
                               float sink, const float* qw, float eps, void* stream) {
    const QkNorm norm{qw, nullptr, nullptr, eps, 0};   // a non-null qw normalizes q; k is taken as it is (csrc/attn_int8.cu:198-201)
    return int8_attn(q, k, v, o, ws, b, lq, lk, h, hk, 128, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs, o_rs,
                     o_hs, scale, DT_BF16, stream, sink, qw ? &norm : nullptr);
}

// gpu_int8_attn with q and k taken through the per-head RMSNorm, weight and RoPE of gpu_qk_norm_rope first, inside the
// quantizers; q and k in memory are left as they are (csrc/attn_int8.cu:163-174).  Head dim 128, bf16.
GPU_API int gpu_int8_attn_norm_rope(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk,
                                    int h, int hk, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs,
                                    int64_t k_hs, int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs,
                                    int64_t o_hs, float scale, const float* qw, const float* kw, float eps,
                                    const float* rope, int rope_mode, void* stream) {
    const QkNorm norm{qw, kw, rope, eps, rope_mode};
    return int8_attn(q, k, v, o, ws, b, lq, lk, h, hk, 128, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs, o_rs,
                     o_hs, scale, DT_BF16, stream, 0.f, &norm);
}

// sage's prepared key mask row for lk keys: each key's bias, then one value per 128-key tile (csrc/attn_int8.cu:178-182).
// The layout kept here (bias * log2e per key of every tile, then one value per 128-key tile) fits the same size.
static int64_t key_mask_width(int lk) {
    const int64_t tiles = (lk + 127) / 128;
    return (tiles * 129 + 3) / 4 * 4;
}

GPU_API int64_t gpu_int8_attn_key_bias_workspace(int b, int h, int hk, int lq, int lk) {
    if (b <= 0 || h <= 0 || hk <= 0 || lq <= 0 || lk <= 0) return 0;
    return gpu_int8_attn_workspace_d(b, h, hk, lq, lk, 128) + (key_mask_width(lk) * 4 + 255) / 256 * 256;
}

// gpu_int8_attn with bias (f32 [lk], the same for every batch item, query and head) added to each key's logits, as an
// additive attention mask; a bias that is not finite masks its key (csrc/attn_int8.cu:184-223).  bf16.
GPU_API int gpu_int8_attn_key_bias(const void* q, const void* k, const void* v, void* o, void* ws, int b, int lq, int lk, int h,
                                   int hk, int64_t q_bs, int64_t q_rs, int64_t q_hs, int64_t k_bs, int64_t k_rs, int64_t k_hs,
                                   int64_t v_bs, int64_t v_rs, int64_t v_hs, int64_t o_bs, int64_t o_rs, int64_t o_hs, float scale,
                                   const float* bias, void* stream) {
    if (!bias) {
        fprintf(stderr, "int8 attention: null key bias\n");
        return -400;
    }
    return int8_attn(q, k, v, o, ws, b, lq, lk, h, hk, 128, q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs, o_rs,
                     o_hs, scale, DT_BF16, stream, 0.f, nullptr, bias);
}

// Test hook: y[i] = v_cvt_pk_u8_f32(x[i]) into byte 0 of zero, so that a test can hold the instruction to
// round-to-nearest-even with saturation, which the probabilities rely on.
namespace {
__global__ void cvt_pk_u8_probe_kernel(const float* x, uint32_t* y, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = __builtin_amdgcn_cvt_pk_u8_f32(x[i], 0, 0u);
}
}  // namespace
GPU_API int gpu_internal_cvt_pk_u8_probe(const float* x, uint32_t* y, int n, void* stream) {
    if (!x || !y || n <= 0) return -400;
    cvt_pk_u8_probe_kernel<<<dim3((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, y, n);
    return hipGetLastError() == hipSuccess ? 0 : -401;
}

// Test hook: the sum of squares of rows of 128 floats as the fused norm takes it (eight lanes per row, sumsq128) and as
// the anchor search takes it (one thread, sumsq128_serial).  out[2 * row] and out[2 * row + 1]; rows a multiple of 8.
namespace {
__global__ void __launch_bounds__(64) sumsq_probe_kernel(const float* x, float* out, int split) {
    const int lane = threadIdx.x, o8 = lane & 7, row = blockIdx.x * 8 + (lane >> 3);
    float v[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = x[row * 128 + o8 * 16 + e];
    const float ss = sumsq128(v, o8, split != 0);
    if (o8 == (row & 7)) out[2 * row] = ss;          // any of the eight lanes holds it: take a different one per row
    if (o8 == 0) out[2 * row + 1] = sumsq128_serial(x + row * 128, split != 0);
}
}  // namespace
GPU_API int gpu_internal_attn_sumsq_probe(const float* x, float* out, int rows, int split, void* stream) {
    if (!x || !out || rows <= 0 || rows % 8) return -400;
    sumsq_probe_kernel<<<dim3(rows / 8), 64, 0, (hipStream_t)stream>>>(x, out, split);
    return hipGetLastError() == hipSuccess ? 0 : -401;
}

// Test hook: where the pieces of the workspace lie (byte offsets), and the tiling.  out[0..9] = qi, ki, qs, ks, vt, vs,
// anchors, vsum, key tile length, key tiles.
GPU_API int gpu_internal_attn_layout_d(int b, int h, int hk, int lq, int lk, int head_dim, int64_t* out) {
    if (b <= 0 || h <= 0 || hk <= 0 || lq <= 0 || lk <= 0 || !out || (head_dim != 64 && head_dim != 128 && head_dim != 256)) return -400;
    const Plan p = plan_for(b, h, hk, lq, lk, head_dim);
    const int64_t v[10] = {p.qi, p.ki, p.qs, p.ks, p.vt, p.vs, p.anchors, p.vsum, p.ck, p.kb};
    for (int i = 0; i < 10; ++i) out[i] = v[i];
    return 0;
}
GPU_API int gpu_internal_attn_layout(int b, int h, int hk, int lq, int lk, int64_t* out) {
    return gpu_internal_attn_layout_d(b, h, hk, lq, lk, 128, out);
}
