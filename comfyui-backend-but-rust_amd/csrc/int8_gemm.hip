// int8 x int8 -> int32 GEMM on gfx950 MFMA with the dequant epilogue fused, D = Out(acc * xs[m] * ws[n] + bias[n]).
//
// Semantics follow the reference's fused CUTLASS kernel (csrc/vendor/cutlass_gemm_int8.cu:84-95 plain epilogue,
// :149-161 residual epilogue, :348-388 argument handling); the design is for CDNA4: A[M,K] and W[N,K] are both
// K-contiguous, which is exactly the operand shape of v_mfma_i32_32x32x32_i8 (each lane feeds 16 consecutive K bytes of
// one row), so tiles go global -> LDS as 16-byte chunks with an XOR swizzle and come back as ds_read_b128 fragments.
// W rides in src0 and A in src1, which leaves every lane holding runs of four consecutive n for one m: the epilogue
// stores 8-byte (bf16/f16) or 16-byte (f32) vectors straight from the accumulators.
#include <atomic>
#include <cstdio>
#include <mutex>

#include "common.hpp"

// Nothing is scheduled across this point: it pins hand-interleaved instruction orders and keeps live ranges short.
#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

namespace {

__device__ __forceinline__ void store16_untracked(void* ptr, uint4 v);
__device__ __forceinline__ void store16_untracked_at(const void* base, uint32_t off, uint4 v);
// A 64-bit value that is the same in every lane, moved to scalar registers.
__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

enum { EPI_PLAIN = 0, EPI_RESID = 1, EPI_ACC = 2 };

struct GemmArgs {
    const int8_t* A;
    const int8_t* W;
    const float* xs;
    const float* ws;
    const void* bias;
    const void* rscale;
    const void* resid;
    void* D;
    int M, N, K;
    int tiles_m, tiles_n;
    uint32_t magic;   // panel_magic(tiles_m, tiles_n), for tile_of_block
    int kslice;   // ring kernel only: K elements per split-K slice (a multiple of 128), 0 = no split
};

template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int OCC_>
struct Cfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_, OCC = OCC_;
    static constexpr int NT = 64 * WGM * WGN;
    static constexpr int WTM = BM / WGM, WTN = BN / WGN;   // wave tile
    static constexpr int TM = WTM / 32, TN = WTN / 32;     // 32x32 MFMA tiles per wave
    static constexpr int CPR = BK / 16;                    // 16-byte chunks per tile row
    static constexpr int A_CHUNKS = BM * CPR / NT, W_CHUNKS = BN * CPR / NT;
    static constexpr int STAGE = (BM + BN) * BK;           // bytes per LDS stage
    static constexpr int SMEM = 2 * STAGE;
    static_assert(BM % (32 * WGM) == 0 && BN % (32 * WGN) == 0, "wave tile must be a multiple of 32x32");
    static_assert((BM * CPR) % NT == 0 && (BN * CPR) % NT == 0, "chunks must divide over the threads");
    static_assert(BK == 64 || BK == 128, "swizzle is written for 64- and 128-byte rows");
};

// Chunk swizzle.  The LDS of gfx950 has 64 banks of 4 bytes, and a ds_read_b128 is served 16 lanes (256 bytes) at a
// time: a fragment read takes 16 consecutive rows at one chunk column, so those 16 rows must land on 16 distinct
// 16-byte bank groups.  Rows are BK bytes apart: with 128-byte rows an even/odd row pair already covers the two halves
// of the bank space, so the chunk index is XORed with bits 1..3 of the row; with 64-byte rows four rows span the banks
// and bits 2..3 are used.  (Measured: XOR with the low row bits instead costs 25 % of the read bandwidth.)
// The lane number from the execution mask counters: two instructions, and no register held across a loop for it.
__device__ __forceinline__ int hw_lane() {
    int l = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(l));
    return l;
}

template <int BK> __device__ __forceinline__ int swz(int row, int chunk) {
    return BK == 64 ? (chunk ^ ((row >> 2) & 3)) : (chunk ^ ((row >> 1) & 7));
}

// The epilogue arithmetic for one value.  t0 = float(acc)*xs; then fma(t0, ws, bias): the reference composes a
// multiply node and an add node (csrc/vendor/cutlass_gemm_int8.cu:90-93) that its compiler is free to contract; this
// kernel always contracts, and likewise for z*rscale + resid (:156-159).
template <int OUT_DT, int EPI>
__device__ __forceinline__ float epi_value(int acc, float xs, float ws, float b, float rs, float res) {
    const float t = __builtin_fmaf((float)acc * xs, ws, b);
    if (EPI == EPI_RESID) return __builtin_fmaf(rnd_dt<OUT_DT>(t), rs, res);
    return t;
}

// Epilogue of one wave tile whose origin is (mb, nb).  acc[in][im][4*rb + j] is the accumulator of
// (m = mb + 32*im + lane%32, n = nb + 32*in + 8*rb + 4*(lane/32) + j): four consecutive n per lane and register group.
template <int TM, int TN, int OUT_DT, int EPI>
__device__ __forceinline__ void epilogue_store(const GemmArgs& p, v16i (&acc)[TN][TM], int mb, int nb, int lane, bool vec_ok) {
    const int frow = lane & 31, fhalf = lane >> 5;
#pragma unroll
    for (int im = 0; im < TM; ++im) {
        const int m = mb + im * 32 + frow;
        if (m >= p.M) continue;
        const float xs = EPI == EPI_ACC ? 0.f : p.xs[m];
#pragma unroll
        for (int in = 0; in < TN; ++in) {
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const int n = nb + in * 32 + rb * 8 + fhalf * 4;
                if (n >= p.N) continue;
                const int64_t o = (int64_t)m * p.N + n;
                if (EPI == EPI_ACC) {
                    int* d = (int*)p.D + o;
                    if (vec_ok) {
                        *reinterpret_cast<v4i*>(d) = v4i{acc[in][im][4 * rb], acc[in][im][4 * rb + 1], acc[in][im][4 * rb + 2], acc[in][im][4 * rb + 3]};
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j) if (n + j < p.N) d[j] = acc[in][im][4 * rb + j];
                    }
                    continue;
                }
                float ws[4], b[4] = {0.f, 0.f, 0.f, 0.f}, rs[4] = {0.f, 0.f, 0.f, 0.f}, res[4] = {0.f, 0.f, 0.f, 0.f}, out[4];
                if (vec_ok) {
                    const float4 w4 = *reinterpret_cast<const float4*>(p.ws + n);
                    ws[0] = w4.x; ws[1] = w4.y; ws[2] = w4.z; ws[3] = w4.w;
                    if (p.bias) load4<OUT_DT>(p.bias, n, b);
                    if (EPI == EPI_RESID) { load4<OUT_DT>(p.rscale, n, rs); load4<OUT_DT>(p.resid, o, res); }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (n + j >= p.N) { ws[j] = 0.f; continue; }
                        ws[j] = p.ws[n + j];
                        if (p.bias) b[j] = ld_dt<OUT_DT>(p.bias, n + j);
                        if (EPI == EPI_RESID) { rs[j] = ld_dt<OUT_DT>(p.rscale, n + j); res[j] = ld_dt<OUT_DT>(p.resid, o + j); }
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) out[j] = epi_value<OUT_DT, EPI>(acc[in][im][4 * rb + j], xs, ws[j], b[j], rs[j], res[j]);
                if (vec_ok) {
                    store4<OUT_DT>(p.D, o, out);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) if (n + j < p.N) st_dt<OUT_DT>(p.D, o + j, out[j]);
                }
            }
        }
    }
}

// Coalesced epilogue: the accumulator layout (lane = one m, four consecutive n per register group) would store 16-byte
// pieces scattered over 32 rows per instruction.  Instead each wave rounds its values to the output type, passes a
// 32-row piece of its tile through a private LDS region (XOR-swizzled 16-byte chunks, conflict-free both ways) and
// writes whole rows: 16 bytes per lane, consecutive lanes on consecutive addresses.  For the residual form the LDS
// holds z = Out(acc*xs*ws + bias), exactly the intermediate the reference rounds, and fma(z, rscale, resid) is applied
// on the way out.  Needs row starts of D (and resid) 16-byte aligned; the caller falls back to epilogue_store otherwise.
// STAGED: the per-column constants (ws and bias as floats, 2 x 32*TN values) are kept in the wave's LDS area `cst` and
// read back per piece, instead of 96 registers that a persistent kernel cannot spare next to its pipeline state.  1: this
// function loads them into `cst` first; 2: the caller has put them there (stage_columns, long before, so that their
// trip from memory is off the epilogue's path), and `xs_lds`, when given, holds the tile's row scales the same way.
// L: the MFMA shape the accumulators come from.  32: v16i acc[TN][TM], a lane holds row lane % 32 of a 32x32 tile and
// the columns 8*rb + 4*(lane / 32) + j.  16: v4i acc[2*TN][2*TM] of 16x16 tiles, a lane holds row lane % 16 and the
// columns 4*(lane / 16) + j; the 32x32 block (in, im) is then the four tiles (2*in + rb, 2*im + hm).
template <int TM, int TN, int OUT_DT, int EPI, int PW = TN * 32, bool UNTRACKED = false, int STAGED = 0, int L = 32, class Acc>
__device__ __forceinline__ void epilogue_shuffle(const GemmArgs& p, Acc& acc, int mb, int nb, int lane, uint8_t* wl,
                                                 uint8_t* wl2 = nullptr, float* cst = nullptr, const float* xs_lds = nullptr) {
    // a piece is 32 rows x PW columns of the wave tile: PW*SZ bytes per LDS row, 32*PW*SZ bytes per wave
    constexpr int SZ = (EPI == EPI_ACC || OUT_DT == DT_F32) ? 4 : 2;
    constexpr int WTN = TN * 32, NP = WTN / PW, TNP = PW / 32;
    constexpr int ROWB = PW * SZ, CPRW = ROWB / 16, MASK = CPRW - 1;
    constexpr int EPC = 16 / SZ;                  // elements per 16-byte chunk
    constexpr int RPI = 64 / CPRW, PASSES = 32 / RPI;
    static_assert(PW % 32 == 0 && WTN % PW == 0, "piece width");
    static_assert((CPRW & MASK) == 0 && CPRW <= 64 && CPRW >= 2, "chunks per row must be a power of two");
    // Everything below is a function of the lane number only, so in a persistent kernel the compiler would hoist dozens
    // of addresses out of the tile loop, keep them live across the K loop and spill them; the reloads then sit between
    // the stores, each behind a full memory wait.  Making the lane number opaque here keeps the address arithmetic local.
    asm volatile("" : "+v"(lane));
    constexpr int NRB = L == 32 ? 4 : 2, NHM = L == 32 ? 1 : 2;   // column runs per 32 columns, row halves per 32 rows
    const int frow = lane & (L - 1), fhalf = lane / L;            // row inside a tile; which four of every 8 (16) columns
    // first column of run rb inside a 32-column block; value j of run rb of block (in, im), row half hm
    auto run_col = [&](int rb) { return L == 32 ? rb * 8 + fhalf * 4 : rb * 16 + fhalf * 4; };
    auto val = [&](int in, int im, int rb, int hm, int j) -> int {
        if constexpr (L == 32) return acc[in][im][4 * rb + j];
        else return acc[2 * in + rb][2 * im + hm][j];
    };

    // per-lane column constants, loaded once and in one batch (no branches between the loads, so a single wait covers
    // them): ws and the raw bias words for the 4 n of every (in, rb).  Columns past N read the last valid vector.
    constexpr int BW = SZ == 4 ? 4 : 2;            // 32-bit words holding 4 bias values
    float wsr[STAGED ? 1 : TN][NRB][4];
    uint32_t braw[STAGED ? 1 : TN][NRB][BW];
    if (EPI != EPI_ACC && STAGED == 1) {
        // two columns per lane and pass
#pragma unroll
        for (int c0 = 0; c0 < WTN; c0 += 128) {
            const int c = c0 + lane * 2;
            if (c < WTN) {
                int n = nb + c;
                n = n < p.N ? n : p.N - 2;
                const float2 w2 = *reinterpret_cast<const float2*>(p.ws + n);
                float2 b2 = make_float2(0.f, 0.f);
                if (p.bias) {
                    b2.x = ld_dt<(SZ == 4 ? DT_F32 : OUT_DT)>(p.bias, n);
                    b2.y = ld_dt<(SZ == 4 ? DT_F32 : OUT_DT)>(p.bias, n + 1);
                }
                *reinterpret_cast<float2*>(cst + c) = w2;
                *reinterpret_cast<float2*>(cst + WTN + c) = b2;
            }
        }
    }
    if (EPI != EPI_ACC && !STAGED) {
#pragma unroll
        for (int in = 0; in < TN; ++in)
#pragma unroll
            for (int rb = 0; rb < NRB; ++rb) {
                int n = nb + in * 32 + run_col(rb);
                n = n < p.N ? n : p.N - 4;
                const float4 w4 = *reinterpret_cast<const float4*>(p.ws + n);
                wsr[in][rb][0] = w4.x; wsr[in][rb][1] = w4.y; wsr[in][rb][2] = w4.z; wsr[in][rb][3] = w4.w;
                if (p.bias) {
                    if (SZ == 4) {
                        const uint4 b4 = *reinterpret_cast<const uint4*>((const uint8_t*)p.bias + (int64_t)n * 4);
                        braw[in][rb][0] = b4.x; braw[in][rb][1] = b4.y; braw[in][rb][BW - 2] = b4.z; braw[in][rb][BW - 1] = b4.w;
                    } else {
                        const uint2 b2 = *reinterpret_cast<const uint2*>((const uint8_t*)p.bias + (int64_t)n * 2);
                        braw[in][rb][0] = b2.x; braw[in][rb][1] = b2.y;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < BW; ++j) braw[in][rb][j] = 0u;
                }
            }
    }
    // bias value j of (in, rb) as float: +0.0 for a null bias
    auto bias_f = [&](int in, int rb, int j) -> float {
        if (SZ == 4) return u2f(braw[in][rb][j]);
        const uint32_t w = braw[in][rb][j >> 1];
        if (OUT_DT == DT_BF16) return (j & 1) ? u2f(w & 0xffff0000u) : u2f(w << 16);
        return f16_to_f((uint16_t)((j & 1) ? (w >> 16) : (w & 0xffffu)));
    };
    const int rrow = lane / CPRW, rc = lane % CPRW;   // read phase: row within a pass, chunk
    // uniform per wave: the wave tile is wholly inside the matrix; where it starts; bytes per output row
    const bool full = __builtin_amdgcn_readfirstlane((int)(mb + TM * 32 <= p.M && nb + WTN <= p.N && p.N < (1 << 21))) != 0;
    const uint64_t row_bytes = (uint64_t)p.N * SZ;
    const uint64_t tile_base = uniform64((uint64_t)(uintptr_t)p.D + ((uint64_t)mb * p.N + nb) * SZ);
    const uint32_t lane_off = __umul24((uint32_t)rrow, (uint32_t)row_bytes) + (uint32_t)(rc * 16);   // both factors < 2^24 when `full`

    // Every global load is issued ahead of the stores that precede its use: the memory counter retires in order, so a
    // load issued after a store cannot be waited for without also waiting for that store to reach memory.
    float xsr[TM][NHM];
#pragma unroll
    for (int im = 0; im < TM; ++im)
#pragma unroll
        for (int hm = 0; hm < NHM; ++hm) {
            const int mrow = mb + im * 32 + hm * 16 + frow;
            if (xs_lds) xsr[im][hm] = EPI == EPI_ACC ? 0.f : xs_lds[im * 32 + hm * 16 + frow];
            else xsr[im][hm] = (EPI == EPI_ACC || mrow >= p.M) ? 0.f : p.xs[mrow];
        }
    float rs[NP][EPC];
    if (EPI == EPI_RESID) {
#pragma unroll
        for (int np = 0; np < NP; ++np) {
            const int ncol = nb + np * PW + rc * EPC;
#pragma unroll
            for (int h = 0; h < EPC / 4; ++h) {
                if (ncol < p.N) load4<OUT_DT>(p.rscale, ncol + 4 * h, rs[np] + 4 * h);
                else { rs[np][4 * h] = 0.f; rs[np][4 * h + 1] = 0.f; rs[np][4 * h + 2] = 0.f; rs[np][4 * h + 3] = 0.f; }
            }
        }
    }
    // residual rows of piece (im, np), in the read phase's layout
    auto load_resid = [&](int im, int np, uint4* rv) {
        const int ncol = nb + np * PW + rc * EPC;
#pragma unroll
        for (int t = 0; t < PASSES; ++t) {
            const int m = mb + im * 32 + t * RPI + rrow;
            if (m < p.M && ncol < p.N) rv[t] = *reinterpret_cast<const uint4*>((const uint8_t*)p.resid + ((int64_t)m * p.N + ncol) * SZ);
            else rv[t] = make_uint4(0, 0, 0, 0);
        }
    };

    // write phase of piece (im, np): this lane's rows of the piece into `buf`
    auto write_piece = [&](int im, int np, uint8_t* buf) {
#pragma unroll
        for (int hm = 0; hm < NHM; ++hm) {
            const float xs = xsr[im][hm];
            const int prow = hm * 16 + frow;   // row inside the 32-row piece
#pragma unroll
            for (int ip = 0; ip < TNP; ++ip)
#pragma unroll
                for (int rb = 0; rb < NRB; ++rb) {
                    const int in = np * TNP + ip;
                    const int byte = (ip * 32 + run_col(rb)) * SZ;
                    uint8_t* dst = buf + prow * ROWB + ((((byte >> 4) ^ prow) & MASK) << 4) + (byte & 15);
                    if (EPI == EPI_ACC) {
                        *reinterpret_cast<v4i*>(dst) = v4i{val(in, im, rb, hm, 0), val(in, im, rb, hm, 1), val(in, im, rb, hm, 2), val(in, im, rb, hm, 3)};
                    } else {
                        float o[4];
                        if (STAGED) {
                            const float4 w4 = *reinterpret_cast<const float4*>(cst + in * 32 + run_col(rb));
                            const float4 b4 = *reinterpret_cast<const float4*>(cst + WTN + in * 32 + run_col(rb));
                            o[0] = __builtin_fmaf((float)val(in, im, rb, hm, 0) * xs, w4.x, b4.x);
                            o[1] = __builtin_fmaf((float)val(in, im, rb, hm, 1) * xs, w4.y, b4.y);
                            o[2] = __builtin_fmaf((float)val(in, im, rb, hm, 2) * xs, w4.z, b4.z);
                            o[3] = __builtin_fmaf((float)val(in, im, rb, hm, 3) * xs, w4.w, b4.w);
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; ++j) o[j] = __builtin_fmaf((float)val(in, im, rb, hm, j) * xs, wsr[in][rb][j], bias_f(in, rb, j));
                        }
                        if (OUT_DT == DT_F32) {
                            *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
                        } else if (OUT_DT == DT_BF16) {
                            *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
                        } else {
                            *reinterpret_cast<uint2*>(dst) = make_uint2((uint32_t)f_to_f16(o[0]) | ((uint32_t)f_to_f16(o[1]) << 16),
                                                                        (uint32_t)f_to_f16(o[2]) | ((uint32_t)f_to_f16(o[3]) << 16));
                        }
                    }
                }
        }
    };
    // read phase, first half: the piece's rows back from `buf`, 16 bytes per lane and pass, all passes in one batch
    auto read_piece = [&](const uint8_t* buf, uint4* v) {
#pragma unroll
        for (int t = 0; t < PASSES; ++t) {
            const int r = t * RPI + rrow;
            v[t] = *reinterpret_cast<const uint4*>(buf + r * ROWB + (((rc ^ r) & MASK) << 4));
        }
    };
    // read phase, second half: whole rows out.  A wave tile that lies wholly inside the matrix stores through one
    // scalar base per pass plus a 32-bit lane offset: no per-pass compares, branches or 64-bit vector address arithmetic
    // (a fifth of the vector instructions of an epilogue that is bound by them).
    auto finish = [&](int np, const uint4& z, const uint4& r) -> uint4 {
        if (EPI != EPI_RESID) return z;
        const uint32_t zw[4] = {z.x, z.y, z.z, z.w}, rw[4] = {r.x, r.y, r.z, r.w};
        uint32_t ow[4];
        if (OUT_DT == DT_F32) {
#pragma unroll
            for (int j = 0; j < 4; ++j) ow[j] = f2u(__builtin_fmaf(u2f(zw[j]), rs[np][j], u2f(rw[j])));
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float z0, z1, r0, r1;
                if (OUT_DT == DT_BF16) {
                    z0 = u2f(zw[j] << 16); z1 = u2f(zw[j] & 0xffff0000u); r0 = u2f(rw[j] << 16); r1 = u2f(rw[j] & 0xffff0000u);
                    ow[j] = pack_bf16x2(__builtin_fmaf(z0, rs[np][2 * j], r0), __builtin_fmaf(z1, rs[np][2 * j + 1], r1));
                } else {
                    z0 = f16_to_f((uint16_t)(zw[j] & 0xffffu)); z1 = f16_to_f((uint16_t)(zw[j] >> 16));
                    r0 = f16_to_f((uint16_t)(rw[j] & 0xffffu)); r1 = f16_to_f((uint16_t)(rw[j] >> 16));
                    ow[j] = (uint32_t)f_to_f16(__builtin_fmaf(z0, rs[np][2 * j], r0)) | ((uint32_t)f_to_f16(__builtin_fmaf(z1, rs[np][2 * j + 1], r1)) << 16);
                }
            }
        }
        return make_uint4(ow[0], ow[1], ow[2], ow[3]);
    };
    auto store_piece = [&](int im, int np, const uint4* v, const uint4* rv) {
        if (full) {
            const uint64_t piece = tile_base + (uint64_t)(im * 32) * row_bytes + (uint64_t)(np * PW * SZ);
#pragma unroll
            for (int t = 0; t < PASSES; ++t) {
                const uint64_t pass = piece + (uint64_t)(t * RPI) * row_bytes;
                const uint4 o = finish(np, v[t], rv[t]);
                if (UNTRACKED) store16_untracked_at((const void*)pass, lane_off, o);
                else *reinterpret_cast<uint4*>((uint8_t*)pass + lane_off) = o;
            }
            return;
        }
        int l = lane;
        asm volatile("" : "+v"(l));   // keeps this path's address arithmetic from being hoisted in front of the branch
        const int row = l / CPRW, ncol = nb + np * PW + (l % CPRW) * EPC;
        uint8_t* base = (uint8_t*)p.D + ((int64_t)(mb + im * 32 + row) * p.N + ncol) * SZ;
        const int64_t step = (int64_t)RPI * p.N * SZ;
#pragma unroll
        for (int t = 0; t < PASSES; ++t) {
            const int m = mb + im * 32 + t * RPI + row;
            if (m >= p.M || ncol >= p.N) continue;
            uint8_t* out = base + t * step;
            const uint4 o = finish(np, v[t], rv[t]);
            if (UNTRACKED) store16_untracked(out, o);
            else *reinterpret_cast<uint4*>(out) = o;
        }
    };

    // Pieces go through the LDS one after the other.  With a second region (wl2) the loop is software-pipelined: the
    // LDS reads of piece i are issued, then the arithmetic and LDS writes of piece i+1 (into the other region) cover
    // their latency, then piece i is stored.  The LDS queue runs one wave's accesses in program order, so a piece's
    // reads see its writes, and a region is rewritten only after the reads of its previous piece have returned (they
    // are waited for by the stores in between).  The residual rows of a piece are requested before its write phase.
    constexpr int NPIECE = TM * NP;
    uint8_t* bufs[2] = {wl, wl2 ? wl2 : wl};
    uint4 rv[2][PASSES];
    if (EPI == EPI_RESID) load_resid(0, 0, rv[0]);
    write_piece(0, 0, bufs[0]);
#pragma unroll
    for (int i = 0; i < NPIECE; ++i) {
        const int im = i / NP, np = i % NP;
        uint4 v[PASSES];
        asm volatile("" ::: "memory");
        read_piece(bufs[i & 1], v);
        asm volatile("" ::: "memory");
        if (wl2 && i + 1 < NPIECE) {
            if (EPI == EPI_RESID) load_resid((i + 1) / NP, (i + 1) % NP, rv[(i + 1) & 1]);
            write_piece((i + 1) / NP, (i + 1) % NP, bufs[(i + 1) & 1]);
        }
        store_piece(im, np, v, rv[i & 1]);
        if (!wl2 && i + 1 < NPIECE) {
            if (EPI == EPI_RESID) load_resid((i + 1) / NP, (i + 1) % NP, rv[(i + 1) & 1]);
            asm volatile("" ::: "memory");
            write_piece((i + 1) / NP, (i + 1) % NP, bufs[0]);
        }
    }
    asm volatile("" ::: "memory");
}

// Chooses the coalesced epilogue when row starts are 16-byte aligned.  Must be called by all waves of the workgroup:
// it begins with a workgroup barrier because the shuffle reuses the LDS of the K loop.
template <int OUT_DT, int EPI>
__host__ __device__ __forceinline__ void epilogue_alignment(const GemmArgs& p, bool& vec_ok, bool& aligned) {
    constexpr int SZ = (EPI == EPI_ACC || OUT_DT == DT_F32) ? 4 : 2;
    constexpr uintptr_t V4 = 4 * SZ - 1;   // mask of a 4-element vector of the output type
    const uintptr_t ptrs = EPI == EPI_ACC ? (uintptr_t)p.D
                                          : ((uintptr_t)p.D | (uintptr_t)p.bias | (uintptr_t)p.rscale | (uintptr_t)p.resid);
    vec_ok = (p.N & 3) == 0 && (ptrs & V4) == 0 && (EPI == EPI_ACC || (((uintptr_t)p.ws) & 15) == 0);
    aligned = vec_ok && (((int64_t)p.N * SZ) & 15) == 0 &&
              (((uintptr_t)p.D | (uintptr_t)p.resid | (uintptr_t)p.rscale) & 15) == 0;
}

template <int TM, int TN, int OUT_DT, int EPI>
__device__ __forceinline__ void epilogue(const GemmArgs& p, v16i (&acc)[TN][TM], int mb, int nb, int lane, int wave, uint8_t* smem) {
    constexpr int SZ = (EPI == EPI_ACC || OUT_DT == DT_F32) ? 4 : 2;
    constexpr int PIECE = 32 * TN * 32 * SZ;   // bytes of one wave's 32-row piece
    bool vec_ok, aligned;
    epilogue_alignment<OUT_DT, EPI>(p, vec_ok, aligned);
    if (aligned) {
        __syncthreads();
        epilogue_shuffle<TM, TN, OUT_DT, EPI>(p, acc, mb, nb, lane, smem + wave * PIECE);
    } else {
        epilogue_store<TM, TN, OUT_DT, EPI>(p, acc, mb, nb, lane, vec_ok);
    }
}

template <class C, int OUT_DT, int EPI>
__global__ void __launch_bounds__(C::NT, C::OCC) int8_gemm_kernel(GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int BM = C::BM, BN = C::BN, BK = C::BK, NT = C::NT, CPR = C::CPR;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / C::WGN, wn = wave % C::WGN;

    int tm, tn;
    tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tm, tn, p.magic);
    const int m0 = tm * BM, n0 = tn * BN;
    const int K = p.K;

    // per-thread global sources (rows clamped into range: out-of-range rows compute garbage that is never stored)
    const int8_t* ga[C::A_CHUNKS];
    const int8_t* gw[C::W_CHUNKS];
    int la[C::A_CHUNKS], lw[C::W_CHUNKS], ka[C::A_CHUNKS], kw[C::W_CHUNKS];
#pragma unroll
    for (int i = 0; i < C::A_CHUNKS; ++i) {
        const int c = tid + i * NT, row = c / CPR, kc = c % CPR;
        const int gr = m0 + row < p.M ? m0 + row : p.M - 1;
        ga[i] = p.A + (int64_t)gr * K + kc * 16;
        ka[i] = kc * 16;
        la[i] = row * BK + (swz<BK>(row, kc) << 4);
    }
#pragma unroll
    for (int i = 0; i < C::W_CHUNKS; ++i) {
        const int c = tid + i * NT, row = c / CPR, kc = c % CPR;
        const int gr = n0 + row < p.N ? n0 + row : p.N - 1;
        gw[i] = p.W + (int64_t)gr * K + kc * 16;
        kw[i] = kc * 16;
        lw[i] = BM * BK + row * BK + (swz<BK>(row, kc) << 4);
    }

    v16i acc[C::TN][C::TM];
#pragma unroll
    for (int in = 0; in < C::TN; ++in)
#pragma unroll
        for (int im = 0; im < C::TM; ++im)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[in][im][r] = 0;

    const int nk = (K + BK - 1) / BK;
    v4i ra[C::A_CHUNKS], rw[C::W_CHUNKS];

    // Only the last K tile can be partial (K % 16 == 0, so whole chunks are in or out); it takes the guarded path.
    auto load_global = [&](int kt) {
        const int k0 = kt * BK;
#pragma unroll
        for (int i = 0; i < C::A_CHUNKS; ++i) ra[i] = *reinterpret_cast<const v4i*>(ga[i] + k0);
#pragma unroll
        for (int i = 0; i < C::W_CHUNKS; ++i) rw[i] = *reinterpret_cast<const v4i*>(gw[i] + k0);
    };
    auto load_global_tail = [&](int kt) {
        const int k0 = kt * BK;
#pragma unroll
        for (int i = 0; i < C::A_CHUNKS; ++i) {
            const bool in = k0 + ka[i] < K;
            ra[i] = *reinterpret_cast<const v4i*>(in ? ga[i] + k0 : ga[i] - ka[i]);  // row start is always readable
            if (!in) ra[i] = v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < C::W_CHUNKS; ++i) {
            const bool in = k0 + kw[i] < K;
            rw[i] = *reinterpret_cast<const v4i*>(in ? gw[i] + k0 : gw[i] - kw[i]);
            if (!in) rw[i] = v4i{0, 0, 0, 0};
        }
    };
    const bool tail = (K % BK) != 0;
    auto load_tile = [&](int kt) {
        if (tail && kt == nk - 1) load_global_tail(kt);
        else load_global(kt);
    };
    auto store_lds = [&](int stage) {
        uint8_t* s = smem + stage * C::STAGE;
#pragma unroll
        for (int i = 0; i < C::A_CHUNKS; ++i) *reinterpret_cast<v4i*>(s + la[i]) = ra[i];
#pragma unroll
        for (int i = 0; i < C::W_CHUNKS; ++i) *reinterpret_cast<v4i*>(s + lw[i]) = rw[i];
    };

    // fragment rows of this lane inside the tile
    const int frow = lane & 31, fhalf = lane >> 5;

    load_tile(0);
    store_lds(0);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) load_tile(kt + 1);
        const uint8_t* sa = smem + cur * C::STAGE;
        const uint8_t* sw = sa + BM * BK;
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk) {
            v4i af[C::TM], wf[C::TN];
#pragma unroll
            for (int im = 0; im < C::TM; ++im) {
                const int r = wm * C::WTM + im * 32 + frow;
                af[im] = *reinterpret_cast<const v4i*>(sa + r * BK + (swz<BK>(r, kk * 2 + fhalf) << 4));
            }
#pragma unroll
            for (int in = 0; in < C::TN; ++in) {
                const int r = wn * C::WTN + in * 32 + frow;
                wf[in] = *reinterpret_cast<const v4i*>(sw + r * BK + (swz<BK>(r, kk * 2 + fhalf) << 4));
            }
#pragma unroll
            for (int in = 0; in < C::TN; ++in)
#pragma unroll
                for (int im = 0; im < C::TM; ++im)
                    acc[in][im] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[in], af[im], acc[in][im], 0, 0, 0);
        }
        if (kt + 1 < nk) store_lds(cur ^ 1);
        __syncthreads();
    }

    static_assert(4 * 32 * C::WTN * 4 <= C::SMEM || C::NT != 256, "epilogue shuffle needs 4 pieces of LDS");
    epilogue<C::TM, C::TN, OUT_DT, EPI>(p, acc, m0 + wm * C::WTM, n0 + wn * C::WTN, lane, wave, smem);
}

// 16-byte global store the compiler's wait-count bookkeeping does not see (see the ring kernel's epilogue)
__device__ __forceinline__ void store16_untracked(void* ptr, uint4 v) {
    const v4i d = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
    // The trailing s_nop gives the two wait states this hardware needs between a store of more than 8 bytes and a
    // vector write to its data registers; the compiler inserts them for its own stores but cannot see into this one.
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(ptr), "v"(d) : "memory");
}
// The same with a scalar base and a 32-bit lane offset.
__device__ __forceinline__ void store16_untracked_at(const void* base, uint32_t off, uint4 v) {
    const v4i d = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
    asm volatile("global_store_dwordx4 %0, %1, %2 nt\n\ts_nop 1" ::"v"(off), "v"(d), "s"(base) : "memory");
}

template <int N> __device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
__device__ __forceinline__ void wg_barrier() { asm volatile("s_barrier" ::: "memory"); }
__device__ __forceinline__ void wait_lgkmcnt0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// ---------------------------------------------------------------------------------------------------------------
// The persistent ring kernel: one workgroup per CU walks its share of the 256x256 output tiles and keeps ONE
// global -> LDS pipeline running across all of them.  Tiles have 128-byte K rows (whole cache lines per DMA lane
// group).  LDS holds two stages of A (2 x 32 KB) and three of W (3 x 32 KB) = 160 KB: in iteration g the DMA fetches
// A of iteration g+1 (it must land before barrier Y of this iteration) and W of iteration g+2 (a full iteration of
// slack), so the last-issued loads of an iteration are never the ones the next wait needs.  Iterations number
// straight through tile boundaries: while the last K tiles of one output tile are multiplied, the first K tiles of
// the next one are already in flight, and the stores of an epilogue drain under the next tile's K loop.
//
// Per iteration (64 MFMAs per wave = four 32-deep sub-steps): barrier X (every wave is done with iteration g-1, whose
// stages are now free); sub-steps 0-2 with A DMA after MFMAs 0,3,..,21 and W DMA after MFMAs 24,28,..,52; vmcnt wait
// that leaves only this iteration's W DMA in flight; barrier Y; sub-step 3, which prefetches the first fragments of
// iteration g+1.  Requires K % 128 == 0 and M*K, N*K < 2^32.
// ---------------------------------------------------------------------------------------------------------------
template <int V> struct ic { static constexpr int value = V; };
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(ic<I>{});
        static_for<N, I + 1>(f);
    }
}

// BN: tile width; WGM x WGN: wave grid of four waves, one per SIMD (up to 512 registers each); NSA: LDS stages of A (2
// when a 256-wide tile leaves no room for a third in 160 KB of LDS; 3 where a narrower tile does).  W always has three
// stages.
template <int BN_, int WGM_, int WGN_, int NSA_, int BM_ = 256>
struct RingCfg {
    static constexpr int BM = BM_, BN = BN_, BK = 128, WGM = WGM_, WGN = WGN_, NW = WGM * WGN, NT = 64 * NW, NSA = NSA_, NSW = 3;
    static constexpr int WTM = BM / WGM, WTN = BN / WGN, TM = WTM / 32, TN = WTN / 32;
    static constexpr int A_LD = BM / (8 * NW), W_LD = BN / (8 * NW);   // DMA instructions per wave per stage (8 rows each)
    static constexpr int NDMA = A_LD + W_LD, NM = TM * TN, NF = TM + TN;
    static constexpr int A_STAGE = BM * BK, W_STAGE = BN * BK;
    static constexpr int W_BASE = NSA * A_STAGE;
    static constexpr int SMEM = NSA * A_STAGE + NSW * W_STAGE;
    static_assert(NW == 4 && BM % (32 * WGM) == 0 && BN % (32 * WGN) == 0 && BN % 32 == 0, "tile shape");
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "whole DMA blocks per wave");
    static_assert(NF <= NM && SMEM <= 160 * 1024, "fragment loads hide behind MFMAs; LDS fits");
    // Slot of the d-th DMA instruction of an iteration (A first, then W), as the number of the MFMA it follows; an
    // iteration has 4*NM MFMAs and barrier Y sits after MFMA 3*NM - 1.  With two A stages the A DMA is needed by this
    // iteration's barrier Y, so it goes first and dense (inside the first one and a half sub-steps); with three,
    // everything has an iteration of slack and is spread evenly.
    static constexpr int slot(int d) {
        return NSA == 2 ? (d < A_LD ? d * ((3 * NM) / (2 * A_LD)) : (3 * NM) / 2 + (d - A_LD) * ((4 * NM - (3 * NM) / 2 - 1) / W_LD))
                        : (d * 4 * NM) / NDMA;
    }
    // DMA instructions of this iteration that may still be in flight at barrier Y
    static constexpr int in_flight_at_y() {
        int n = 0;
        for (int d = (NSA == 2 ? A_LD : 0); d < NDMA; ++d) n += slot(d) < 3 * NM ? 1 : 0;
        return n;
    }
    static constexpr bool slots_ok() {
        for (int d = 0; d < NDMA; ++d) {
            if (slot(d) >= 4 * NM) return false;
            if (d > 0 && slot(d) <= slot(d - 1)) return false;
            if (NSA == 2 && d < A_LD && slot(d) >= 2 * NM) return false;
        }
        return true;
    }
    static_assert(slots_ok(), "DMA slots must be distinct, inside the iteration, and early for a two-stage A");
    // columns of one epilogue shuffle piece for an output element of SZ bytes: 128-byte LDS rows (four 16-byte vectors
    // per lane in flight between the read and the store half of a piece) where the wave tile's width allows
    static constexpr int piece_cols(int sz) { return WTN % (128 / sz) == 0 ? 128 / sz : 32; }
    // Epilogue scratch of one wave inside a stage that was just multiplied: a shuffle piece in each of an A and a W
    // stage; the wave's column constants (2 x WTN floats) sit behind the piece in the W stage.
    static constexpr bool STAGED = true;
    static constexpr int A_REGION = A_STAGE / NW, W_REGION = W_STAGE / NW;
    static constexpr int piece_bytes(int sz) { return 32 * piece_cols(sz) * sz; }
    static constexpr bool scratch_ok(int sz) {
        return piece_bytes(sz) <= A_REGION && piece_bytes(sz) + (STAGED ? 2 * WTN * 4 : 0) <= W_REGION;
    }
    static_assert(scratch_ok(2) && scratch_ok(4), "epilogue scratch fits the stages");
};

template <class C, int OUT_DT, int EPI>
__global__ void __launch_bounds__(C::NT, 1) int8_gemm_ring_kernel(GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int BK = C::BK, TM = C::TM, TN = C::TN, NM = C::NM, NF = C::NF, NSA = C::NSA;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / C::WGN, wn = wave % C::WGN;
    const int ld = p.K;                                  // row stride of A and W
    // split K: workgroup row blockIdx.y multiplies K slice [k_lo, k_lo + nk*128) and writes its own int32 plane
    const int k_lo = p.kslice ? (int)blockIdx.y * p.kslice : 0;
    const int k_len = p.kslice ? (p.K - k_lo < p.kslice ? p.K - k_lo : p.kslice) : p.K;
    const int nk = k_len / BK;
    if (p.kslice) p.D = (uint8_t*)p.D + (int64_t)blockIdx.y * p.M * p.N * 4;
    const int8_t* Ab = p.A + k_lo;
    const int8_t* Wb = p.W + k_lo;
    const int G = gridDim.x, ntiles = p.tiles_m * p.tiles_n;
    const int nt_b = (ntiles - (int)blockIdx.x + G - 1) / G;   // tiles of this workgroup: blockIdx, blockIdx + G, ...

    auto tile_origin = [&](int i, int& m0, int& n0) {
        int tm, tn;
        tile_of_block((int)blockIdx.x + i * G, ntiles, p.tiles_m, p.tiles_n, tm, tn, p.magic);
        m0 = tm * C::BM;
        n0 = tn * C::BN;
    };

    // DMA streams.  Each walks (tile, K tile) pairs in the order the MFMAs will consume them and stops on the last one
    // (re-fetching it into a stage nothing reads again keeps the loop free of branches around the DMA slots).
    // rows come in blocks of 8 (block index wave + NW*j has the parity of wave): swz<128> of the row
    uint32_t ga[C::A_LD], gw[C::W_LD];
    int a_tile = 0, a_kt = 0, a_stage = 0, w_tile = 0, w_kt = 0, w_stage = 0;
    // The row and chunk of a lane are recomputed from the hardware lane number each time a stream moves to its next
    // tile: as loop invariants the compiler would keep sixteen of them live across the K loop, spill them, and reload
    // them here behind full memory waits that drain the DMA pipeline (a spilled copy of the lane number does the same).
    auto set_a = [&](int i) {
        int m0, n0;
        tile_origin(i, m0, n0);
        const int l = hw_lane();
        const int lr = l >> 3, lc = ((l & 7) ^ (((wave & 1) << 2) | (lr >> 1))) * 16;
#pragma unroll
        for (int j = 0; j < C::A_LD; ++j) {
            const int row = (wave + C::NW * j) * 8 + lr;
            const int gr = m0 + row < p.M ? m0 + row : p.M - 1;
            ga[j] = (uint32_t)gr * (uint32_t)ld + lc;
        }
    };
    auto set_w = [&](int i) {
        int m0, n0;
        tile_origin(i, m0, n0);
        const int l = hw_lane();
        const int lr = l >> 3, lc = ((l & 7) ^ (((wave & 1) << 2) | (lr >> 1))) * 16;
#pragma unroll
        for (int j = 0; j < C::W_LD; ++j) {
            const int row = (wave + C::NW * j) * 8 + lr;
            const int gr = n0 + row < p.N ? n0 + row : p.N - 1;
            gw[j] = (uint32_t)gr * (uint32_t)ld + lc;
        }
    };
    // The DMA is written as inline assembly: through the builtin the compiler, unable to prove that a fragment read and
    // an in-flight DMA touch different stages, puts a full vmcnt(0) wait in front of the fragment reads, which serializes
    // the whole pipeline.  Ordering is kept by hand instead (wait_vmcnt + barriers).  scalar base + 32-bit lane offset.
    const uint32_t lds_base = (uint32_t)(uintptr_t)smem;   // LDS byte address of the dynamic segment
    auto dma_a = [&](int j) {
        const int8_t* base = Ab + (int64_t)a_kt * BK;
        const uint32_t dst = lds_base + a_stage * C::A_STAGE + (wave + C::NW * j) * 1024;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(ga[j]), "s"(base) : "memory", "m0");
    };
    auto dma_w = [&](int j) {
        const int8_t* base = Wb + (int64_t)w_kt * BK;
        const uint32_t dst = lds_base + C::W_BASE + w_stage * C::W_STAGE + (wave + C::NW * j) * 1024;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(gw[j]), "s"(base) : "memory", "m0");
    };
    auto advance_a = [&]() {
        a_stage = a_stage == NSA - 1 ? 0 : a_stage + 1;
        if (a_tile == nt_b - 1 && a_kt == nk - 1) return;
        if (++a_kt == nk) { a_kt = 0; set_a(++a_tile); }
    };
    auto advance_w = [&]() {
        w_stage = w_stage == C::NSW - 1 ? 0 : w_stage + 1;
        if (w_tile == nt_b - 1 && w_kt == nk - 1) return;
        if (++w_kt == nk) { w_kt = 0; set_w(++w_tile); }
    };

    // fragment addresses inside a stage: row r at r*128, chunk c at slot c ^ ((r>>1)&7); K sub-step kk flips bits 5 and 6
    const int frow = lane & 31, fhalf = lane >> 5;
    const int fsw = (fhalf ^ ((frow >> 1) & 7)) << 4;
    int aoff[4], woff[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        aoff[kk] = ((wm * C::WTM + frow) * BK + fsw) ^ (kk << 5);
        woff[kk] = ((wn * C::WTN + frow) * BK + fsw) ^ (kk << 5);
    }
    auto frag = [&](const uint8_t* sa, const uint8_t* sw, int kk, int j) -> v4i {
        if (j < TM) return *reinterpret_cast<const v4i*>(sa + aoff[kk] + j * 32 * BK);
        return *reinterpret_cast<const v4i*>(sw + woff[kk] + (j - TM) * 32 * BK);
    };

    v16i acc[TN][TM];
    v4i f0[NF], f1[NF];

    // One sub-step: NM MFMAs on `cur`; the NF fragment loads of the next sub-step ride behind the first MFMAs; DMA
    // instructions sit in their slots (this sub-step's MFMAs are numbers BASE .. BASE + NM - 1 of the iteration).
    auto substep = [&](auto BASE, v4i* cur, v4i* nxt, const uint8_t* sa_n, const uint8_t* sw_n, int kk_n) {
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            const int in = i / TM, im = i % TM;
            acc[in][im] = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur[TM + in], cur[im], acc[in][im], 0, 0, 0);
            SCHED_FENCE();
#pragma unroll
            for (int d = 0; d < C::NDMA; ++d) {
                if (C::slot(d) == decltype(BASE)::value + i) {
                    if (d < C::A_LD) dma_a(d);
                    else dma_w(d - C::A_LD);
                    SCHED_FENCE();
                }
            }
            if (i < NF) { nxt[i] = frag(sa_n, sw_n, kk_n, i); SCHED_FENCE(); }
        }
    };

    // prologue: A(0), W(0), [A(1),] W(1) in flight; A(0) and W(0) must land
    set_a(0);
    set_w(0);
#pragma unroll
    for (int j = 0; j < C::A_LD; ++j) dma_a(j);
    advance_a();
#pragma unroll
    for (int j = 0; j < C::W_LD; ++j) dma_w(j);
    advance_w();
    if (NSA == 3) {
#pragma unroll
        for (int j = 0; j < C::A_LD; ++j) dma_a(j);
        advance_a();
    }
#pragma unroll
    for (int j = 0; j < C::W_LD; ++j) dma_w(j);
    advance_w();
    wait_vmcnt<(NSA == 3 ? C::A_LD : 0) + C::W_LD>();
    wg_barrier();
#pragma unroll
    for (int j = 0; j < NF; ++j) f0[j] = frag(smem, smem + C::W_BASE, 0, j);

    int ca = 0, cw = 0;   // stages of the iteration being multiplied
    for (int ti = 0; ti < nt_b; ++ti) {
#pragma unroll
        for (int in = 0; in < TN; ++in)
#pragma unroll
            for (int im = 0; im < TM; ++im)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[in][im][r] = 0;
        // The epilogue's stores are issued from inline assembly: were they visible to the compiler, it would assume
        // them pending at the K loop's header and park a vmcnt(0) inside the loop, in front of the first fragment read,
        // draining the DMA pipeline every iteration.  (Waits it derives for its own loads stay correct: the memory
        // counter retires in order, so instructions it does not know about only make those waits stricter.)

        int pa = 0, pw = 0;
        for (int kt = 0; kt < nk; ++kt) {
            const uint8_t* sa = smem + ca * C::A_STAGE;
            const uint8_t* sw = smem + C::W_BASE + cw * C::W_STAGE;
            const int na = ca == NSA - 1 ? 0 : ca + 1, nw = cw == C::NSW - 1 ? 0 : cw + 1;
            wg_barrier();                                                   // X
            substep(ic<0>{}, f0, f1, sa, sw, 1);
            substep(ic<NM>{}, f1, f0, sa, sw, 2);
            substep(ic<2 * NM>{}, f0, f1, sa, sw, 3);
            wait_vmcnt<C::in_flight_at_y()>();
            wg_barrier();                                                   // Y
            substep(ic<3 * NM>{}, f1, f0, smem + na * C::A_STAGE, smem + C::W_BASE + nw * C::W_STAGE, 0);
            advance_a();
            advance_w();
            pa = ca;
            pw = cw;
            ca = na;
            cw = nw;
        }

        // epilogue of tile ti; the A stage that was just multiplied is the shuffle scratch (8 KB per wave).
        // (The launcher only picks this kernel when the coalesced epilogue's alignment conditions hold.)
        int m0, n0;
        tile_origin(ti, m0, n0);
        __syncthreads();   // every wave is done reading that stage
        constexpr int SZ = (EPI == EPI_ACC || OUT_DT == DT_F32) ? 4 : 2;
        constexpr int PW = C::piece_cols(SZ);
        // Shuffle scratch, 8 KB per wave and region: the A stage and the W stage that were just multiplied (the DMA in
        // flight fills the other stages; the next write into these two is issued inside the next iteration).
        uint8_t* ra = smem + pa * C::A_STAGE + wave * C::A_REGION;
        uint8_t* rw = smem + C::W_BASE + pw * C::W_STAGE + wave * C::W_REGION;
        epilogue_shuffle<TM, TN, OUT_DT, EPI, PW, true, C::STAGED>(p, acc, m0 + wm * C::WTM, n0 + wn * C::WTN, hw_lane(), ra, rw,
                                                               reinterpret_cast<float*>(rw + C::piece_bytes(SZ)));
        // The first fragments of the next tile were prefetched by the last sub-step; fetching them again here instead of
        // carrying 32 registers across the epilogue keeps the epilogue free of spills.
#pragma unroll
        for (int j = 0; j < NF; ++j) f0[j] = frag(smem + ca * C::A_STAGE, smem + C::W_BASE + cw * C::W_STAGE, 0, j);
    }
    wait_vmcnt<0>();   // no DMA may still be writing this workgroup's LDS when it retires
}

// ---------------------------------------------------------------------------------------------------------------
// The two-group persistent kernel for large shapes.  A global_load_lds_dwordx4 keeps the wave that issues it busy for
// about 68 cycles (measured: one wave alone, 16 of them back to back, 1088 cycles), twice the 32 cycles of a
// v_mfma_i32_32x32x32_i8, so a wave that issues its own DMA between its MFMAs leaves the matrix pipe of its SIMD idle
// for part of each one.  Here a workgroup has eight waves, two per SIMD, in two groups of four: group g owns rows
// 128g..128g+127 of a 256x256 tile (wave tiles 128x64).  The groups alternate between two kinds of phase, with one
// workgroup barrier between phases:
//   compute: the 64 MFMAs (16x16x64, 16 cycles each) of one 128-deep K step, on fragments already in registers, and
//            nothing else;
//   memory:  the 24 fragment reads of the group's next K step and 8 DMA instructions per wave.
// While one wave of a SIMD is in its memory phase the other is in its compute phase, so the matrix pipe always has an
// MFMA to run and no MFMA waits behind a DMA.
//
// LDS (160 KB): three 32 KB stages of W (both groups read them) and two 16 KB stages of A for each group.  With global
// step s = tile * nk + k tile, group 0 computes step s in phase 2s and group 1 in phase 2s + 1.  Group 0's memory phase
// before step s fetches A of group 1 for step s + 1 and rows 0..127 of W for step s + 2; group 1's fetches A of group 0
// and rows 128..255 of W, both for step s + 2.  Every memory phase ends with a wait that leaves only its own 8 DMA
// instructions in flight, so what a phase fetches is visible to everybody two phases later, and each stage is refilled
// only after the barrier that follows its last reader.  Steps run straight through tile boundaries.
//
// End of a tile: group 0 runs its epilogue while group 1 multiplies its last step and then runs its own; the shuffle
// scratch is the W stage of that step (4 KB per wave), which no DMA in flight targets.  Group 0 follows its epilogue with
// the memory phase of the next tile's first step (under group 1's epilogue), one barrier, and the alternation resumes
// with group 0 multiplying.
// Requires K % 128 == 0, M*K and N*K < 2^32, and the coalesced epilogue's alignment.
// ---------------------------------------------------------------------------------------------------------------
// GM: rows of a group.  128 gives the 256x256 tile (wave tiles 128x64); 64 gives a 128x256 tile (wave tiles 64x64) for
// the rows a whole number of rounds of the large tile leaves over: half the work per tile, so the last, partly filled
// round costs half as much, at a step that is bound by its 6 DMA instructions per wave rather than by its 16 MFMAs.
template <int GM_>
struct PpCfg {
    static constexpr int GM = GM_, BM = 2 * GM, BN = 256, BK = 128, NT = 512;
    static constexpr int TM = GM / 32, TN = 2, WTN = 64;                            // wave tile GM x 64
    static constexpr int W_STAGE = BN * BK, A_STAGE = GM * BK, NSW = 3, NSA = 2;
    static constexpr int A_BASE = NSW * W_STAGE;                                    // group g's A ring at A_BASE + g*NSA*A_STAGE
    static constexpr int SMEM = NSW * W_STAGE + 2 * NSA * A_STAGE;
    static constexpr int NLA = GM / 32, NLW = 4;       // DMA instructions per wave for a group's A half / a 128-row W half
    static_assert(GM % 32 == 0 && SMEM <= 160 * 1024, "tile shape; LDS fits");
    static constexpr int piece_cols(int sz) { return sz == 2 ? 64 : 32; }           // 4 KB shuffle pieces
};
using PpL = PpCfg<128>;
using PpS = PpCfg<64>;

// The work of workgroup `bid` of `G` on problem p.
template <class C, int OUT_DT, int EPI>
__device__ __forceinline__ void pp_gemm_tiles(const GemmArgs& p, uint8_t* smem, const int bid, const int G) {
    constexpr int BK = C::BK, TM = C::TM, TN = C::TN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, wq = wave & 3;            // group; wave within the group = its column quarter
    const int ld = p.K, nk = p.K / BK;
    const int ntiles = p.tiles_m * p.tiles_n;
    const int nt_b = (ntiles - bid + G - 1) / G;         // tiles of this workgroup: bid, bid + G, ...
    const int S = nt_b * nk;                             // steps of this workgroup
    auto tile_origin = [&](int i, int& m0, int& n0) {
        int tm, tn;
        tile_of_block(bid + i * G, ntiles, p.tiles_m, p.tiles_n, tm, tn, p.magic);
        m0 = tm * C::BM;
        n0 = tn * C::BN;
    };
    const uint32_t lds_base = (uint32_t)(uintptr_t)smem;
    auto dma = [&](uint32_t dst, uint32_t off, const int8_t* base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(base) : "memory", "m0");
    };

    // DMA streams of this wave.  A wave fetches 8-row blocks wq, wq + 4, ... of the OTHER group's A rows and of its own
    // half of the W tile (group 0: rows 0..127, group 1: rows 128..255).
    // Lane offsets carry the chunk swizzle (bits 1..3 of the row) on the global side, as in the ring kernel.
    uint32_t ga[C::NLA], gw[C::NLW];
    // a stream's position: the (tile, k tile) it fetches next and the stage that goes to.  A stream stops on the last step
    // and keeps re-fetching it, into the stage it would have used, which nothing reads again.
    int a_tile, a_kt, a_stage, w_tile = 0, w_kt = 0, w_stage = 0;
    auto set_rows = [&](uint32_t* g, auto n, int origin, int limit) {
        const int l = hw_lane();
        const int lr = l >> 3, lc = ((l & 7) ^ (((wq & 1) << 2) | (lr >> 1))) * 16;
#pragma unroll
        for (int j = 0; j < decltype(n)::value; ++j) {
            const int row = origin + (wq + 4 * j) * 8 + lr;
            g[j] = (uint32_t)(row < limit ? row : limit - 1) * (uint32_t)ld + lc;
        }
    };
    auto set_a = [&](int tile) { int m0, n0; tile_origin(tile, m0, n0); set_rows(ga, ic<C::NLA>{}, m0 + (grp ^ 1) * C::GM, p.M); };
    // W: a wave fetches the four CONSECUTIVE 8-row blocks 4*wq .. 4*wq + 3 of its group's half, which are exactly the 4 KB
    // of the stage that serve as this wave's shuffle scratch in the epilogue: group 0 may then refill the stage right
    // after its own epilogue, while other waves are still in theirs.  (A block's parity, which the swizzle needs, is j's.)
    auto set_w = [&](int tile) {
        int m0, n0;
        tile_origin(tile, m0, n0);
        const int l = hw_lane();
        const int lr = l >> 3;
#pragma unroll
        for (int j = 0; j < C::NLW; ++j) {
            const int row = n0 + grp * 128 + (4 * wq + j) * 8 + lr;
            const int lc = ((l & 7) ^ (((j & 1) << 2) | (lr >> 1))) * 16;
            gw[j] = (uint32_t)(row < p.N ? row : p.N - 1) * (uint32_t)ld + lc;
        }
    };
    auto fetch_a = [&]() {
        const int8_t* base = p.A + (int64_t)a_kt * BK;
        const uint32_t dst = lds_base + C::A_BASE + ((grp ^ 1) * C::NSA + a_stage) * C::A_STAGE + wq * 1024;
#pragma unroll
        for (int j = 0; j < C::NLA; ++j) dma(dst + j * 4096, ga[j], base);
        a_stage = a_stage == C::NSA - 1 ? 0 : a_stage + 1;
        if (a_tile == nt_b - 1 && a_kt == nk - 1) return;
        if (++a_kt == nk) { a_kt = 0; set_a(++a_tile); }
    };
    auto fetch_w = [&]() {
        const int8_t* base = p.W + (int64_t)w_kt * BK;
        const uint32_t dst = lds_base + w_stage * C::W_STAGE + grp * 128 * BK + wq * 4096;
#pragma unroll
        for (int j = 0; j < C::NLW; ++j) dma(dst + j * 1024, gw[j], base);
        w_stage = w_stage == C::NSW - 1 ? 0 : w_stage + 1;
        if (w_tile == nt_b - 1 && w_kt == nk - 1) return;
        if (++w_kt == nk) { w_kt = 0; set_w(++w_tile); }
    };

    // The tiles are multiplied with v_mfma_i32_16x16x64_i8: as many operations per cycle as the 32x32x32 form and the same
    // fragment bytes per K, but an accumulator is touched once per 64 K instead of once per 32.  On this power-limited
    // part that is worth clock: a loop of nothing but MFMAs on random bits sustains 3.95 POP/s in this form against 3.4,
    // and this kernel ran 9-11 % faster with it.  A wave tile is FM x FN tiles of 16 x 16, four accumulator registers each.
    // Fragment addresses inside a stage: row r at r*128, chunk c at slot c ^ ((r>>1)&7); a lane reads row lane % 16,
    // chunk 4*kk + lane / 16 of K half kk (which flips bit 6).
    constexpr int FM = 2 * TM, FN = 2 * TN;
    v4i acc[FN][FM];
    v4i f[2][FM + FN];
    int ra_stage = 0, rw_stage = 0;   // stages this group's next fragments come from
    auto load_frags = [&]() {
        const int l = hw_lane();
        const int frow = l & 15, fq = l >> 4;
        const int x = frow * BK + ((fq ^ ((frow >> 1) & 7)) << 4);
        const uint8_t* sa = smem + C::A_BASE + (grp * C::NSA + ra_stage) * C::A_STAGE;
        const uint8_t* sw = smem + rw_stage * C::W_STAGE + wq * C::WTN * BK;
        ra_stage = ra_stage == C::NSA - 1 ? 0 : ra_stage + 1;
        rw_stage = rw_stage == C::NSW - 1 ? 0 : rw_stage + 1;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int xk = x ^ (kk << 6);
#pragma unroll
            for (int j = 0; j < FM; ++j) f[kk][j] = *reinterpret_cast<const v4i*>(sa + xk + j * 16 * BK);
#pragma unroll
            for (int j = 0; j < FN; ++j) f[kk][FM + j] = *reinterpret_cast<const v4i*>(sw + xk + j * 16 * BK);
        }
    };
    // a tile's first MFMAs take C = 0 instead of cleared accumulators
    auto compute = [&](bool first) {
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int in = 0; in < FN; ++in)
#pragma unroll
                for (int im = 0; im < FM; ++im) {
                    const v4i c = (first && kk == 0) ? v4i{0, 0, 0, 0} : acc[in][im];
                    acc[in][im] = __builtin_amdgcn_mfma_i32_16x16x64_i8(f[kk][FM + in], f[kk][im], c, 0, 0, 0);
                    SCHED_FENCE();
                }
        __builtin_amdgcn_s_setprio(0);
    };
    // memory phase before this group's next step
    auto memory = [&]() {
        load_frags();
        SCHED_FENCE();
        fetch_a();
        fetch_w();
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(C::NLA + C::NLW) : "memory");   // everything but this phase's own DMA has landed
    };

    // prologue: every group fetches its OWN A for step 0 (group 0 also for step 1: group 1's first memory phase fetches
    // A0 of step 2) and its half of W for steps 0 and 1; then the streams move to where the memory phases expect them
    {
        int m0, n0;
        const int own_a = C::A_BASE + grp * C::NSA * C::A_STAGE;
        const int t1 = (nk == 1 && nt_b > 1) ? 1 : 0, k1 = nk > 1 ? 1 : 0;   // step 1 as (tile, k tile); step 0 again if S == 1
        tile_origin(0, m0, n0);
        set_rows(ga, ic<C::NLA>{}, m0 + grp * C::GM, p.M);
#pragma unroll
        for (int j = 0; j < C::NLA; ++j) dma(lds_base + own_a + (wq + 4 * j) * 1024, ga[j], p.A);
        if (grp == 0) {
            if (t1) { tile_origin(1, m0, n0); set_rows(ga, ic<C::NLA>{}, m0, p.M); }
#pragma unroll
            for (int j = 0; j < C::NLA; ++j) dma(lds_base + own_a + C::A_STAGE + (wq + 4 * j) * 1024, ga[j], p.A + (int64_t)k1 * BK);
        }
        set_w(0);
        fetch_w();
        fetch_w();
        // the A stream of the OTHER group's tile: group 0 starts at step 1, group 1 at step 2 (clamped to the last step)
        int st = grp == 0 ? 1 : 2;
        a_stage = st % C::NSA;
        if (st > S - 1) st = S - 1;
        a_tile = st / nk;
        a_kt = st - a_tile * nk;
        set_a(a_tile);
        wait_vmcnt<0>();
        wg_barrier();
    }

    constexpr int SZ = (EPI == EPI_ACC || OUT_DT == DT_F32) ? 4 : 2;
    constexpr int PW = C::piece_cols(SZ);
    auto run_epilogue = [&](int ti, int s_last) {
        int m0, n0;
        tile_origin(ti, m0, n0);
        uint8_t* scratch = smem + (s_last % C::NSW) * C::W_STAGE + wave * 4096;
        epilogue_shuffle<TM, TN, OUT_DT, EPI, PW, true, false, 16>(p, acc, m0 + grp * C::GM, n0 + wq * C::WTN, hw_lane(), scratch);
    };

    // Both groups run the same loop; group 1 is one phase behind (the barrier in front) and multiplies its last step of a
    // tile in the phase in which group 0 already runs its epilogue.  Group 0 goes from its epilogue straight into the
    // memory phase of the next tile's first step, while group 1 is still in its epilogue: what that phase reads landed
    // before the tile's last compute phases, and what it fetches goes to stages that neither epilogue uses (group 1's A
    // stage of the step before last, and the half of the last step's W stage that was group 0's own shuffle scratch).
    // After the one barrier that follows the epilogues group 0 multiplies at once and the alternation is back.
    if (grp == 1) wg_barrier();
    int s = 0;
    for (int ti = 0; ti < nt_b; ++ti) {
        for (int kt = 0; kt < nk; ++kt, ++s) {
            memory();
            wait_lgkmcnt0();
            wg_barrier();
            compute(kt == 0);
            if (grp == 0 || kt + 1 < nk) wg_barrier();
        }
        run_epilogue(ti, s - 1);
        // the barrier behind the epilogues; group 0 meets it after the next tile's first memory phase (the loop's first
        // barrier), so it skips this one when a tile follows
        if (grp == 1 || ti + 1 == nt_b) wg_barrier();
    }
    wait_vmcnt<0>();   // no DMA may still be writing this workgroup's LDS when it retires
}

// Workgroups 0 .. g_main-1 walk the 256x256 tiles of `main`; the rest walk the 128x256 tiles of `rest` (the rows that
// whole rounds of large tiles leave over, or nothing).  One launch: the hardware starts a workgroup of the second kind
// on each CU as its workgroup of the first kind retires, with no gap between two launches.
template <int OUT_DT, int EPI>
__global__ void __launch_bounds__(PpL::NT, 1) int8_gemm_pp_kernel(GemmArgs main, GemmArgs rest, int g_main) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int bid = (int)blockIdx.x;
    if (bid < g_main) pp_gemm_tiles<PpL, OUT_DT, EPI>(main, smem, bid, g_main);
    else pp_gemm_tiles<PpS, OUT_DT, EPI>(rest, smem, bid - g_main, (int)gridDim.x - g_main);
}

// ---------------------------------------------------------------------------------------------------------------
// Weight-streaming kernel for skinny M (M <= 256): one row of 256 x 96 tiles, every weight read from HBM exactly once.
// Eight waves form two groups of four (one wave of each group per SIMD), and group g multiplies the K tiles
// t = g, g + 2, ... of the workgroup's K range, all 256 x 96 outputs of them (wave tile 64 x 96, 4 x 6 tiles of
// v_mfma_i32_16x16x64_i8), into accumulators of its own.  The groups alternate between two kinds of phase, with one
// workgroup barrier per phase:
//   compute: the 48 MFMAs of the group's K tile; the six W fragments of the second 64 K bytes are read behind the
//            first MFMAs, and the wave's three DMA instructions of W follow the last one;
//   memory:  the other 14 fragment reads of the group's next K tile with the wave's eight DMA instructions of A spread
//            between them.
// A group fetches only the K tiles it multiplies itself, so every wait for data is a wait of a wave on its own memory
// counter, placed at the end of its compute phase.
//
// LDS: A in three stages of 32 KB, W in five of 12 KB (K tile t sits in stage t % 3 and t % 5), 2 KB of constants for the
// epilogue.  In its memory phase before K tile t a group fetches A(t+2) into the stage of K tile t-1, whose fragments
// the other group read a phase earlier; after multiplying K tile t it fetches W(t+4) into the W stage of K tile t-1,
// whose second half the other group read during that earlier phase.  W, which comes from HBM, has three phases to land;
// A, which comes from L2 behind it in the CU's in-order return path, has one and a half.
//
// What bounds this tile is how much a CU can keep in flight: 44 KB enter it per K tile, a third of them at HBM's
// latency, and a kernel of any structure built on this tile (separate loader waves in lock step or free-running on LDS
// counters, loads in registers instead of DMA) ran its K tile in the same 1350-1450 cycles.
//
// At the end the two groups swap halves of their accumulators through the LDS (the ring is dead by then) and each
// finishes 32 of a wave tile's 64 rows; the tile's column constants and row scales were requested at the start and wait
// in LDS.  Requires K % 128 == 0 and M*K, N*K < 2^32.
// ---------------------------------------------------------------------------------------------------------------
struct TurnCfg {
    static constexpr int BM = 256, BN = 96, BK = 128, NSA = 3, NSW = 5, NT = 512;
    static constexpr int TM = 2, TN = 3;                                       // wave tile 64 x 96 as 32 x 32 blocks
    static constexpr int A_STAGE = BM * BK, W_STAGE = BN * BK, W_BASE = NSA * A_STAGE;
    static constexpr int NLA = BM / 32, NLW = BN / 32;                         // DMA instructions (8 rows each) per wave and K tile
    static constexpr int RING = W_BASE + NSW * W_STAGE;
    static constexpr int CST_BASE = RING, CST_FLOATS = 2 * BN + BM, SMEM = RING + 2048;   // ws[96], bias[96], xs[256] as floats
    static constexpr int HALF_ACC = 2 * TM * TN * 1024;                        // half of one wave's accumulators
    static_assert(SMEM <= 160 * 1024 && CST_FLOATS * 4 <= 2048, "LDS budget");
    static_assert(8 * HALF_ACC <= W_BASE && 8 * 4096 <= NSW * W_STAGE, "hand-over area and epilogue scratch fit the dead ring");
};

template <int OUT_DT, int EPI>
__global__ void __launch_bounds__(TurnCfg::NT, 1) int8_gemm_turn_kernel(GemmArgs p) {
    using C = TurnCfg;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int BK = C::BK, TM = C::TM, TN = C::TN, FM = 2 * TM, FN = 2 * TN;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int grp = wave >> 2, wq = wave & 3;   // group; wave within the group = its 64-row quarter and its DMA blocks
    const int ld = p.K;
    // split K: workgroup row blockIdx.y multiplies K slice [k_lo, k_lo + nk*128) and writes its own int32 plane
    const int k_lo = p.kslice ? (int)blockIdx.y * p.kslice : 0;
    const int k_len = p.kslice ? (p.K - k_lo < p.kslice ? p.K - k_lo : p.kslice) : p.K;
    const int nk = k_len / BK;
    if (p.kslice) p.D = (uint8_t*)p.D + (int64_t)blockIdx.y * p.M * p.N * 4;
    const int G = gridDim.x, ntiles = p.tiles_m * p.tiles_n;
    const int nt_b = (ntiles - (int)blockIdx.x + G - 1) / G;   // tiles of this workgroup: blockIdx, blockIdx + G, ...
    // The K tiles are walked from a start that differs between the workgroups of an XCD (the int32 sums do not depend
    // on the order), so that they do not all ask that XCD's L2 for the same lines of A at the same moment.
    const int rot = (int)(((blockIdx.x >> 3) & 31) * (unsigned)nk) >> 5;
    auto rk = [&](int kt) { kt = kt < nk ? kt : nk - 1; return kt + rot < nk ? kt + rot : kt + rot - nk; };
    const uint32_t lds_base = (uint32_t)(uintptr_t)smem;
    auto dma = [&](uint32_t dst, uint32_t off, const int8_t* base) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(base) : "memory", "m0");
    };

    // DMA streams of this wave: 8-row blocks wq, wq + 4, ... of the A tile and of the W tile, of this group's K tiles.
    // The chunk swizzle (bits 1..3 of the row) is applied on the global side; a block's parity is the wave's.
    // (Giving W to one wave of the group and A to the other three, so that no wave's A loads queue behind its own W
    // loads, was measured and is slower: what A waits behind is the CU's return path, not the wave's counter.)
    uint32_t ga[C::NLA], gw[C::NLW];
    auto set_rows = [&](int m0, int n0) {
        const int l = hw_lane();
        const int lr = l >> 3, lc = ((l & 7) ^ (((wq & 1) << 2) | (lr >> 1))) * 16;
#pragma unroll
        for (int j = 0; j < C::NLA; ++j) {
            const int row = m0 + (wq + 4 * j) * 8 + lr;
            ga[j] = (uint32_t)(row < p.M ? row : p.M - 1) * (uint32_t)ld + lc;
        }
#pragma unroll
        for (int j = 0; j < C::NLW; ++j) {
            const int row = n0 + (wq + 4 * j) * 8 + lr;
            gw[j] = (uint32_t)(row < p.N ? row : p.N - 1) * (uint32_t)ld + lc;
        }
    };
    // K tile and stage each stream fetches next (a stream past the last K tile re-fetches it, into a stage that nothing
    // reads again: the number of instructions per phase, which the wait counts assume, stays fixed)
    int a_t, a_st, w_t, w_st, r_sa, r_sw;
    // source and destination of the A blocks a memory phase fetches
    const int8_t* base_a;
    uint32_t dst_a;
    auto fetch_one = [&](auto D) { dma(dst_a + decltype(D)::value * 4096, ga[decltype(D)::value], base_a); };
    auto fetch_w = [&]() {
        const int8_t* base = p.W + k_lo + (int64_t)rk(w_t) * BK;
        const uint32_t dst = lds_base + C::W_BASE + w_st * C::W_STAGE + wq * 1024;
#pragma unroll
        for (int j = 0; j < C::NLW; ++j) dma(dst + j * 4096, gw[j], base);
        w_t += 2;
        w_st = w_st >= 3 ? w_st - 3 : w_st + 2;
    };
    auto fetch_a = [&]() {
        const int8_t* base = p.A + k_lo + (int64_t)rk(a_t) * BK;
        const uint32_t dst = lds_base + a_st * C::A_STAGE + wq * 1024;
#pragma unroll
        for (int j = 0; j < C::NLA; ++j) dma(dst + j * 4096, ga[j], base);
        a_t += 2;
        a_st = a_st == 0 ? 2 : a_st - 1;
    };

    // Fragments: row r of a stage at r*128, chunk c at slot c ^ ((r>>1)&7); a lane reads row lane % 16, chunk
    // 4*kk + lane / 16 of K half kk (which flips bit 6 of the address).
    v4i acc[FN][FM];
    v4i f[2][FM + FN];
    // The memory phase: 14 fragment reads of the group's next K tile (all of A, and W for the first 64 K bytes) with the
    // wave's 8 DMA instructions of A spread between them.  The six W fragments of the second 64 K bytes are read in the
    // compute phase, behind the first MFMAs, and the three DMA instructions of W follow the last MFMA: a compute phase
    // (768 cycles of MFMA) would otherwise be a third shorter than the memory phase beside it, whose reads return at the
    // SIMD's pace of about 25 cycles each and whose DMA instructions hold the wave about 50 cycles each.  W can move
    // because its ring has the room (a stage stays readable for one phase more), A cannot.
    const uint8_t* sw_cur = smem;   // W stage of the K tile whose fragments are in registers (its second half still in LDS)
    int fx = 0;
    auto memory = [&]() {
        constexpr int ND = C::NLA;
        const int l = hw_lane();
        const int frow = l & 15, fq = l >> 4;
        const int x = frow * BK + ((fq ^ ((frow >> 1) & 7)) << 4);
        const uint8_t* sa = smem + r_sa * C::A_STAGE + wq * 64 * BK;
        const uint8_t* sw = smem + C::W_BASE + r_sw * C::W_STAGE;
        sw_cur = sw;
        fx = x ^ 64;
        r_sa = r_sa == 0 ? 2 : r_sa - 1;
        r_sw = r_sw >= 3 ? r_sw - 3 : r_sw + 2;
        base_a = p.A + k_lo + (int64_t)rk(a_t) * BK;
        dst_a = lds_base + a_st * C::A_STAGE + wq * 1024;
        a_t += 2;
        a_st = a_st == 0 ? 2 : a_st - 1;            // + 2 mod 3
        constexpr int NF = 2 * FM + FN;
        static_for<NF>([&](auto I) {
            constexpr int i = decltype(I)::value;
            if constexpr (i < FM) f[0][i] = *reinterpret_cast<const v4i*>(sa + x + i * 16 * BK);
            else if constexpr (i < FM + FN) f[0][i] = *reinterpret_cast<const v4i*>(sw + x + (i - FM) * 16 * BK);
            else f[1][i - FM - FN] = *reinterpret_cast<const v4i*>(sa + (x ^ 64) + (i - FM - FN) * 16 * BK);
            SCHED_FENCE();
            // DMA instruction d goes behind read (d * NF) / ND + 1
            static_for<ND>([&](auto D) {
                if constexpr ((decltype(D)::value * NF) / ND + 1 == i) { fetch_one(D); SCHED_FENCE(); }
            });
        });
        static_for<ND>([&](auto D) {
            if constexpr ((decltype(D)::value * NF) / ND + 1 >= NF) { fetch_one(D); SCHED_FENCE(); }
        });
    };
    auto compute = [&]() {
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int in = 0; in < FN; ++in)
#pragma unroll
            for (int im = 0; im < FM; ++im) {
                acc[in][im] = __builtin_amdgcn_mfma_i32_16x16x64_i8(f[0][FM + in], f[0][im], acc[in][im], 0, 0, 0);
                SCHED_FENCE();
                if (im == 1) {   // one W fragment of the second half behind every fourth MFMA
                    f[1][FM + in] = *reinterpret_cast<const v4i*>(sw_cur + fx + in * 16 * BK);
                    SCHED_FENCE();
                }
            }
#pragma unroll
        for (int in = 0; in < FN; ++in)
#pragma unroll
            for (int im = 0; im < FM; ++im) {
                acc[in][im] = __builtin_amdgcn_mfma_i32_16x16x64_i8(f[1][FM + in], f[1][im], acc[in][im], 0, 0, 0);
                SCHED_FENCE();
            }
        __builtin_amdgcn_s_setprio(0);
        fetch_w();                                 // W(t + 4), into the stage whose second half the other group read a phase ago
    };

    for (int ti = 0; ti < nt_b; ++ti) {
        int m0, n0;
        {
            int tm, tn;
            tile_of_block((int)blockIdx.x + ti * G, ntiles, p.tiles_m, p.tiles_n, tm, tn, p.magic);
            m0 = tm * C::BM;
            n0 = tn * C::BN;
        }
        set_rows(m0, n0);
#pragma unroll
        for (int in = 0; in < FN; ++in)
#pragma unroll
            for (int im = 0; im < FM; ++im) acc[in][im] = v4i{0, 0, 0, 0};
        // The column constants and row scales of the tile are requested now and parked in LDS at the end of the K loop, so
        // that the epilogue finds them there instead of waiting for memory.
        float2 c_ws = make_float2(0.f, 0.f), c_b = make_float2(0.f, 0.f);
        float c_xs[4] = {0.f, 0.f, 0.f, 0.f};
        const bool stager = EPI != EPI_ACC && wave == 7;
        if (stager) {
            const int l = hw_lane();
            int n = n0 + 2 * l;
            n = n < p.N ? n : p.N - 2;
            if (2 * l < C::BN) {
                c_ws = *reinterpret_cast<const float2*>(p.ws + n);
                if (p.bias) {
                    c_b.x = ld_dt<(EPI == EPI_ACC || OUT_DT == DT_F32) ? DT_F32 : OUT_DT>(p.bias, n);
                    c_b.y = ld_dt<(EPI == EPI_ACC || OUT_DT == DT_F32) ? DT_F32 : OUT_DT>(p.bias, n + 1);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) c_xs[j] = m0 + l + 64 * j < p.M ? p.xs[m0 + l + 64 * j] : 0.f;
        }
        // prologue.  Group 0 asks for its first K tile (W first: it has the longer way), then group 1 for its first, so
        // that what the first compute phase needs is at the head of the CU's return path.
        a_t = grp; w_t = grp;
        a_st = grp; w_st = grp;
        r_sa = grp; r_sw = grp;
        if (grp == 0) {
            fetch_w();
            fetch_a();
            wg_barrier();
            fetch_w();
            wait_vmcnt<C::NLW>();              // all but the second W tile
        } else {
            wg_barrier();
            fetch_w();
            fetch_a();
            fetch_w();
        }
        wg_barrier();
        if (grp == 1) wait_vmcnt<C::NLW>();
        // Both groups run the same loop, group 1 one phase behind.
        if (grp == 1) wg_barrier();
        for (int t = grp; t < nk; t += 2) {
            memory();                          // fragments of K tile t; A(t + 2)
            wait_lgkmcnt0();
            wg_barrier();
            compute();                         // K tile t; W(t + 4)
            wait_vmcnt<C::NLW>();              // everything but the W tile fetched last has landed
            wg_barrier();
        }
        if ((nk & 1) == grp) wg_barrier();     // the group with fewer K tiles sits out the last phase
        wait_vmcnt<0>();
        if (stager) {
            float* cst = reinterpret_cast<float*>(smem + C::CST_BASE);
            const int l = hw_lane();
            if (2 * l < C::BN) {
                *reinterpret_cast<float2*>(cst + 2 * l) = c_ws;
                *reinterpret_cast<float2*>(cst + C::BN + 2 * l) = c_b;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) cst[2 * C::BN + l + 64 * j] = c_xs[j];
        }
        __syncthreads();                       // no DMA in flight, nobody reads fragments: the LDS is free
        // Each group finishes half of every wave tile: group 0 the 16-row tiles 0 and 1 of its waves' 64 rows, group 1
        // tiles 2 and 3.  A wave parks the other group's half of its accumulators in LDS and adds the half it is handed.
        v4i fin[FN][2];
        {
            uint8_t* mine = smem + wave * C::HALF_ACC + hw_lane() * 16;
            const uint8_t* theirs = smem + (wave ^ 4) * C::HALF_ACC + hw_lane() * 16;
            if (nk > 1) {
#pragma unroll
                for (int in = 0; in < FN; ++in)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        *reinterpret_cast<v4i*>(mine + (in * 2 + h) * 1024) = grp == 0 ? acc[in][2 + h] : acc[in][h];
                        fin[in][h] = grp == 0 ? acc[in][h] : acc[in][2 + h];
                    }
                __syncthreads();
#pragma unroll
                for (int in = 0; in < FN; ++in)
#pragma unroll
                    for (int h = 0; h < 2; ++h) fin[in][h] += *reinterpret_cast<const v4i*>(theirs + (in * 2 + h) * 1024);
            } else {   // one K tile: group 0 holds all of it and hands group 1 its half
#pragma unroll
                for (int in = 0; in < FN; ++in)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        if (grp == 0) *reinterpret_cast<v4i*>(mine + (in * 2 + h) * 1024) = acc[in][2 + h];
                        fin[in][h] = acc[in][h];
                    }
                __syncthreads();
                if (grp == 1) {
#pragma unroll
                    for (int in = 0; in < FN; ++in)
#pragma unroll
                        for (int h = 0; h < 2; ++h) fin[in][h] = *reinterpret_cast<const v4i*>(theirs + (in * 2 + h) * 1024);
                }
            }
        }
        {
            uint8_t* scratch = smem + C::W_BASE + wave * 4096;   // a 4 KB shuffle piece per wave
            float* cst = reinterpret_cast<float*>(smem + C::CST_BASE);
            const int rows = wq * 64 + grp * 32;
            epilogue_shuffle<1, TN, OUT_DT, EPI, 32, true, 2, 16>(p, fin, m0 + rows, n0, hw_lane(), scratch, nullptr, cst, cst + 2 * C::BN + rows);
        }
        if (ti + 1 < nt_b) __syncthreads();    // the next tile's prologue overwrites what the epilogue reads
    }
}

// Sum of the int32 planes of a split-K run, then the epilogue.  planes[s][M][N]; four consecutive n per thread.
template <int OUT_DT, int EPI>
__global__ void __launch_bounds__(256) splitk_epilogue_kernel(GemmArgs p, const int* planes, int slices) {
    const int64_t nvec = (int64_t)p.M * p.N / 4, plane = (int64_t)p.M * p.N;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        const int64_t o = i * 4;
        const int m = (int)(o / p.N), n = (int)(o - (int64_t)m * p.N);
        // the planes' loads go out in batches of four with nothing between them: one trip to memory instead of `slices`
        const int* src = planes + o;
        v4i acc = *reinterpret_cast<const v4i*>(src);
        int s = 1;
        for (; s + 3 < slices; s += 4) {
            const v4i a0 = *reinterpret_cast<const v4i*>(src + s * plane), a1 = *reinterpret_cast<const v4i*>(src + (s + 1) * plane);
            const v4i a2 = *reinterpret_cast<const v4i*>(src + (s + 2) * plane), a3 = *reinterpret_cast<const v4i*>(src + (s + 3) * plane);
            acc += (a0 + a1) + (a2 + a3);
        }
        for (; s < slices; ++s) acc += *reinterpret_cast<const v4i*>(src + s * plane);
        if (EPI == EPI_ACC) {   // the caller asked for the accumulators themselves: no scales to apply
            *reinterpret_cast<v4i*>((int*)p.D + o) = acc;
            continue;
        }
        const float xs = p.xs[m];
        const float4 w4 = *reinterpret_cast<const float4*>(p.ws + n);
        const float ws[4] = {w4.x, w4.y, w4.z, w4.w};
        float b[4] = {0.f, 0.f, 0.f, 0.f}, rs[4] = {0.f, 0.f, 0.f, 0.f}, res[4] = {0.f, 0.f, 0.f, 0.f}, out[4];
        if (p.bias) load4<OUT_DT>(p.bias, n, b);
        if (EPI == EPI_RESID) { load4<OUT_DT>(p.rscale, n, rs); load4<OUT_DT>(p.resid, o, res); }
#pragma unroll
        for (int j = 0; j < 4; ++j) out[j] = epi_value<OUT_DT, EPI>(acc[j], xs, ws[j], b[j], rs[j], res[j]);
        store4<OUT_DT>(p.D, o, out);
    }
}

// Tile shapes of the register-staged kernel, the fallback for K % 128 != 0, unaligned outputs and small problems.
// M: 128x128, two workgroups per CU.  S: 64x64 for small M or N.
using CfgM = Cfg<128, 128, 64, 2, 2, 2>;
using CfgS = Cfg<64, 64, 64, 2, 2, 4>;

template <class C, int OUT_DT, int EPI>
int launch_cfg(GemmArgs a, hipStream_t st) {
    a.tiles_m = (a.M + C::BM - 1) / C::BM;
    a.tiles_n = (a.N + C::BN - 1) / C::BN;
    a.magic = panel_magic(a.tiles_m, a.tiles_n);
    const int64_t nblocks = (int64_t)a.tiles_m * a.tiles_n;
    if (nblocks > 0x7fffffff) return -1;
    auto kern = int8_gemm_kernel<C, OUT_DT, EPI>;
    if (C::SMEM > 48 * 1024) {
        static PerDeviceOnce once;
        if (const int e = allow_dynamic_lds((const void*)kern, C::SMEM, once)) return e;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(C::NT), C::SMEM, st, a);
    KCHECK();
    return 0;
}

int device_cu_count() {
    static std::atomic<int> cached[64];   // compute units per device ordinal, 0 = not asked yet
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    const bool keep = dev >= 0 && dev < 64;
    if (keep && (n = cached[dev].load(std::memory_order_relaxed)) > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
    if (keep) cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

// Launches the persistent ring kernel on `slices` K slices (1 = whole K).  With slices > 1, EPI must be EPI_ACC and
// a.D the int32 planes.
template <class C, int OUT_DT, int EPI>
int launch_ring_cfg(GemmArgs a, int slices, hipStream_t st) {
    a.tiles_m = (a.M + C::BM - 1) / C::BM;
    a.tiles_n = (a.N + C::BN - 1) / C::BN;
    a.magic = panel_magic(a.tiles_m, a.tiles_n);
    const int64_t ntiles = (int64_t)a.tiles_m * a.tiles_n;
    if (ntiles > 0x7fffffff) return -1;
    auto kern = int8_gemm_ring_kernel<C, OUT_DT, EPI>;
    static PerDeviceOnce once;
    if (const int e = allow_dynamic_lds((const void*)kern, C::SMEM, once)) return e;
    const int num_cu = device_cu_count();
    const int64_t per_slice = slices > 1 ? (num_cu / slices > 0 ? num_cu / slices : 1) : num_cu;
    const unsigned grid = (unsigned)(ntiles < per_slice ? ntiles : per_slice);
    hipLaunchKernelGGL(kern, dim3(grid, (unsigned)slices), dim3(C::NT), C::SMEM, st, a);
    KCHECK();
    return 0;
}

using RingS = RingCfg<192, 2, 2, 3, 128>;    // 128x192, waves 2x2 of 64x96: shapes with too few 256x256 tiles for the CUs

// Rows [row0, row0 + rows) of the problem as a problem of its own.
template <int OUT_DT, int EPI>
GemmArgs row_band(const GemmArgs& a, int64_t row0, int64_t rows) {
    constexpr int SZ = (EPI == EPI_ACC || OUT_DT == DT_F32) ? 4 : 2;
    GemmArgs b = a;
    b.A = a.A + row0 * a.K;
    b.xs = a.xs ? a.xs + row0 : nullptr;
    b.D = (uint8_t*)a.D + row0 * a.N * SZ;
    b.resid = a.resid ? (const uint8_t*)a.resid + row0 * a.N * SZ : nullptr;
    b.M = (int)rows;
    return b;
}

// Large shapes on the two-group kernel.  Every CU gets whole 256x256 tiles; when the tile count is not a multiple of the
// CU count, the last round would keep only some CUs busy for a full tile's time (864 tiles on 256 CUs: 96 busy, 160
// idle, a sixth of the run).  The tile rows that fill whole rounds are then run as 256x256 tiles and the rows left over
// as 128x256 tiles by further workgroups of the same launch, when that is estimated to be shorter (a small tile costs
// about 0.6 of a large one).
template <int OUT_DT, int EPI>
int launch_pp(GemmArgs a, hipStream_t st) {
    bool vec_ok, aligned;
    epilogue_alignment<OUT_DT, EPI>(a, vec_ok, aligned);
    if (!aligned) return launch_cfg<CfgM, OUT_DT, EPI>(a, st);   // this kernel has only the coalesced epilogue
    const int64_t G = device_cu_count();
    const int64_t tm = (a.M + PpL::BM - 1) / PpL::BM, tn = (a.N + PpL::BN - 1) / PpL::BN;
    const int64_t full = tm * tn / G, rem = tm * tn % G;
    GemmArgs main = a, rest = a;
    int64_t n_main = tm * tn, n_rest = 0;
    if (full >= 1 && rem > 0 && tm > 1) {
        int64_t main_rows = full * G / tn;
        if (main_rows >= tm) main_rows = tm - 1;
        const int64_t m_main = main_rows * PpL::BM, m_rest = a.M - m_main;
        const int64_t small = ((m_rest + PpS::BM - 1) / PpS::BM) * tn;
        const double split_cost = (double)((main_rows * tn + G - 1) / G) + 0.6 * (double)((small + G - 1) / G);
        if (main_rows > 0 && split_cost < (double)(full + 1) - 0.1) {
            main = row_band<OUT_DT, EPI>(a, 0, m_main);
            rest = row_band<OUT_DT, EPI>(a, m_main, m_rest);
            n_main = main_rows * tn;
            n_rest = small;
        }
    }
    if (n_main > 0x7fffffff) return -1;
    main.tiles_m = (main.M + PpL::BM - 1) / PpL::BM;
    main.tiles_n = (int)tn;
    rest.tiles_m = (rest.M + PpS::BM - 1) / PpS::BM;
    rest.tiles_n = (int)tn;
    main.magic = panel_magic(main.tiles_m, main.tiles_n);
    rest.magic = panel_magic(rest.tiles_m, rest.tiles_n);
    const int g_main = (int)(n_main < G ? n_main : G), g_rest = (int)(n_rest < G ? n_rest : G);
    auto kern = int8_gemm_pp_kernel<OUT_DT, EPI>;
    static PerDeviceOnce once;
    if (const int e = allow_dynamic_lds((const void*)kern, PpL::SMEM, once)) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g_main + g_rest)), dim3(PpL::NT), PpL::SMEM, st, main, rest, g_main);
    KCHECK();
    return 0;
}


// The 128x192 ring kernel on the whole problem: shapes with too few 256x256 tiles to fill the CUs.
template <int OUT_DT, int EPI>
int launch_ring_small(GemmArgs a, hipStream_t st) {
    bool vec_ok, aligned;
    epilogue_alignment<OUT_DT, EPI>(a, vec_ok, aligned);
    if (!aligned) return launch_cfg<CfgM, OUT_DT, EPI>(a, st);
    return launch_ring_cfg<RingS, OUT_DT, EPI>(a, 1, st);
}

// ---------------------------------------------------------------------------------------------------------------
// Scratch of the entry point that allocates nothing (gpu_int8_gemm_static): the int32 planes of a split-K run live in
// this file-scope device array instead of a stream-ordered allocation.  Every GPU the library runs on holds its own
// copy at its own address until the process ends; the array's name is only a host-side handle, so the device address
// is looked up once per device and host code uses that pointer from then on.  24 MiB covers every shape the skinny
// path splits on a GPU with up to 256 CUs: slices * N <= 256 * 96 columns and M <= 256 rows of int32.
// ---------------------------------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = (size_t)24 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each device, null until looked up

// Device address of the scratch array on the current device; 0 and a hipError_t / -210 in *rc on failure.
void* static_scratch(int* rc) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { *rc = (int)e; return nullptr; }
    if (dev < 0 || dev >= kMaxDevices) { *rc = -210; return nullptr; }
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));   // the current device's copy
        if (e != hipSuccess || !ptr) { *rc = e != hipSuccess ? (int)e : -210; return nullptr; }
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // every thread finds the same address
    }
    *rc = 0;
    return ptr;
}

// Set by gpu_int8_gemm_static around its dispatch: split-K planes go to this buffer instead of a stream-ordered
// allocation.  Thread-local, so calls from other threads through the other entry points are not affected.
thread_local void* tl_scratch = nullptr;
thread_local size_t tl_scratch_bytes = 0;

// Keep freed scratch in the device's default pool instead of returning it to the driver at every synchronization, as
// the reference's runtime layer does at start-up (src/cuda.rs:88-97): otherwise each call that needs scratch pays a
// fresh allocation.
void retain_pool_memory() {
    static PerDeviceOnce once;
    const int dev = PerDeviceOnce::current();
    if (dev < 0 || once.is_done(dev)) return;
    hipMemPool_t pool;
    uint64_t keep = ~(uint64_t)0;
    if (hipDeviceGetDefaultMemPool(&pool, dev) == hipSuccess && hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep) == hipSuccess)
        once.mark(dev);
}

// Split-K planes of the allocating entry points: one buffer per (device, stream), made on that stream's first split
// call and kept until the process ends.  Work on one stream is ordered, so its calls can share a buffer, and a
// stream-ordered allocation per call costs about 7 us on the stream's timeline (measured: 31 against 24 us per call at
// M=256, K=12288, N=4096).  The buffer has the one size every shape that the dispatcher splits fits into (slices *
// column tiles <= CUs, so slices * N <= CUs * 96, times 256 rows of int32: 24 MiB on 256 CUs) and is never grown or
// freed, so a captured graph that holds its address stays valid.  At most kStreamPlanes streams per process are served;
// a call on any further stream, a first call made under capture, or a shape beyond the size (a forced configuration)
// falls back to a stream-ordered allocation, and so does hipStreamPerThread (one handle for a different stream in every
// thread).  A stream handle that the runtime reuses after hipStreamDestroy inherits
// the destroyed stream's buffer; work still queued on the destroyed stream at that moment would share it.
struct StreamPlanes { int dev; hipStream_t st; void* ptr; size_t bytes; };
constexpr int kStreamPlanes = 8;
std::mutex g_planes_mu;
StreamPlanes g_planes[kStreamPlanes];
int g_planes_n = 0;

void* stream_planes(hipStream_t st, size_t need, int num_cu) {
    if (st == hipStreamPerThread) return nullptr;   // one handle, a different stream in every thread: nothing to key on
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_planes_mu);
    for (int i = 0; i < g_planes_n; ++i)
        if (g_planes[i].dev == dev && g_planes[i].st == st) return need <= g_planes[i].bytes ? g_planes[i].ptr : nullptr;
    const size_t bytes = (size_t)num_cu * TurnCfg::BN * TurnCfg::BM * sizeof(int);
    if (g_planes_n == kStreamPlanes || need > bytes) return nullptr;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;
    }
    void* ptr = nullptr;
    if (hipMalloc(&ptr, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_planes[g_planes_n++] = StreamPlanes{dev, st, ptr, bytes};
    return ptr;
}

// Launches the weight-streaming kernel on `slices` K slices (1 = whole K).  With slices > 1, EPI must be EPI_ACC and a.D
// the int32 planes.
template <int OUT_DT, int EPI>
int launch_stream(GemmArgs a, int slices, hipStream_t st) {
    using C = TurnCfg;
    a.tiles_m = (a.M + C::BM - 1) / C::BM;
    a.tiles_n = (a.N + C::BN - 1) / C::BN;
    a.magic = panel_magic(a.tiles_m, a.tiles_n);
    const int64_t ntiles = (int64_t)a.tiles_m * a.tiles_n;
    if (ntiles > 0x7fffffff) return -1;
    auto kern = int8_gemm_turn_kernel<OUT_DT, EPI>;
    static PerDeviceOnce once;
    if (const int e = allow_dynamic_lds((const void*)kern, C::SMEM, once)) return e;
    const int num_cu = device_cu_count();
    const int64_t per_slice = slices > 1 ? (num_cu / slices > 0 ? num_cu / slices : 1) : num_cu;
    const unsigned grid = (unsigned)(ntiles < per_slice ? ntiles : per_slice);
    hipLaunchKernelGGL(kern, dim3(grid, (unsigned)slices), dim3(C::NT), C::SMEM, st, a);
    KCHECK();
    return 0;
}

// M <= 256: one row of 256 x 96 tiles, the weights are read once and the run is bound by how fast they stream.  When N
// is too small to give every CU a column slab, K is split as well: each slice writes an int32 plane (exact, so the
// order of the sum does not matter) into the stream's scratch buffer and a second kernel adds the planes and applies
// the epilogue.
template <int OUT_DT, int EPI>
int launch_skinny(GemmArgs a, hipStream_t st) {
    bool vec_ok, aligned;
    epilogue_alignment<OUT_DT, EPI>(a, vec_ok, aligned);
    if (!aligned) return launch_cfg<CfgM, OUT_DT, EPI>(a, st);
    const int num_cu = device_cu_count();
    const int t96 = (a.N + 95) / 96, nk = a.K / 128;
    int slices = t96 * 4 >= num_cu * 3 ? 1 : num_cu / t96;
    if (slices > nk) slices = nk;
    if (slices > 1) {
        const int per = (nk + slices - 1) / slices;   // K tiles per slice
        slices = (nk + per - 1) / per;                // no empty slice
    }
    if (slices <= 1) return launch_stream<OUT_DT, EPI>(a, 1, st);
    const int per = (nk + slices - 1) / slices;
    const size_t need = (size_t)slices * a.M * a.N * sizeof(int);
    int* planes = nullptr;
    bool own = false;   // planes come from the stream-ordered pool and go back to it
    if (tl_scratch == nullptr) {
        planes = (int*)stream_planes(st, need, num_cu);
        if (!planes) {
            own = true;
            retain_pool_memory();
            hipError_t e = hipMallocAsync((void**)&planes, need, st);
            if (e != hipSuccess) return (int)e;
        }
    } else {
        if (need > tl_scratch_bytes) {
            fprintf(stderr, "gpu_int8_gemm_static: M=%d N=%d K=%d needs %zu bytes of split-K scratch, the static buffer has %zu\n",
                    a.M, a.N, a.K, need, tl_scratch_bytes);
            return -210;
        }
        planes = (int*)tl_scratch;   // every plane element is written before it is read: nothing to clear
    }
    GemmArgs pa = a;
    pa.D = planes;
    pa.kslice = per * 128;
    int rc = launch_stream<DT_F32, EPI_ACC>(pa, slices, st);
    if (rc == 0) {
        const int64_t nvec = (int64_t)a.M * a.N / 4;
        const unsigned grid = (unsigned)((nvec + 255) / 256 < 4096 ? (nvec + 255) / 256 : 4096);
        hipLaunchKernelGGL((splitk_epilogue_kernel<OUT_DT, EPI>), dim3(grid), dim3(256), 0, st, a, (const int*)planes, slices);
        hipError_t le = hipGetLastError();
        if (le != hipSuccess) rc = (int)le;
    }
    if (own) {
        hipError_t e = hipFreeAsync(planes, st);
        if (rc == 0 && e != hipSuccess) rc = (int)e;
    }
    return rc;
}

// Kernel family forced by the test hook (-1 = choose by shape).  Process-wide and only meant for tests and benchmarks:
// relaxed atomic, so a concurrent call sees either the old or the new value, never a torn one.
std::atomic<int> g_force_cfg{-1};

int choose_cfg(int64_t M, int64_t N, int64_t K) {
    const int force = g_force_cfg.load(std::memory_order_relaxed);
    const bool dma_ok = M * K < ((int64_t)1 << 32) && N * K < ((int64_t)1 << 32);   // 32-bit lane offsets
    if (force == 6 || force == 7 || force == 9) return (dma_ok && (K % 128) == 0) ? force : 1;
    if (force == 1 || force == 2) return force;
    if (M <= 256 && N >= 1024 && (K % 128) == 0 && K >= 512 && dma_ok) {
        // The weight-streaming kernel pays a fixed price per call (a prologue that waits for HBM, two launches when K
        // is split), which long K repays and short K does not.  Measured with weights from HBM, M = 16..256, K =
        // 1024..12288, N = 1024..24576: it wins from K = 3072 on at M > 128 and from K = 1536 on below; under that the
        // 128 x 192 ring tiles win for M > 128 (all N at K >= 1536, N >= 8192 below) and the small register-staged
        // tiles for the rest.
        if (K >= (M > 128 ? 3072 : 1536)) return 6;
        if (M > 128 && (K >= 1536 || N >= 8192)) return 7;
        return 2;
    }
    // Everything below was chosen from measured grids of shapes (weights from HBM, every family forced in turn).  A
    // round of 128 x 192 ring tiles costs about two thirds of a round of 256 x 256 two-group tiles, so the large tiles
    // win as soon as the small ones need a second round, i.e. more than one per CU.
    const int64_t tiles_s = ((M + 127) / 128) * ((N + 191) / 192);
    if (M >= 512 && N >= 512 && tiles_s > device_cu_count()) return (dma_ok && (K % 128) == 0) ? 9 : 1;
    if (dma_ok && (K % 128) == 0) {
        // a few hundred rows, long K, few columns: the ring tiles leave most CUs idle, the weight-streaming kernel splits
        // K over them (not for the entry point that may not allocate: its planes are sized for 256 rows)
        if (M <= 512 && N >= 1024 && K >= 8192 && tiles_s <= 96 && tl_scratch == nullptr) return 6;
        if (M > 128 && N >= 192 && (tiles_s >= 96 || (tiles_s >= 40 && K >= 2048))) return 7;
    }
    const int64_t tiles_m = ((M + 127) / 128) * ((N + 127) / 128);
    if (M > 64 && N > 64 && tiles_m >= 256) return 1;
    return 2;
}

template <int OUT_DT, int EPI>
int dispatch_cfg(const GemmArgs& a, hipStream_t st) {
    switch (choose_cfg(a.M, a.N, a.K)) {
        case 6: return launch_skinny<OUT_DT, EPI>(a, st);
        case 7: return launch_ring_small<OUT_DT, EPI>(a, st);
        case 9: return launch_pp<OUT_DT, EPI>(a, st);
        case 1: return launch_cfg<CfgM, OUT_DT, EPI>(a, st);
        default: return launch_cfg<CfgS, OUT_DT, EPI>(a, st);
    }
}

template <int EPI>
int dispatch_dt(const GemmArgs& a, int out_dt, hipStream_t st) {
    switch (out_dt) {
        case DT_F32: return dispatch_cfg<DT_F32, EPI>(a, st);
        case DT_F16: return dispatch_cfg<DT_F16, EPI>(a, st);
        case DT_BF16: return dispatch_cfg<DT_BF16, EPI>(a, st);
        default: return -1;
    }
}

bool shape_ok(int64_t M, int64_t N, int64_t K) {
    return M <= 0x7fffffff && N <= 0x7fffffff && K <= 0x7fffffff - 8 && (K % 8) == 0 && M * N < (int64_t)1 << 40;
}

// K % 16 == 8 (the reference's alignment-8 tile configurations, csrc/vendor/cutlass_gemm_int8.cu:191,237-247,265): the
// kernels here read 16-byte vectors of K, so such a call runs on copies of A and W whose rows carry eight more zero
// bytes, which leave every int32 sum as it was.  The copies live in one stream-ordered allocation for the length of
// the call.  No model in the reference's tree has such a K; the path exists so that the call is not refused.
__global__ void __launch_bounds__(256) pad_k_rows_kernel(const int8_t* src, int8_t* dst, int64_t rows, int k8) {
    const int64_t n = rows * (k8 + 1);   // 8-byte pieces of the destination
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / (k8 + 1);
        const int c = (int)(i - r * (k8 + 1));
        uint2 v = make_uint2(0u, 0u);
        if (c < k8) v = *reinterpret_cast<const uint2*>(src + (r * k8 + c) * 8);
        *reinterpret_cast<uint2*>(dst + i * 8) = v;
    }
}

struct PaddedK {
    int8_t* buf = nullptr;
    hipStream_t st;
    int rc = 0;
    // replaces A, W and K by the padded copies when K % 16 != 0
    PaddedK(const int8_t*& A, const int8_t*& W, int64_t M, int64_t N, int64_t& K, hipStream_t stream) : st(stream) {
        if ((K % 16) == 0) return;
        if ((((uintptr_t)A | (uintptr_t)W) & 7) != 0) { rc = -1; return; }
        const int64_t k16 = K + 8;
        retain_pool_memory();
        hipError_t e = hipMallocAsync((void**)&buf, (size_t)((M + N) * k16), st);
        if (e != hipSuccess) { buf = nullptr; rc = (int)e; return; }
        const int8_t* src[2] = {A, W};
        int8_t* dst[2] = {buf, buf + M * k16};
        const int64_t rows[2] = {M, N};
        for (int i = 0; i < 2; ++i) {
            const int64_t pieces = rows[i] * (k16 / 8);
            const unsigned grid = (unsigned)((pieces + 255) / 256 < 8192 ? (pieces + 255) / 256 : 8192);
            hipLaunchKernelGGL(pad_k_rows_kernel, dim3(grid), dim3(256), 0, st, src[i], dst[i], rows[i], (int)(K / 8));
        }
        hipError_t le = hipGetLastError();
        if (le != hipSuccess) rc = (int)le;
        A = dst[0];
        W = dst[1];
        K = k16;
    }
    ~PaddedK() { if (buf) (void)hipFreeAsync(buf, st); }
};

__global__ void mfma_layout_probe_kernel(int* out) {
    const int lane = threadIdx.x;
    v16i di, dj;
#pragma unroll
    for (int r = 0; r < 16; ++r) { di[r] = 0; dj[r] = 0; }
    const bool k0 = lane < 32;                       // lanes that feed the first 16 K bytes
    const v4i row = v4i{k0 ? (lane & 31) : 0, 0, 0, 0};  // byte 0 = row index
    const v4i one = v4i{k0 ? 1 : 0, 0, 0, 0};
    di = __builtin_amdgcn_mfma_i32_32x32x32_i8(row, one, di, 0, 0, 0);  // D[i][j] = i
    dj = __builtin_amdgcn_mfma_i32_32x32x32_i8(one, row, dj, 0, 0, 0);  // D[i][j] = j
#pragma unroll
    for (int r = 0; r < 16; ++r) out[lane * 16 + r] = di[r] * 32 + dj[r];
}

// Nothing but v_mfma_i32_32x32x32_i8: four waves per CU, sixteen independent accumulator tiles per wave (the register
// shape of the GEMM kernels), operands held in registers.  What this loop sustains is the matrix pipes' ceiling under
// the chip's power management for the given operand bits; the shader-clock count per workgroup gives the clock.
__global__ void __launch_bounds__(256, 1) mfma_ceiling_kernel(int iters, int random_bits, int form, long long* cycles, int* sink) {
    const uint32_t tid = threadIdx.x + blockIdx.x * 256u;
    auto hash = [](uint32_t x) { x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16; return x; };
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            a[i][r] = random_bits ? (int)hash(tid * 977u + i * 17u + r) : 0;
            b[i][r] = random_bits ? (int)hash(tid * 613u + i * 29u + r + 99991u) : 0;
        }
    if (form == 16) {   // v_mfma_i32_16x16x64_i8: 32 accumulator tiles with their own operand pairs, the same operations per iteration
        v4i c4[32];
        v4i a2[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) a2[i][r] = random_bits ? (int)hash(tid * 331u + i * 41u + r + 77777u) : 0;
#pragma unroll
        for (int i = 0; i < 32; ++i) c4[i] = v4i{0, 0, 0, 0};
        const long long t0 = (long long)__builtin_readcyclecounter();
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                for (int i = 0; i < 32; ++i) {
                    c4[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b[(i >> 2) & 3], i < 16 ? a[i & 3] : a2[i & 3], c4[i], 0, 0, 0);
                    SCHED_FENCE();
                }
        }
        const long long t1 = (long long)__builtin_readcyclecounter();
        int s = 0;
#pragma unroll
        for (int i = 0; i < 32; ++i) s += c4[i][0] + c4[i][1] + c4[i][2] + c4[i][3];
        if (s == 0x7fffffff) sink[0] = s;   // keeps the accumulators alive
        if (threadIdx.x == 0) cycles[blockIdx.x] = t1 - t0;
        return;
    }
    v16i acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    const long long t0 = (long long)__builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[i >> 2], a[i & 3], acc[i], 0, 0, 0);
                SCHED_FENCE();
            }
    }
    const long long t1 = (long long)__builtin_readcyclecounter();
    int s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    if (s == 0x7fffffff) sink[0] = s;   // keeps the accumulators alive
    if (threadIdx.x == 0) cycles[blockIdx.x] = t1 - t0;
}

}  // namespace

GPU_API int gpu_int8_gemm(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias, void* D,
                          int64_t M, int64_t N, int64_t K, int out_dt, void* stream) {
    if (M == 0 || N == 0 || K == 0) return 0;  // csrc/vendor/cutlass_gemm_int8.cu:377
    if (out_dt < DT_F32 || out_dt > DT_BF16 || M < 0 || N < 0 || K < 0 || !shape_ok(M, N, K)) return -200;
    PaddedK pad(A, W, M, N, K, (hipStream_t)stream);
    if (pad.rc != 0) return pad.rc < 0 ? -200 : pad.rc;
    GemmArgs a{A, W, xs, ws, bias, nullptr, nullptr, D, (int)M, (int)N, (int)K, 0, 0, 0};
    const int rc = dispatch_dt<EPI_PLAIN>(a, out_dt, (hipStream_t)stream);
    return rc < 0 ? -200 : rc;
}

GPU_API int gpu_int8_gemm_residual(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias,
                                   const void* rscale, const void* resid, void* D, int64_t M, int64_t N, int64_t K,
                                   int out_dt, void* stream) {
    if (M == 0 || N == 0) return 0;                       // csrc/vendor/cutlass_gemm_int8.cu:353
    if (K == 0 || !rscale || !resid) return -201;         // :355-357
    if (out_dt < DT_F32 || out_dt > DT_BF16 || M < 0 || N < 0 || K < 0 || !shape_ok(M, N, K)) return -201;
    PaddedK pad(A, W, M, N, K, (hipStream_t)stream);
    if (pad.rc != 0) return pad.rc < 0 ? -201 : pad.rc;
    GemmArgs a{A, W, xs, ws, bias, rscale, resid, D, (int)M, (int)N, (int)K, 0, 0, 0};
    const int rc = dispatch_dt<EPI_RESID>(a, out_dt, (hipStream_t)stream);
    return rc < 0 ? -201 : rc;
}

GPU_API int gpu_int8_gemm_static(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias, void* D,
                                 int64_t M, int64_t N, int64_t K, int out_dt, void* stream) {
    if (M == 0 || N == 0 || K == 0) return 0;
    if (out_dt < DT_F32 || out_dt > DT_BF16 || M < 0 || N < 0 || K < 0 || !shape_ok(M, N, K)) return -200;
    if ((K % 16) != 0) return -200;   // the K % 16 == 8 path allocates its padded copies
    int rc = 0;
    void* ptr = static_scratch(&rc);
    if (!ptr) return rc;
    GemmArgs a{A, W, xs, ws, bias, nullptr, nullptr, D, (int)M, (int)N, (int)K, 0, 0, 0};
    tl_scratch = ptr;
    tl_scratch_bytes = kStaticScratchBytes;
    rc = dispatch_dt<EPI_PLAIN>(a, out_dt, (hipStream_t)stream);
    tl_scratch = nullptr;
    tl_scratch_bytes = 0;
    return rc == -210 ? -210 : rc < 0 ? -200 : rc;
}

GPU_API int64_t gpu_int8_gemm_static_limit(void) { return (int64_t)kStaticScratchBytes; }

GPU_API int gpu_int8_gemm_acc(const int8_t* A, const int8_t* W, int32_t* acc, int64_t M, int64_t N, int64_t K, void* stream) {
    if (M == 0 || N == 0 || K == 0) return 0;
    if (M < 0 || N < 0 || K < 0 || !shape_ok(M, N, K)) return -200;
    PaddedK pad(A, W, M, N, K, (hipStream_t)stream);
    if (pad.rc != 0) return pad.rc < 0 ? -200 : pad.rc;
    GemmArgs a{A, W, nullptr, nullptr, nullptr, nullptr, nullptr, acc, (int)M, (int)N, (int)K, 0, 0, 0};
    const int rc = dispatch_cfg<DT_F32, EPI_ACC>(a, (hipStream_t)stream);
    return rc < 0 ? -200 : rc;
}

// Test hook: force a kernel family (1 = 128x128, 2 = 64x64 register-staged tiles; 6 = weight streaming; 7 = persistent
// ring, 128x192; 9 = two-group kernel; -1 or anything else = automatic).
GPU_API int gpu_int8_gemm_force_config(int cfg) {
    g_force_cfg.store(cfg, std::memory_order_relaxed);
    return 0;
}

GPU_API int gpu_mfma_ceiling_probe(int iters, int random_bits, int64_t* cycles, int32_t* sink, void* stream) {
    if (iters <= 0) return 0;
    // random_bits: 0 = zero operands, 1 = random; + 2 = the 16x16x64 form of the instruction instead of 32x32x32
    hipLaunchKernelGGL(mfma_ceiling_kernel, dim3((unsigned)device_cu_count()), dim3(256), 0, (hipStream_t)stream, iters, random_bits & 1,
                       (random_bits & 2) ? 16 : 32, (long long*)cycles, (int*)sink);
    KCHECK();
    return 0;
}

GPU_API int gpu_mfma_layout_probe(int32_t* out, void* stream) {
    hipLaunchKernelGGL(mfma_layout_probe_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, out);
    KCHECK();
    return 0;
}
