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
// C = 0) that is folded into the fp32 accumulators.  A workgroup of eight waves owns a 256 x 128 tile; per iteration g:
//   * LDS-DMA brings A(g+2) (256 x 128 int8, three stages), the packed weights of group g+2 (128 rows x 96 bytes, two
//     stages) and the 128 scales of group g+2 (four stages) straight into LDS.  Every wave issues the same seven
//     instructions, one after every other MFMA, so one counted wait serves all waves;
//   * the packed weights are wave-local: wave w fetches rows 16w..16w+15 itself (1.5 KB), waits for its own fetch, and
//     expands its 128 twelve-byte pieces (two per lane) of group g+1 into 16 int8 each, written in the swizzled
//     fragment layout (conflict-free both ways).  Only the expanded tile crosses waves, behind the iteration's barrier;
//   * each wave (2 x 4 grid, 128 x 32 outputs, 8 x 2 tiles of v_mfma_i32_16x16x64_i8) multiplies group g in two halves
//     of eight tiles; the fp32 fold of the first half rides between the MFMAs of the second.
// The fold costs two VALU operations per output and group and the unpack about six per code word: together more issue
// slots than the MFMAs, so the kernel is bound by VALU issue, not by the matrix pipe.  Two waves share a SIMD; the upper
// four waves fold their second half at the end of an iteration, the lower four at the start of the next, so that on
// every SIMD one wave's VALU-only stretch meets the other's MFMAs.
#include "common.hpp"
#include <atomic>

#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

namespace {

struct W6Args {
    const int8_t* A;
    const uint8_t* Wp;
    const int8_t* W8;   // the weights already expanded to int8 [N, K] (the W8 form of the kernel), or null
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
constexpr int NSA = 3, NSS = 4;   // stages of A and of the scales (the deferred fold still reads group g-1 in iteration g)
constexpr int U_BASE = NSA * A_STAGE;
// Fused unpack: two stages of expanded weights and two of packed ones.  W8 form (weights expanded beforehand, fetched
// like A): three stages of expanded weights, none of packed ones.
template <bool W8> struct Lay {
    static constexpr int NSU = W8 ? 3 : 2;
    static constexpr int R_BASE = U_BASE + NSU * U_STAGE, S_BASE = R_BASE + (W8 ? 0 : 2 * R_STAGE);
    static constexpr int SMEM = S_BASE + NSS * S_STAGE;
    static_assert(SMEM <= 160 * 1024, "LDS budget");
};
constexpr int RAW_WAVE = 16 * RAW_ROW;   // bytes of packed weights a wave owns per group: 16 rows
constexpr int NT = 512;         // eight waves, 2 (m) x 4 (n)

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
template <int N> __device__ __forceinline__ void wait_vmcnt_n() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
__device__ __forceinline__ void wait_all_dma() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void dma4(uint32_t lds_dst, uint32_t lane_off, const void* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_dst), "v"(lane_off), "s"(base) : "memory", "m0");
}

// ABL (measurement only, wrong results): bit 0 leaves out the fp32 fold, bit 1 the unpack, bit 2 the DMA of the MFMA
// waves after the prologue; what remains shows what each part costs next to the MFMAs.
template <int OUT_DT, bool DUMP, int ABL = 0, bool W8 = false>
__global__ void __launch_bounds__(NT, 1) w6a8_group_gemm_kernel(W6Args p) {
    constexpr int R_BASE = Lay<W8>::R_BASE, S_BASE = Lay<W8>::S_BASE;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    int tm, tn;
    tile_of_block((int)blockIdx.x, (int)gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN, ng = p.ng;
    const uint32_t lds_base = (uint32_t)(uintptr_t)smem;

    // DMA sources: 32-bit lane offsets from a per-group scalar base.  Rows past the edge re-read the last valid row;
    // what they produce is never stored.
    // The swizzle (chunk ^ bits 1..3 of the row: 16 consecutive rows of a chunk column then cover all 64 LDS banks) is
    // applied on the global side; rows come in blocks of 8 whose index wave + 8j has the parity of wave.
    const int lrow = lane >> 3, lch = ((lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1))) * 16;
    uint32_t ga[4], gr[2], gs;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = (wave + 8 * j) * 8 + lrow;
        const int r = m0 + row < p.M ? m0 + row : p.M - 1;
        ga[j] = (uint32_t)r * (uint32_t)p.K + lch;
    }
    const uint32_t wrow = (uint32_t)p.K / 4 * 3;                   // bytes per packed weight row
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        if (W8) {                                                  // expanded weights: 8-row blocks wave, wave + 8, as for A
            const int row = (wave + 8 * j) * 8 + lrow;
            const int r = n0 + row < p.N ? n0 + row : p.N - 1;
            gr[j] = (uint32_t)r * (uint32_t)p.K + lch;
            continue;
        }
        // the wave's own 1.5 KB of packed weights: one full and one half instruction
        const int b = (64 * j + (j ? (lane & 31) : lane)) * 16;    // byte inside the wave's block of 16 rows x 96 bytes
        const int row = 16 * wave + b / RAW_ROW, col = b % RAW_ROW;
        const int r = n0 + row < p.N ? n0 + row : p.N - 1;
        gr[j] = (uint32_t)r * wrow + col;
    }
    {
        const int row = 16 * wave + (lane & 15);
        const int r = n0 + row < p.N ? n0 + row : p.N - 1;
        gs = (uint32_t)r * (uint32_t)ng * 4u;
    }
    // The seven DMA instructions a wave issues per group.  Groups past the end re-fetch the last one (into stages that
    // nothing reads again), which keeps the loop free of branches and the count per iteration fixed.
    auto dma_a = [&](int g, int stage, int j) {
        dma16(lds_base + stage * A_STAGE + (wave + 8 * j) * 1024, ga[j], p.A + (int64_t)(g < ng ? g : ng - 1) * BK);
    };
    auto dma_raw = [&](int g, int stage, int j) {
        if (W8) {   // `stage` is then a stage of expanded weights
            dma16(lds_base + U_BASE + stage * U_STAGE + (wave + 8 * j) * 1024, gr[j], p.W8 + (int64_t)(g < ng ? g : ng - 1) * BK);
            return;
        }
        const uint8_t* base = p.Wp + (int64_t)(g < ng ? g : ng - 1) * RAW_ROW;
        const uint32_t dst = lds_base + R_BASE + stage * R_STAGE + wave * RAW_WAVE + j * 1024;
        if (j == 0) dma16(dst, gr[0], base);
        else if (lane < 32) dma16(dst, gr[1], base);
    };
    auto dma_scales = [&](int g, int stage) {
        if (lane < 16) dma4(lds_base + S_BASE + stage * S_STAGE + wave * 64, gs, p.sw + (g < ng ? g : ng - 1));
    };
    // Piece e of the wave's block is bytes [12e, 12e+12): row 16*wave + e/8, codes 16*(e%8) .. +15 -> one 16-byte
    // chunk.  Reading the three words and expanding them are separate steps so that the LDS latency hides behind
    // other work.
    auto raw_read = [&](int rstage, int i, uint32_t (&d)[3]) {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(smem + R_BASE + rstage * R_STAGE + wave * RAW_WAVE + 12 * (lane + 64 * i));
        d[0] = src[0]; d[1] = src[1]; d[2] = src[2];
    };
    auto unpack_write = [&](int ustage, int i, const uint32_t (&d)[3]) {
        const int e = lane + 64 * i;
        const v4i out = v4i{spread6(d[0]), spread6(__builtin_amdgcn_alignbit(d[1], d[0], 24)),
                            spread6(__builtin_amdgcn_alignbit(d[2], d[1], 16)), spread6(d[2] >> 8)};
        const int r = 16 * wave + (e >> 3), pc = e & 7;
        *reinterpret_cast<v4i*>(smem + U_BASE + ustage * U_STAGE + r * BK + ((pc ^ ((r >> 1) & 7)) << 4)) = out;
    };

    // The tiles are multiplied with v_mfma_i32_16x16x64_i8 (the same operations per cycle as the 32x32x32 form, less
    // accumulator traffic per operation, which this power-limited part pays back as clock): a wave's 128 x 32 outputs are
    // 8 x 2 tiles of 16 x 16, four registers each.  A lane holds row lane % 16 of a tile and columns 4*(lane / 16) + c.
    // Fragment addresses inside a stage: row r at r*128, chunk c at slot c ^ ((r>>1)&7); a lane reads row lane % 16, chunk
    // 4*h + lane / 16 of K half h (which flips bit 6).
    const int frow = lane & 15, fq = lane >> 4;
    const int fsw = (fq ^ ((frow >> 1) & 7)) << 4;
    const int aoff = (wm * 128 + frow) * BK + fsw, woff = (wn * 32 + frow) * BK + fsw;
    constexpr int FM = 8, FN = 2;

    v4i part[FN][FM];        // int32 partial of the current group
    float accf[FN][FM][4];   // fp32 accumulators
#pragma unroll
    for (int in = 0; in < FN; ++in)
#pragma unroll
        for (int im = 0; im < FM; ++im)
#pragma unroll
            for (int r = 0; r < 4; ++r) accf[in][im][r] = 0.f;

    // prologue: groups 0 and 1 of everything land; the wave's rows of group 0 are unpacked
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        dma_raw(g, g, 0);
        dma_raw(g, g, 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) dma_a(g, g, j);
        dma_scales(g, g);
    }
    wait_all_dma();
    if (!W8) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint32_t d[3];
            raw_read(0, i, d);
            unpack_write(0, i, d);
        }
    }
    __syncthreads();

    const bool defer = wm == 0;   // these waves fold their second half at the start of the next iteration
#pragma unroll
    for (int in = 0; in < FN; ++in)
#pragma unroll
        for (int im = 0; im < FM; ++im) part[in][im] = v4i{0, 0, 0, 0};

    // fp32 fold of one tile's four values.  accf += float(part) * sw[n, g]
    auto fold = [&](int in, int im, const float4& s4) {
        if (ABL & 1) {   // keep the partials alive with one operation per tile instead of eight
            accf[in][im][0] += __builtin_bit_cast(float, part[in][im][0] ^ part[in][im][1] ^ part[in][im][2] ^ part[in][im][3]);
            return;
        }
        const float sv[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) accf[in][im][c] = __builtin_fmaf((float)part[in][im][c], sv[c], accf[in][im][c]);
    };

    int a_cur = 0, s_cur = 0;   // stages of group g: g mod 3 (A), g mod 4 (scales)
    for (int g = 0; g < ng; ++g) {
        const int a_new = a_cur == 0 ? 2 : a_cur - 1;                  // (g + 2) mod 3
        const int s = W8 ? a_new : g & 1;                              // the stage dma_raw fills with group g+2
        const int s_new = (s_cur + 2) & 3, s_prev = (s_cur + 3) & 3;   // (g + 2) mod 4, (g - 1) mod 4
        const uint8_t* sa = smem + a_cur * A_STAGE;
        const uint8_t* su = smem + U_BASE + (W8 ? a_cur : g & 1) * U_STAGE;
        const float* sc = reinterpret_cast<const float*>(smem + S_BASE + s_cur * S_STAGE);
        const float* sc_prev = reinterpret_cast<const float*>(smem + S_BASE + s_prev * S_STAGE);

        v4i fa[4][2], fw[FN][2], na[4][2];   // A fragments of row tiles 0..3 / 4..7 and W fragments, per K half
        float4 sv[FN];
        uint32_t raw[2][3];
        // Sixteen MFMAs of one half of the wave tile (row tiles imb .. imb+3, both column tiles, both K halves; a tile's two
        // MFMAs are eight apart); between(i) is issued after the i-th of them.
        auto mma_half = [&](int imb, v4i (&a)[4][2], auto&& between) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const int in = t & 1, il = t >> 1;
                    const v4i c = h == 0 ? v4i{0, 0, 0, 0} : part[in][imb + il];
                    part[in][imb + il] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[in][h], a[il][h], c, 0, 0, 0);
                    SCHED_FENCE();
                    between(h * 8 + t);
                    SCHED_FENCE();
                }
        };

        // The wave's own packed rows of group g+1 were the first two DMA instructions of the previous iteration; the
        // five issued after them may still be in flight.
        if (ABL & 4) wait_all_dma();
        else if (!W8) wait_vmcnt_n<5>();
        // everything this iteration reads from LDS early: fragments of the first half, the group's scales, packed words
#pragma unroll
        for (int in = 0; in < FN; ++in)
#pragma unroll
            for (int h = 0; h < 2; ++h) fw[in][h] = *reinterpret_cast<const v4i*>(su + ((woff + in * 16 * BK) ^ (h << 6)));
#pragma unroll
        for (int il = 0; il < 4; ++il)
#pragma unroll
            for (int h = 0; h < 2; ++h) fa[il][h] = *reinterpret_cast<const v4i*>(sa + ((aoff + il * 16 * BK) ^ (h << 6)));
#pragma unroll
        for (int in = 0; in < FN; ++in) sv[in] = *reinterpret_cast<const float4*>(sc + wn * 32 + 16 * in + 4 * fq);
#pragma unroll
        for (int i = 0; i < 2; ++i)
            if (!(ABL & 2) && !W8) raw_read(s ^ 1, i, raw[i]);
        SCHED_FENCE();
        if (defer && g > 0) {   // the fold the previous iteration left over
#pragma unroll
            for (int in = 0; in < FN; ++in) {
                const float4 sp = *reinterpret_cast<const float4*>(sc_prev + wn * 32 + 16 * in + 4 * fq);
#pragma unroll
                for (int il = 0; il < 4; ++il) fold(in, 4 + il, sp);
            }
            SCHED_FENCE();
        }
        // The second half's A fragments are read while the first half is multiplied.  DMA targets: the packed stage of
        // group g (expanded during iteration g-1) or the expanded stage of group g-1, the A stage of group g-1 and the scale
        // stage of group g-2, all of them last read before the barrier that ended iteration g-1.
        mma_half(0, fa, [&](int i) {
            if (i < 8) na[i >> 1][i & 1] = *reinterpret_cast<const v4i*>(sa + ((aoff + (4 + (i >> 1)) * 16 * BK) ^ ((i & 1) << 6)));
            if (!(ABL & 4)) {
                if (i == 2) dma_raw(g + 2, s, 0);
                if (i == 6) dma_raw(g + 2, s, 1);
                if (i == 10) dma_a(g + 2, a_new, 0);
                if (i == 14) dma_a(g + 2, a_new, 1);
            }
            if (!(ABL & 2) && !W8) {
                if (i == 4) unpack_write(s ^ 1, 0, raw[0]);
                if (i == 8) unpack_write(s ^ 1, 1, raw[1]);
            }
        });
        mma_half(4, na, [&](int i) {
            if (i & 1) fold((i >> 1) & 1, i >> 2, sv[(i >> 1) & 1]);   // the first half's eight tiles, one every other MFMA
            if (!(ABL & 4)) {
                if (i == 2) dma_a(g + 2, a_new, 2);
                if (i == 6) dma_a(g + 2, a_new, 3);
                if (i == 10) dma_scales(g + 2, s_new);
            }
        });
        if (!defer) {
#pragma unroll
            for (int in = 0; in < FN; ++in)
#pragma unroll
                for (int il = 0; il < 4; ++il) fold(in, 4 + il, sv[in]);
        }

        if (DUMP) {   // test hook: the exact int32 partials, [M, N, ng]
#pragma unroll
            for (int in = 0; in < FN; ++in)
#pragma unroll
                for (int im = 0; im < FM; ++im)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int m = m0 + wm * 128 + im * 16 + frow;
                        const int n = n0 + wn * 32 + 16 * in + 4 * fq + c;
                        if (m < p.M && n < p.N) p.partials[((int64_t)m * p.N + n) * ng + g] = part[in][im][c];
                    }
            wait_all_dma();   // the dump's stores share the counter: drain it rather than count them
        }
        if (ABL & 4) wait_all_dma();
        else wait_vmcnt_n<7>();   // everything older than this iteration's seven has landed: A and scales of group g+1
        __syncthreads();     // ... for every wave, and the expanded weights of group g+1 are written
        a_cur = a_cur == 2 ? 0 : a_cur + 1;
        s_cur = (s_cur + 1) & 3;
    }
    wait_all_dma();   // nothing may still be writing this workgroup's LDS when it retires or reuses it
    if (defer) {
        const float* sc_last = reinterpret_cast<const float*>(smem + S_BASE + ((s_cur + 3) & 3) * S_STAGE);
#pragma unroll
        for (int in = 0; in < FN; ++in) {
            const float4 sp = *reinterpret_cast<const float4*>(sc_last + wn * 32 + 16 * in + 4 * fq);
#pragma unroll
            for (int il = 0; il < 4; ++il) fold(in, 4 + il, sp);
        }
    }
    __syncthreads();   // every wave's DMA is drained before the epilogue reuses the stages

    // Epilogue.  A lane holds one m per row tile and four consecutive n per column tile, so storing straight from the
    // registers would touch 16 rows per instruction.  When the rows of D are 16-byte aligned each wave instead passes its
    // tile, 32 rows at a time, through a private 4 KB of LDS (16-byte chunks XOR-swizzled by row) and writes whole row
    // segments, 16 bytes per lane.
    constexpr int SZ = dt_size<OUT_DT>::value;
    const bool vec_ok = (p.N & 3) == 0 && ((uintptr_t)p.D & (4 * SZ - 1)) == 0 && ((uintptr_t)p.bias & (4 * SZ - 1)) == 0;
    const bool rows_ok = vec_ok && (((int64_t)p.N * SZ) & 15) == 0 && ((uintptr_t)p.D & 15) == 0;
    const int nb = n0 + wn * 32;
    float bv[FN][4];
#pragma unroll
    for (int in = 0; in < FN; ++in) {
        const int n = nb + 16 * in + 4 * fq;
#pragma unroll
        for (int c = 0; c < 4; ++c) bv[in][c] = 0.f;
        if (p.bias && n < p.N) {
            if (vec_ok) {
                load4<OUT_DT>(p.bias, n, bv[in]);
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) if (n + c < p.N) bv[in][c] = ld_dt<OUT_DT>(p.bias, n + c);
            }
        }
    }
    if (rows_ok) {
        constexpr int ROWB = 32 * SZ, CPR = ROWB / 16;          // bytes and 16-byte chunks per LDS row (32 columns)
        constexpr int RPI = 64 / CPR, NI = 32 / RPI;            // rows per store instruction, instructions per piece
        uint8_t* wl = smem + wave * 4096;                        // the stages are idle: the loop ended with a barrier
#pragma unroll
        for (int ip = 0; ip < FM / 2; ++ip) {                    // a piece: row tiles 2*ip and 2*ip + 1
            const int mb = m0 + wm * 128 + ip * 32;
#pragma unroll
            for (int hm = 0; hm < 2; ++hm) {
                const int prow = hm * 16 + frow;
                const float xs = p.xs[mb + prow < p.M ? mb + prow : p.M - 1];
#pragma unroll
                for (int in = 0; in < FN; ++in) {
                    float out[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) out[c] = __builtin_fmaf(accf[in][2 * ip + hm][c], xs, bv[in][c]);
                    const int byte = (16 * in + 4 * fq) * SZ;    // columns 16*in + 4*fq .. +3 of row prow
                    uint8_t* dst = wl + prow * ROWB + ((((byte >> 4) ^ (prow & (CPR - 1))) << 4) | (byte & 15));
                    if (OUT_DT == DT_F32) {
                        *reinterpret_cast<float4*>(dst) = make_float4(out[0], out[1], out[2], out[3]);
                    } else if (OUT_DT == DT_BF16) {
                        *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(out[0], out[1]), pack_bf16x2(out[2], out[3]));
                    } else {
                        *reinterpret_cast<uint2*>(dst) = make_uint2((uint32_t)f_to_f16(out[0]) | ((uint32_t)f_to_f16(out[1]) << 16),
                                                                    (uint32_t)f_to_f16(out[2]) | ((uint32_t)f_to_f16(out[3]) << 16));
                    }
                }
            }
            asm volatile("" ::: "memory");   // the wave's own LDS writes are ordered before its reads
#pragma unroll
            for (int t = 0; t < NI; ++t) {
                const int row = t * RPI + lane / CPR, ch = lane % CPR;
                const uint4 v = *reinterpret_cast<const uint4*>(wl + row * ROWB + ((ch ^ (row & (CPR - 1))) << 4));
                const int m = mb + row, n = nb + ch * (16 / SZ);
                if (m < p.M && n < p.N) *reinterpret_cast<uint4*>((uint8_t*)p.D + ((int64_t)m * p.N + n) * SZ) = v;
            }
            asm volatile("" ::: "memory");   // ... and the reads before the next piece's writes
        }
        return;
    }
    // fallback for unaligned rows: four consecutive n per lane and tile, straight from the accumulators
#pragma unroll
    for (int im = 0; im < FM; ++im) {
        const int m = m0 + wm * 128 + im * 16 + frow;
        if (m >= p.M) continue;
        const float xs = p.xs[m];
#pragma unroll
        for (int in = 0; in < FN; ++in) {
            const int n = nb + 16 * in + 4 * fq;
            if (n >= p.N) continue;
            const int64_t o = (int64_t)m * p.N + n;
            float out[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) out[c] = __builtin_fmaf(accf[in][im][c], xs, bv[in][c]);
            if (vec_ok) {
                store4<OUT_DT>(p.D, o, out);
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) if (n + c < p.N) st_dt<OUT_DT>(p.D, o + c, out[c]);
            }
        }
    }
}

template <int OUT_DT, bool DUMP, int ABL = 0, bool W8 = false>
int launch(W6Args a, hipStream_t st) {
    auto kern = w6a8_group_gemm_kernel<OUT_DT, DUMP, ABL, W8>;
    constexpr int SMEM = Lay<W8>::SMEM;
    static PerDeviceOnce once;
    if (const int e = allow_dynamic_lds((const void*)kern, SMEM, once)) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)(a.tiles_m * a.tiles_n)), dim3(NT), SMEM, st, a);
    KCHECK();
    return 0;
}

template <int OUT_DT>
int launch_dt(const W6Args& a, hipStream_t st) {
    if (a.W8) return a.partials ? launch<OUT_DT, true, 0, true>(a, st) : launch<OUT_DT, false, 0, true>(a, st);
    return a.partials ? launch<OUT_DT, true>(a, st) : launch<OUT_DT, false>(a, st);
}

// The packed weights expanded to int8 [N, K]: a thread turns one 12-byte piece into 16 codes.
__global__ void __launch_bounds__(256) w6_words_to_int8_kernel(const uint8_t* Wp, int8_t* out, int64_t pieces) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (int64_t)gridDim.x * 256) {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(Wp + i * 12);
        const uint32_t d0 = src[0], d1 = src[1], d2 = src[2];
        *reinterpret_cast<v4i*>(out + i * 16) = v4i{spread6(d0), spread6(__builtin_amdgcn_alignbit(d1, d0, 24)),
                                                   spread6(__builtin_amdgcn_alignbit(d2, d1, 16)), spread6(d2 >> 8)};
    }
}

// From this many rows of A on, the weights are expanded once into a stream-ordered scratch and the kernel fetches them
// like A; below, every workgroup expands its own 128 columns as it goes.  Each weight is used by M / 256 workgroups:
// expanding it that many times costs the large-M shapes more vector issue slots than the int8 round trip through HBM
// costs them time (M = 8192: 9 % faster; M = 2048: 10 % slower, the expansion being a fixed 25-30 us).
constexpr int64_t kExpandFirstRows = 4096;
std::atomic<int> g_mode{-1};   // test hook: 0 = always fused, 1 = always expand first, -1 = by M

// 32-bit DMA lane offsets into A, the packed weights and the scales; a tile count that fits the grid
bool shape_fits(int64_t M, int64_t N, int64_t K) {
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return false;
    if (M * K >= ((int64_t)1 << 32) || N * (K / 4 * 3) >= ((int64_t)1 << 32) || N * (K / 128) * 4 >= ((int64_t)1 << 32)) return false;
    return ((M + BM - 1) / BM) * ((N + BN - 1) / BN) <= 0x7fffffff;
}

}  // namespace

GPU_API int gpu_w6a8_group_gemm(const int8_t* A, const void* Wp, const float* xs, const float* sw, const void* bias,
                                void* D, int32_t* partials, int64_t M, int64_t N, int64_t K, int out_dt, void* stream) {
    if (K < 0 || (K % 128) != 0) return -1;
    if (out_dt < DT_F32 || out_dt > DT_BF16 || M < 0 || N < 0) return -200;
    if (M == 0 || N == 0) return 0;
    if (K == 0 || !shape_fits(M, N, K)) return -200;
    W6Args a{A, (const uint8_t*)Wp, nullptr, xs, sw, bias, D, partials, (int)M, (int)N, (int)K, (int)(K / 128), 0, 0};
    a.tiles_m = (int)((M + BM - 1) / BM);
    a.tiles_n = (int)((N + BN - 1) / BN);
    hipStream_t st = (hipStream_t)stream;
    const int mode = g_mode.load(std::memory_order_relaxed);
    int8_t* w8 = nullptr;
    if ((mode == 1 || (mode != 0 && M >= kExpandFirstRows)) && N * K < ((int64_t)1 << 32) && ((uintptr_t)Wp & 3) == 0) {
        hipError_t e = hipMallocAsync((void**)&w8, (size_t)(N * K), st);
        if (e != hipSuccess) return (int)e;
        const int64_t pieces = N * K / 16;
        const unsigned grid = (unsigned)((pieces + 255) / 256 < 256 * 32 ? (pieces + 255) / 256 : 256 * 32);
        hipLaunchKernelGGL(w6_words_to_int8_kernel, dim3(grid), dim3(256), 0, st, (const uint8_t*)Wp, w8, pieces);
        a.W8 = w8;
    }
    int rc;
    switch (out_dt) {
        case DT_F32: rc = launch_dt<DT_F32>(a, st); break;
        case DT_F16: rc = launch_dt<DT_F16>(a, st); break;
        default: rc = launch_dt<DT_BF16>(a, st); break;
    }
    if (w8) {
        hipError_t e = hipFreeAsync(w8, st);
        if (rc == 0 && e != hipSuccess) rc = (int)e;
    }
    return rc;
}

// Test hook, no reference counterpart: 0 = gpu_w6a8_group_gemm always expands the weights inside the kernel, 1 = always
// expands them first, -1 = chooses by M.
GPU_API int gpu_internal_w6a8_group_gemm_mode(int mode) {
    g_mode.store(mode, std::memory_order_relaxed);
    return 0;
}

// Measurement hook, no reference counterpart: gpu_w6a8_group_gemm (bf16 output) with parts of the kernel left out --
// ablate bit 0 the fp32 fold, bit 1 the unpack, bit 2 the LDS-DMA after the prologue; bit 3 (8, 9, 12, 13) the form that
// fetches expanded weights, with Wp then pointing at int8 [N, K].  D receives meaningless values.
GPU_API int gpu_internal_w6a8_group_gemm_ablate(int ablate, const int8_t* A, const void* Wp, const float* xs, const float* sw,
                                                void* D, int64_t M, int64_t N, int64_t K, void* stream) {
    if (K <= 0 || (K % 128) != 0 || M <= 0 || N <= 0 || !shape_fits(M, N, K)) return -200;
    if ((ablate & 8) && N * K >= ((int64_t)1 << 32)) return -200;
    W6Args a{A, (const uint8_t*)Wp, nullptr, xs, sw, nullptr, D, nullptr, (int)M, (int)N, (int)K, (int)(K / 128), 0, 0};
    a.tiles_m = (int)((M + BM - 1) / BM);
    a.tiles_n = (int)((N + BN - 1) / BN);
    hipStream_t st = (hipStream_t)stream;
    if (ablate & 8) a.W8 = (const int8_t*)Wp;   // the caller passes expanded weights, int8 [N, K]
    switch (ablate) {
        case 0: return launch<DT_BF16, false, 0>(a, st);
        case 1: return launch<DT_BF16, false, 1>(a, st);
        case 2: return launch<DT_BF16, false, 2>(a, st);
        case 3: return launch<DT_BF16, false, 3>(a, st);
        case 4: return launch<DT_BF16, false, 4>(a, st);
        case 5: return launch<DT_BF16, false, 5>(a, st);
        case 6: return launch<DT_BF16, false, 6>(a, st);
        case 7: return launch<DT_BF16, false, 7>(a, st);
        case 8: return launch<DT_BF16, false, 0, true>(a, st);
        case 9: return launch<DT_BF16, false, 1, true>(a, st);
        case 12: return launch<DT_BF16, false, 4, true>(a, st);
        case 13: return launch<DT_BF16, false, 5, true>(a, st);
        default: return -200;
    }
}
