// int8 x int8 -> int32 GEMM on gfx950 MFMA with the dequant epilogue fused, D = Out(acc * xs[m] * ws[n] + bias[n]).
//
// Semantics follow the reference's fused CUTLASS kernel (csrc/vendor/cutlass_gemm_int8.cu:84-95 plain epilogue,
// :149-161 residual epilogue, :348-388 argument handling); the design is for CDNA4: A[M,K] and W[N,K] are both
// K-contiguous, which is exactly the operand shape of v_mfma_i32_32x32x32_i8 (each lane feeds 16 consecutive K bytes of
// one row), so tiles go global -> LDS as 16-byte chunks with an XOR swizzle and come back as ds_read_b128 fragments.
// W rides in src0 and A in src1, which leaves every lane holding runs of four consecutive n for one m: the epilogue
// stores 8-byte (bf16/f16) or 16-byte (f32) vectors straight from the accumulators.
#include "common.hpp"

namespace {

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

// Chunk swizzle: rows are BK bytes apart, so 8 consecutive rows of one chunk column would share banks; XOR the chunk
// index with row bits so that any 8 consecutive rows land on 8 distinct 16-byte bank groups.
template <int BK> __device__ __forceinline__ int swz(int row, int chunk) {
    return BK == 64 ? (chunk ^ ((row >> 1) & 3)) : (chunk ^ (row & 7));
}

// Workgroup -> tile.  Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so first renumber them
// XCD-contiguously, then walk tiles in panels of 4 tile rows so that the 32 workgroups an XCD runs at once cover a
// 4 x 8 patch of tiles and share A rows / W rows in that XCD's L2.
__device__ __forceinline__ void tile_of_block(int b, int nblocks, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int base = nblocks >> 3, rem = nblocks & 7;
    const int xcd = b & 7, idx = b >> 3;
    const int lin = xcd * base + (xcd < rem ? xcd : rem) + idx;
    constexpr int GM = 4;
    const int per_panel = GM * tiles_n;
    const int panel = lin / per_panel;
    const int first_m = panel * GM;
    const int rows = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int in_panel = lin - panel * per_panel;
    tm = first_m + in_panel % rows;
    tn = in_panel / rows;
}

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
        u.x = (uint32_t)f_to_bf16(v[0]) | ((uint32_t)f_to_bf16(v[1]) << 16);
        u.y = (uint32_t)f_to_bf16(v[2]) | ((uint32_t)f_to_bf16(v[3]) << 16);
        *reinterpret_cast<uint2*>((uint16_t*)p + i) = u;
    } else {
        uint2 u;
        u.x = (uint32_t)f_to_f16(v[0]) | ((uint32_t)f_to_f16(v[1]) << 16);
        u.y = (uint32_t)f_to_f16(v[2]) | ((uint32_t)f_to_f16(v[3]) << 16);
        *reinterpret_cast<uint2*>((uint16_t*)p + i) = u;
    }
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

template <class C, int OUT_DT, int EPI>
__global__ void __launch_bounds__(C::NT, C::OCC) int8_gemm_kernel(GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int BM = C::BM, BN = C::BN, BK = C::BK, NT = C::NT, CPR = C::CPR;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / C::WGN, wn = wave % C::WGN;

    int tm, tn;
    tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tm, tn);
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

    // Epilogue.  acc[in][im][4*rb + j] is (n = nb + 8*rb + 4*fhalf + j, m = mb + frow).
    const bool vec_ok = (p.N & 3) == 0;
#pragma unroll
    for (int im = 0; im < C::TM; ++im) {
        const int m = m0 + wm * C::WTM + im * 32 + frow;
        if (m >= p.M) continue;
        const float xs = EPI == EPI_ACC ? 0.f : p.xs[m];
#pragma unroll
        for (int in = 0; in < C::TN; ++in) {
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const int n = n0 + wn * C::WTN + in * 32 + rb * 8 + fhalf * 4;
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

// Tile shapes.  L: the large-shape workhorse, one workgroup per CU, each of 4 waves owns a 128x128 accumulator tile
// (256 accumulator registers).  M: 128x128 for mid-size problems and better wave quantization.  S: 64x64 for small M or N.
using CfgL = Cfg<256, 256, 64, 2, 2, 1>;
using CfgM = Cfg<128, 128, 64, 2, 2, 2>;
using CfgS = Cfg<64, 64, 64, 2, 2, 4>;

template <class C, int OUT_DT, int EPI>
int launch_cfg(GemmArgs a, hipStream_t st) {
    a.tiles_m = (a.M + C::BM - 1) / C::BM;
    a.tiles_n = (a.N + C::BN - 1) / C::BN;
    const int64_t nblocks = (int64_t)a.tiles_m * a.tiles_n;
    if (nblocks > 0x7fffffff) return -1;
    auto kern = int8_gemm_kernel<C, OUT_DT, EPI>;
    if (C::SMEM > 48 * 1024) {
        static bool once = false;  // benign race: the attribute is idempotent
        if (!once) {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM);
            if (e != hipSuccess) return (int)e;
            once = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(C::NT), C::SMEM, st, a);
    KCHECK();
    return 0;
}

// 0 = L, 1 = M, 2 = S; -1 = choose by shape.
int g_force_cfg = -1;

int choose_cfg(int64_t M, int64_t N) {
    if (g_force_cfg >= 0) return g_force_cfg;
    const int64_t tiles_l = ((M + 255) / 256) * ((N + 255) / 256);
    if (M >= 512 && N >= 512 && tiles_l >= 192) return 0;
    const int64_t tiles_m = ((M + 127) / 128) * ((N + 127) / 128);
    if (M > 64 && N > 64 && tiles_m >= 128) return 1;
    return 2;
}

template <int OUT_DT, int EPI>
int dispatch_cfg(const GemmArgs& a, hipStream_t st) {
    switch (choose_cfg(a.M, a.N)) {
        case 0: return launch_cfg<CfgL, OUT_DT, EPI>(a, st);
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
    return M <= 0x7fffffff && N <= 0x7fffffff && K <= 0x7fffffff && (K % 16) == 0 && M * N < (int64_t)1 << 40;
}

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

}  // namespace

GPU_API int gpu_int8_gemm(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias, void* D,
                          int64_t M, int64_t N, int64_t K, int out_dt, void* stream) {
    if (M == 0 || N == 0 || K == 0) return 0;  // csrc/vendor/cutlass_gemm_int8.cu:377
    if (out_dt < DT_F32 || out_dt > DT_BF16 || M < 0 || N < 0 || K < 0 || !shape_ok(M, N, K)) return -200;
    GemmArgs a{A, W, xs, ws, bias, nullptr, nullptr, D, (int)M, (int)N, (int)K, 0, 0};
    const int rc = dispatch_dt<EPI_PLAIN>(a, out_dt, (hipStream_t)stream);
    return rc < 0 ? -200 : rc;
}

GPU_API int gpu_int8_gemm_residual(const int8_t* A, const int8_t* W, const float* xs, const float* ws, const void* bias,
                                   const void* rscale, const void* resid, void* D, int64_t M, int64_t N, int64_t K,
                                   int out_dt, void* stream) {
    if (M == 0 || N == 0) return 0;                       // csrc/vendor/cutlass_gemm_int8.cu:353
    if (K == 0 || !rscale || !resid) return -201;         // :355-357
    if (out_dt < DT_F32 || out_dt > DT_BF16 || M < 0 || N < 0 || K < 0 || !shape_ok(M, N, K)) return -201;
    GemmArgs a{A, W, xs, ws, bias, rscale, resid, D, (int)M, (int)N, (int)K, 0, 0};
    const int rc = dispatch_dt<EPI_RESID>(a, out_dt, (hipStream_t)stream);
    return rc < 0 ? -201 : rc;
}

GPU_API int gpu_int8_gemm_acc(const int8_t* A, const int8_t* W, int32_t* acc, int64_t M, int64_t N, int64_t K, void* stream) {
    if (M == 0 || N == 0 || K == 0) return 0;
    if (M < 0 || N < 0 || K < 0 || !shape_ok(M, N, K)) return -200;
    GemmArgs a{A, W, nullptr, nullptr, nullptr, nullptr, nullptr, acc, (int)M, (int)N, (int)K, 0, 0};
    const int rc = dispatch_cfg<DT_F32, EPI_ACC>(a, (hipStream_t)stream);
    return rc < 0 ? -200 : rc;
}

// Test hook: force a tile configuration (0 = 256x256, 1 = 128x128, 2 = 64x64, -1 = automatic).
GPU_API int gpu_int8_gemm_force_config(int cfg) {
    g_force_cfg = cfg;
    return 0;
}

GPU_API int gpu_mfma_layout_probe(int32_t* out, void* stream) {
    hipLaunchKernelGGL(mfma_layout_probe_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, out);
    KCHECK();
    return 0;
}
