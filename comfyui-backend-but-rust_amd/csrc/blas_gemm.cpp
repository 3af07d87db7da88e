// Dense floating-point GEMM for the linears around the quantized path (timestep MLPs, first/last layers, the text
// encoders' fp32 GEMMs): a plan cache over hipBLASLt.  Replaces gpu_blas_init / gpu_gemm, csrc/gemm.cu:46-110.
// Built as a library of its own so that the int8 path does not depend on hipBLASLt being loadable.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdint>
#include <map>
#include <mutex>
#include <tuple>

#include "../../include/gpu_blas_api.h"

#define BLAS_API extern "C" __attribute__((visibility("default")))

namespace {

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };

hipDataType hip_type(int dt) { return dt == DT_F32 ? HIP_R_32F : dt == DT_F16 ? HIP_R_16F : HIP_R_16BF; }

// One matmul problem as hipBLASLt sees it, with the algorithm its heuristic picked.
struct Plan {
    hipblasLtMatmulDesc_t op = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, x = nullptr, y = nullptr;
    hipblasLtMatmulAlgo_t algo;
};

using Key = std::tuple<int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, int, int, bool>;

class Blas {
public:
    int init(size_t workspace_bytes) {
        std::lock_guard<std::mutex> hold(mu_);
        if (lt_) return 0;
        if (hipblasLtCreate(&lt_) != HIPBLAS_STATUS_SUCCESS) { lt_ = nullptr; return -1; }
        if (workspace_bytes && hipMalloc(&ws_, workspace_bytes) != hipSuccess) {
            hipblasLtDestroy(lt_);
            lt_ = nullptr;
            return -2;
        }
        ws_bytes_ = workspace_bytes;
        return 0;
    }
    bool ready() const { return lt_ != nullptr; }

    // Row-major D[M,N] = alpha * A[M,K] . op(B) + beta * D (+ bias[N]).  hipBLASLt is column-major: it computes
    // D^T[N,M] = op'(B)[N,K] . A^T[K,M], where the row-major buffers are read as their transposes.
    int run(const void* A, int64_t lda, const void* B, int64_t ldb, void* D, int64_t ldd, const void* bias, int64_t M, int64_t N,
            int64_t K, int transb, int in_dt, int out_dt, float alpha, float beta, hipStream_t st) {
        Plan plan;
        {
            std::lock_guard<std::mutex> hold(mu_);
            const Key key{M, N, K, lda, ldb, ldd, transb, in_dt, out_dt, bias != nullptr};
            auto it = plans_.find(key);
            if (it == plans_.end()) {
                Plan p;
                const int rc = make_plan(p, M, N, K, lda, ldb, ldd, transb, in_dt, out_dt, bias != nullptr);
                if (rc) return rc;
                it = plans_.emplace(key, p).first;
            }
            plan = it->second;
            if (bias) hipblasLtMatmulDescSetAttribute(plan.op, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
            // the launch stays under the lock: the bias pointer lives in the shared descriptor
            const hipblasStatus_t s = hipblasLtMatmul(lt_, plan.op, &alpha, B, plan.w, A, plan.x, &beta, D, plan.y, D, plan.y,
                                                      &plan.algo, ws_, ws_bytes_, st);
            return s == HIPBLAS_STATUS_SUCCESS ? 0 : -(int)s - 1000;
        }
    }

private:
    int make_plan(Plan& p, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldd, int transb, int in_dt,
                  int out_dt, bool has_bias) {
        const hipDataType tin = hip_type(in_dt), tout = hip_type(out_dt);
        // fp32 accumulation for every input type; plain HIPBLAS_COMPUTE_32F never narrows fp32 inputs
        if (hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return -101;
        const hipblasOperation_t opw = transb ? HIPBLAS_OP_T : HIPBLAS_OP_N, opx = HIPBLAS_OP_N;
        hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSA, &opw, sizeof(opw));
        hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSB, &opx, sizeof(opx));
        if (has_bias) {
            const hipblasLtEpilogue_t ep = HIPBLASLT_EPILOGUE_BIAS;
            hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_EPILOGUE, &ep, sizeof(ep));
            hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &tout, sizeof(tout));
        }
        // a Linear weight [N,K] row-major is a K x N column-major matrix to transpose; a [K,N] one is N x K as it lies
        if (transb) hipblasLtMatrixLayoutCreate(&p.w, tin, K, N, ldb);
        else hipblasLtMatrixLayoutCreate(&p.w, tin, N, K, ldb);
        hipblasLtMatrixLayoutCreate(&p.x, tin, K, M, lda);
        hipblasLtMatrixLayoutCreate(&p.y, tout, N, M, ldd);
        hipblasLtMatmulPreference_t pref;
        hipblasLtMatmulPreferenceCreate(&pref);
        const uint64_t cap = ws_bytes_;
        hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &cap, sizeof(cap));
        hipblasLtMatmulHeuristicResult_t found[4];
        int n = 0;
        const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(lt_, p.op, p.w, p.x, p.y, p.y, pref, 4, found, &n);
        hipblasLtMatmulPreferenceDestroy(pref);
        if (s != HIPBLAS_STATUS_SUCCESS || n == 0) {
            hipblasLtMatrixLayoutDestroy(p.w);
            hipblasLtMatrixLayoutDestroy(p.x);
            hipblasLtMatrixLayoutDestroy(p.y);
            hipblasLtMatmulDescDestroy(p.op);
            return -101;
        }
        p.algo = found[0].algo;
        return 0;
    }

    std::mutex mu_;
    hipblasLtHandle_t lt_ = nullptr;
    void* ws_ = nullptr;
    size_t ws_bytes_ = 0;
    std::map<Key, Plan> plans_;
};

Blas g_blas;

}  // namespace

BLAS_API int gpu_blas_init(size_t workspace_bytes) { return g_blas.init(workspace_bytes); }

BLAS_API int gpu_gemm(const void* A, int64_t lda, const void* B, int64_t ldb, void* D, int64_t ldd, const void* bias, int64_t M,
                      int64_t N, int64_t K, int transb, int in_dt, int out_dt, float alpha, float beta, void* stream) {
    if (!g_blas.ready()) return -100;
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || in_dt < 0 || in_dt > 2 || out_dt < 0 || out_dt > 2) return -101;
    return g_blas.run(A, lda, B, ldb, D, ldd, bias, M, N, K, transb, in_dt, out_dt, alpha, beta, (hipStream_t)stream);
}
