// Dense fp16 mat-muls of long prompt chunks through hipBLASLt: y[t][row] = W[row][:] . xn[t][:] with fp32 accumulation and
// fp32 output.  The reference hands the same products to cuBLAS (ggml_cuda_op_mul_mat_cublas, ggml-cuda.cu:7662-7756); they are
// plain library GEMMs with nothing of the sparse path in them.  The epilogues of pi_k_gemm_f16 are kept: a single residual rides
// along as the C operand (beta = 1), the second residual, ReLU and the fp16 copy of the result run as one small kernel.
#include "runtime.hpp"
#include "device_utils.hpp"
#include "../../include/powerinfer_hip.h"

#include <hip/hip_fp16.h>
#include <hipblaslt/hipblaslt.h>

#include <vector>

namespace {

struct Plan {
    int rows, cols, T;
    bool with_c;
    uint64_t last_use;
    hipblasLtMatmulDesc_t op;
    hipblasLtMatrixLayout_t a, b, c;
    hipblasLtMatmulHeuristicResult_t heur;
};

// y = relu(y) | y += add2, and the fp16 copy, in one pass over the result
__global__ void gemm_lib_post_kernel(float * __restrict__ y, const float * __restrict__ add2, __half * __restrict__ y16, int relu, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        float v = y[i];
        if (relu) v = fmaxf(v, 0.0f);
        if (add2) v = __fadd_rn(v, add2[i]);
        if (relu || add2) y[i] = v;
        if (y16) y16[i] = __float2half_rn(v);
    }
}

}  // namespace

struct pi_gemm_lib {
    hipblasLtHandle_t handle = nullptr;
    void * ws = nullptr;
    size_t ws_bytes = 0;
    std::vector<Plan> plans;          // at most kMaxPlans; the least recently used one makes room for a new shape
    uint64_t clock = 0;
};
constexpr size_t kMaxPlans = 64;

static void destroy_plan(Plan & p) {
    if (p.a) (void)hipblasLtMatrixLayoutDestroy(p.a);
    if (p.b) (void)hipblasLtMatrixLayoutDestroy(p.b);
    if (p.c) (void)hipblasLtMatrixLayoutDestroy(p.c);
    if (p.op) (void)hipblasLtMatmulDescDestroy(p.op);
    p.a = p.b = p.c = nullptr; p.op = nullptr;
}

#define PI_TRY(expr) do { int _rc = (expr); if (_rc != PI_OK) return _rc; } while (0)
#define PI_LT_TRY(expr)                                                                                                 \
    do {                                                                                                                \
        const hipblasStatus_t s_ = (expr);                                                                              \
        if (s_ != HIPBLAS_STATUS_SUCCESS) {                                                                             \
            char msg_[160];                                                                                             \
            snprintf(msg_, sizeof msg_, "%s: hipBLASLt status %d", #expr, (int)s_);                                     \
            return pi::fail(PI_E_HIP, msg_);                                                                            \
        }                                                                                                               \
    } while (0)

// A plan is used only to enqueue its product (the descriptors are read at enqueue time), so evicting one between two calls is safe.
// Prompt remainders of every length ask for their own plans: a server would otherwise run into the cap after a few dozen prompts.
static int make_plan(pi_gemm_lib * g, int rows, int cols, int T, bool with_c, Plan ** out) {
    for (Plan & p : g->plans)
        if (p.rows == rows && p.cols == cols && p.T == T && p.with_c == with_c) { p.last_use = ++g->clock; *out = &p; return PI_OK; }
    Plan p{};
    p.rows = rows; p.cols = cols; p.T = T; p.with_c = with_c;
    const auto build = [&]() -> int {
        // column-major view: D (rows x T, ld rows) = W^T-as-stored (cols x rows, ld cols) transposed  x  xn-as-stored (cols x T, ld cols)
        PI_LT_TRY(hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F));
        const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
        PI_LT_TRY(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof ta));
        PI_LT_TRY(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof tb));
        PI_LT_TRY(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16F, cols, rows, cols));
        PI_LT_TRY(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16F, cols, T, cols));
        PI_LT_TRY(hipblasLtMatrixLayoutCreate(&p.c, HIP_R_32F, rows, T, rows));
        hipblasLtMatmulPreference_t pref;
        PI_LT_TRY(hipblasLtMatmulPreferenceCreate(&pref));
        const uint64_t wsb = g->ws_bytes;
        hipblasStatus_t hs = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &wsb, sizeof wsb);
        int found = 0;
        if (hs == HIPBLAS_STATUS_SUCCESS) hs = hipblasLtMatmulAlgoGetHeuristic(g->handle, p.op, p.a, p.b, p.c, p.c, pref, 1, &p.heur, &found);
        (void)hipblasLtMatmulPreferenceDestroy(pref);
        if (hs != HIPBLAS_STATUS_SUCCESS || found < 1) return pi::fail(PI_E_UNSUPPORTED, "pi_gemm_lib_f16: hipBLASLt offers no kernel for this shape");
        return PI_OK;
    };
    const int rc = build();
    if (rc != PI_OK) { destroy_plan(p); return rc; }
    p.last_use = ++g->clock;
    if (g->plans.size() < kMaxPlans) {
        g->plans.push_back(p);
        *out = &g->plans.back();
    } else {
        size_t victim = 0;
        for (size_t i = 1; i < g->plans.size(); ++i) if (g->plans[i].last_use < g->plans[victim].last_use) victim = i;
        destroy_plan(g->plans[victim]);
        g->plans[victim] = p;
        *out = &g->plans[victim];
    }
    return PI_OK;
}

extern "C" {

pi_gemm_lib * pi_gemm_lib_create(size_t workspace_bytes) {
    pi_gemm_lib * g = new pi_gemm_lib;
    if (hipblasLtCreate(&g->handle) != HIPBLAS_STATUS_SUCCESS) { pi::set_error("hipblasLtCreate failed"); delete g; return nullptr; }
    g->ws_bytes = workspace_bytes;
    if (workspace_bytes) {
        g->ws = pi_malloc(workspace_bytes);
        if (!g->ws) { (void)hipblasLtDestroy(g->handle); delete g; return nullptr; }
    }
    g->plans.reserve(kMaxPlans);
    return g;
}

int pi_gemm_lib_destroy(pi_gemm_lib * g) {
    if (!g) return PI_OK;
    for (Plan & p : g->plans) destroy_plan(p);
    if (g->ws) { (void)pi_sync(); (void)pi_free(g->ws); }
    (void)hipblasLtDestroy(g->handle);
    delete g;
    return PI_OK;
}

int pi_gemm_lib_f16(pi_gemm_lib * g, const void * W_f16, int rows, int cols, const void * xn_f16, int T, int epilogue,
                    const float * add1, const float * add2, float * y, void * y_f16, pi_stream_t stream) {
    if (!g || !W_f16 || !xn_f16 || !y || rows <= 0 || cols <= 0 || T <= 0) return pi::fail(PI_E_ARG, "pi_gemm_lib_f16: bad arguments");
    if (epilogue < PI_EPI_NONE || epilogue > PI_EPI_ADD2) return pi::fail(PI_E_ARG, "pi_gemm_lib_f16: unknown epilogue");
    if ((epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2)) return pi::fail(PI_E_ARG, "pi_gemm_lib_f16: residual operand missing");
    const bool with_c = epilogue >= PI_EPI_ADD;
    Plan * p = nullptr;
    PI_TRY(make_plan(g, rows, cols, T, with_c, &p));
    const float alpha = 1.0f, beta = with_c ? 1.0f : 0.0f;
    hipStream_t st = (hipStream_t)stream;
    PI_LT_TRY(hipblasLtMatmul(g->handle, p->op, &alpha, W_f16, p->a, xn_f16, p->b, &beta, with_c ? (const void *)add1 : (const void *)y, p->c, y, p->c,
                              &p->heur.algo, g->ws, g->ws_bytes, st));
    const bool relu = epilogue == PI_EPI_RELU;
    if (relu || epilogue == PI_EPI_ADD2 || y_f16) {
        const size_t n = (size_t)rows * T;
        size_t blocks = (n + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(gemm_lib_post_kernel, dim3((unsigned)blocks), dim3(256), 0, st, y, epilogue == PI_EPI_ADD2 ? add2 : nullptr, (__half *)y_f16, relu ? 1 : 0, n);
        return pi::check_launch("pi_gemm_lib_f16");
    }
    return PI_OK;
}

}  // extern "C"
