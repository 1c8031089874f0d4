/*
 * Plain linear layers through the vendor GEMM library, when it is present.
 *
 * iris_dev_linear_f32 / _bf16 (iris_dev.h:48-53) are plain GEMMs, y = x W^T
 * with bf16 operands and f32 accumulation; the reference backend hands them
 * to cuBLAS / hipBLAS (iris_cuda.cu:456-505). Here they go to hipBLASLt,
 * which on this GPU sustains 1.1-1.4 PFLOP/s on the models' shapes against
 * 0.7-0.9 for this library's own MFMA kernel (gemm_conv_gfx950.hip). The own
 * kernel stays as the path for everything the library refuses and for hosts
 * without it: hipBLASLt is opened with dlopen at the first call, so
 * libiris_dev.so itself does not depend on it.
 *
 * Column-major reading of the row-major operands: y^T [out x rows] =
 * W [out x in] . x^T [in x rows], i.e. m = out, n = rows, k = in, A = W stored
 * as [k x m] with op T, B = x stored as [k x n] with op N, D = y with
 * ld = out: the library's "TN" case.
 *
 * One plan (descriptors + the heuristic's first algorithm) is kept per
 * distinct (out, rows, in, output type); a model uses a handful.
 */
#include <hip/hip_runtime_api.h>
#include <hipblaslt/hipblaslt.h>

#include <dlfcn.h>
#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "iris_kernels_hip.h"

namespace {

struct Api {
    decltype(&hipblasLtCreate) create;
    decltype(&hipblasLtDestroy) destroy;
    decltype(&hipblasLtMatmulDescCreate) desc_create;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic;
    decltype(&hipblasLtMatmul) matmul;
};

struct Plan {
    int out, rows, in, out_bf16;
    bool usable;
    hipblasLtMatmulDesc_t desc;
    hipblasLtMatrixLayout_t a, b, d;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace;
};

constexpr size_t WORKSPACE_BYTES = (size_t)64 << 20;

int g_state = 0;                 /* 0 not tried, 1 ready, -1 unavailable */
void *g_dl = nullptr;
Api g_api;
hipblasLtHandle_t g_handle = nullptr;
void *g_workspace = nullptr;
std::vector<Plan> g_plans;

template <typename F>
bool sym(F &f, const char *name) {
    f = reinterpret_cast<F>(dlsym(g_dl, name));
    return f != nullptr;
}

bool open_library() {
    if (g_state) return g_state > 0;
    g_state = -1;
    for (const char *name : {"libhipblaslt.so.1", "libhipblaslt.so", "/opt/rocm/lib/libhipblaslt.so.1"}) {
        g_dl = dlopen(name, RTLD_NOW | RTLD_LOCAL);
        if (g_dl) break;
    }
    if (!g_dl) return false;
    Api &a = g_api;
    if (!(sym(a.create, "hipblasLtCreate") && sym(a.destroy, "hipblasLtDestroy") &&
          sym(a.desc_create, "hipblasLtMatmulDescCreate") && sym(a.desc_destroy, "hipblasLtMatmulDescDestroy") &&
          sym(a.desc_set, "hipblasLtMatmulDescSetAttribute") && sym(a.layout_create, "hipblasLtMatrixLayoutCreate") &&
          sym(a.layout_destroy, "hipblasLtMatrixLayoutDestroy") && sym(a.pref_create, "hipblasLtMatmulPreferenceCreate") &&
          sym(a.pref_destroy, "hipblasLtMatmulPreferenceDestroy") &&
          sym(a.pref_set, "hipblasLtMatmulPreferenceSetAttribute") &&
          sym(a.heuristic, "hipblasLtMatmulAlgoGetHeuristic") && sym(a.matmul, "hipblasLtMatmul")))
        return false;
    if (a.create(&g_handle) != HIPBLAS_STATUS_SUCCESS) return false;
    if (hipMalloc(&g_workspace, WORKSPACE_BYTES) != hipSuccess) {
        (void)hipGetLastError();
        a.destroy(g_handle);
        g_handle = nullptr;
        g_workspace = nullptr;
        return false;
    }
    g_state = 1;
    return true;
}

void destroy_plan(Plan &p) {
    if (p.desc) g_api.desc_destroy(p.desc);
    if (p.a) g_api.layout_destroy(p.a);
    if (p.b) g_api.layout_destroy(p.b);
    if (p.d) g_api.layout_destroy(p.d);
    p.desc = nullptr;
    p.a = p.b = p.d = nullptr;
}

Plan make_plan(int out, int rows, int in, int out_bf16) {
    Plan p{};
    p.out = out; p.rows = rows; p.in = in; p.out_bf16 = out_bf16;
    const Api &a = g_api;
    const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    hipblasLtMatmulPreference_t pref = nullptr;
    hipblasLtMatmulHeuristicResult_t found{};
    int n_found = 0;
    const uint64_t ws = WORKSPACE_BYTES;
    bool ok = a.desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS &&
              a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof op_t) == HIPBLAS_STATUS_SUCCESS &&
              a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof op_n) == HIPBLAS_STATUS_SUCCESS &&
              a.layout_create(&p.a, HIP_R_16BF, (uint64_t)in, (uint64_t)out, in) == HIPBLAS_STATUS_SUCCESS &&
              a.layout_create(&p.b, HIP_R_16BF, (uint64_t)in, (uint64_t)rows, in) == HIPBLAS_STATUS_SUCCESS &&
              a.layout_create(&p.d, out_bf16 ? HIP_R_16BF : HIP_R_32F, (uint64_t)out, (uint64_t)rows, out) ==
                  HIPBLAS_STATUS_SUCCESS &&
              a.pref_create(&pref) == HIPBLAS_STATUS_SUCCESS &&
              a.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof ws) == HIPBLAS_STATUS_SUCCESS &&
              a.heuristic(g_handle, p.desc, p.a, p.b, p.d, p.d, pref, 1, &found, &n_found) == HIPBLAS_STATUS_SUCCESS &&
              n_found > 0 && found.state == HIPBLAS_STATUS_SUCCESS && found.workspaceSize <= WORKSPACE_BYTES;
    if (pref) a.pref_destroy(pref);
    if (ok) {
        p.algo = found.algo;
        p.workspace = found.workspaceSize;
        p.usable = true;
    } else {
        destroy_plan(p);          /* remembered as unusable: the caller's own kernel takes this shape */
    }
    return p;
}

}  // namespace

/* 0 = the product was enqueued on `stream`; 1 = not handled (library absent, or it offers no
 * algorithm for this problem): the caller runs its own kernel instead. */
extern "C" int iris_lt_linear(void *stream, void *y, int out_bf16, const uint16_t *x, const uint16_t *W,
                              int rows, int in, int out) {
    if (rows <= 0 || in <= 0 || out <= 0) return 1;
    if (!open_library()) return 1;
    Plan *plan = nullptr;
    for (Plan &p : g_plans)
        if (p.out == out && p.rows == rows && p.in == in && p.out_bf16 == out_bf16) { plan = &p; break; }
    if (!plan) {
        g_plans.push_back(make_plan(out, rows, in, out_bf16));
        plan = &g_plans.back();
    }
    if (!plan->usable) return 1;
    const float alpha = 1.0f, beta = 0.0f;
    const hipblasStatus_t st =
        g_api.matmul(g_handle, plan->desc, &alpha, W, plan->a, x, plan->b, &beta, y, plan->d, y, plan->d, &plan->algo,
                     g_workspace, plan->workspace, (hipStream_t)stream);
    if (st != HIPBLAS_STATUS_SUCCESS) {
        plan->usable = false;     /* do not ask again; nothing was enqueued */
        return 1;
    }
    return 0;
}

/* 1 when the library has been opened and is in use */
extern "C" int iris_lt_available(void) { return open_library() ? 1 : 0; }

/* Releases plans, workspace and the handle (the caller has synchronised the stream). The
 * library stays mapped: unloading it while the HIP runtime still knows its code objects is
 * not worth the risk for a few MB of address space. */
extern "C" void iris_lt_release(void) {
    if (g_state <= 0) return;
    for (Plan &p : g_plans) destroy_plan(p);
    g_plans.clear();
    if (g_workspace) (void)hipFree(g_workspace);
    g_workspace = nullptr;
    if (g_handle) g_api.destroy(g_handle);
    g_handle = nullptr;
    g_state = 0;                  /* a later iris_dev_init() may open it again */
}
