// Large bfloat16 products through the vendor's GEMM library (hipBLASLt), called directly.
//
// The reference hands all its products to a library (cuBLAS: candle-core/src/cuda_backend/mod.rs:2260-2305); here
// the library takes the products of more rows than the kernels of this package are made for.  Through torch a
// product costs the host 18 us whatever its size (descriptors, layouts and the search for a kernel are made anew
// for every call), which is more than the GPU needs for the products of a small model: a prompt of 512 tokens at
// the smallest shape was bound by the host.  Here descriptors, layouts and the library's choice of kernel are
// made once for every shape (rows, features, k) and kept; a call is then one `hipblasLtMatmul`.
//
// The library is the one that the process already holds (torch brings its own copy, with its kernels beside it):
// it is opened by its path and its entry points are looked up by name, so nothing is linked against a second
// copy.  Only the header's types are used at compile time.
#include "common.h"
#include "api.h"

#if !__has_include(<hipblaslt/hipblaslt.h>)
// (an installation without the library's header: its products go through torch, and the caller is told so)
extern "C" int ia_vendor_gemm_init(const char*) { IA_CHECK(false, "vendor_gemm: built without the header of hipBLASLt"); }
extern "C" int ia_vendor_gemm_ready(void) { return 0; }
extern "C" int ia_vendor_gemm_bf16(void*, const void*, const void*, int, int, int, void*, long long, hipStream_t) {
    IA_CHECK(false, "vendor_gemm: built without the header of hipBLASLt");
}
#else
#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdint>
#include <mutex>
#include <unordered_map>

namespace {

struct Library {
    void* handle = nullptr;
    decltype(&hipblasLtCreate) create = nullptr;
    decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
    decltype(&hipblasLtMatmul) matmul = nullptr;
};

// What is kept for a shape: the operation, the three layouts and the library's first choice of kernel.
struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, x = nullptr, out = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
};

#define VENDOR_DEVICES 64
Library g_lib;
hipblasLtHandle_t g_handles[VENDOR_DEVICES];
std::unordered_map<uint64_t, Plan> g_plans[VENDOR_DEVICES];
std::mutex g_lock;

template <typename F>
bool lookup(F& fn, const char* name) {
    fn = (F)dlsym(g_lib.handle, name);
    return fn != nullptr;
}

}  // namespace

// Opens the library at `path` (the copy that the process has loaded already, or else loads it) and looks its
// entry points up.  0: ready.
extern "C" int ia_vendor_gemm_init(const char* path) {
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_lib.handle != nullptr) return 0;
    IA_CHECK(path != nullptr && path[0] != 0, "vendor_gemm: no path of the library");
    void* handle = dlopen(path, RTLD_NOW | RTLD_LOCAL | RTLD_NOLOAD);
    if (handle == nullptr) handle = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    IA_CHECK(handle != nullptr, "vendor_gemm: cannot open %s: %s", path, dlerror());
    g_lib.handle = handle;
    const bool ok = lookup(g_lib.create, "hipblasLtCreate") && lookup(g_lib.desc_create, "hipblasLtMatmulDescCreate") &&
                    lookup(g_lib.desc_set, "hipblasLtMatmulDescSetAttribute") &&
                    lookup(g_lib.layout_create, "hipblasLtMatrixLayoutCreate") &&
                    lookup(g_lib.pref_create, "hipblasLtMatmulPreferenceCreate") &&
                    lookup(g_lib.pref_set, "hipblasLtMatmulPreferenceSetAttribute") &&
                    lookup(g_lib.pref_destroy, "hipblasLtMatmulPreferenceDestroy") &&
                    lookup(g_lib.heuristic, "hipblasLtMatmulAlgoGetHeuristic") && lookup(g_lib.matmul, "hipblasLtMatmul");
    if (!ok) {
        g_lib = Library();
        IA_CHECK(false, "vendor_gemm: %s lacks an entry point of hipBLASLt", path);
    }
    return 0;
}

extern "C" int ia_vendor_gemm_ready(void) { return g_lib.handle != nullptr ? 1 : 0; }

// out [M, N] = x [M, K] . w [N, K]^T, all bfloat16 and contiguous, sums in 32-bit.  Returns 0, IA_VENDOR_NO_KERNEL when
// the library's search names no kernel for the shape (nothing has run then), or 1 with an error.  `workspace`: device memory of
// `workspace_bytes` for kernels that want some (a kernel is only chosen among those it suffices for).
// In the library's column-major terms: out^T [N x M] = w^T (w as [K x N], transposed) . x^T (x as [K x M]).
extern "C" int ia_vendor_gemm_bf16(void* out, const void* x, const void* w, int M, int N, int K, void* workspace,
                                   long long workspace_bytes, hipStream_t stream) {
    IA_CHECK(g_lib.handle != nullptr, "vendor_gemm: ia_vendor_gemm_init has not been called");
    IA_CHECK(M > 0 && N > 0 && K > 0 && M < (1 << 21) && N < (1 << 21) && K < (1 << 21), "vendor_gemm: bad sizes %d x %d x %d", M, N, K);
    IA_CHECK(workspace_bytes >= 0 && (workspace != nullptr || workspace_bytes == 0), "vendor_gemm: a workspace size without a workspace");
    int dev = 0;
    IA_CHECK(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < VENDOR_DEVICES, "vendor_gemm: no current device");
    Plan plan;
    {
        std::lock_guard<std::mutex> guard(g_lock);
        if (g_handles[dev] == nullptr)
            IA_CHECK(g_lib.create(&g_handles[dev]) == HIPBLAS_STATUS_SUCCESS, "vendor_gemm: hipblasLtCreate failed");
        const uint64_t key = ((uint64_t)M << 42) | ((uint64_t)N << 21) | (uint64_t)K;
        auto found = g_plans[dev].find(key);
        if (found == g_plans[dev].end()) {
            if (g_plans[dev].size() >= 8192) g_plans[dev].clear();          // (descriptors of shapes long gone)
            Plan p;
            IA_CHECK(g_lib.desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS, "vendor_gemm: no descriptor");
            const hipblasOperation_t t = HIPBLAS_OP_T, n = HIPBLAS_OP_N;
            IA_CHECK(g_lib.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &t, sizeof(t)) == HIPBLAS_STATUS_SUCCESS &&
                     g_lib.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &n, sizeof(n)) == HIPBLAS_STATUS_SUCCESS,
                     "vendor_gemm: the descriptor refuses the transposes");
            IA_CHECK(g_lib.layout_create(&p.w, HIP_R_16BF, (uint64_t)K, (uint64_t)N, (int64_t)K) == HIPBLAS_STATUS_SUCCESS &&
                     g_lib.layout_create(&p.x, HIP_R_16BF, (uint64_t)K, (uint64_t)M, (int64_t)K) == HIPBLAS_STATUS_SUCCESS &&
                     g_lib.layout_create(&p.out, HIP_R_16BF, (uint64_t)N, (uint64_t)M, (int64_t)N) == HIPBLAS_STATUS_SUCCESS,
                     "vendor_gemm: no layouts for %d x %d x %d", M, N, K);
            hipblasLtMatmulPreference_t pref = nullptr;
            IA_CHECK(g_lib.pref_create(&pref) == HIPBLAS_STATUS_SUCCESS, "vendor_gemm: no preference");
            const uint64_t most = (uint64_t)workspace_bytes;
            g_lib.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &most, sizeof(most));
            hipblasLtMatmulHeuristicResult_t result;
            int returned = 0;
            const hipblasStatus_t status = g_lib.heuristic(g_handles[dev], p.desc, p.w, p.x, p.out, p.out, pref, 1, &result, &returned);
            g_lib.pref_destroy(pref);
            if (!(status == HIPBLAS_STATUS_SUCCESS && returned >= 1 && result.state == HIPBLAS_STATUS_SUCCESS)) {
                // (a shape the library's search has nothing for, an odd k for instance: the caller goes another way)
                ia_set_error("vendor_gemm: the library names no kernel for %d x %d x %d (status %d)", M, N, K, (int)status);
                return IA_VENDOR_NO_KERNEL;
            }
            p.algo = result.algo;
            p.workspace = result.workspaceSize;
            found = g_plans[dev].emplace(key, p).first;
        }
        plan = found->second;
    }
    IA_CHECK(plan.workspace <= (size_t)workspace_bytes, "vendor_gemm: the chosen kernel wants %zu bytes of workspace, %lld are there",
             plan.workspace, workspace_bytes);
    const float one = 1.0f, zero = 0.0f;
    const hipblasStatus_t status = g_lib.matmul(g_handles[dev], plan.desc, &one, w, plan.w, x, plan.x, &zero, out, plan.out, out,
                                                plan.out, &plan.algo, workspace, (size_t)workspace_bytes, stream);
    IA_CHECK(status == HIPBLAS_STATUS_SUCCESS, "vendor_gemm: hipblasLtMatmul failed for %d x %d x %d (status %d)", M, N, K, (int)status);
    return 0;
}
#endif
