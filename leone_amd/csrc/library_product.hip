// The library's matrix product for prompt portions (more rows than the own kernels take), with the library's
// algorithm chosen by measurement.
//
// The reference leaves a prompt's products to the vendor library (cuBLASLt: crates/leone-cuda/cuda/ie_cuda.cu,
// the `ie_gemm_*` entry points); here that is hipBLASLt.  The library offers hundreds of algorithms for one
// problem and names one by a heuristic; for the shapes of a decoder layer the heuristic's choice is up to 15 %
// slower than the best of its own candidates, so `leone_library_product_tune` times the candidates on the
// caller's operands once and `leone_library_product` then runs the winner for exactly that problem.  Problems
// that were not tuned are not served here: the caller keeps its ordinary call of the library for them.
//
// hipBLASLt is looked up at run time (the copy already in the process if there is one), through its C interface
// only; nothing here links against it, and without it the entry points say so.
//
//   Y[M,N] (+)= X[M,K] . W[N,K]^T      X, W bfloat16 row-major; Y bfloat16 or float32; float accumulation
#include "common.h"
#include "leone_hip.h"

#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

namespace leone {

namespace {

struct Library {
    decltype(&hipblasLtCreate) create = nullptr;
    decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
    decltype(&hipblasLtMatmul) matmul = nullptr;
    // the library's C++ extension, by its mangled names: every algorithm it has, not only what its heuristic
    // lists; optional
    decltype(&hipblaslt_ext::getAllAlgos) all_algorithms = nullptr;
    decltype(&hipblaslt_ext::matmulIsAlgoSupported) supported = nullptr;
    bool ok = false;
};

const Library& lt() {
    static const Library lib = [] {
        Library l;
        void* h = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_GLOBAL);
        if (!h) h = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_GLOBAL);
        if (!h) return l;
#define LEONE_LT_SYMBOL(field, name)                                   \
    l.field = reinterpret_cast<decltype(l.field)>(dlsym(h, #name));    \
    if (!l.field) return l;
        LEONE_LT_SYMBOL(create, hipblasLtCreate)
        LEONE_LT_SYMBOL(desc_create, hipblasLtMatmulDescCreate)
        LEONE_LT_SYMBOL(desc_destroy, hipblasLtMatmulDescDestroy)
        LEONE_LT_SYMBOL(desc_set, hipblasLtMatmulDescSetAttribute)
        LEONE_LT_SYMBOL(layout_create, hipblasLtMatrixLayoutCreate)
        LEONE_LT_SYMBOL(layout_destroy, hipblasLtMatrixLayoutDestroy)
        LEONE_LT_SYMBOL(pref_create, hipblasLtMatmulPreferenceCreate)
        LEONE_LT_SYMBOL(pref_destroy, hipblasLtMatmulPreferenceDestroy)
        LEONE_LT_SYMBOL(pref_set, hipblasLtMatmulPreferenceSetAttribute)
        LEONE_LT_SYMBOL(heuristic, hipblasLtMatmulAlgoGetHeuristic)
        LEONE_LT_SYMBOL(matmul, hipblasLtMatmul)
#undef LEONE_LT_SYMBOL
        l.all_algorithms = reinterpret_cast<decltype(l.all_algorithms)>(dlsym(
            h, "_ZN13hipblaslt_ext11getAllAlgosEPvNS_8GemmTypeE18hipblasOperation_tS2_11hipDataTypeS3_S3_S3_"
               "20hipblasComputeType_tRSt6vectorI33_hipblasLtMatmulHeuristicResult_tSaIS6_EE"));
        l.supported = reinterpret_cast<decltype(l.supported)>(dlsym(
            h, "_ZN13hipblaslt_ext21matmulIsAlgoSupportedEPvP27hipblasLtMatmulDescOpaque_tPKvP29hipblasLtMatrixLayout"
               "Opaque_tS6_S4_S6_S6_R22_hipblasLtMatmulAlgo_tRm"));
        if (!l.all_algorithms || !l.supported) l.all_algorithms = nullptr, l.supported = nullptr;
        l.ok = true;
        return l;
    }();
    return lib;
}

constexpr size_t kWorkspaceBytes = 64u << 20;      // what the library's algorithms may use beside the operands
constexpr int kMaxCandidates = 1024;

// One device's handle and workspace; made at the device's first call and kept until the process ends.
struct Device {
    hipblasLtHandle_t handle = nullptr;
    void* workspace = nullptr;
};

// A problem: the three layouts, the operation, and the algorithm that won the measurement.
struct Problem {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, x = nullptr, y = nullptr;
    hipblasLtMatmulAlgo_t algo{};
    bool tuned = false;
};

using Key = std::tuple<int, int, int, int, int, int>;   // device, m, n, k, out type, accumulate

std::mutex g_mutex;
std::map<int, Device> g_devices;
std::map<Key, Problem> g_problems;

bool device_state(int device, Device** out) {
    Device& d = g_devices[device];
    if (!d.handle) {
        if (lt().create(&d.handle) != HIPBLAS_STATUS_SUCCESS) {
            set_error("library product: the library gave no handle");
            return false;
        }
        if (hipMalloc(&d.workspace, kWorkspaceBytes) != hipSuccess) {
            set_error("library product: no memory for the library's workspace");
            return false;
        }
    }
    *out = &d;
    return true;
}

bool make_problem(int m, int n, int k, int out_dtype, Problem* p) {
    const Library& l = lt();
    const hipDataType out = out_dtype == kF32 ? HIP_R_32F : HIP_R_16BF;
    // The library counts in columns: Y^T [N,M] = W [N,K] (a K x N matrix, transposed) . X^T [K,M].
    const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
    bool ok = l.desc_create(&p->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && l.desc_set(p->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && l.desc_set(p->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && l.layout_create(&p->w, HIP_R_16BF, k, n, k) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && l.layout_create(&p->x, HIP_R_16BF, k, m, k) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && l.layout_create(&p->y, out, n, m, n) == HIPBLAS_STATUS_SUCCESS;
    if (!ok) set_error("library product: the library refused the description of %d x %d x %d", m, n, k);
    return ok;
}

void drop_problem(Problem* p) {
    const Library& l = lt();
    if (p->y) l.layout_destroy(p->y);
    if (p->x) l.layout_destroy(p->x);
    if (p->w) l.layout_destroy(p->w);
    if (p->desc) l.desc_destroy(p->desc);
    *p = Problem{};
}

hipblasStatus_t run(const Device& d, const Problem& p, const hipblasLtMatmulAlgo_t& algo, const void* x, const void* w,
                    void* y, int accumulate, hipStream_t stream) {
    const float one = 1.f, beta = accumulate ? 1.f : 0.f;
    return lt().matmul(d.handle, p.desc, &one, w, p.w, x, p.x, &beta, y, p.y, y, p.y, &algo, d.workspace,
                       kWorkspaceBytes, stream);
}

bool checked_shape(const char* who, int m, int n, int k, int out_dtype) {
    if (!lt().ok) {
        set_error("%s: hipBLASLt could not be loaded", who);
        return false;
    }
    if (m <= 0 || n <= 0 || k <= 0 || k % 8 != 0 || (out_dtype != kF32 && out_dtype != kBF16)) {
        set_error("%s: %d x %d x %d (inner size a multiple of 8), output bfloat16 or float32", who, m, n, k);
        return false;
    }
    return true;
}

}  // namespace

}  // namespace leone

using namespace leone;

extern "C" int leone_library_product_available() { return !lt().ok ? 0 : lt().all_algorithms ? 2 : 1; }

extern "C" int leone_library_product_tuned(int m, int n, int k, int out_dtype, int accumulate) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lock(g_mutex);
    auto found = g_problems.find(Key{device, m, n, k, out_dtype, accumulate ? 1 : 0});
    return found != g_problems.end() && found->second.tuned ? 1 : 0;
}

extern "C" int leone_library_product_forget(int m, int n, int k, int out_dtype, int accumulate) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return 1;
    std::lock_guard<std::mutex> lock(g_mutex);
    auto found = g_problems.find(Key{device, m, n, k, out_dtype, accumulate ? 1 : 0});
    if (found != g_problems.end()) {
        drop_problem(&found->second);
        g_problems.erase(found);
    }
    return 0;
}

extern "C" int leone_library_product(const void* x, const void* w, void* y, int m, int n, int k, int out_dtype,
                                     int accumulate, hipStream_t stream) {
    LEONE_REQUIRE(x && w && y, "library product: null pointer");
    if (!checked_shape("library product", m, n, k, out_dtype)) return 1;
    int device = 0;
    LEONE_REQUIRE(hipGetDevice(&device) == hipSuccess, "library product: no current device");
    std::lock_guard<std::mutex> lock(g_mutex);
    auto found = g_problems.find(Key{device, m, n, k, out_dtype, accumulate ? 1 : 0});
    LEONE_REQUIRE(found != g_problems.end() && found->second.tuned,
                  "library product: %d x %d x %d was not tuned on this device", m, n, k);
    Device* d = nullptr;
    if (!device_state(device, &d)) return 1;
    const hipblasStatus_t status = run(*d, found->second, found->second.algo, x, w, y, accumulate, stream);
    LEONE_REQUIRE(status == HIPBLAS_STATUS_SUCCESS, "library product: the library returned status %d", static_cast<int>(status));
    return 0;
}

extern "C" int leone_library_product_tune(const void* x, const void* const* ws, int n_ws, void* y, int m, int n, int k,
                                          int out_dtype, int accumulate, int max_candidates, int every_algorithm,
                                          float* first_us, float* best_us, int* candidates_timed, hipStream_t stream) {
    LEONE_REQUIRE(x && ws && y && n_ws > 0, "library product tune: null pointer");
    for (int i = 0; i < n_ws; ++i) LEONE_REQUIRE(ws[i], "library product tune: weight %d is null", i);
    if (!checked_shape("library product tune", m, n, k, out_dtype)) return 1;
    LEONE_REQUIRE(max_candidates >= 1 && max_candidates <= kMaxCandidates,
                  "library product tune: 1 to %d candidates, not %d", kMaxCandidates, max_candidates);
    int device = 0;
    LEONE_REQUIRE(hipGetDevice(&device) == hipSuccess, "library product tune: no current device");
    std::lock_guard<std::mutex> lock(g_mutex);
    Device* d = nullptr;
    if (!device_state(device, &d)) return 1;
    const Key key{device, m, n, k, out_dtype, accumulate ? 1 : 0};
    Problem& p = g_problems[key];
    if (!p.desc && !make_problem(m, n, k, out_dtype, &p)) {
        drop_problem(&p);
        g_problems.erase(key);
        return 1;
    }
    p.tuned = false;
    const Library& l = lt();
    hipblasLtMatmulPreference_t pref = nullptr;
    std::vector<hipblasLtMatmulHeuristicResult_t> found(max_candidates);
    int n_found = 0;
    bool ok = l.pref_create(&pref) == HIPBLAS_STATUS_SUCCESS;
    const size_t workspace = kWorkspaceBytes;
    ok = ok && l.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace, sizeof(workspace)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && l.heuristic(d->handle, p.desc, p.w, p.x, p.y, p.y, pref, max_candidates, found.data(), &n_found) == HIPBLAS_STATUS_SUCCESS;
    if (pref) l.pref_destroy(pref);
    if (ok && n_found > 0 && every_algorithm && l.all_algorithms) {
        // every algorithm the library has for these types that takes this problem, after the heuristic's list
        // (whose first stays first)
        found.resize(n_found);
        std::vector<hipblasLtMatmulHeuristicResult_t> all;
        const hipDataType out = out_dtype == kF32 ? HIP_R_32F : HIP_R_16BF;
        if (l.all_algorithms(d->handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, HIP_R_16BF,
                             HIP_R_16BF, out, out, HIPBLAS_COMPUTE_32F, all) == HIPBLAS_STATUS_SUCCESS) {
            const float one = 1.f, beta = accumulate ? 1.f : 0.f;
            for (auto& candidate : all) {
                size_t needs = 0;
                if (l.supported(d->handle, p.desc, &one, p.w, p.x, &beta, p.y, p.y, candidate.algo, needs) != HIPBLAS_STATUS_SUCCESS ||
                    needs > kWorkspaceBytes)
                    continue;
                candidate.state = HIPBLAS_STATUS_SUCCESS;
                candidate.workspaceSize = needs;
                found.push_back(candidate);
            }
            n_found = static_cast<int>(found.size());
        }
    }
    if (!ok || n_found <= 0) {
        set_error("library product tune: the library names no algorithm for %d x %d x %d", m, n, k);
        drop_problem(&p);
        g_problems.erase(key);
        return 1;
    }
    hipEvent_t begin = nullptr, end = nullptr;
    LEONE_REQUIRE(hipEventCreate(&begin) == hipSuccess && hipEventCreate(&end) == hipSuccess,
                  "library product tune: no events");
    // The weights take turns, as the layers of a model do: none of them is still in a cache when it is read.
    int turn = 0;
    auto time_of = [&](const hipblasLtMatmulAlgo_t& algo, int warm, int reps) -> float {
        for (int i = 0; i < warm; ++i)
            if (run(*d, p, algo, x, ws[turn++ % n_ws], y, accumulate, stream) != HIPBLAS_STATUS_SUCCESS) return -1.f;
        if (hipEventRecord(begin, stream) != hipSuccess) return -1.f;
        for (int i = 0; i < reps; ++i)
            if (run(*d, p, algo, x, ws[turn++ % n_ws], y, accumulate, stream) != HIPBLAS_STATUS_SUCCESS) return -1.f;
        float ms = 0.f;
        if (hipEventRecord(end, stream) != hipSuccess || hipEventSynchronize(end) != hipSuccess ||
            hipEventElapsedTime(&ms, begin, end) != hipSuccess)
            return -1.f;
        return ms * 1e3f / static_cast<float>(reps);
    };
    std::vector<std::pair<float, int>> timed;
    for (int i = 0; i < n_found; ++i) {
        if (found[i].state != HIPBLAS_STATUS_SUCCESS || found[i].workspaceSize > kWorkspaceBytes) continue;
        const float us = time_of(found[i].algo, 1, 3);
        if (us > 0.f) timed.push_back({us, i});
    }
    std::sort(timed.begin(), timed.end());
    // the heuristic's own choice and the eight that looked best, measured at length
    const float first = time_of(found[0].algo, 2, 16);
    float best = first;
    int best_index = first > 0.f ? 0 : -1;
    for (size_t i = 0; i < timed.size() && i < 8; ++i) {
        if (timed[i].second == 0) continue;
        const float us = time_of(found[timed[i].second].algo, 2, 16);
        if (us > 0.f && (best_index < 0 || us < best)) {
            best = us;
            best_index = timed[i].second;
        }
    }
    hipEventDestroy(begin);
    hipEventDestroy(end);
    if (best_index < 0) {
        set_error("library product tune: no algorithm ran for %d x %d x %d", m, n, k);
        drop_problem(&p);
        g_problems.erase(key);
        return 1;
    }
    p.algo = found[best_index].algo;
    p.tuned = true;
    if (first_us) *first_us = first;
    if (best_us) *best_us = best;
    if (candidates_timed) *candidates_timed = static_cast<int>(timed.size());
    return 0;
}
