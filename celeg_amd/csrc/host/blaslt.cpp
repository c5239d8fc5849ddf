// bfloat16 matrix products of many rows through hipBLASLt, called directly.
//
// The products of a prompt's rows are the library's, as in the reference (cuBLASLt there:
// src/backend/cuda/model/prefill_batched/non_attention.cpp:175-201).  A product is one call of
// hipblasLtMatmul with descriptors and an algorithm that are looked up by the sizes and made
// once.  The library is opened at run time: the copy that the process has loaded already (a
// Python process with torch has one) or the one on the loader's path, so that it goes with the
// HIP runtime in use.
//
// out[M, N] = x[M, K] w[N, K]^T, all row-major.  In the library's column-major terms that is
// D (N x M, ld ldo) = A^T B with A = w (K x N, ld K) and B = x (K x M, ld ldx).
#include "blaslt.hpp"

#include <dlfcn.h>

#include <cstring>

namespace celeg {

namespace {
constexpr int HIPBLAS_OP_N = 111, HIPBLAS_OP_T = 112;
constexpr int HIPBLAS_COMPUTE_32F = 2;
constexpr int HIP_R_32F = 0, HIP_R_16BF = 14;
constexpr int DESC_TRANSA = 0, DESC_TRANSB = 1;
constexpr int PREF_MAX_WORKSPACE_BYTES = 1;
constexpr size_t WORKSPACE_BYTES = 32u << 20;

struct Algo {
    uint8_t data[16];
    size_t max_workspace_bytes;
};
struct Heuristic {
    Algo algo;
    size_t workspace_size;
    int state;
    float waves_count;
    int reserved[4];
};
}  // namespace

struct BlasLt::Api {
    void* handle = nullptr;
    int (*Create)(void**) = nullptr;
    int (*Destroy)(void*) = nullptr;
    int (*DescCreate)(void**, int, int) = nullptr;
    int (*DescSetAttribute)(void*, int, const void*, size_t) = nullptr;
    int (*LayoutCreate)(void**, int, uint64_t, uint64_t, int64_t) = nullptr;
    int (*PrefCreate)(void**) = nullptr;
    int (*PrefSetAttribute)(void*, int, const void*, size_t) = nullptr;
    int (*GetHeuristic)(void*, void*, void*, void*, void*, void*, void*, int, Heuristic*, int*) = nullptr;
    int (*Matmul)(void*, void*, const void*, const void*, void*, const void*, void*, const void*, const void*, void*,
                  void*, void*, const void*, void*, size_t, hipStream_t) = nullptr;
};

struct BlasLt::Plan {
    void *a = nullptr, *b = nullptr, *d = nullptr;
    Algo algo;
    bool usable = false;
};

static void ok(int status, const char* what) {
    if (status != 0) throw KernelError(std::string(what) + " failed with hipblasStatus " + std::to_string(status));
}

BlasLt::BlasLt() : api_(new Api) {
    void* lib = nullptr;
    for (const char* name : {"libhipblaslt.so", "libhipblaslt.so.1", "libhipblaslt.so.0"}) {
        lib = dlopen(name, RTLD_NOW | RTLD_NOLOAD);      // a copy the process holds already
        if (lib) break;
    }
    if (!lib)
        for (const char* name : {"libhipblaslt.so.1", "libhipblaslt.so", "/opt/rocm/lib/libhipblaslt.so"}) {
            lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
            if (lib) break;
        }
    if (!lib) throw KernelError("libhipblaslt.so was not found (looked among the loaded libraries and on the loader's path)");
    api_->handle = lib;
    auto sym = [&](const char* name) {
        void* p = dlsym(lib, name);
        if (!p) throw KernelError(std::string("libhipblaslt.so has no ") + name);
        return p;
    };
#define LOAD(field, name) api_->field = reinterpret_cast<decltype(api_->field)>(sym(name))
    LOAD(Create, "hipblasLtCreate");
    LOAD(Destroy, "hipblasLtDestroy");
    LOAD(DescCreate, "hipblasLtMatmulDescCreate");
    LOAD(DescSetAttribute, "hipblasLtMatmulDescSetAttribute");
    LOAD(LayoutCreate, "hipblasLtMatrixLayoutCreate");
    LOAD(PrefCreate, "hipblasLtMatmulPreferenceCreate");
    LOAD(PrefSetAttribute, "hipblasLtMatmulPreferenceSetAttribute");
    LOAD(GetHeuristic, "hipblasLtMatmulAlgoGetHeuristic");
    LOAD(Matmul, "hipblasLtMatmul");
#undef LOAD
    ok(api_->Create(&handle_), "hipblasLtCreate");
    ok(api_->DescCreate(&desc_, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
    const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    ok(api_->DescSetAttribute(desc_, DESC_TRANSA, &ta, 4), "hipblasLtMatmulDescSetAttribute");
    ok(api_->DescSetAttribute(desc_, DESC_TRANSB, &tb, 4), "hipblasLtMatmulDescSetAttribute");
    ok(api_->PrefCreate(&pref_), "hipblasLtMatmulPreferenceCreate");
    const uint64_t size = WORKSPACE_BYTES;
    ok(api_->PrefSetAttribute(pref_, PREF_MAX_WORKSPACE_BYTES, &size, 8), "hipblasLtMatmulPreferenceSetAttribute");
    workspace_ = DeviceBuffer(WORKSPACE_BYTES);
}

BlasLt::~BlasLt() {
    if (handle_ && api_->Destroy) api_->Destroy(handle_);
}

bool BlasLt::matmul(const void* x, long long ldx, const void* w, void* out, long long ldo, int M, int N, int K,
                    hipStream_t stream) {
    const std::array<long long, 5> key{M, N, K, ldx, ldo};
    auto it = plans_.find(key);
    if (it == plans_.end()) {
        auto plan = std::make_unique<Plan>();
        ok(api_->LayoutCreate(&plan->a, HIP_R_16BF, static_cast<uint64_t>(K), static_cast<uint64_t>(N), K), "hipblasLtMatrixLayoutCreate");
        ok(api_->LayoutCreate(&plan->b, HIP_R_16BF, static_cast<uint64_t>(K), static_cast<uint64_t>(M), ldx), "hipblasLtMatrixLayoutCreate");
        ok(api_->LayoutCreate(&plan->d, HIP_R_16BF, static_cast<uint64_t>(N), static_cast<uint64_t>(M), ldo), "hipblasLtMatrixLayoutCreate");
        Heuristic result;
        std::memset(&result, 0, sizeof result);
        int found = 0;
        const int status = api_->GetHeuristic(handle_, desc_, plan->a, plan->b, plan->d, plan->d, pref_, 1, &result, &found);
        // no kernel for these sizes: the caller takes another way
        plan->usable = status == 0 && found >= 1 && result.state == 0 && result.workspace_size <= WORKSPACE_BYTES;
        plan->algo = result.algo;
        it = plans_.emplace(key, std::move(plan)).first;
    }
    const Plan& plan = *it->second;
    if (!plan.usable) return false;
    const float one = 1.0f, zero = 0.0f;
    const int status = api_->Matmul(handle_, desc_, &one, w, plan.a, x, plan.b, &zero, out, plan.d, out, plan.d,
                                    &plan.algo, workspace_.ptr(), WORKSPACE_BYTES, stream);
    if (status != 0)
        throw KernelError("hipblasLtMatmul failed with hipblasStatus " + std::to_string(status) + " for M, N, K = " +
                          std::to_string(M) + ", " + std::to_string(N) + ", " + std::to_string(K));
    return true;
}

}  // namespace celeg
