// hipBLASLt, opened at run time; see blaslt.cpp.
#pragma once
#include <array>
#include <map>
#include <memory>

#include "device.hpp"

namespace celeg {

class BlasLt {
public:
    BlasLt();
    ~BlasLt();
    BlasLt(const BlasLt&) = delete;
    // out = x w^T for bfloat16 x [M, K] (rows ldx apart), w [N, K] (dense) and out [M, N] (rows
    // ldo apart) on `stream`.  False if the library has no kernel for these sizes (nothing was
    // launched).
    bool matmul(const void* x, long long ldx, const void* w, void* out, long long ldo, int M, int N, int K,
                hipStream_t stream);

private:
    struct Api;
    struct Plan;
    std::unique_ptr<Api> api_;
    void* handle_ = nullptr;
    void* desc_ = nullptr;
    void* pref_ = nullptr;
    DeviceBuffer workspace_;
    std::map<std::array<long long, 5>, std::unique_ptr<Plan>> plans_;
};

}  // namespace celeg
