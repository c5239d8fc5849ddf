// Device memory, tensor views and the workspace of reusable buffers.
//
// The host keeps no tensor library: a Tensor is a typed view (pointer, sizes, strides in
// elements) of device memory that a DeviceBuffer or the Workspace owns.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "spec.hpp"

namespace celeg {

// the numbers the kernels' entry points take for a dtype (CELEG_F32 = 0, CELEG_BF16 = 1)
enum class DType : int { F32 = 0, BF16 = 1, I32 = 2, U8 = 3 };

inline size_t dtype_size(DType d) {
    switch (d) {
        case DType::F32: return 4;
        case DType::BF16: return 2;
        case DType::I32: return 4;
        default: return 1;
    }
}
inline const char* dtype_name(DType d) {
    switch (d) {
        case DType::F32: return "float32";
        case DType::BF16: return "bfloat16";
        case DType::I32: return "int32";
        default: return "uint8";
    }
}
DType parse_dtype(const std::string& name);   // "bfloat16" | "bf16" | "float32" | "fp32" | "f32"

void hip_check(hipError_t code, const char* what);
#define CELEG_HIP(expr) ::celeg::hip_check((expr), #expr)
// the return value of a kernel's entry point (0 or a hipError_t)
void kernel_check(int code, const char* what);
// CELEG_SYNC_LAUNCHES=1 in the environment: kernel_check also waits for the kernel and checks how
// it ended, so that an asynchronous fault is named by the launch that caused it, and no step is
// recorded into or replayed from a graph (the reference's CELEG_DEBUG_SYNC build,
// include/celeg/backend/cuda/utils.cuh:109-116, synchronises the stream behind every launch)
bool sync_launches();

// bfloat16 <-> float on the host (round to nearest even, like the device's conversion)
inline uint16_t float_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40);   // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}
inline float bf16_to_float(uint16_t b) {
    const uint32_t u = static_cast<uint32_t>(b) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
float half_to_float(uint16_t h);

class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t bytes, bool zero = false);
    ~DeviceBuffer();
    DeviceBuffer(DeviceBuffer&& o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
    DeviceBuffer& operator=(DeviceBuffer&& o) noexcept;
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    void* ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }
    template <typename T>
    T* as() const { return static_cast<T*>(ptr_); }

private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
};

// Pinned host memory (allocated, never registered).
class PinnedBuffer {
public:
    PinnedBuffer() = default;
    explicit PinnedBuffer(size_t bytes);
    ~PinnedBuffer();
    PinnedBuffer(PinnedBuffer&& o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_), pinned_(o.pinned_) { o.ptr_ = nullptr; }
    PinnedBuffer& operator=(PinnedBuffer&& o) noexcept;
    PinnedBuffer(const PinnedBuffer&) = delete;
    void* ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }
    template <typename T>
    T* as() const { return static_cast<T*>(ptr_); }

private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
    bool pinned_ = false;
};

// A view of up to four dimensions; strides in elements.
struct Tensor {
    void* data = nullptr;
    DType dtype = DType::F32;
    int ndim = 0;
    long long shape[4] = {0, 0, 0, 0};
    long long stride[4] = {0, 0, 0, 0};

    bool defined() const { return data != nullptr; }
    long long numel() const {
        long long n = 1;
        for (int i = 0; i < ndim; ++i) n *= shape[i];
        return n;
    }
    size_t bytes() const { return static_cast<size_t>(numel()) * dtype_size(dtype); }
    template <typename T>
    T* as() const { return static_cast<T*>(data); }
    bool contiguous() const {
        long long expect = 1;
        for (int i = ndim - 1; i >= 0; --i) {
            if (shape[i] != 1 && stride[i] != expect) return false;
            expect *= shape[i];
        }
        return true;
    }
    static Tensor make(void* data, DType dtype, std::initializer_list<long long> dims) {
        Tensor t;
        t.data = data;
        t.dtype = dtype;
        t.ndim = static_cast<int>(dims.size());
        int i = 0;
        for (long long d : dims) t.shape[i++] = d;
        long long s = 1;
        for (int k = t.ndim - 1; k >= 0; --k) { t.stride[k] = s; s *= t.shape[k]; }
        return t;
    }
    // rows [begin, begin + count) of a tensor whose first dimension are rows
    Tensor rows(long long begin, long long count) const {
        Tensor t = *this;
        t.data = static_cast<char*>(data) + static_cast<size_t>(begin * stride[0]) * dtype_size(dtype);
        t.shape[0] = count;
        return t;
    }
    // columns [begin, begin + count) of a 2-D tensor (rows keep their stride)
    Tensor cols(long long begin, long long count) const {
        Tensor t = *this;
        t.data = static_cast<char*>(data) + static_cast<size_t>(begin * stride[1]) * dtype_size(dtype);
        t.shape[1] = count;
        return t;
    }
    // the stride between rows of a 2-D tensor with dense rows
    long long row_stride() const { return shape[0] > 1 ? stride[0] : (stride[0] > shape[1] ? stride[0] : shape[1]); }
};

// Reusable buffers by name, sized for the largest use so far.  `generation` changes whenever
// a buffer moves, which invalidates recorded graphs; while `frozen` (a graph is being
// recorded) a buffer that would move is an error.  Buffers that recorded graphs may still
// point into are kept until the workspace goes.
class Workspace {
public:
    Tensor buf(const std::string& name, DType dtype, std::initializer_list<long long> dims);
    void* raw(const std::string& name, size_t bytes);
    unsigned long long generation = 0;
    bool frozen = false;
    size_t bytes() const;

private:
    std::map<std::string, DeviceBuffer> buffers_;
    std::vector<DeviceBuffer> retired_;
};

// Times of the phases of a step, for finding where a step's time goes: events on the stream at
// the phase boundaries, read when the step has run.  The reference brackets its phases with
// events under CELEG_PROFILE_DECODE / CELEG_PROFILE_PREFILL and prints ms per token
// (include/celeg/backend/cuda/phase_profile.hpp:11-186); like there, a step that is timed is
// not replayed from a recorded graph.
class PhaseTimer {
public:
    explicit PhaseTimer(hipStream_t stream) : stream_(stream) {}
    ~PhaseTimer();
    PhaseTimer(const PhaseTimer&) = delete;
    void begin();                               // a step begins
    void mark(const std::string& phase);        // what ran since the last mark belongs to `phase`
    void end(long long tokens);                 // waits for the step and adds its times up
    // {"steps", "tokens", "phases": {name: {"ms": total, "calls": n}}}
    Json report() const;
    std::string table() const;                  // the same for people: ms per step and share, by phase

private:
    hipEvent_t event();
    hipStream_t stream_;
    std::vector<hipEvent_t> events_;
    size_t used_ = 0;
    std::vector<std::pair<std::string, size_t>> marks_;
    std::vector<std::string> order_;
    std::map<std::string, std::pair<double, long long>> totals_;
    long long steps_ = 0, tokens_ = 0;
};

}  // namespace celeg
