#include "device.hpp"

#include <cstdio>
#include <cstdlib>

namespace celeg {

DType parse_dtype(const std::string& name) {
    if (name == "bfloat16" || name == "bf16") return DType::BF16;
    if (name == "float32" || name == "fp32" || name == "f32") return DType::F32;
    throw ConfigError("unknown dtype '" + name + "': bfloat16 or float32");
}

void hip_check(hipError_t code, const char* what) {
    if (code != hipSuccess)
        throw KernelError(std::string(what) + ": " + hipGetErrorString(code) + " (HIP error " +
                          std::to_string(static_cast<int>(code)) + ")");
}

bool sync_launches() {
    static const bool on = [] {
        const char* v = std::getenv("CELEG_SYNC_LAUNCHES");
        return v && *v && std::string(v) != "0";
    }();
    return on;
}

void kernel_check(int code, const char* what) {
    if (code != 0) throw KernelError(std::string(what) + ": HIP error " + std::to_string(code));
    if (!sync_launches()) return;
    // the launch is waited for, so that a fault while the kernel ran is reported under the
    // kernel's name and not by whatever call comes next
    const hipError_t ran = hipDeviceSynchronize();
    if (ran != hipSuccess)
        throw KernelError(std::string(what) + ": failed while it ran: " + hipGetErrorString(ran) + " (" +
                          std::to_string(static_cast<int>(ran)) + ")");
}

float half_to_float(uint16_t h) {
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else {              // subnormal: normalise
            exp = 127 - 15 + 1;
            while (!(man & 0x400u)) { man <<= 1; --exp; }
            u = sign | (exp << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

DeviceBuffer::DeviceBuffer(size_t bytes, bool zero) : bytes_(bytes) {
    if (bytes == 0) return;
    const hipError_t err = hipMalloc(&ptr_, bytes);
    if (err != hipSuccess) {
        ptr_ = nullptr;
        throw KernelError("hipMalloc of " + std::to_string(bytes) + " bytes failed: " + hipGetErrorString(err));
    }
    if (zero) CELEG_HIP(hipMemset(ptr_, 0, bytes));
}

DeviceBuffer::~DeviceBuffer() {
    if (ptr_) (void)hipFree(ptr_);
}

DeviceBuffer& DeviceBuffer::operator=(DeviceBuffer&& o) noexcept {
    if (this != &o) {
        if (ptr_) (void)hipFree(ptr_);
        ptr_ = o.ptr_;
        bytes_ = o.bytes_;
        o.ptr_ = nullptr;
        o.bytes_ = 0;
    }
    return *this;
}

PinnedBuffer::PinnedBuffer(size_t bytes) : bytes_(bytes) {
    if (bytes == 0) return;
    if (hipHostMalloc(&ptr_, bytes, hipHostMallocDefault) == hipSuccess) {
        pinned_ = true;
    } else {
        (void)hipGetLastError();
        ptr_ = std::malloc(bytes);        // no GPU: ordinary memory, for the host-only paths
        if (!ptr_) throw std::bad_alloc();
    }
}

PinnedBuffer::~PinnedBuffer() {
    if (!ptr_) return;
    if (pinned_) (void)hipHostFree(ptr_);
    else std::free(ptr_);
}

PinnedBuffer& PinnedBuffer::operator=(PinnedBuffer&& o) noexcept {
    if (this != &o) {
        this->~PinnedBuffer();
        ptr_ = o.ptr_;
        bytes_ = o.bytes_;
        pinned_ = o.pinned_;
        o.ptr_ = nullptr;
    }
    return *this;
}

void* Workspace::raw(const std::string& name, size_t bytes) {
    auto it = buffers_.find(name);
    if (it == buffers_.end() || it->second.bytes() < bytes) {
        if (frozen)
            throw KernelError("workspace buffer '" + name + "' would move while a graph is being recorded");
        DeviceBuffer fresh(bytes < 256 ? 256 : bytes);
        if (it != buffers_.end()) {
            retired_.push_back(std::move(it->second));    // recorded graphs may still point at it
            it->second = std::move(fresh);
        } else {
            it = buffers_.emplace(name, std::move(fresh)).first;
        }
        ++generation;
    }
    return it->second.ptr();
}

Tensor Workspace::buf(const std::string& name, DType dtype, std::initializer_list<long long> dims) {
    long long count = 1;
    for (long long d : dims) count *= d;
    void* p = raw(name + ":" + dtype_name(dtype), static_cast<size_t>(count < 1 ? 1 : count) * dtype_size(dtype));
    return Tensor::make(p, dtype, dims);
}

size_t Workspace::bytes() const {
    size_t n = 0;
    for (const auto& b : buffers_) n += b.second.bytes();
    return n;
}

// ---------------------------------------------------------------------------- phase times
PhaseTimer::~PhaseTimer() {
    for (hipEvent_t e : events_) (void)hipEventDestroy(e);
}

hipEvent_t PhaseTimer::event() {
    if (used_ == events_.size()) {
        hipEvent_t e;
        CELEG_HIP(hipEventCreate(&e));
        events_.push_back(e);
    }
    hipEvent_t e = events_[used_++];
    CELEG_HIP(hipEventRecord(e, stream_));
    return e;
}

void PhaseTimer::begin() {
    used_ = 0;
    marks_.clear();
    event();
}

void PhaseTimer::mark(const std::string& phase) {
    if (used_ == 0) return;      // outside a step
    marks_.emplace_back(phase, used_);
    event();
}

void PhaseTimer::end(long long tokens) {
    if (used_ == 0) return;
    CELEG_HIP(hipStreamSynchronize(stream_));
    for (const auto& m : marks_) {
        float ms = 0.0f;
        CELEG_HIP(hipEventElapsedTime(&ms, events_[m.second - 1], events_[m.second]));
        auto it = totals_.find(m.first);
        if (it == totals_.end()) {
            order_.push_back(m.first);
            it = totals_.emplace(m.first, std::make_pair(0.0, 0LL)).first;
        }
        it->second.first += ms;
        it->second.second += 1;
    }
    ++steps_;
    tokens_ += tokens;
    used_ = 0;
    marks_.clear();
}

Json PhaseTimer::report() const {
    Json phases = Json::object();
    for (const std::string& name : order_) {
        const auto& t = totals_.at(name);
        phases.set(name, Json::object().set("ms", t.first).set("calls", t.second));
    }
    return Json::object().set("steps", steps_).set("tokens", tokens_).set("phases", phases);
}

std::string PhaseTimer::table() const {
    double all = 0.0;
    for (const auto& t : totals_) all += t.second.first;
    std::string out = "phase times over " + std::to_string(steps_) + " steps, " + std::to_string(tokens_) + " tokens\n";
    char line[160];
    for (const std::string& name : order_) {
        const auto& t = totals_.at(name);
        std::snprintf(line, sizeof line, "  %-28s %10.4f ms/step %6.1f %%  (%lld calls)\n", name.c_str(),
                      steps_ ? t.first / static_cast<double>(steps_) : 0.0, all > 0 ? 100.0 * t.first / all : 0.0, t.second);
        out += line;
    }
    std::snprintf(line, sizeof line, "  %-28s %10.4f ms/step\n", "all phases", steps_ ? all / static_cast<double>(steps_) : 0.0);
    out += line;
    return out;
}

}  // namespace celeg
