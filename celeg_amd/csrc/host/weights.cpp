#include "weights.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <fstream>
#include <set>
#include <sstream>

namespace celeg {

namespace {
size_t file_dtype_size(const std::string& d) {
    if (d == "F32" || d == "I32") return 4;
    if (d == "F16" || d == "BF16" || d == "I16") return 2;
    if (d == "I64") return 8;
    if (d == "I8" || d == "U8") return 1;
    return 0;
}
std::string shape_text(const std::vector<long long>& s) {
    std::string out = "(";
    for (size_t i = 0; i < s.size(); ++i) out += (i ? ", " : "") + std::to_string(s[i]);
    if (s.size() == 1) out += ",";
    return out + ")";
}
bool is_file(const std::string& path) {
    struct stat st;
    return ::stat(path.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}
}  // namespace

// ---------------------------------------------------------------------------- one file
SafetensorsFile::SafetensorsFile(const std::string& path) : path_(path) {
    fd_ = ::open(path.c_str(), O_RDONLY);
    if (fd_ < 0) throw SafetensorsError("cannot open " + path);
    struct stat st;
    if (::fstat(fd_, &st) != 0) { ::close(fd_); throw SafetensorsError("cannot stat " + path); }
    size_ = static_cast<size_t>(st.st_size);
    auto fail = [&](const std::string& message) {
        if (map_) ::munmap(const_cast<uint8_t*>(map_), size_);
        ::close(fd_);
        map_ = nullptr;
        fd_ = -1;
        throw SafetensorsError(message);
    };
    if (size_ < 8) fail("invalid safetensors file: too small: " + path);
    void* m = ::mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (m == MAP_FAILED) fail("cannot map " + path);
    map_ = static_cast<const uint8_t*>(m);
    uint64_t header_len = 0;
    for (int i = 7; i >= 0; --i) header_len = (header_len << 8) | map_[i];
    if (header_len == 0 || header_len > size_ - 8)
        fail("invalid safetensors header length " + std::to_string(header_len) + " in " + path);
    Json header;
    try {
        header = Json::parse(std::string(reinterpret_cast<const char*>(map_ + 8), header_len));
    } catch (const JsonError& e) {
        const std::string what = e.what();
        if (what.rfind("duplicate name: ", 0) == 0) fail("duplicate tensor name: " + what.substr(16));
        fail("invalid safetensors header in " + path + ": " + what);
    }
    if (!header.is_object()) fail("invalid safetensors header in " + path + ": not an object");
    data_start_ = 8 + static_cast<size_t>(header_len);
    const size_t data_size = size_ - data_start_;
    std::vector<std::pair<std::pair<size_t, size_t>, std::string>> spans;
    for (const auto& member : header.members()) {
        const std::string& name = member.first;
        if (name == "__metadata__") continue;
        const Json& e = member.second;
        TensorInfo info;
        info.name = name;
        long long begin = 0, end = 0;
        try {
            info.dtype = e["dtype"].as_string();
            for (const Json& s : e["shape"].items()) info.shape.push_back(s.as_int());
            if (e["data_offsets"].size() != 2) throw JsonError("offsets");
            begin = e["data_offsets"][0].as_int();
            end = e["data_offsets"][1].as_int();
        } catch (const std::exception&) {
            fail("malformed header entry for tensor " + name + " in " + path);
        }
        const size_t esize = file_dtype_size(info.dtype);
        if (esize == 0) fail("unsupported dtype " + info.dtype + " for tensor " + name + " in " + path);
        if (begin < 0 || end < begin || static_cast<size_t>(end) > data_size)
            fail("out-of-range tensor " + name + " in " + path);
        unsigned long long count = 1;
        for (long long s : info.shape) {
            if (s < 0) fail("negative dimension in tensor " + name + " in " + path);
            count *= static_cast<unsigned long long>(s);
        }
        if (count * esize != static_cast<unsigned long long>(end - begin))
            fail("byte count does not match shape for tensor " + name + " in " + path);
        info.begin = static_cast<size_t>(begin);
        info.end = static_cast<size_t>(end);
        if (end > begin) spans.push_back({{info.begin, info.end}, name});
        index_[name] = tensors_.size();
        tensors_.push_back(std::move(info));
    }
    std::sort(spans.begin(), spans.end());
    for (size_t i = 1; i < spans.size(); ++i)
        if (spans[i].first.first < spans[i - 1].first.second)
            fail("overlapping tensor ranges: " + spans[i - 1].second + " and " + spans[i].second + " in " + path);
}

SafetensorsFile::~SafetensorsFile() {
    if (map_) ::munmap(const_cast<uint8_t*>(map_), size_);
    if (fd_ >= 0) ::close(fd_);
}

const TensorInfo* SafetensorsFile::find(const std::string& name) const {
    auto it = index_.find(name);
    return it == index_.end() ? nullptr : &tensors_[it->second];
}

// ---------------------------------------------------------------------------- a folder
void Checkpoint::add_file(const std::string& path) {
    files_.push_back(std::make_unique<SafetensorsFile>(path));
    const size_t f = files_.size() - 1;
    for (const auto& info : files_[f]->tensors()) {
        index_[info.name] = where_.size();
        where_.push_back({info.name, {f, &info}});
    }
}

Checkpoint::Checkpoint(const std::string& model_dir) : dir_(model_dir) {
    const std::string single = model_dir + "/model.safetensors";
    const std::string index = model_dir + "/model.safetensors.index.json";
    if (is_file(single)) {
        add_file(single);
    } else if (is_file(index)) {
        std::ifstream in(index, std::ios::binary);
        std::ostringstream ss;
        ss << in.rdbuf();
        Json doc;
        try {
            doc = Json::parse(ss.str());
        } catch (const JsonError& e) {
            throw SafetensorsError("invalid " + index + ": " + e.what());
        }
        std::map<std::string, size_t> file_of;
        if (doc["weight_map"].is_object()) {
            for (const auto& m : doc["weight_map"].members()) {
                const std::string shard = m.second.as_string();
                const std::string path = model_dir + "/" + shard;
                auto it = file_of.find(path);
                if (it == file_of.end()) {
                    if (!is_file(path)) throw SafetensorsError("missing safetensors shard: " + path);
                    files_.push_back(std::make_unique<SafetensorsFile>(path));
                    it = file_of.emplace(path, files_.size() - 1).first;
                }
                const TensorInfo* info = files_[it->second]->find(m.first);
                if (!info) throw SafetensorsError("missing tensor: " + m.first + " (index names shard " + shard + ")");
                index_[m.first] = where_.size();
                where_.push_back({m.first, {it->second, info}});
            }
        }
    } else if (is_file(model_dir) && model_dir.size() > 12 &&
               model_dir.compare(model_dir.size() - 12, 12, ".safetensors") == 0) {
        add_file(model_dir);
    } else {
        throw SafetensorsError("no model.safetensors or model.safetensors.index.json found in " + model_dir);
    }
}

std::vector<std::string> Checkpoint::names() const {
    std::vector<std::string> out;
    for (const auto& w : where_) out.push_back(w.first);
    return out;
}

const TensorInfo& Checkpoint::info(const std::string& name) const {
    auto it = index_.find(name);
    if (it == index_.end()) throw SafetensorsError("missing tensor: " + name);
    return *where_[it->second].second.second;
}

const uint8_t* Checkpoint::bytes(const std::string& name) const {
    auto it = index_.find(name);
    if (it == index_.end()) throw SafetensorsError("missing tensor: " + name);
    const auto& w = where_[it->second].second;
    return files_[w.first]->bytes(*w.second);
}

TensorShapes Checkpoint::shapes() const {
    TensorShapes out;
    for (const auto& w : where_) out[w.first] = w.second.second->shape;
    return out;
}

// ---------------------------------------------------------------------------- checking
std::vector<std::string> check_tensors(const Checkpoint& ckpt, const ExpectedTensors& expected, bool strict) {
    std::set<std::string> have;
    for (const auto& n : ckpt.names()) have.insert(n);
    std::set<std::string> wanted;
    std::vector<std::string> missing, unexpected, wrong;
    for (const auto& e : expected) {
        wanted.insert(e.first);
        if (!have.count(e.first)) { missing.push_back(e.first); continue; }
        const TensorInfo& info = ckpt.info(e.first);
        bool fits = info.shape == e.second.shape;
        for (const auto& s : e.second.also) fits = fits || info.shape == s;
        if (!fits)
            wrong.push_back(e.first + " is " + shape_text(info.shape) + ", expected " + shape_text(e.second.shape));
        else if (!info.is_float())
            wrong.push_back(e.first + " is dtype " + info.dtype + ", expected a floating dtype");
    }
    for (const auto& n : have)
        if (!wanted.count(n)) unexpected.push_back(n);
    std::sort(missing.begin(), missing.end());
    missing.erase(std::unique(missing.begin(), missing.end()), missing.end());
    std::sort(unexpected.begin(), unexpected.end());
    // Tensors are bound by name and what nobody asks for is left alone, as the reference does
    // (include/celeg/checkpoint/weight_repository.hpp:14-20: a repository answers requests by
    // name; src/checkpoint/formats/safetensors.cpp:283-297 fails on a missing tensor only): a tied
    // model that still carries lm_head.weight, or an exported buffer, loads.  `strict` refuses them.
    if (missing.empty() && wrong.empty() && (unexpected.empty() || !strict)) return unexpected;
    auto join = [](const std::vector<std::string>& v) {
        std::string out;
        for (size_t i = 0; i < v.size(); ++i) out += (i ? ", " : "") + v[i];
        return out;
    };
    std::string message = "checkpoint " + ckpt.model_dir() + " does not fit the model:";
    if (!missing.empty()) message += "\n  missing tensors (" + std::to_string(missing.size()) + "): " + join(missing);
    if (!unexpected.empty())
        message += "\n  unexpected tensors (" + std::to_string(unexpected.size()) + "): " + join(unexpected);
    for (const auto& w : wrong) message += "\n  wrong shape: " + w;
    throw WeightError(message, missing, unexpected, wrong);
}

// ---------------------------------------------------------------------------- to the device
DType stored_as(const TensorInfo& info, const std::string& kind, DType engine_dtype) {
    if (!info.is_float()) return DType::I32;
    if (kind == "vector" || engine_dtype == DType::F32 || info.dtype == "F32") return DType::F32;
    return DType::BF16;
}

std::shared_ptr<DeviceTensor> device_tensor(DType dtype, std::initializer_list<long long> dims) {
    long long count = 1;
    for (long long d : dims) count *= d;
    auto t = std::make_shared<DeviceTensor>();
    t->buffer = DeviceBuffer(static_cast<size_t>(count < 1 ? 1 : count) * dtype_size(dtype));
    t->view = Tensor::make(t->buffer.ptr(), dtype, dims);
    return t;
}

static std::shared_ptr<DeviceTensor> upload(const Checkpoint& ckpt, const std::string& name, const std::string& kind,
                                            DType engine_dtype) {
    const TensorInfo& info = ckpt.info(name);
    const uint8_t* src = ckpt.bytes(name);
    const DType target = stored_as(info, kind, engine_dtype);
    size_t count = 1;
    for (long long s : info.shape) count *= static_cast<size_t>(s);
    auto t = std::make_shared<DeviceTensor>();
    t->buffer = DeviceBuffer(std::max<size_t>(count, 1) * dtype_size(target));
    t->view.data = t->buffer.ptr();
    t->view.dtype = target;
    t->view.ndim = static_cast<int>(std::min<size_t>(info.shape.size(), 4));
    if (info.shape.size() > 4) throw SafetensorsError("tensor " + name + " has more than four dimensions");
    long long stride = 1;
    for (int i = t->view.ndim - 1; i >= 0; --i) {
        t->view.shape[i] = info.shape[static_cast<size_t>(i)];
        t->view.stride[i] = stride;
        stride *= t->view.shape[i];
    }
    if (count == 0) return t;
    const bool same = (target == DType::F32 && info.dtype == "F32") || (target == DType::BF16 && info.dtype == "BF16") ||
                      (target == DType::I32 && info.dtype == "I32");
    if (same) {
        CELEG_HIP(hipMemcpy(t->buffer.ptr(), src, count * dtype_size(target), hipMemcpyHostToDevice));
        return t;
    }
    std::vector<uint8_t> staged(count * dtype_size(target));
    if (target == DType::I32) {
        int32_t* out = reinterpret_cast<int32_t*>(staged.data());
        for (size_t i = 0; i < count; ++i) {
            long long v = 0;
            if (info.dtype == "I64") { int64_t x; std::memcpy(&x, src + 8 * i, 8); v = x; }
            else if (info.dtype == "I16") { int16_t x; std::memcpy(&x, src + 2 * i, 2); v = x; }
            else if (info.dtype == "I8") v = static_cast<int8_t>(src[i]);
            else v = src[i];
            out[i] = static_cast<int32_t>(v);
        }
    } else {
        auto read = [&](size_t i) -> float {
            if (info.dtype == "F32") { float f; std::memcpy(&f, src + 4 * i, 4); return f; }
            uint16_t h;
            std::memcpy(&h, src + 2 * i, 2);
            return info.dtype == "BF16" ? bf16_to_float(h) : half_to_float(h);
        };
        if (target == DType::F32) {
            float* out = reinterpret_cast<float*>(staged.data());
            for (size_t i = 0; i < count; ++i) out[i] = read(i);
        } else {
            uint16_t* out = reinterpret_cast<uint16_t*>(staged.data());
            for (size_t i = 0; i < count; ++i) out[i] = float_to_bf16(read(i));
        }
    }
    CELEG_HIP(hipMemcpy(t->buffer.ptr(), staged.data(), staged.size(), hipMemcpyHostToDevice));
    return t;
}

WeightMap load_tensors(const Checkpoint& ckpt, const ExpectedTensors& expected, DType engine_dtype, bool strict,
                       std::vector<std::string>* unused) {
    std::vector<std::string> left = check_tensors(ckpt, expected, strict);
    if (unused) *unused = std::move(left);
    WeightMap out;
    for (const auto& e : expected)
        if (!out.count(e.first)) out[e.first] = upload(ckpt, e.first, e.second.kind, engine_dtype);
    return out;
}

std::shared_ptr<DeviceTensor> concat_rows(const std::vector<std::shared_ptr<DeviceTensor>>& parts) {
    long long rows = 0;
    const Tensor& first = parts.at(0)->view;
    for (const auto& p : parts) {
        if (p->view.ndim != 2 || p->view.shape[1] != first.shape[1] || p->view.dtype != first.dtype || !p->view.contiguous())
            throw KernelError("concat_rows: the matrices differ in width or dtype");
        rows += p->view.shape[0];
    }
    auto out = device_tensor(first.dtype, {rows, first.shape[1]});
    size_t offset = 0;
    for (const auto& p : parts) {
        CELEG_HIP(hipMemcpy(static_cast<char*>(out->buffer.ptr()) + offset, p->view.data, p->view.bytes(),
                            hipMemcpyDeviceToDevice));
        offset += p->view.bytes();
    }
    return out;
}

std::vector<float> to_host_floats(const Tensor& t) {
    if (!t.contiguous()) throw KernelError("to_host_floats: the tensor is not contiguous");
    const size_t n = static_cast<size_t>(t.numel());
    std::vector<float> out(n);
    if (t.dtype == DType::F32) {
        CELEG_HIP(hipMemcpy(out.data(), t.data, n * 4, hipMemcpyDeviceToHost));
    } else if (t.dtype == DType::BF16) {
        std::vector<uint16_t> raw(n);
        CELEG_HIP(hipMemcpy(raw.data(), t.data, n * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < n; ++i) out[i] = bf16_to_float(raw[i]);
    } else {
        throw KernelError("to_host_floats: not a floating tensor");
    }
    return out;
}

std::shared_ptr<DeviceTensor> from_host_floats(const std::vector<float>& values, DType dtype,
                                               std::initializer_list<long long> dims) {
    auto t = device_tensor(dtype, dims);
    if (static_cast<long long>(values.size()) != t->view.numel())
        throw KernelError("from_host_floats: the sizes differ");
    if (values.empty()) return t;
    if (dtype == DType::F32) {
        CELEG_HIP(hipMemcpy(t->buffer.ptr(), values.data(), values.size() * 4, hipMemcpyHostToDevice));
    } else if (dtype == DType::BF16) {
        std::vector<uint16_t> raw(values.size());
        for (size_t i = 0; i < values.size(); ++i) raw[i] = float_to_bf16(values[i]);
        CELEG_HIP(hipMemcpy(t->buffer.ptr(), raw.data(), raw.size() * 2, hipMemcpyHostToDevice));
    } else {
        throw KernelError("from_host_floats: not a floating dtype");
    }
    return t;
}

}  // namespace celeg
