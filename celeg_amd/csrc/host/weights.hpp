// Weights by tensor name: the safetensors container, a model folder's checkpoint (one file
// or a sharded index), the check of a checkpoint against what the model's parts expect, and
// the way to the device.
//
// Container: an 8-byte little-endian header length, a JSON header
// {name: {dtype, shape, data_offsets}} and the data section (the reference's reader:
// src/checkpoint/formats/safetensors.cpp:93-239, dtype table 28-38).  Files are memory-mapped
// and only the bytes that are asked for are touched.
//
// Dtypes: floating tensors stored in 16-bit are held in bfloat16 by a bfloat16 engine and
// widened by a 32-bit engine; a tensor stored in 32-bit stays 32-bit; integer tensors become
// int32; "vector" tensors (norm scales, biases, filter taps) are always widened to 32-bit,
// which is exact.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "config.hpp"
#include "device.hpp"

namespace celeg {

struct SafetensorsError : std::runtime_error { using std::runtime_error::runtime_error; };

// The checkpoint does not fit the model: one error that lists everything.
struct WeightError : std::runtime_error {
    WeightError(const std::string& message, std::vector<std::string> missing_, std::vector<std::string> unexpected_,
                std::vector<std::string> wrong_)
        : std::runtime_error(message), missing(std::move(missing_)), unexpected(std::move(unexpected_)),
          wrong_shape(std::move(wrong_)) {}
    std::vector<std::string> missing, unexpected, wrong_shape;
};

struct TensorInfo {
    std::string name, dtype;              // dtype as the file spells it: F32, F16, BF16, I64, I32, I16, I8, U8
    std::vector<long long> shape;
    size_t begin = 0, end = 0;            // byte range inside the data section
    bool is_float() const { return dtype == "F32" || dtype == "F16" || dtype == "BF16"; }
};

class SafetensorsFile {
public:
    explicit SafetensorsFile(const std::string& path);   // validates the whole header
    ~SafetensorsFile();
    SafetensorsFile(const SafetensorsFile&) = delete;
    const std::string& path() const { return path_; }
    const std::vector<TensorInfo>& tensors() const { return tensors_; }
    const TensorInfo* find(const std::string& name) const;
    const uint8_t* bytes(const TensorInfo& info) const { return map_ + data_start_ + info.begin; }

private:
    std::string path_;
    int fd_ = -1;
    const uint8_t* map_ = nullptr;
    size_t size_ = 0, data_start_ = 0;
    std::vector<TensorInfo> tensors_;
    std::map<std::string, size_t> index_;
};

// The tensors of a model folder, across shards (src/checkpoint/repositories/safetensors.cpp:24-83).
class Checkpoint {
public:
    explicit Checkpoint(const std::string& model_dir);
    const std::string& model_dir() const { return dir_; }
    std::vector<std::string> names() const;
    const TensorInfo& info(const std::string& name) const;
    const uint8_t* bytes(const std::string& name) const;
    TensorShapes shapes() const;

private:
    std::string dir_;
    std::vector<std::unique_ptr<SafetensorsFile>> files_;
    std::vector<std::pair<std::string, std::pair<size_t, const TensorInfo*>>> where_;   // in file order
    std::map<std::string, size_t> index_;
    void add_file(const std::string& path);
};

// A tensor a part wants.  kind: "matrix" follows the engine's dtype, "vector" is always held
// in 32-bit.  init picks the distribution of the random-weights mode: "normal" is N(0, std),
// "around_one" is 1 + N(0, std).  `also` lists other shapes of the same tensor that are accepted.
struct WeightSpec {
    std::vector<long long> shape;
    std::string kind = "matrix";
    std::string init = "normal";
    std::vector<std::vector<long long>> also;
};
using ExpectedTensors = std::vector<std::pair<std::string, WeightSpec>>;   // checkpoint name -> spec

// One WeightError that lists every missing tensor, every tensor the model has no use for and
// every wrong shape, if a tensor is missing or has a wrong shape or dtype.  Tensors that the model
// has no use for are no error by themselves unless `strict`: their names are returned (sorted),
// for the caller to warn about.
std::vector<std::string> check_tensors(const Checkpoint& ckpt, const ExpectedTensors& expected, bool strict = false);

struct DeviceTensor {
    DeviceBuffer buffer;
    Tensor view;
};
using WeightMap = std::map<std::string, std::shared_ptr<DeviceTensor>>;

DType stored_as(const TensorInfo& info, const std::string& kind, DType engine_dtype);
// check_tensors, then every expected tensor converted and copied to the device
WeightMap load_tensors(const Checkpoint& ckpt, const ExpectedTensors& expected, DType engine_dtype, bool strict = false,
                       std::vector<std::string>* unused = nullptr);

// device-side helpers parts use while they re-lay their weights at load time
std::shared_ptr<DeviceTensor> device_tensor(DType dtype, std::initializer_list<long long> dims);
std::shared_ptr<DeviceTensor> concat_rows(const std::vector<std::shared_ptr<DeviceTensor>>& parts);
std::vector<float> to_host_floats(const Tensor& t);
std::shared_ptr<DeviceTensor> from_host_floats(const std::vector<float>& values, DType dtype,
                                               std::initializer_list<long long> dims);

}  // namespace celeg
