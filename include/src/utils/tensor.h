// Host-side tensor descriptors with the reference's names and members (src/utils/tensor.h):
//   Device / DataType enums, getTensorType<T>(), Tensor {location, dtype, shape},
//   TensorWrapper<T> : Tensor {T* data} (non-owning), TensorMap (name -> Tensor*).
// A TensorWrapper never owns `data`; launch* functions read `shape` and `data` only.
// `half` is HIP's __half.
#pragma once
#include <hip/hip_fp16.h>

#include <cstdint>
#include <functional>
#include <numeric>
#include <string>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "src/utils/macro.h"
#include "src/utils/string_utils.h"

enum Device { CPU_PINNED, CPU, GPU };

enum DataType { FP32, FP16, INT8, INT32, BOOL, BYTES, UNSUPPORTED };

template <typename T>
DataType getTensorType() {
    using U = typename std::remove_cv<T>::type;
    if (std::is_same<U, float>::value) return FP32;
    if (std::is_same<U, half>::value) return FP16;
    if (std::is_same<U, int>::value) return INT32;
    if (std::is_same<U, int8_t>::value) return INT8;
    if (std::is_same<U, bool>::value) return BOOL;
    if (std::is_same<U, char>::value) return BYTES;
    return UNSUPPORTED;
}

inline const char* isp_device_name(Device d) {
    switch (d) {
        case CPU: return "CPU";
        case CPU_PINNED: return "CPU_PINNED";
        case GPU: return "GPU";
    }
    return "?";
}

inline const char* isp_dtype_name(DataType t) {
    switch (t) {
        case FP32: return "FP32";
        case FP16: return "FP16";
        case INT8: return "INT8";
        case INT32: return "INT32";
        case BOOL: return "BOOL";
        case BYTES: return "BYTES";
        default: return "UNSUPPORTED";
    }
}

template <typename T>
class TensorWrapper;

struct Tensor {
    Device location;
    DataType dtype;
    std::vector<int> shape;

    Tensor() = default;
    Tensor(const Device location_, const DataType dtype_, const std::vector<int> shape_)
        : location(location_), dtype(dtype_), shape(shape_) {}
    virtual ~Tensor() = default;

    // number of elements; 0 for a tensor without a shape
    virtual int size() const {
        if (shape.empty()) return 0;
        return std::accumulate(shape.begin(), shape.end(), 1, std::multiplies<int>());
    }

    template <typename T>
    TensorWrapper<T>* as() {
        return static_cast<TensorWrapper<T>*>(this);
    }

    std::string DeviceString() const { return isp_device_name(location); }

    virtual std::string toString() const {
        return fmtstr("Tensor[where=%s, type=%s, shape=%s]", isp_device_name(location),
                      isp_dtype_name(dtype), vec2str(shape).c_str());
    }
};

template <typename T>
class TensorWrapper : public Tensor {
public:
    T* data = nullptr;

    TensorWrapper(Device location, DataType dtype, std::vector<int> shape)
        : Tensor(location, dtype, shape) {}

    TensorWrapper(Device location, DataType dtype, std::vector<int> shape, T* data)
        : Tensor(location, dtype, shape), data(data) {
        LLM_CHECK_WITH_INFO(getTensorType<T>() == dtype,
                            "when build TensorWrapper, the passed in data type should be same as "
                            "dtype in params");
    }

    // a wrapper without storage counts as empty
    int size() const override { return data == nullptr ? 0 : Tensor::size(); }

    // element access is only meaningful for host tensors
    inline T getVal(int id) const {
        LLM_CHECK(location == CPU);
        return data[id];
    }
    inline T getVal() const {
        LLM_CHECK(location == CPU);
        return getVal(0);
    }
    inline T* getPtr() const { return data; }
    inline T* getPtrByOffset(int offset) const { return data + offset; }

    std::string toString() const override {
        return fmtstr("Tensor[where=%s, type=%s, shape=%s, data=%p]", isp_device_name(location),
                      isp_dtype_name(dtype), vec2str(shape).c_str(), (void*)data);
    }
};

// Named collection of (non-owned) tensors; tensors without storage are rejected.
struct TensorMap {
    std::unordered_map<std::string, Tensor*> tensor_map_;

    TensorMap() = default;
    TensorMap(std::initializer_list<std::pair<std::string, Tensor*>> tensors) {
        for (const auto& kv : tensors) {
            LLM_CHECK_WITH_INFO(isValid(kv.second),
                                fmtstr("%s is not a valid tensor, skipping insert into TensorMap",
                                       kv.first.c_str()));
            insert(kv.first, kv.second);
        }
    }
    explicit TensorMap(const std::unordered_map<std::string, Tensor*>& tensors) {
        for (const auto& kv : tensors)
            if (isValid(kv.second)) insert(kv.first, kv.second);
    }

    inline size_t size() const { return tensor_map_.size(); }
    inline bool isExist(const std::string& key) const { return tensor_map_.count(key) != 0; }
    inline bool isValid(const Tensor* tensor) { return tensor != nullptr && tensor->size() > 0; }
    inline void insert(const std::string& key, Tensor* value) { tensor_map_[key] = value; }
    inline void insert(std::pair<std::string, Tensor*> p) { tensor_map_.insert(p); }

    inline Tensor* at(const std::string& key) {
        LLM_CHECK_WITH_INFO(isExist(key),
                            fmtstr("Cannot find a tensor of name %s in the tensor map (keys: %s)",
                                   key.c_str(), vec2str(keys()).c_str()));
        return tensor_map_.at(key);
    }
    inline Tensor* operator[](const std::string& key) { return at(key); }

    std::vector<std::string> keys() const {
        std::vector<std::string> names;
        names.reserve(tensor_map_.size());
        for (const auto& kv : tensor_map_) names.push_back(kv.first);
        return names;
    }

    std::string toString() {
        std::string out = "{";
        bool first = true;
        for (const auto& kv : tensor_map_) {
            if (!first) out += ", ";
            out += kv.first + ": " + kv.second->toString();
            first = false;
        }
        return out + "}";
    }
};
