// Tensor / TensorMap: the named-tensor currency of the layer API.
// Same names, enumerators and insertion semantics as the reference's
// src/fastertransformer/utils/Tensor.h:37-120 (DataType, MemoryType, Tensor) and :286-504 (TensorMap):
//   * TensorMap constructed from a list / unordered_map silently drops tensors with null data or zero
//     size (utils/Tensor.cc:348-377);
//   * insert(key, tensor) throws on such a tensor or on a duplicate key (Tensor.h:333-338);
//   * insert(pair) performs no check, so an output key may exist with a null pointer
//     (Tensor.h:347-350) and layers must treat it like an absent tensor;
//   * slice(shape, offset) is a bounds-checked pointer offset that passes null through
//     (utils/Tensor.cc:334-346).
#pragma once
#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <string>
#include <type_traits>
#include <unordered_map>
#include <utility>
#include <vector>

#include "src/fastertransformer/utils/ft_common.h"

namespace fastertransformer {

// 16-bit storage types of the logits. Host code never does arithmetic on them.
struct half {
    uint16_t bits;
};
struct bfloat16 {
    uint16_t bits;
};
typedef unsigned int uint;

typedef enum datatype_enum {
    TYPE_INVALID,
    TYPE_BOOL,
    TYPE_UINT8,
    TYPE_UINT16,
    TYPE_UINT32,
    TYPE_UINT64,
    TYPE_INT8,
    TYPE_INT16,
    TYPE_INT32,
    TYPE_INT64,
    TYPE_FP16,
    TYPE_FP32,
    TYPE_FP64,
    TYPE_BYTES,
    TYPE_BF16,
    TYPE_FP8_E4M3,
    TYPE_STR,
    TYPE_VOID,
} DataType;

template<typename T>
DataType getTensorType()
{
    typedef typename std::remove_cv<T>::type U;
    if (std::is_same<U, float>::value) {
        return TYPE_FP32;
    }
    if (std::is_same<U, half>::value) {
        return TYPE_FP16;
    }
    if (std::is_same<U, bfloat16>::value) {
        return TYPE_BF16;
    }
    if (std::is_same<U, int>::value) {
        return TYPE_INT32;
    }
    if (std::is_same<U, int8_t>::value) {
        return TYPE_INT8;
    }
    if (std::is_same<U, uint>::value) {
        return TYPE_UINT32;
    }
    if (std::is_same<U, unsigned long long int>::value || std::is_same<U, uint64_t>::value) {
        return TYPE_UINT64;
    }
    if (std::is_same<U, bool>::value) {
        return TYPE_BOOL;
    }
    if (std::is_same<U, char>::value) {
        return TYPE_BYTES;
    }
    return TYPE_INVALID;
}

typedef enum memorytype_enum {
    MEMORY_CPU,
    MEMORY_CPU_PINNED,
    MEMORY_GPU
} MemoryType;

struct Tensor {
    MemoryType          where;
    DataType            type;
    std::vector<size_t> shape;
    const void*         data;

    Tensor(): where(MEMORY_CPU), type(TYPE_INVALID), shape({}), data(nullptr) {}
    Tensor(MemoryType _where, DataType _type, std::vector<size_t> _shape, const void* _data):
        where(_where), type(_type), shape(std::move(_shape)), data(_data)
    {
    }

    size_t size() const
    {
        if (data == nullptr || shape.empty()) {
            return 0;
        }
        size_t n = 1;
        for (size_t d : shape) {
            n *= d;
        }
        return n;
    }
    size_t sizeBytes() const
    {
        return size() * getTypeSize(type);
    }
    static size_t getTypeSize(DataType type);
    std::string   whereToString() const;
    std::string   toString() const;

    template<typename T>
    T getVal(size_t index) const
    {
        FT_CHECK(where == MEMORY_CPU);
        FT_CHECK(data != nullptr);
        FT_CHECK_WITH_INFO(index < size(), "index is larger than buffer size");
        return ((const T*)data)[index];
    }
    template<typename T>
    T getVal() const
    {
        return getVal<T>(0);
    }
    template<typename T>
    T* getPtr() const
    {
        return (T*)data;
    }
    void* getPtrWithOffset(size_t offset) const
    {
        if (data == nullptr) {
            return nullptr;
        }
        FT_CHECK_WITH_INFO(offset < size(), "offset is larger than buffer size");
        return (void*)((char*)data + offset * getTypeSize(type));
    }
    template<typename T>
    T* getPtrWithOffset(size_t offset) const
    {
        if (data == nullptr) {
            return nullptr;
        }
        FT_CHECK_WITH_INFO(offset < size(), fmtstr("offset (%lu) is larger than buffer size (%lu)", offset, size()));
        return ((T*)data) + offset;
    }
    template<typename T>
    T max() const
    {
        FT_CHECK_WITH_INFO(shape.size() > 0 && data != nullptr, "Should be a non-empty tensor.");
        FT_CHECK_WITH_INFO(where == MEMORY_CPU || where == MEMORY_CPU_PINNED,
                           "max() supports MEMORY_CPU or MEMORY_CPU_PINNED tensor.");
        T best = ((const T*)data)[0];
        for (size_t i = 1; i < size(); ++i) {
            const T v = ((const T*)data)[i];
            best      = v > best ? v : best;
        }
        return best;
    }
    template<typename T>
    T min() const
    {
        FT_CHECK_WITH_INFO(shape.size() > 0 && data != nullptr, "Should be a non-empty tensor.");
        FT_CHECK_WITH_INFO(where == MEMORY_CPU || where == MEMORY_CPU_PINNED,
                           "min() supports MEMORY_CPU or MEMORY_CPU_PINNED tensor.");
        T best = ((const T*)data)[0];
        for (size_t i = 1; i < size(); ++i) {
            const T v = ((const T*)data)[i];
            best      = v < best ? v : best;
        }
        return best;
    }

    Tensor slice(std::vector<size_t> shape, size_t offset = 0) const;
};

class TensorMap {
    std::unordered_map<std::string, Tensor> tensor_map_;

    static bool isValid(const Tensor& tensor)
    {
        return tensor.size() > 0 && tensor.data != nullptr;
    }

public:
    TensorMap() = default;
    TensorMap(const std::unordered_map<std::string, Tensor>& tensor_map);
    TensorMap(const std::vector<Tensor>& tensor_map);
    TensorMap(std::initializer_list<std::pair<std::string, Tensor>> tensor_map);

    size_t size() const
    {
        return tensor_map_.size();
    }
    bool isExist(const std::string& key) const
    {
        return tensor_map_.find(key) != tensor_map_.end();
    }
    std::vector<std::string> keys() const;

    void insert(const std::string& key, const Tensor& value)
    {
        FT_CHECK_WITH_INFO(!isExist(key), fmtstr("Duplicated key %s", key.c_str()));
        FT_CHECK_WITH_INFO(isValid(value), fmtstr("A none tensor or nullptr is not allowed (key is %s)", key.c_str()));
        tensor_map_.insert({key, value});
    }
    void insertIfValid(const std::string& key, const Tensor& value)
    {
        if (isValid(value)) {
            insert({key, value});
        }
    }
    void insert(std::pair<std::string, Tensor> p)
    {
        tensor_map_.insert(p);
    }

    Tensor at(int)    = delete;
    Tensor at(size_t) = delete;

    Tensor& at(const std::string& key)
    {
        FT_CHECK_WITH_INFO(isExist(key),
                           fmtstr("Cannot find a tensor of name %s in the tensor map (keys: %s)", key.c_str(),
                                  vec2str(keys()).c_str()));
        return tensor_map_.at(key);
    }
    Tensor at(const std::string& key) const
    {
        FT_CHECK_WITH_INFO(isExist(key),
                           fmtstr("Cannot find a tensor of name %s in the tensor map (keys: %s)", key.c_str(),
                                  vec2str(keys()).c_str()));
        return tensor_map_.at(key);
    }
    Tensor at(const std::string& key, const Tensor& default_tensor) const
    {
        return isExist(key) ? tensor_map_.at(key) : default_tensor;
    }
    template<typename T>
    T getVal(const std::string& key) const
    {
        return at(key).getVal<T>();
    }
    template<typename T>
    T getVal(const std::string& key, T default_value) const
    {
        return isExist(key) ? tensor_map_.at(key).getVal<T>() : default_value;
    }
    template<typename T>
    T* getPtr(const std::string& key) const
    {
        return at(key).getPtr<T>();
    }
    template<typename T>
    T* getPtr(const std::string& key, T* default_ptr) const
    {
        return isExist(key) ? tensor_map_.at(key).getPtr<T>() : default_ptr;
    }
    template<typename T>
    T* getPtrWithOffset(const std::string& key, size_t index) const
    {
        return at(key).getPtrWithOffset<T>(index);
    }
    std::unordered_map<std::string, Tensor> getMap() const
    {
        return tensor_map_;
    }
    std::unordered_map<std::string, Tensor>::iterator begin()
    {
        return tensor_map_.begin();
    }
    std::unordered_map<std::string, Tensor>::iterator end()
    {
        return tensor_map_.end();
    }
    std::string toString();
};

}  // namespace fastertransformer
