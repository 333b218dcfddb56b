#include "src/fastertransformer/utils/Tensor.h"

#include <numeric>
#include <sstream>

namespace fastertransformer {

size_t Tensor::getTypeSize(DataType type)
{
    switch (type) {
        case TYPE_BOOL:
        case TYPE_UINT8:
        case TYPE_INT8:
        case TYPE_BYTES:
        case TYPE_FP8_E4M3:
            return 1;
        case TYPE_UINT16:
        case TYPE_INT16:
        case TYPE_FP16:
        case TYPE_BF16:
            return 2;
        case TYPE_UINT32:
        case TYPE_INT32:
        case TYPE_FP32:
            return 4;
        case TYPE_UINT64:
        case TYPE_INT64:
        case TYPE_FP64:
            return 8;
        default:
            return 0;
    }
}

std::string Tensor::whereToString() const
{
    return where == MEMORY_CPU ? "CPU" : where == MEMORY_CPU_PINNED ? "CPU_PINNED" : "GPU";
}

std::string Tensor::toString() const
{
    static const char* names[] = {"invalid", "bool", "uint8", "uint16", "uint32", "uint64", "int8",  "int16", "int32",
                                  "int64",   "fp16", "fp32",  "fp64",   "bytes",  "bf16",   "fp8",   "str",   "void"};
    return fmtstr("Tensor[where=%s, type=%s, shape=%s, data=%p]", whereToString().c_str(), names[(int)type],
                  vec2str(shape).c_str(), data);
}

Tensor Tensor::slice(std::vector<size_t> new_shape, size_t offset) const
{
    if (data != nullptr) {
        const size_t n_elts        = size();
        const size_t n_sliced_elts = std::accumulate(new_shape.begin(), new_shape.end(), (size_t)1,
                                                     std::multiplies<size_t>());
        FT_CHECK_WITH_INFO(n_sliced_elts + offset <= n_elts,
                           fmtstr("The number (%ld) of elements of sliced tensor exceeds that (%ld) of the original "
                                  "tensor",
                                  n_sliced_elts + offset, n_elts));
    }
    return Tensor(where, type, new_shape, getPtrWithOffset(offset));
}

TensorMap::TensorMap(const std::unordered_map<std::string, Tensor>& tensor_map)
{
    for (auto& kv : tensor_map) {
        if (isValid(kv.second)) {
            insert(kv.first, kv.second);
        }
    }
}

TensorMap::TensorMap(const std::vector<Tensor>& tensor_map)
{
    for (size_t i = 0; i < tensor_map.size(); i++) {
        insert(std::to_string(i), tensor_map[i]);
    }
}

TensorMap::TensorMap(std::initializer_list<std::pair<std::string, Tensor>> tensor_map)
{
    for (auto& pair : tensor_map) {
        if (isValid(pair.second)) {
            insert(pair.first, pair.second);
        }
    }
}

std::vector<std::string> TensorMap::keys() const
{
    std::vector<std::string> key_names;
    for (auto& kv : tensor_map_) {
        key_names.push_back(kv.first);
    }
    return key_names;
}

std::string TensorMap::toString()
{
    std::stringstream ss;
    ss << "{";
    bool first = true;
    for (auto& kv : tensor_map_) {
        ss << (first ? "" : ", ") << kv.first << ": " << kv.second.toString();
        first = false;
    }
    ss << "}";
    return ss.str();
}

}  // namespace fastertransformer
