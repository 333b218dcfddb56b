// Device / pinned-host buffer allocator of the layers.
// Interface of the reference's src/fastertransformer/utils/allocator.h:64-117 (IAllocator with
// malloc / free / reMalloc / memSet / setStream); reMalloc rounds to 32 bytes and reuses, grows or
// shrinks a tracked buffer. The concrete allocator uses the HIP runtime: hipMalloc for device
// memory, hipHostMalloc for pinned host memory.
#pragma once
#include <cstring>
#include <unordered_map>

#include "src/fastertransformer/utils/ft_common.h"

namespace fastertransformer {

enum class AllocatorType {
    HIP
};

enum class ReallocType {
    INCREASE,
    REUSE,
    DECREASE,
};

class IAllocator {
public:
    virtual ~IAllocator(){};

    virtual void*       malloc(size_t size, const bool is_set_zero = true, bool is_host = false) = 0;
    virtual void        free(void** ptr, bool is_host = false) const                             = 0;
    virtual void        setStream(hipStream_t stream)                                            = 0;
    virtual hipStream_t returnStream()                                                           = 0;
    virtual void        memSet(void* ptr, const int val, const size_t size)                      = 0;

    template<typename T>
    void* reMalloc(T* ptr, size_t size, const bool is_set_zero = true, bool is_host = false)
    {
        size           = ((size + 31) / 32) * 32;
        void* void_ptr = (void*)ptr;
        if (isExist(void_ptr)) {
            const ReallocType realloc_type = isReMalloc(void_ptr, size);
            if (realloc_type == ReallocType::INCREASE || realloc_type == ReallocType::DECREASE) {
                free((void**)(&void_ptr), is_host);
                return malloc(size, is_set_zero, is_host);
            }
            if (is_set_zero) {
                memSet(void_ptr, 0, size);
            }
            return void_ptr;
        }
        return malloc(size, is_set_zero, is_host);
    }

protected:
    virtual bool        isExist(void* address) const                 = 0;
    virtual ReallocType isReMalloc(void* address, size_t size) const = 0;
};

template<AllocatorType AllocType_>
class Allocator;

template<>
class Allocator<AllocatorType::HIP>: public IAllocator {
    const int                                            device_id_;
    hipStream_t                                          stream_ = nullptr;
    mutable std::unordered_map<void*, std::pair<size_t, bool>> pointer_mapping_;  // ptr -> (bytes, is_host)

    bool isExist(void* address) const override
    {
        return address != nullptr && pointer_mapping_.count(address) > 0;
    }
    ReallocType isReMalloc(void* address, size_t size) const override
    {
        const size_t have = pointer_mapping_.at(address).first;
        return have < size ? ReallocType::INCREASE : have == size ? ReallocType::REUSE : ReallocType::DECREASE;
    }

public:
    explicit Allocator(int device_id): device_id_(device_id) {}
    ~Allocator() override
    {
        while (!pointer_mapping_.empty()) {
            void* p = pointer_mapping_.begin()->first;
            free(&p, pointer_mapping_.begin()->second.second);
        }
    }
    void setStream(hipStream_t stream) override
    {
        stream_ = stream;
    }
    hipStream_t returnStream() override
    {
        return stream_;
    }
    void* malloc(size_t size, const bool is_set_zero = true, bool is_host = false) override
    {
        if (size == 0) {
            return nullptr;
        }
        void* ptr = nullptr;
        int   cur = 0;
        check_hip_error(hipGetDevice(&cur));
        if (cur != device_id_) {
            check_hip_error(hipSetDevice(device_id_));
        }
        if (is_host) {
            check_hip_error(hipHostMalloc(&ptr, size, hipHostMallocDefault));
        }
        else {
            check_hip_error(hipMalloc(&ptr, size));
        }
        if (is_set_zero) {
            if (is_host) {
                std::memset(ptr, 0, size);
            }
            else {
                check_hip_error(hipMemsetAsync(ptr, 0, size, stream_));
            }
        }
        if (cur != device_id_) {
            check_hip_error(hipSetDevice(cur));
        }
        pointer_mapping_[ptr] = {size, is_host};
        return ptr;
    }
    void free(void** ptr, bool is_host = false) const override
    {
        (void)is_host;
        if (ptr == nullptr || *ptr == nullptr) {
            return;
        }
        auto it = pointer_mapping_.find(*ptr);
        if (it != pointer_mapping_.end()) {
            if (it->second.second) {
                check_hip_error(hipHostFree(*ptr));
            }
            else {
                check_hip_error(hipFree(*ptr));
            }
            pointer_mapping_.erase(it);
        }
        else {
            FT_LOG_WARNING("pointer %p is not tracked by this allocator; not freed", *ptr);
        }
        *ptr = nullptr;
    }
    void memSet(void* ptr, const int val, const size_t size) override
    {
        auto it = pointer_mapping_.find(ptr);
        if (it != pointer_mapping_.end() && it->second.second) {
            std::memset(ptr, val, size);
        }
        else {
            check_hip_error(hipMemsetAsync(ptr, val, size, stream_));
        }
    }
};

}  // namespace fastertransformer
