#include "ft_decode_c.h"

#include <memory>
#include <string>

#include "src/fastertransformer/layers/DynamicDecodeLayer.h"
#include "src/fastertransformer/layers/beam_search_layers/OnlineBeamSearchLayer.h"

namespace ft = fastertransformer;

namespace {

thread_local std::string g_last_error;

struct DecodeHandle {
    int                                                    dtype;
    std::unique_ptr<ft::Allocator<ft::AllocatorType::HIP>> allocator;
    std::unique_ptr<ft::DynamicDecodeLayer<float>>         f32;
    std::unique_ptr<ft::DynamicDecodeLayer<ft::half>>      f16;
    std::unique_ptr<ft::DynamicDecodeLayer<ft::bfloat16>>  bf16;
};

struct BeamHandle {
    std::unique_ptr<ft::Allocator<ft::AllocatorType::HIP>> allocator;
    std::unique_ptr<ft::DynamicDecodeBaseLayer>            layer;
};

ft::TensorMap toMap(int n, const char* const* names, const ft_tensor* tensors)
{
    ft::TensorMap map;
    for (int i = 0; i < n; ++i) {
        const ft_tensor&    t = tensors[i];
        std::vector<size_t> shape(t.shape, t.shape + t.ndim);
        // unchecked insertion: a key may carry a null pointer
        map.insert({std::string(names[i]), ft::Tensor((ft::MemoryType)t.where, (ft::DataType)t.type, shape, t.data)});
    }
    return map;
}

template<typename F>
int guarded(F&& f)
{
    try {
        f();
        return FT_OK;
    }
    catch (const std::domain_error& e) {
        g_last_error = e.what();
        return FT_DOMAIN_ERROR;
    }
    catch (const std::runtime_error& e) {
        g_last_error = e.what();
        return FT_RUNTIME_ERROR;
    }
    catch (const std::exception& e) {
        g_last_error = e.what();
        return FT_OTHER_ERROR;
    }
}

}  // namespace

extern "C" {

const char* ft_decode_last_error(void)
{
    return g_last_error.c_str();
}

void* ft_dynamic_decode_create(int dtype, size_t vocab_size, size_t vocab_size_padded, int end_id, void* stream,
                               int is_free_buffer_after_forward)
{
    DecodeHandle* h  = nullptr;
    const int     rc = guarded([&]() {
        int device = 0;
        check_hip_error(hipGetDevice(&device));
        std::unique_ptr<DecodeHandle> p(new DecodeHandle());
        p->dtype = dtype;
        p->allocator.reset(new ft::Allocator<ft::AllocatorType::HIP>(device));
        p->allocator->setStream((hipStream_t)stream);
        const bool free_after = is_free_buffer_after_forward != 0;
        if (dtype == FTK_DTYPE_F32) {
            p->f32.reset(new ft::DynamicDecodeLayer<float>(vocab_size, vocab_size_padded, end_id, (hipStream_t)stream,
                                                           nullptr, p->allocator.get(), free_after, nullptr));
        }
        else if (dtype == FTK_DTYPE_F16) {
            p->f16.reset(new ft::DynamicDecodeLayer<ft::half>(vocab_size, vocab_size_padded, end_id,
                                                              (hipStream_t)stream, nullptr, p->allocator.get(),
                                                              free_after, nullptr));
        }
        else if (dtype == FTK_DTYPE_BF16) {
            p->bf16.reset(new ft::DynamicDecodeLayer<ft::bfloat16>(vocab_size, vocab_size_padded, end_id,
                                                                   (hipStream_t)stream, nullptr, p->allocator.get(),
                                                                   free_after, nullptr));
        }
        else {
            throw std::runtime_error("unsupported dtype");
        }
        h = p.release();
    });
    return rc == FT_OK ? h : nullptr;
}

void ft_dynamic_decode_destroy(void* handle)
{
    DecodeHandle* h = (DecodeHandle*)handle;
    if (h != nullptr) {
        // layers free their buffers through the allocator: destroy them first
        h->f32.reset();
        h->f16.reset();
        h->bf16.reset();
        delete h;
    }
}

int ft_dynamic_decode_set_stream(void* handle, void* stream)
{
    DecodeHandle* h = (DecodeHandle*)handle;
    return guarded([&]() {
        h->allocator->setStream((hipStream_t)stream);
        if (h->f32) {
            h->f32->setStream((hipStream_t)stream);
        }
        if (h->f16) {
            h->f16->setStream((hipStream_t)stream);
        }
        if (h->bf16) {
            h->bf16->setStream((hipStream_t)stream);
        }
    });
}

int ft_dynamic_decode_setup(void* handle, size_t batch_size, size_t beam_width, int n, const char* const* names,
                            const ft_tensor* tensors)
{
    DecodeHandle* h = (DecodeHandle*)handle;
    return guarded([&]() {
        ft::TensorMap args = toMap(n, names, tensors);
        if (h->f32) {
            h->f32->setup(batch_size, beam_width, &args);
        }
        else if (h->f16) {
            h->f16->setup(batch_size, beam_width, &args);
        }
        else {
            h->bf16->setup(batch_size, beam_width, &args);
        }
    });
}

int ft_dynamic_decode_forward(void* handle, int n_in, const char* const* in_names, const ft_tensor* in_tensors,
                              int n_out, const char* const* out_names, const ft_tensor* out_tensors)
{
    DecodeHandle* h = (DecodeHandle*)handle;
    return guarded([&]() {
        ft::TensorMap in  = toMap(n_in, in_names, in_tensors);
        ft::TensorMap out = toMap(n_out, out_names, out_tensors);
        if (h->f32) {
            h->f32->forward(&out, &in);
        }
        else if (h->f16) {
            h->f16->forward(&out, &in);
        }
        else {
            h->bf16->forward(&out, &in);
        }
    });
}

void* ft_online_beam_search_create(int dtype, size_t vocab_size, size_t vocab_size_padded, void* stream)
{
    BeamHandle* h  = nullptr;
    const int   rc = guarded([&]() {
        int device = 0;
        check_hip_error(hipGetDevice(&device));
        std::unique_ptr<BeamHandle> p(new BeamHandle());
        p->allocator.reset(new ft::Allocator<ft::AllocatorType::HIP>(device));
        p->allocator->setStream((hipStream_t)stream);
        hipStream_t st = (hipStream_t)stream;
        if (dtype == FTK_DTYPE_F32) {
            p->layer.reset(new ft::OnlineBeamSearchLayer<float>(0, 0, 0, 0, vocab_size, vocab_size_padded, 0, 0.0f, 1.0f,
                                                                0.0f, 1.0f, st, nullptr, p->allocator.get(), false));
        }
        else if (dtype == FTK_DTYPE_F16) {
            p->layer.reset(new ft::OnlineBeamSearchLayer<ft::half>(0, 0, 0, 0, vocab_size, vocab_size_padded, 0, 0.0f,
                                                                   1.0f, 0.0f, 1.0f, st, nullptr, p->allocator.get(),
                                                                   false));
        }
        else if (dtype == FTK_DTYPE_BF16) {
            p->layer.reset(new ft::OnlineBeamSearchLayer<ft::bfloat16>(0, 0, 0, 0, vocab_size, vocab_size_padded, 0,
                                                                       0.0f, 1.0f, 0.0f, 1.0f, st, nullptr,
                                                                       p->allocator.get(), false));
        }
        else {
            throw std::runtime_error("unsupported dtype");
        }
        h = p.release();
    });
    return rc == FT_OK ? h : nullptr;
}

void ft_online_beam_search_destroy(void* handle)
{
    BeamHandle* h = (BeamHandle*)handle;
    if (h != nullptr) {
        h->layer.reset();  // frees its workspace through the allocator
        delete h;
    }
}

int ft_online_beam_search_forward(void* handle, int n_in, const char* const* in_names, const ft_tensor* in_tensors,
                                  int n_out, const char* const* out_names, const ft_tensor* out_tensors)
{
    BeamHandle* h = (BeamHandle*)handle;
    return guarded([&]() {
        ft::TensorMap in  = toMap(n_in, in_names, in_tensors);
        ft::TensorMap out = toMap(n_out, out_names, out_tensors);
        h->layer->forward(&out, &in);
    });
}

}  // extern "C"
