/*
 * C handle API over the host C++ layers of libft_decode.so, for language bindings (ctypes, a
 * PyTorch-ROCm extension, cgo ...). It exposes fastertransformer::DynamicDecodeLayer<T>
 * (setup / forward with named tensors, reference: src/fastertransformer/layers/DynamicDecodeLayer.h:59-74)
 * the way the reference's TorchScript binding does (src/fastertransformer/th_op/common/DynamicDecodeOp.cc:86-186):
 * tensors are passed by name; exceptions become return codes plus a message.
 */
#ifndef FT_DECODE_C_H
#define FT_DECODE_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* values of fastertransformer::MemoryType / DataType (utils/Tensor.h) */
enum { FT_MEMORY_CPU = 0, FT_MEMORY_CPU_PINNED = 1, FT_MEMORY_GPU = 2 };
enum {
    FT_TYPE_INVALID = 0, FT_TYPE_BOOL = 1, FT_TYPE_UINT8 = 2, FT_TYPE_UINT16 = 3, FT_TYPE_UINT32 = 4,
    FT_TYPE_UINT64 = 5, FT_TYPE_INT8 = 6, FT_TYPE_INT16 = 7, FT_TYPE_INT32 = 8, FT_TYPE_INT64 = 9,
    FT_TYPE_FP16 = 10, FT_TYPE_FP32 = 11, FT_TYPE_FP64 = 12, FT_TYPE_BYTES = 13, FT_TYPE_BF16 = 14
};

typedef struct ft_tensor {
    int         where;
    int         type;
    int         ndim;
    size_t      shape[4];
    const void* data; /* may be NULL: the key then exists with a null pointer, as in the reference tests */
} ft_tensor;

enum { FT_OK = 0, FT_RUNTIME_ERROR = 1, FT_DOMAIN_ERROR = 2, FT_OTHER_ERROR = 3 };

/* message of the last failing call on this thread */
const char* ft_decode_last_error(void);

/* dtype: FTK_DTYPE_F32 / F16 / BF16. `stream` is a hipStream_t (NULL = default stream). */
void* ft_dynamic_decode_create(int dtype, size_t vocab_size, size_t vocab_size_padded, int end_id, void* stream,
                               int is_free_buffer_after_forward);
void  ft_dynamic_decode_destroy(void* handle);
int   ft_dynamic_decode_set_stream(void* handle, void* stream);

int ft_dynamic_decode_setup(void* handle, size_t batch_size, size_t beam_width, int n, const char* const* names,
                            const ft_tensor* tensors);

int ft_dynamic_decode_forward(void* handle, int n_in, const char* const* in_names, const ft_tensor* in_tensors,
                              int n_out, const char* const* out_names, const ft_tensor* out_tensors);

/* fastertransformer::OnlineBeamSearchLayer<T> (reference: layers/beam_search_layers/OnlineBeamSearchLayer.h:24-64,
 * BaseBeamSearchLayer.h:27-71): one beam-search step per forward call, tensors by name as the reference's layer
 * documents them (inputs: logits, step, ite, max_input_length, end_id, src_cache_indirection, optional
 * embedding_bias, input_lengths, temperature, len_penalty, beam_search_diversity_rate, repetition_penalty or
 * presence_penalty, min_length; outputs: output_ids, finished, cum_log_probs, parent_ids, sequence_length,
 * tgt_cache_indirection, optional output_log_probs and beam_hyps = a host pointer to an ftk_beam_hypotheses).
 * The layer keeps no state between steps apart from its workspace. */
void* ft_online_beam_search_create(int dtype, size_t vocab_size, size_t vocab_size_padded, void* stream);
void  ft_online_beam_search_destroy(void* handle);
int   ft_online_beam_search_forward(void* handle, int n_in, const char* const* in_names, const ft_tensor* in_tensors,
                                    int n_out, const char* const* out_names, const ft_tensor* out_tensors);

#ifdef __cplusplus
}
#endif
#endif
