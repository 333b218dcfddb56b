// PyTorch-ROCm custom class over DynamicDecodeLayer: torch.classes.FasterTransformer.DynamicDecodeOp.
//
// Same class name, constructor, positional `setup` / `forward` argument order and placement rules as
// the reference's src/fastertransformer/th_op/common/DynamicDecodeOp.h:160-226 and
// DynamicDecodeOp.cc:248-453 (runtime arguments of `setup` on the CPU, top-p decay tensors and every
// per-step tensor on the GPU, `should_stop` returned as a 0-d CPU bool).
//
// Differences:
//   * tensor_para_size and pipeline_para_size must be 1: this build runs one GPU and holds no
//     communicator; `broadcast_from_last_pipeline` is then the reference's own early return.
//   * torch.bfloat16 is accepted next to float and half.
//   * the decay tensor reaches the layer under the key "top_p_decay", the one the layer reads. The
//     reference inserts it as "top_p_decay_opt" (DynamicDecodeOp.cc:101, :165), so its layer never
//     sees a decay passed through this class.
//   * beam_width > 1 raises: beam search is not part of this library.
#pragma once
#include <memory>
#include <vector>

#include <torch/custom_class.h>
#include <torch/script.h>

namespace torch_ext {

namespace th = torch;

// type-erased DynamicDecodeLayer<T> with its allocator
class IFtDynamicDecode {
public:
    virtual ~IFtDynamicDecode() {}
    // `args` and `outs`: (key, tensor, element type id of fastertransformer::DataType)
    struct Named {
        const char* key;
        th::Tensor  tensor;
        int         type;
    };
    virtual void setup(size_t batch_size, size_t beam_width, const std::vector<Named>& args)          = 0;
    virtual void forward(int step, int max_input_length, unsigned ite, int local_batch_size, bool* should_stop,
                         const std::vector<Named>& ins, const std::vector<Named>& outs)                = 0;
};

class DynamicDecodeOp: public th::jit::CustomClassHolder {
public:
    DynamicDecodeOp(const int64_t vocab_size, const int64_t vocab_size_padded, const int64_t tensor_para_size,
                    const int64_t pipeline_para_size, at::ScalarType scalar_type);
    ~DynamicDecodeOp();

    void setup(int64_t batch_size, int64_t beam_width, th::optional<th::Tensor> runtime_top_k_opt,
               th::optional<th::Tensor> runtime_top_p_opt, th::optional<th::Tensor> temperature_opt,
               th::optional<th::Tensor> repetition_penalty_opt, th::optional<th::Tensor> presence_penalty_opt,
               th::optional<th::Tensor> min_length_opt, th::optional<th::Tensor> length_penalty_opt,
               th::optional<th::Tensor> beam_search_diversity_rate_opt, th::optional<th::Tensor> random_seed_opt,
               th::optional<th::Tensor> top_p_decay_opt, th::optional<th::Tensor> top_p_min_opt,
               th::optional<th::Tensor> top_p_reset_ids_opt);

    th::Tensor forward(th::Tensor logits,  // (batch_size, beam_width, vocab_size_padded)
                       int64_t step, int64_t max_input_length, int64_t ite, int64_t local_batch_size,
                       th::Tensor end_id, th::optional<th::Tensor> runtime_top_k_opt,
                       th::optional<th::Tensor> runtime_top_p_opt, th::optional<th::Tensor> temperature_opt,
                       th::optional<th::Tensor> repetition_penalty_opt,
                       th::optional<th::Tensor> presence_penalty_opt, th::optional<th::Tensor> min_length_opt,
                       th::optional<th::Tensor> length_penalty_opt,
                       th::optional<th::Tensor> beam_search_diversity_rate_opt,
                       th::optional<th::Tensor> top_p_decay_opt, th::optional<th::Tensor> top_p_min_opt,
                       th::optional<th::Tensor> top_p_reset_ids_opt, th::optional<th::Tensor> embedding_bias_opt,
                       th::optional<th::Tensor> input_lengths_opt,
                       th::optional<th::Tensor> sequence_limit_length_opt,
                       th::optional<th::Tensor> stop_words_list_opt, th::optional<th::Tensor> bad_words_list_opt,
                       th::optional<th::Tensor> src_cache_indirection_opt,
                       // output buffers
                       th::Tensor output_token_ids, th::optional<th::Tensor> finished_opt,
                       th::optional<th::Tensor> sequence_lengths_opt, th::optional<th::Tensor> cum_log_probs_opt,
                       th::optional<th::Tensor> output_log_probs_opt, th::optional<th::Tensor> parent_ids_opt,
                       th::optional<th::Tensor> tgt_cache_indirection_opt);

    void broadcastFromLastPipeline(std::vector<th::Tensor> tensors);

private:
    size_t         vocab_size_;
    size_t         vocab_size_padded_;
    int            tensor_para_size_;
    int            pipeline_para_size_;
    at::ScalarType scalar_type_;  // type of the logits

    std::unique_ptr<IFtDynamicDecode> dynamic_decode_;
};

}  // namespace torch_ext
