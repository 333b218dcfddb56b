// See DynamicDecodeOp.h. Checks and argument tables follow the reference's
// src/fastertransformer/th_op/common/DynamicDecodeOp.cc:248-453 and th_op/th_utils.h:28-50.
#include "src/fastertransformer/th_op/common/DynamicDecodeOp.h"

#include <c10/hip/HIPStream.h>

#include "src/fastertransformer/layers/DynamicDecodeLayer.h"
#include "src/fastertransformer/utils/allocator.h"

namespace ft = fastertransformer;

namespace torch_ext {

namespace {

void check_type(const th::Tensor& t, at::ScalarType st, const char* name)
{
    TORCH_CHECK(t.scalar_type() == st, name, ": inconsistent tensor type, expected ", c10::toString(st), " but got ",
                c10::toString(t.scalar_type()));
}

// a device tensor: on the GPU, contiguous, of the given type (CHECK_INPUT)
void check_input(const th::Tensor& t, at::ScalarType st, const char* name)
{
    TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    check_type(t, st, name);
}

// a host tensor: on the CPU, contiguous, of the given type (CHECK_CPU_INPUT)
void check_cpu_input(const th::Tensor& t, at::ScalarType st, const char* name)
{
    TORCH_CHECK(!t.is_cuda(), name, " must be a CPU tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    check_type(t, st, name);
}

void check_optional_input(const th::optional<th::Tensor>& t, at::ScalarType st, const char* name)
{
    if (t.has_value()) {
        check_input(t.value(), st, name);
    }
}

void check_optional_cpu_input(const th::optional<th::Tensor>& t, at::ScalarType st, const char* name)
{
    if (t.has_value()) {
        check_cpu_input(t.value(), st, name);
    }
}

ft::Tensor convert_tensor(const th::Tensor& t, ft::DataType type)
{
    std::vector<size_t> shape;
    for (int64_t d : t.sizes()) {
        shape.push_back((size_t)d);
    }
    return ft::Tensor(t.is_cuda() ? ft::MEMORY_GPU : ft::MEMORY_CPU, type, shape, t.data_ptr());
}

void add(std::vector<IFtDynamicDecode::Named>& v, const char* key, const th::optional<th::Tensor>& t, ft::DataType type)
{
    if (t.has_value()) {
        v.push_back({key, t.value(), (int)type});
    }
}

template<typename T>
class FtDynamicDecode: public IFtDynamicDecode {
public:
    FtDynamicDecode(size_t vocab_size, size_t vocab_size_padded)
    {
        int device = 0;
        check_hip_error(hipGetDevice(&device));
        allocator_.reset(new ft::Allocator<ft::AllocatorType::HIP>(device));
        layer_.reset(new ft::DynamicDecodeLayer<T>(vocab_size, vocab_size_padded, 0, stream(), nullptr,
                                                   allocator_.get(), false, nullptr));
    }

    void setup(size_t batch_size, size_t beam_width, const std::vector<Named>& args) override
    {
        layer_->setStream(stream());
        ft::TensorMap runtime_args;
        for (const Named& a : args) {
            runtime_args.insert(a.key, convert_tensor(a.tensor, (ft::DataType)a.type));
        }
        layer_->setup(batch_size, beam_width, &runtime_args);
    }

    void forward(int step, int max_input_length, unsigned ite, int local_batch_size, bool* should_stop,
                 const std::vector<Named>& ins, const std::vector<Named>& outs) override
    {
        layer_->setStream(stream());
        ft::TensorMap input_tensors{
            {"step", ft::Tensor(ft::MEMORY_CPU, ft::TYPE_INT32, {1}, &step)},
            {"max_input_length", ft::Tensor(ft::MEMORY_CPU, ft::TYPE_INT32, {1}, &max_input_length)},
            {"ite", ft::Tensor(ft::MEMORY_CPU, ft::TYPE_UINT32, {1}, &ite)},
            {"local_batch_size", ft::Tensor(ft::MEMORY_CPU, ft::TYPE_INT32, {1}, &local_batch_size)}};
        for (const Named& a : ins) {
            input_tensors.insert(a.key, convert_tensor(a.tensor, (ft::DataType)a.type));
        }
        ft::TensorMap output_tensors{{"should_stop", ft::Tensor(ft::MEMORY_CPU, ft::TYPE_BOOL, {1}, should_stop)}};
        for (const Named& a : outs) {
            output_tensors.insert(a.key, convert_tensor(a.tensor, (ft::DataType)a.type));
        }
        layer_->forward(&output_tensors, &input_tensors);
    }

private:
    static hipStream_t stream()
    {
        return c10::hip::getCurrentHIPStream().stream();
    }

    std::unique_ptr<ft::Allocator<ft::AllocatorType::HIP>> allocator_;
    std::unique_ptr<ft::DynamicDecodeLayer<T>>            layer_;
};

}  // namespace

DynamicDecodeOp::DynamicDecodeOp(const int64_t vocab_size, const int64_t vocab_size_padded,
                                 const int64_t tensor_para_size, const int64_t pipeline_para_size,
                                 at::ScalarType scalar_type):
    vocab_size_((size_t)vocab_size),
    vocab_size_padded_((size_t)vocab_size_padded),
    tensor_para_size_((int)tensor_para_size),
    pipeline_para_size_((int)pipeline_para_size),
    scalar_type_(scalar_type)
{
    TORCH_CHECK(tensor_para_size_ == 1 && pipeline_para_size_ == 1,
                "this build runs one GPU: tensor_para_size and pipeline_para_size must be 1");
    switch (scalar_type_) {
        case at::ScalarType::Float:
            dynamic_decode_.reset(new FtDynamicDecode<float>(vocab_size_, vocab_size_padded_));
            break;
        case at::ScalarType::Half:
            dynamic_decode_.reset(new FtDynamicDecode<ft::half>(vocab_size_, vocab_size_padded_));
            break;
        case at::ScalarType::BFloat16:
            dynamic_decode_.reset(new FtDynamicDecode<ft::bfloat16>(vocab_size_, vocab_size_padded_));
            break;
        default:
            throw std::runtime_error("Wrong tensor type.");
    }
}

DynamicDecodeOp::~DynamicDecodeOp() {}

void DynamicDecodeOp::setup(int64_t batch_size, int64_t beam_width, th::optional<th::Tensor> runtime_top_k_opt,
                            th::optional<th::Tensor> runtime_top_p_opt, th::optional<th::Tensor> temperature_opt,
                            th::optional<th::Tensor> repetition_penalty_opt,
                            th::optional<th::Tensor> presence_penalty_opt, th::optional<th::Tensor> min_length_opt,
                            th::optional<th::Tensor> length_penalty_opt,
                            th::optional<th::Tensor> beam_search_diversity_rate_opt,
                            th::optional<th::Tensor> random_seed_opt, th::optional<th::Tensor> top_p_decay_opt,
                            th::optional<th::Tensor> top_p_min_opt, th::optional<th::Tensor> top_p_reset_ids_opt)
{
    check_optional_cpu_input(runtime_top_k_opt, torch::kInt32, "runtime_top_k");
    check_optional_cpu_input(runtime_top_p_opt, torch::kFloat, "runtime_top_p");
    check_optional_cpu_input(temperature_opt, torch::kFloat, "temperature");
    check_optional_cpu_input(repetition_penalty_opt, torch::kFloat, "repetition_penalty");
    check_optional_cpu_input(presence_penalty_opt, torch::kFloat, "presence_penalty");
    check_optional_cpu_input(min_length_opt, torch::kInt32, "min_length");
    check_optional_cpu_input(length_penalty_opt, torch::kFloat, "len_penalty");
    check_optional_cpu_input(beam_search_diversity_rate_opt, torch::kFloat, "beam_search_diversity_rate");
    check_optional_cpu_input(random_seed_opt, torch::kInt64, "random_seed");
    check_optional_input(top_p_decay_opt, torch::kFloat, "top_p_decay");
    check_optional_input(top_p_min_opt, torch::kFloat, "top_p_min");
    check_optional_input(top_p_reset_ids_opt, torch::kInt32, "top_p_reset_ids");

    std::vector<IFtDynamicDecode::Named> args;
    add(args, "runtime_top_k", runtime_top_k_opt, ft::TYPE_UINT32);
    add(args, "runtime_top_p", runtime_top_p_opt, ft::TYPE_FP32);
    add(args, "temperature", temperature_opt, ft::TYPE_FP32);
    add(args, "repetition_penalty", repetition_penalty_opt, ft::TYPE_FP32);
    add(args, "presence_penalty", presence_penalty_opt, ft::TYPE_FP32);
    add(args, "min_length", min_length_opt, ft::TYPE_INT32);
    add(args, "len_penalty", length_penalty_opt, ft::TYPE_FP32);
    add(args, "beam_search_diversity_rate", beam_search_diversity_rate_opt, ft::TYPE_FP32);
    add(args, "random_seed", random_seed_opt, ft::TYPE_UINT64);
    add(args, "top_p_decay", top_p_decay_opt, ft::TYPE_FP32);
    add(args, "top_p_min", top_p_min_opt, ft::TYPE_FP32);
    add(args, "top_p_reset_ids", top_p_reset_ids_opt, ft::TYPE_UINT32);
    dynamic_decode_->setup((size_t)batch_size, (size_t)beam_width, args);
}

th::Tensor DynamicDecodeOp::forward(
    th::Tensor logits, int64_t step, int64_t max_input_length, int64_t ite, int64_t local_batch_size,
    th::Tensor end_id, th::optional<th::Tensor> runtime_top_k_opt, th::optional<th::Tensor> runtime_top_p_opt,
    th::optional<th::Tensor> temperature_opt, th::optional<th::Tensor> repetition_penalty_opt,
    th::optional<th::Tensor> presence_penalty_opt, th::optional<th::Tensor> min_length_opt,
    th::optional<th::Tensor> length_penalty_opt, th::optional<th::Tensor> beam_search_diversity_rate_opt,
    th::optional<th::Tensor> top_p_decay_opt, th::optional<th::Tensor> top_p_min_opt,
    th::optional<th::Tensor> top_p_reset_ids_opt, th::optional<th::Tensor> embedding_bias_opt,
    th::optional<th::Tensor> input_lengths_opt, th::optional<th::Tensor> sequence_limit_length_opt,
    th::optional<th::Tensor> stop_words_list_opt, th::optional<th::Tensor> bad_words_list_opt,
    th::optional<th::Tensor> src_cache_indirection_opt, th::Tensor output_token_ids,
    th::optional<th::Tensor> finished_opt, th::optional<th::Tensor> sequence_lengths_opt,
    th::optional<th::Tensor> cum_log_probs_opt, th::optional<th::Tensor> output_log_probs_opt,
    th::optional<th::Tensor> parent_ids_opt, th::optional<th::Tensor> tgt_cache_indirection_opt)
{
    check_input(logits, scalar_type_, "logits");
    TORCH_CHECK(logits.dim() == 3, "logits is of shape (batch_size, beam_width, vocab_size_padded), but got dim=",
                logits.dim(), " shape=", logits.sizes());
    TORCH_CHECK((size_t)logits.size(2) == vocab_size_padded_, "logits is of shape (batch_size, beam_width, vocab_size(",
                vocab_size_padded_, ")), but got the last dim=", logits.size(2), ".");
    check_input(end_id, torch::kInt32, "end_id");
    check_optional_cpu_input(runtime_top_k_opt, torch::kInt32, "runtime_top_k");
    check_optional_cpu_input(runtime_top_p_opt, torch::kFloat, "runtime_top_p");
    check_optional_cpu_input(temperature_opt, torch::kFloat, "temperature");
    check_optional_cpu_input(repetition_penalty_opt, torch::kFloat, "repetition_penalty");
    check_optional_cpu_input(presence_penalty_opt, torch::kFloat, "presence_penalty");
    check_optional_cpu_input(min_length_opt, torch::kInt32, "min_length");
    check_optional_cpu_input(length_penalty_opt, torch::kFloat, "len_penalty");
    check_optional_cpu_input(beam_search_diversity_rate_opt, torch::kFloat, "beam_search_diversity_rate");
    check_optional_input(top_p_decay_opt, torch::kFloat, "top_p_decay");
    check_optional_input(top_p_min_opt, torch::kFloat, "top_p_min");
    check_optional_input(top_p_reset_ids_opt, torch::kInt32, "top_p_reset_ids");
    check_optional_input(embedding_bias_opt, scalar_type_, "embedding_bias");
    check_optional_input(input_lengths_opt, torch::kInt32, "input_lengths");
    check_optional_input(sequence_limit_length_opt, torch::kInt32, "sequence_limit_length");
    check_optional_input(stop_words_list_opt, torch::kInt32, "stop_words_list");
    check_optional_input(bad_words_list_opt, torch::kInt32, "bad_words_list");
    check_optional_input(src_cache_indirection_opt, torch::kInt32, "src_cache_indirection");
    check_input(output_token_ids, torch::kInt32, "output_token_ids");
    check_optional_input(finished_opt, torch::kBool, "finished");
    check_optional_input(sequence_lengths_opt, torch::kInt32, "sequence_lengths");
    check_optional_input(cum_log_probs_opt, torch::kFloat32, "cum_log_probs");
    check_optional_input(output_log_probs_opt, torch::kFloat32, "output_log_probs");
    check_optional_input(parent_ids_opt, torch::kInt32, "parent_ids");
    check_optional_input(tgt_cache_indirection_opt, torch::kInt32, "tgt_cache_indirection");

    const ft::DataType logits_type = scalar_type_ == at::ScalarType::Float ? ft::TYPE_FP32 :
                                     scalar_type_ == at::ScalarType::Half  ? ft::TYPE_FP16 :
                                                                             ft::TYPE_BF16;
    std::vector<IFtDynamicDecode::Named> ins;
    ins.push_back({"logits", logits, (int)logits_type});
    ins.push_back({"end_id", end_id, (int)ft::TYPE_INT32});
    add(ins, "runtime_top_k", runtime_top_k_opt, ft::TYPE_UINT32);
    add(ins, "runtime_top_p", runtime_top_p_opt, ft::TYPE_FP32);
    add(ins, "temperature", temperature_opt, ft::TYPE_FP32);
    add(ins, "repetition_penalty", repetition_penalty_opt, ft::TYPE_FP32);
    add(ins, "presence_penalty", presence_penalty_opt, ft::TYPE_FP32);
    add(ins, "min_length", min_length_opt, ft::TYPE_INT32);
    add(ins, "len_penalty", length_penalty_opt, ft::TYPE_FP32);
    add(ins, "beam_search_diversity_rate", beam_search_diversity_rate_opt, ft::TYPE_FP32);
    add(ins, "top_p_decay", top_p_decay_opt, ft::TYPE_FP32);
    add(ins, "top_p_min", top_p_min_opt, ft::TYPE_FP32);
    add(ins, "top_p_reset_ids", top_p_reset_ids_opt, ft::TYPE_UINT32);
    add(ins, "embedding_bias", embedding_bias_opt, logits_type);
    add(ins, "input_lengths", input_lengths_opt, ft::TYPE_INT32);
    add(ins, "sequence_limit_length", sequence_limit_length_opt, ft::TYPE_INT32);
    add(ins, "stop_words_list", stop_words_list_opt, ft::TYPE_INT32);
    add(ins, "bad_words_list", bad_words_list_opt, ft::TYPE_INT32);
    add(ins, "src_cache_indirection", src_cache_indirection_opt, ft::TYPE_INT32);

    std::vector<IFtDynamicDecode::Named> outs;
    outs.push_back({"output_ids", output_token_ids, (int)ft::TYPE_INT32});
    add(outs, "finished", finished_opt, ft::TYPE_BOOL);
    add(outs, "sequence_length", sequence_lengths_opt, ft::TYPE_INT32);
    add(outs, "parent_ids", parent_ids_opt, ft::TYPE_INT32);
    add(outs, "cum_log_probs", cum_log_probs_opt, ft::TYPE_FP32);
    add(outs, "output_log_probs", output_log_probs_opt, ft::TYPE_FP32);
    add(outs, "tgt_cache_indirection", tgt_cache_indirection_opt, ft::TYPE_INT32);

    th::Tensor should_stop = torch::zeros({}, torch::dtype(torch::kBool).requires_grad(false));
    dynamic_decode_->forward((int)step, (int)max_input_length, (unsigned)ite, (int)local_batch_size,
                             should_stop.data_ptr<bool>(), ins, outs);
    return should_stop;
}

void DynamicDecodeOp::broadcastFromLastPipeline(std::vector<th::Tensor> tensors)
{
    for (const th::Tensor& t : tensors) {
        TORCH_CHECK(t.is_cuda(), "tensor must be a CUDA tensor");
        TORCH_CHECK(t.is_contiguous(), "tensor must be contiguous");
    }
    // one pipeline stage: every tensor is already where it is needed (DynamicDecodeOp.cc:192-194)
}

}  // namespace torch_ext

static auto fasterTransformerDynamicDecodeTHS =
    torch::jit::class_<torch_ext::DynamicDecodeOp>("FasterTransformer", "DynamicDecodeOp")
        .def(torch::jit::init<int64_t, int64_t, int64_t, int64_t, at::ScalarType>())
        .def("setup", &torch_ext::DynamicDecodeOp::setup)
        .def("forward", &torch_ext::DynamicDecodeOp::forward)
        .def("broadcast_from_last_pipeline", &torch_ext::DynamicDecodeOp::broadcastFromLastPipeline);
