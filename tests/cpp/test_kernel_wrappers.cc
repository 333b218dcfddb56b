// Every launcher template of the reference-named headers instantiates for the three element types, and the calls
// that need no device (size queries, argument refusals) behave: compiled and run by tests/test_cabi.py.
#include "src/fastertransformer/kernels/ban_bad_words.h"
#include "src/fastertransformer/kernels/beam_search_penalty_kernels.h"
#include "src/fastertransformer/kernels/beam_search_topk_kernels.h"
#include "src/fastertransformer/kernels/online_softmax_beamsearch_kernels.h"
#include "src/fastertransformer/kernels/sampling_penalty_kernels.h"
#include "src/fastertransformer/kernels/sampling_topk_kernels.h"
#include "src/fastertransformer/kernels/sampling_topp_kernels.h"
#include "src/fastertransformer/kernels/stop_criteria_kernels.h"

#include <cstdio>
#include <stdexcept>

using namespace fastertransformer;

template<typename T>
static int instantiate()
{
    const void* launchers[] = {
        (const void*)&invokeAddBiasEndMask<T>,
        (const void*)&invokeBatchTopKSampling<T>,
        (const void*)&invokeTopKSampling<T>,
        (const void*)&invokeTopKTopPSampling<T>,
        (const void*)&invokeAddBiasSoftMax<T>,
        (const void*)&invokeBatchTopPSampling<T>,
        (const void*)&invokeTopPSampling<T>,
        (const void*)&invokeFusedTopPStep<T>,
        (const void*)&invokeApplyRepetitionPenalty<T>,
        (const void*)&invokeBatchApplyRepetitionPenalty<T>,
        (const void*)&invokeBatchApplyFrequencyPenalty<T>,
        (const void*)&invokeApplyTemperaturePenalty<T>,
        (const void*)&invokeBatchApplyTemperaturePenalty<T>,
        (const void*)&invokeMinLengthPenalty<T>,
        (const void*)&invokeBanBadWords<T>,
        (const void*)&invokeLogProbFromLogits<T>,
        (const void*)&invokeTopkSoftMax<T>,
        (const void*)&invokeAddBiasApplyPenalties<T>,
        (const void*)&topkSoftMaxWorkspaceBytes<T>,
    };
    int n = 0;
    for (const void* p : launchers) {
        n += p != nullptr;
    }
    return n;
}

int main()
{
    if (instantiate<float>() != 19 || instantiate<half>() != 19 || instantiate<bfloat16>() != 19) {
        return 1;
    }
    // size queries run on the host
    if (topkSoftMaxWorkspaceBytes<half>(32, 4, 50257) == 0) {
        std::printf("beam workspace query returned 0\n");
        return 1;
    }
    size_t need = 0;
    invokeFusedTopPStep<float>(nullptr, need, nullptr, nullptr, 50257, 50264, 8, nullptr, nullptr, nullptr, nullptr,
                               nullptr, nullptr, nullptr, nullptr, 0.5f, nullptr, nullptr, nullptr, nullptr, nullptr,
                               nullptr, nullptr);
    if (need == 0) {
        std::printf("top-p step workspace query returned 0\n");
        return 1;
    }
    // the reference's dispatch throws for beam widths it has no kernel for; so does the wrapper
    BeamHypotheses hyps{};
    bool           thrown = false;
    try {
        invokeTopkSoftMax<float>(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, &hyps, 1, 65,
                                 1000, nullptr, 0.0f, 0.0f, nullptr);
    }
    catch (const std::exception&) {
        thrown = true;
    }
    if (!thrown) {
        std::printf("beam width 65 was accepted\n");
        return 1;
    }
    return 0;
}
