// Same enumerators and default values as the reference's src/fastertransformer/kernels/penalty_types.h:26-43.
#pragma once

namespace fastertransformer {

enum class RepetitionPenaltyType {
    Additive,        // the presence penalty
    Multiplicative,  // the repetition penalty
    None             // no repetition penalty
};

inline float getDefaultPenaltyValue(RepetitionPenaltyType penalty_type)
{
    return penalty_type == RepetitionPenaltyType::Multiplicative ? 1.0f : 0.0f;
}

}  // namespace fastertransformer
