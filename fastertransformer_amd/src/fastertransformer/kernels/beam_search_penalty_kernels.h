// Header name of the reference (src/fastertransformer/kernels/beam_search_penalty_kernels.h), kept so that a call
// site's #include line resolves unchanged. invokeAddBiasApplyPenalties is declared, for this engine, in
// sampling_kernels.h.
#pragma once
#include "src/fastertransformer/kernels/sampling_kernels.h"
