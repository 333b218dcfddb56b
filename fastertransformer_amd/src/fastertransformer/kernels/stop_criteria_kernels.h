// Header name of the reference (src/fastertransformer/kernels/stop_criteria_kernels.h), kept so that a call site's
// #include line resolves unchanged. The launchers it declares there (invokeStopWordsCriterion, invokeLengthCriterion)
// are declared, for this engine, in sampling_kernels.h.
#pragma once
#include "src/fastertransformer/kernels/sampling_kernels.h"
