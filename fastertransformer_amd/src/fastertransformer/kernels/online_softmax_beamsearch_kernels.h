// Header name of the reference (src/fastertransformer/kernels/online_softmax_beamsearch_kernels.h), kept so that a call site's
// #include line resolves unchanged. Of what it declares there, invokeTopkSoftMax is declared, for this engine, in
// sampling_kernels.h; the other launchers of the reference's file are not built.
#pragma once
#include "src/fastertransformer/kernels/sampling_kernels.h"
