// Header name of the reference (src/fastertransformer/layers/beam_search_layers/BaseBeamSearchLayer.h), kept so
// that a call site's #include line resolves unchanged; the class lives in BeamSearchLayers.h.
#pragma once
#include "src/fastertransformer/layers/beam_search_layers/BeamSearchLayers.h"
