// The Tezinex decoder, from its config.json to a description of parts: a residual stream in 32-bit with sinusoidal
// positions added to the embedding, layers listed one by one in the configuration (each a mixer between two norms,
// optionally a dense feed-forward between two more, then a learned weighted sum over the stream's earlier states),
// mixers that are either softmax attention (biases, capped scores, a window that keeps the first keys, a sink per
// head, optionally another layer's keys and values) or the gated delta rule with a decay per key channel, a head tied
// to the embedding and capped logits.
#pragma once
#include "spec.h"

namespace vosti {

ModelSpec tezinex_model_spec(const Json& config);

}  // namespace vosti
