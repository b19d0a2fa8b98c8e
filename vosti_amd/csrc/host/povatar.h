// The Povatar decoder, from its config.json to a description of parts: an embedding times a constant onto a residual
// stream in 32-bit, layers listed one by one in the configuration, each adding a mixer's and a routed feed-forward's
// output to the stream, both computed from norms of the same stream (x <- x + mixer(norm1 x) + experts(norm2 x)).  The
// mixer is the mean of two mixers that read the same input, each RMS-normed over the width with a weight of its own:
// softmax attention (grouped heads, a rotation of the first dimensions of every head with stretched frequencies,
// visible keys limited to the query's own block of positions, a constant 1 in the softmax's denominator) and a
// state-space recurrence with one decay per head.  The feed-forward is a mixture of small experts with squared-relu
// activation, chosen per token by a softmax router.  Then the model's norm and an untied vocabulary projection.
#pragma once
#include "spec.h"

namespace vosti {

ModelSpec povatar_model_spec(const Json& config);

}  // namespace vosti
