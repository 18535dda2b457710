// The Pabavik decoder, from its config.json to a description of parts: an embedding times a constant onto a residual
// stream in 32-bit, layers listed one by one in the configuration, each with a norm before and after both sublayers
// (x <- x + norm_b(mixer(norm_a x)); x <- x + norm_d(ff(norm_c x)), weights stored around zero).  The mixer is softmax
// attention (grouped heads, q and k normed per head, a rotation of the first dimensions of every head, a sliding window,
// a constant 1 in the softmax's denominator, an output gate, optionally on the keys and values of an earlier layer) or
// gated linear attention (per head a state of outer products k v^T with a decay per key channel).  The feed-forward is
// a mixture of gated experts with clamped inputs, chosen per token by a router with a bias whose chosen logits are
// soft-maxed, beside an expert that every token uses.  Then the model's norm, an untied vocabulary projection and capped logits.
#pragma once
#include "spec.h"

namespace vosti {

ModelSpec pabavik_model_spec(const Json& config);

}  // namespace vosti
