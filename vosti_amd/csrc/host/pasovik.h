// The Pasovik decoder, from its config.json to a description of parts: an embedding onto a residual stream in 32-bit, layers
// listed one by one in the configuration whose sublayers read the stream as it is and whose outputs alone are normed
// (x <- x + n1(mixer(x)); x <- x + n2(ff(x)), plain weights), and after them what a layer adds from the token's own
// second embedding (x <- x + n(W_proj (gelu(W_gate x) * e)), e the layer's slice of that table's row).  The mixer is softmax
// attention (grouped heads, q and k normed per head, neighbouring entries rotated in pairs with all frequencies divided by
// a constant, capped scores), attention through a latent (queries and keys/values projected down, normed and up again, one
// rotated key part for all heads, an output gate, optionally on the latent of an earlier layer), or linear attention with
// a fixed decay per head.  The feed-forward is dense (silu-gated) or a mixture of clamped gated experts whose logistic
// router scores scale what the chosen experts read.  Then the model's norm and an untied vocabulary projection.
#pragma once
#include "spec.h"

namespace vosti {

ModelSpec pasovik_model_spec(const Json& config);

}  // namespace vosti
