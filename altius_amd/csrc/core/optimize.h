// Graph rewrites that produce the fused operators this backend has kernels for.
// Mirrors altius_core::optimize (crates/core/src/optimize/layer_norm_fusion.rs,
// gelu_fusion.rs, fast_gelu_fusion.rs, identity_elim.rs).  Each pass returns the
// number of subgraphs it rewrote.
#pragma once

#include "model.h"

namespace altius {

// ReduceMean -> Sub -> Pow -> ReduceMean -> Add -> Sqrt -> Div -> Mul -> Add  =>  LayerNormalization
// (axis -1, epsilon taken from the first Add's initializer, stash_type 1), inputs
// (x, Mul's second input, last Add's second input).  Like the reference, the match
// follows the chain of users and does not inspect axes or the Pow exponent; where the
// reference takes whichever user its hash set yields first, this pass takes the user
// that continues the pattern, so it matches whenever the reference can.
size_t fuse_layer_norm(Model &model);

// Div(x, ~sqrt 2) -> Erf -> Add 1 -> Mul x -> Mul 0.5  =>  Gelu(x)
size_t fuse_gelu(Model &model);

// Pow(x,3) -> Mul 0.044715 -> Add x -> Mul 0.79788 -> Tanh -> Add 1 -> Mul(Mul(x, 0.5), .)  =>  Gelu(x)
size_t fuse_fast_gelu(Model &model);

// Rewires the users of every Identity node to its input and drops the node; an
// Identity that feeds a graph output is kept.
size_t eliminate_identity(Model &model);

}  // namespace altius
