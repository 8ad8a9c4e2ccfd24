// Graph rewrites that produce the fused operators this backend has kernels for.
// Mirrors altius_core::optimize (crates/core/src/optimize/layer_norm_fusion.rs,
// gelu_fusion.rs, fast_gelu_fusion.rs, identity_elim.rs).  Each pass returns the
// number of subgraphs it rewrote.
#pragma once

#include <string>

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

// Chains of element-wise operators => one FusedElemwise node (crates/core/src/optimize/elemwise_fusion.rs:12-138).
//
// ReferenceRule restates the reference's pass: operators of Op::is_elemwise with one output; a node
// continues a chain when its first input is the previous node's output, that output has no other
// reader, the previous node is binary, its remaining inputs are not produced by other nodes, and (if
// it is binary) its second operand has the shape of the previous node's second operand.
//
// ExtendedRule is this backend's own: the previous result may be any operand (also both), the other
// operands may be any values computed outside the chain with any shapes that broadcast, and the
// approximated unary functions (Erf, Gelu, Sigmoid, Tanh, Exp, Round) count as element-wise, as long as
// every tensor involved is f32 with a known shape, the chain has at most 16 steps and reads at most 6
// distinct values.  Greater is left out (its result is not f32).
//
// Under both rules a value that is also a graph output ends the chain (the reference would drop such an
// output).  Needs every shape it looks at to be inferable; returns false with *err set when shape
// inference fails.  *count receives the number of chains fused.
// Not in the reference.  [Mul | Div by a one-element f32 initializer] -> [Add of a mask] -> Softmax(last axis)
// => one Softmax node with inputs (x, scale?, mask?) and Op::prologue_scale / prologue_mask set, which the
// session runs as one kernel with the bits of the separate nodes.  Either prologue operator may be absent (not
// both); intermediates must have no other reader and must not be graph outputs; the mask must be f32 of
// known shape, broadcast onto x without changing x's shape, and constant along every axis but the first and
// the last ([N,1,1,C], [1,1,1,C], [C]).  Returns the number of Softmax nodes rewritten.
size_t fuse_softmax_prologue(Model &model);

// Not in the reference.  MatMul(x, W) -> Add(., b) with b one value per output column (shape [N], [1, N], ...),
// the product having no other reader: the MatMul node takes b as a third input and the session adds it in the
// product's epilogue -- the same single addition per element, without the extra pass over the output.
// Returns the number of MatMul nodes rewritten.
size_t fuse_matmul_bias(Model &model);

// Transpose of the last two axes (perm [1,0], [0,2,1] or [0,1,3,2]) in front of a MatMul operand is folded into
// the product: the MatMul node reads the untransposed tensor and carries trans_a / trans_b.  The reference has
// this pass switched off (crates/core/src/optimize/transpose_fusion.rs:10-104 emits a Gemm its interpreter cannot
// run on batched operands, mod.rs:7); here the MatMul kernel takes the flags.  Unlike the reference's draft, a
// Transpose that has other readers is kept for them.  Returns the number of MatMul nodes rewritten.
size_t fuse_transpose_matmul(Model &model);

enum class ElemwiseFusionRule { ReferenceRule = 0, ExtendedRule = 1 };
bool fuse_elemwise_ops(Model &model, ElemwiseFusionRule rule, size_t *count, std::string *err);

}  // namespace altius
