// optimizer.h -- NetDef -> NetDef rewrites of the offline optimizer that matter on this path.
//
// The reference's optimizer (blaze/optimizer/, blaze/graph/pattern/) is a library of some thirty passes; the one
// the FC stack of a CTR model depends on is the parallel-Gemm fusion of
// blaze/graph/pattern/in_parallel/parallel_gemm_fusion_pattern_impl.cc:20-250: Gemm operators that read the same
// tensor and have constant weights of one shape become one FusedParallelGemm over the stacked weights, followed by a
// Split along axis 0 that hands every former Gemm's output name its slice.  That pass is rebuilt here, with the
// removal of the constants it orphans.  The second one is the in-order Gemm -> Gemm folding of
// blaze/graph/pattern/in_order/gemm_gemm_fusion_pattern_impl.cc:15-298: two FC layers with nothing between them are
// one layer on the product of their weights.  Blaze_OptimizeBlaze runs both.  Everything else of the optimizer is out
// of scope.
#pragma once

#include <string>

#include "blaze/proto.h"

namespace blaze {

// returns the number of groups fused (0: the net is unchanged)
int FuseParallelGemms(NetDef* net);

// Gemm(X, W0[, b0]) read only by Gemm(., W1[, b1]), all operands ConstantFill, no transA:
//   alpha1 * ((alpha0 * X * op(W0)) + beta0 * b0) * op(W1) + beta1 * b1
//     = (alpha0 * alpha1) * X * (op(W0) * op(W1)) + (beta0 * b0 * op(W1) + beta1 * b1)     (the reference's formula)
// The second Gemm stays, reading X, with `alpha` = alpha0 * alpha1 and `beta` = 1 as its only arguments; its weight
// constant holds op(W0) * op(W1) untransposed, its bias constant (the second one's, else the first one's) the folded
// bias; the first Gemm and the constants only it read disappear.  Returns the number of pairs folded.
int FuseGemmChains(NetDef* net);

}  // namespace blaze
