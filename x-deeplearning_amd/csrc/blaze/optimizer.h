// optimizer.h -- NetDef -> NetDef rewrites of the offline optimizer that matter on this path.
//
// The reference's optimizer (blaze/optimizer/, blaze/graph/pattern/) is a library of some thirty passes; the one
// the FC stack of a CTR model depends on is the parallel-Gemm fusion of
// blaze/graph/pattern/in_parallel/parallel_gemm_fusion_pattern_impl.cc:20-250: Gemm operators that read the same
// tensor and have constant weights of one shape become one FusedParallelGemm over the stacked weights, followed by a
// Split along axis 0 that hands every former Gemm's output name its slice.  That pass is rebuilt here, with the
// removal of the constants it orphans; Blaze_OptimizeBlaze runs it.  Everything else of the optimizer is out of scope.
#pragma once

#include <string>

#include "blaze/proto.h"

namespace blaze {

// returns the number of groups fused (0: the net is unchanged)
int FuseParallelGemms(NetDef* net);

}  // namespace blaze
