// The FC kernels of fc_fused_impl.h for bf16 operands.
#include "fc_fused_impl.h"

int bz::fc_run_bf16(const bz_fc_desc& d, const bz::fc::Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st) {
  return run_typed<BZ_BF16, __hip_bfloat16>(d, ep, vec_a, vec_w, st);
}
