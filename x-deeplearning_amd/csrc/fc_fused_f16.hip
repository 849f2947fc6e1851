// The FC kernels of fc_fused_impl.h for fp16 operands.
#include "fc_fused_impl.h"

int bz::fc_run_f16(const bz_fc_desc& d, const bz::fc::Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st) {
  return run_typed<BZ_F16, __half>(d, ep, vec_a, vec_w, st);
}
