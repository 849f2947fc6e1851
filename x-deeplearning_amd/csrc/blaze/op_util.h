// op_util.h -- small helpers shared by the operator implementations.
#pragma once

#include "blaze/common.h"
#include "blaze/runtime.h"
#include "blaze_hip.h"

namespace blaze {

inline int BzType(int data_type) {
  switch (data_type) {
    case kFloat: return BZ_F32;
    case kFloat16: return BZ_F16;
    case kInt32: return BZ_I32;
    case kInt64: return BZ_I64;
    default: BLAZE_THROW("Unsupported type: ", data_type);
  }
}

// fp32 device copy of a small parameter blob (the activation kernels read fp32 parameters); converted again only
// when the blob's buffer changed
struct ParamF32 {
  float* ptr = nullptr;
  size_t cap = 0;
  const void* src = nullptr;
  uint64_t src_version = 0;
  size_t src_size = 0;
  ~ParamF32() {
    if (ptr) (void)hipFree(ptr);
  }
  const float* Get(Blob* b, hipStream_t st, bool constant = true) {
    if (b->data_type() == kFloat) return b->as<float>();
    BLAZE_CONDITION_THROW(b->data_type() == kFloat16, "Unsupported type: ", b->data_type());
    const int n = (int)b->size();
    const int64_t ld = (n + 7) / 8 * 8;
    if ((size_t)ld > cap) {
      if (ptr) (void)hipFree(ptr);
      ptr = nullptr;
      HIP_CHECK(hipMalloc((void**)&ptr, ld * sizeof(float)));
      cap = ld;
      src = nullptr;
    }
    if (constant && src == b->data() && src_version == b->version() && src_size == b->size()) return ptr;
    BZ_CHECK(bz_fc_pack_weight(b->data(), BZ_F16, 1, n, 1, ptr, BZ_F32, ld, st));
    src = b->data();
    src_version = b->version();
    src_size = b->size();
    return ptr;
  }
};

}  // namespace blaze
