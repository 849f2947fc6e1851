#include "blaze/runtime.h"

#include <stdlib.h>

#include <atomic>
#include <mutex>
#include <unordered_set>

namespace blaze {

namespace {
// host blocks that came from hipHostMalloc (the rest came from malloc, when no device is usable)
std::mutex g_pinned_mu;
std::unordered_set<void*>& PinnedSet() {
  static std::unordered_set<void*> s;
  return s;
}
}  // namespace

std::atomic<int64_t>& AllocationCount() {
  static std::atomic<int64_t> n{0};
  return n;
}

void* Alloc(size_t bytes, int device_type, int device_id) {
  if (bytes == 0) bytes = 16;
  ++AllocationCount();
  void* p = nullptr;
  if (device_type == kCPU) {
    // pinned, so that Feed / Output copies are real DMA transfers instead of the runtime's staged pageable path
    if (hipHostMalloc(&p, bytes, hipHostMallocDefault) == hipSuccess && p != nullptr) {
      std::lock_guard<std::mutex> lock(g_pinned_mu);
      PinnedSet().insert(p);
      return p;
    }
    (void)hipGetLastError();
    p = malloc(bytes);
    BLAZE_CONDITION_THROW(p != nullptr, "malloc of ", bytes, " bytes failed");
    return p;
  }
  int cur = 0;
  HIP_CHECK(hipGetDevice(&cur));
  if (cur != device_id) HIP_CHECK(hipSetDevice(device_id));
  HIP_CHECK(hipMalloc(&p, bytes));
  if (cur != device_id) HIP_CHECK(hipSetDevice(cur));
  return p;
}

void Free(void* ptr, int device_type, int) {
  if (ptr == nullptr) return;
  if (device_type == kCPU) {
    bool pinned;
    {
      std::lock_guard<std::mutex> lock(g_pinned_mu);
      pinned = PinnedSet().erase(ptr) != 0;
    }
    if (pinned)
      (void)hipHostFree(ptr);
    else
      free(ptr);
  } else {
    (void)hipFree(ptr);
  }
}

void HIPContext::Activate() const {
  static thread_local int current = -1;
  if (current != device_id_) {
    HIP_CHECK(hipSetDevice(device_id_));
    current = device_id_;
  }
}

namespace {
struct ThreadStreams {
  std::vector<std::vector<hipStream_t>> per_device;
  ~ThreadStreams() {
    for (auto& v : per_device)
      for (auto s : v)
        if (s) (void)hipStreamDestroy(s);
  }
  hipStream_t& at(int device_id, int stream_id) {
    BLAZE_CONDITION_THROW(device_id >= 0 && stream_id >= 0 && stream_id < kMaxStreamNum, "device_id=", device_id, " stream_id=", stream_id);
    if ((int)per_device.size() <= device_id) per_device.resize(device_id + 1);
    auto& v = per_device[device_id];
    if (v.empty()) v.resize(kMaxStreamNum, nullptr);
    return v[stream_id];
  }
};
ThreadStreams& StreamsOfThisThread() {
  static thread_local ThreadStreams tls;
  return tls;
}
}  // namespace

hipStream_t HIPContext::hip_stream(int device_id, int stream_id) {
  hipStream_t& s = StreamsOfThisThread().at(device_id, stream_id);
  if (s == nullptr) {
    int cur = 0;
    HIP_CHECK(hipGetDevice(&cur));
    if (cur != device_id) HIP_CHECK(hipSetDevice(device_id));
    HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    if (cur != device_id) HIP_CHECK(hipSetDevice(cur));
  }
  return s;
}

void HIPContext::AdoptThreadStream(int device_id, int stream_id, hipStream_t stream) {
  hipStream_t& s = StreamsOfThisThread().at(device_id, stream_id);
  if (s != nullptr && s != stream) {
    HIP_CHECK(hipStreamSynchronize(s));
    HIP_CHECK(hipStreamDestroy(s));
  }
  s = stream;
}

void CopyBytes(void* dst, int dst_device_type, const void* src, int src_device_type, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return;
  if (dst_device_type == kCPU && src_device_type == kCPU) {
    memcpy(dst, src, bytes);
    return;
  }
  hipMemcpyKind kind = dst_device_type == kCPU ? hipMemcpyDeviceToHost
                                               : (src_device_type == kCPU ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice);
  HIP_CHECK(hipMemcpyAsync(dst, src, bytes, kind, stream));
  HIP_CHECK(hipStreamSynchronize(stream));
}

}  // namespace blaze
