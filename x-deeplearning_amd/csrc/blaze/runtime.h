// runtime.h -- Blob (typed buffer that owns its memory) and the device contexts.
//
// Follows the ownership rules of the reference (blaze/common/blob.h:17-103): Reshape grows capacity and never
// shrinks it, RefReshape borrows foreign memory, operators never free their inputs.  The accelerator context
// replaces CUDAContext (blaze/common/context.h:123-182): streams are thread local per (device, stream id), so a
// serving thread that owns a Predictor owns its stream, and kernels are stream ordered with no device
// synchronisation inside operators.
#pragma once

#include <atomic>
#include <memory>
#include <vector>

#include "blaze/common.h"
#include "blaze/proto.h"

namespace blaze {

// cudaMalloc / malloc twins of blaze/common/allocator.h:33-71.  Host memory for device_type kCPU is pinned
// (hipHostMalloc) whenever a device is usable, so Feed / Output copies run at full PCIe rate; plain malloc otherwise.
void* Alloc(size_t bytes, int device_type, int device_id);
void Free(void* ptr, int device_type, int device_id);
// number of device / pinned-host allocations the host layer has made in this process (Alloc above plus the feed
// arenas and the Embedding operator's slot and offset buffers): lets a serving loop check that its steady state
// allocates nothing
std::atomic<int64_t>& AllocationCount();

class Blob {
 public:
  explicit Blob(const DeviceOption& device_option) : device_option_(device_option) {}
  Blob(const DeviceOption& device_option, const std::vector<TIndex>& dims, DataType data_type)
      : device_option_(device_option), data_type_(data_type) {
    Reshape(dims);
  }
  ~Blob() { Destroy(); }
  Blob(const Blob&) = delete;
  Blob& operator=(const Blob&) = delete;

  void Reshape(const std::vector<TIndex>& dims) {
    if (slices_ && slices_->parent != this && ReshapeAsSlice(dims)) return;
    TIndex n = 1;
    for (auto d : dims) n *= d;
    if (arena_view_) {
      // a view of a slice of its predictor's feed arena (Predictor::FeedMany): the next FeedMany places it again, so
      // a new shape allocates nothing.  A shape that outgrows the slice leaves the blob "unplaced" until it is fed;
      // Predictor::Forward refuses to run a net with an unplaced input.
      size_ = n;
      dims_ = dims;
      if (size_ > capacity_) unplaced_ = true;
      return;
    }
    size_ = n;
    if (size_ > capacity_ || !own_handle_) {
      Destroy();
      own_handle_ = true;
      slice_view_ = false;
      pitch_ = 0;
      capacity_ = size_;
      data_ = blaze::Alloc(capacity_ * DataTypeSize(data_type_), device_option_.device_type(), device_option_.device_id());
      ++version_;
      if (slices_ && slices_->parent == this) RefreshSlices();
    }
    dims_ = dims;
  }
  // the shape alone, for the output of an operator whose work its consumer has taken over: readers may ask the shape,
  // nobody reads the data (a later Reshape allocates as usual)
  void SetShapeOnly(const std::vector<TIndex>& dims) {
    TIndex n = 1;
    for (auto d : dims) n *= d;
    size_ = n;
    dims_ = dims;
  }
  // arena_view: `handle` is a slice of the owning predictor's feed arena (see Reshape)
  void RefReshape(const std::vector<TIndex>& dims, void* handle, bool arena_view = false) {
    if (own_handle_ || data_ != handle) {  // (re-aliasing the same buffer keeps the version)
      Destroy();
      own_handle_ = false;
      data_ = handle;
      ++version_;
    }
    arena_view_ = arena_view;
    unplaced_ = false;
    pitch_ = 0;
    slice_view_ = false;
    TIndex n = 1;
    for (auto d : dims) n *= d;
    size_ = capacity_ = n;
    dims_ = dims;
  }

  // ---- column slices: the inputs of a Concat along the last axis of 2-D tensors living directly in the
  // Concat's output, so that their producers write in place and the Concat has nothing to copy.  `children` are
  // the Concat's inputs in order; widths[i] is child i's column count (0 = not known yet).  A child becomes a
  // view (row pitch = the parent's width) when it is reshaped to 2-D while every width is known; any other
  // Reshape gives it memory of its own again.  The parent refreshes the views whenever its buffer moves.
  struct SliceGroup {
    Blob* parent = nullptr;
    std::vector<Blob*> children;
    std::vector<TIndex> widths;
  };
  static void LinkColumnSlices(Blob* parent, const std::vector<Blob*>& children, const std::vector<TIndex>& static_widths) {
    auto g = std::make_shared<SliceGroup>();
    g->parent = parent;
    g->children = children;
    g->widths = static_widths;
    parent->slices_ = g;
    for (Blob* c : children) c->slices_ = g;
  }
  // true after a Reshape beyond the feed-arena slice this blob views, until the next feed gives it memory
  bool unplaced() const { return unplaced_; }
  // gives an arena view memory of its own again (a single-input Feed after a FeedMany)
  void DropArenaView() {
    if (!arena_view_) return;
    arena_view_ = unplaced_ = false;
    data_ = nullptr;
    capacity_ = 0;
    own_handle_ = true;
    ++version_;
  }
  // elements between consecutive rows when this blob is a column slice, else 0 (rows are contiguous)
  TIndex pitch() const { return pitch_; }
  // whether this blob currently is the view of `parent`'s columns [col, col + shape[1])
  bool IsColumnSliceOf(const Blob* parent, TIndex col) const {
    return slice_view_ && slices_ && slices_->parent == parent && parent->data_ != nullptr &&
           parent->dims_.size() == 2 && pitch_ == parent->dims_[1] &&
           data_ == (const char*)parent->data_ + col * DataTypeSize(data_type_);
  }
  const DeviceOption& device_option() const { return device_option_; }
  int device_type() const { return device_option_.device_type(); }
  int device_id() const { return device_option_.device_id(); }
  // changing the element type of a blob that already holds memory re-sizes its capacity in elements
  void set_data_type(DataType t) {
    if (t != data_type_ && data_ != nullptr && own_handle_) capacity_ = capacity_ * DataTypeSize(data_type_) / DataTypeSize(t);
    data_type_ = t;
  }
  int data_type() const { return data_type_; }
  std::vector<TIndex>& shape() { return dims_; }
  const std::vector<TIndex>& shape() const { return dims_; }
  TIndex capacity() const { return capacity_; }
  TIndex size() const { return size_; }
  TIndex size(int start, int end) const {
    TIndex s = 1;
    for (int k = start; k < end; ++k) s *= dims_[k];
    return s;
  }
  TIndex dim(size_t index) const {
    BLAZE_CONDITION_THROW(index < dims_.size(), "index=", index, " dims_.size()=", dims_.size());
    return dims_[index];
  }
  template <typename T>
  T* as() { return reinterpret_cast<T*>(data_); }
  void* data() { return data_; }
  const void* data() const { return data_; }
  // bumps whenever the buffer address may have changed: lets operators cache descriptors that embed pointers
  uint64_t version() const { return version_; }

 private:
  bool ReshapeAsSlice(const std::vector<TIndex>& dims) {
    SliceGroup& g = *slices_;
    size_t me = 0;
    while (me < g.children.size() && g.children[me] != this) ++me;
    if (me == g.children.size() || dims.size() != 2 || g.parent->data_type_ != data_type_) return false;
    g.widths[me] = dims[1];
    TIndex total = 0;
    for (TIndex w : g.widths) {
      if (w == 0) return false;
      total += w;
    }
    if (own_handle_) Destroy();
    if (!slice_view_) data_ = nullptr;
    own_handle_ = false;
    slice_view_ = true;
    dims_ = dims;
    size_ = capacity_ = dims[0] * dims[1];
    g.parent->Reshape({dims[0], total});  // grows the buffer when needed
    g.parent->RefreshSlices();            // widths may have moved every view
    return true;
  }
  void RefreshSlices() {
    SliceGroup& g = *slices_;
    TIndex total = 0;
    for (TIndex w : g.widths) total += w;
    TIndex col = 0;
    for (size_t i = 0; i < g.children.size(); ++i) {
      Blob* c = g.children[i];
      if (c->slice_view_) {
        void* p = (char*)data_ + col * DataTypeSize(data_type_);
        if (c->data_ != p || c->pitch_ != total) ++c->version_;
        c->data_ = p;
        c->pitch_ = total;
      }
      col += g.widths[i];
    }
  }
  void Destroy() {
    if (data_ != nullptr && own_handle_)
      blaze::Free(data_, device_option_.device_type(), device_option_.device_id());
    data_ = nullptr;
    capacity_ = 0;
  }
  DeviceOption device_option_;
  void* data_ = nullptr;
  TIndex capacity_ = 0, size_ = 0;
  std::vector<TIndex> dims_;
  DataType data_type_ = kFloat;
  bool own_handle_ = true;
  uint64_t version_ = 0;
  TIndex pitch_ = 0;
  bool slice_view_ = false;
  bool arena_view_ = false;
  bool unplaced_ = false;
  std::shared_ptr<SliceGroup> slices_;
};

constexpr int kMaxStreamNum = 4;  // blaze/common/context.h:121

class CPUContext {
 public:
  explicit CPUContext(const DeviceOption& option) : device_option_(option) {}
  void SwitchToDevice(int) {}
  void FinishDeviceComputation() {}
  void* device_stream() const { return nullptr; }
  int device_type() const { return kCPU; }
  int stream_id() const { return 0; }
  const DeviceOption& device_option() const { return device_option_; }

 private:
  DeviceOption device_option_;
};

class HIPContext {
 public:
  explicit HIPContext(const DeviceOption& option) : device_option_(option), device_id_(option.device_id()) {}
  void SwitchToDevice(int stream_id) {
    stream_id_ = stream_id;
    Activate();
  }
  void Activate() const;                 // hipSetDevice when the thread is on another device
  hipStream_t hip_stream() const { return hip_stream(device_id_, stream_id_); }
  void* device_stream() const { return (void*)hip_stream(); }
  static hipStream_t hip_stream(int device_id, int stream_id);  // thread-local, created on first use
  // makes `stream` (created on device_id, default priority) the calling thread's stream from now on; the thread owns it:
  // it is destroyed when the thread ends, like one created on first use.  A stream the thread already had is
  // waited for and destroyed.
  static void AdoptThreadStream(int device_id, int stream_id, hipStream_t stream);
  void FinishDeviceComputation() {
    Activate();
    HIP_CHECK(hipStreamSynchronize(hip_stream()));
  }
  int device_type() const { return kHIP; }
  int device_id() const { return device_id_; }
  int stream_id() const { return stream_id_; }
  const DeviceOption& device_option() const { return device_option_; }

 private:
  DeviceOption device_option_;
  int device_id_ = 0;
  int stream_id_ = 0;
};

// copies between blobs of any two devices on `stream` (nullptr: the thread's stream 0), synchronous on return
void CopyBytes(void* dst, int dst_device_type, const void* src, int src_device_type, size_t bytes, hipStream_t stream);

}  // namespace blaze
