// sparse_puller.h -- the sparse-store plugin interface of the Embedding operator.
//
// Same ABI as the reference's blaze/store/sparse_puller.h:40-105 and store.h:15-35: a store is created by name
// through REGISTER_SPARSE_PULLER_CREATION, loaded once per PredictorManager, shared by every predictor (so Get
// must be re-entrant and read-only), and receives one SparsePullerInput / SparsePullerOutput per feature group.
// Get takes HOST pointers, as in the reference; GetOnStream (an extension: the reference's store runs on the host) takes
// the same structs with DEVICE pointers and enqueues its work on the caller's stream.
#pragma once

#include <functional>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

namespace blaze {
namespace store {

enum Status { kOK = 0, kTimeout, kFail };
enum UDFType { kSum = 0, kAvg, kAssign };
enum TruncDirection { kOrder = 0, kReverse };

struct SparsePullerInput {
  std::string version;
  std::string name;       // table name
  void* key = nullptr;    // ids
  void* key_num = nullptr;  // per-sample id counts
  size_t key_num_size = 0;  // batch
  void* value = nullptr;
  int key_type = 0, value_type = 0, num_type = 0;  // blaze DataType values
  int dim = 0;
  struct Param {
    UDFType udf_type = kSum;
    TruncDirection trunc_direction = kReverse;
    int trunc_num = 0;
  };
  std::vector<Param> in_item;
  size_t key_size = 0;    // number of ids (extension: lets a device store validate without reading key_num)
};

struct SparsePullerOutput {
  struct OutItem {
    void* out = nullptr;  // block base + item offset; element type = out_type
    size_t stride = 0;    // elements between samples
    // extension: elements between consecutive positions of a kAssign item; 0 = the group's dim (positions contiguous)
    size_t assign_pitch = 0;
  };
  std::vector<OutItem> out_item;
  int out_type = 0;       // extension: blaze DataType of the block (kFloat or kFloat16); 0 = same as value_type
};

class SparsePuller {
 public:
  virtual ~SparsePuller() {}
  virtual Status Load(const std::string& url) { return kFail; }
  virtual Status Get(const std::vector<SparsePullerInput>& input, std::vector<SparsePullerOutput>& output) { return kFail; }
  // device stores: Get with the stream to enqueue on and a caller-owned cache slot that keeps device-side
  // launch descriptors alive between calls (one per Embedding operator instance)
  struct DeviceCache {
    virtual ~DeviceCache() {}
  };
  virtual Status GetOnStream(const std::vector<SparsePullerInput>& input, std::vector<SparsePullerOutput>& output,
                             void* stream, std::unique_ptr<DeviceCache>* cache) {
    return Get(input, output);
  }
  virtual bool on_device() const { return false; }
};

using FCreateSparsePuller = std::function<SparsePuller*(void)>;

struct SparsePullerCreationRegisterer {
  static SparsePullerCreationRegisterer* Get();
  bool Register(const std::string& name, FCreateSparsePuller fcs);
  SparsePuller* CreateSparsePuller(const std::string& name);  // throws for an unknown name (sparse_puller.cc:21-25)

 private:
  std::unordered_map<std::string, FCreateSparsePuller> fcs_map_;
};

#define BLAZE_SP_CONCAT_(a, b) a##b
#define BLAZE_SP_CONCAT(a, b) BLAZE_SP_CONCAT_(a, b)
#define REGISTER_SPARSE_PULLER_CREATION(name, fcs) \
  static bool BLAZE_SP_CONCAT(sparse_puller_status_, __COUNTER__) = ::blaze::store::SparsePullerCreationRegisterer::Get()->Register(name, fcs);

}  // namespace store
}  // namespace blaze
