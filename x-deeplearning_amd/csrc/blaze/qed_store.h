// qed_store.h -- "qed_hip_sparse_puller": the QED embedding store served from device memory.
//
// Load reads the reference's on-disk format (blaze/store/quick_embedding/quick_embedding_dict.cc:29-74):
//   31-byte magic "ALIMAMA_MODEL_SERVING_EMBEDDING", u32 version = 2000 + {0 fp32, 1 fp16, 2 int8}
//   (version_verifier.cc:40-63); u64 length + trie bytes, nodes {u16 value, u8 nbranch, (u8 ch, u32 offset)*}
//   in BFS order (trie.cc:70-124); then per table {u16 gid; u32 nbucket; 8-byte buckets {offset:40,size:24};
//   u64 bytes + (u64 key, u64 blob offset) pairs (hashtable.cc:96-118); u64 bytes + weight blob whose byte 0 is a
//   pad so that offset 0 means "none" (weight_blob.h:20,65-84)}.
// Rows are repacked to a 16-byte-aligned pitch and uploaded; the hash index is uploaded with row numbers as
// values, or dropped when the keys are exactly 0..n-1 (row = key).  Get launches the pooling kernel of
// include/blaze_hip.h on the caller's stream; it keeps the semantics of QuickEmbeddingDict::Get (:76-148): unknown
// table -> block left zero, unknown key -> skipped, kAvg divides by the id count including unknown keys.
#pragma once

#include <map>
#include <memory>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <vector>

#include "blaze/common.h"
#include "blaze/sparse_puller.h"

namespace blaze {
namespace store {

struct DeviceTable {
  int value_type = kFloat;  // kFloat | kFloat16 | kInt8 (int8 needs row_scale; not loadable from a QED file)
  int dim = 0;
  int64_t rows = 0;
  int pitch = 0;
  void* data = nullptr;       // device
  float* row_scale = nullptr; // device: scale of row r at byte offset r * scale_pitch (inside `data` when scale_pitch == pitch)
  int scale_pitch = 0;
  uint64_t* hash_buckets = nullptr;
  uint64_t* hash_pairs = nullptr;
  uint32_t hash_bucket_size = 0;
  bool owns = true;
  ~DeviceTable();
};

class QedHipSparsePuller : public SparsePuller {
 public:
  QedHipSparsePuller() {}
  ~QedHipSparsePuller() override {}
  Status Load(const std::string& url) override;
  // host pointers, as the reference's interface passes them: staged through the device (copy in, the same pooling
  // kernel, copy back, wait); nothing is computed on the host
  Status Get(const std::vector<SparsePullerInput>& input, std::vector<SparsePullerOutput>& output) override;
  Status GetOnStream(const std::vector<SparsePullerInput>& input, std::vector<SparsePullerOutput>& output, void* stream,
                     std::unique_ptr<DeviceCache>* cache) override;
  bool on_device() const override { return true; }

  // Registers a table that is already in memory (synthetic benchmarks, tables produced on the device).
  // rows_ptr holds [rows, dim] elements of value_type, row major, on the device (on_device) or the host;
  // keys == nullptr: ids are row numbers.  scale: per-row fp32 scale for kInt8.  No reference counterpart.
  Status AddTable(const std::string& table_name, int value_type, int64_t rows, int dim, const void* rows_ptr, bool on_device,
                  const int64_t* keys, const float* scale);
  // table name -> gid exactly as Trie::Lookup answers (trie.cc:44-68), interior nodes included
  bool LookupGid(const std::string& name, uint16_t* gid) const;
  // (both take the store's lock shared; a table handed out stays alive while the caller holds the pointer, also
  // when AddTable / Load replace it meanwhile)
  std::shared_ptr<const DeviceTable> table(uint16_t gid) const;

 private:
  Status LoadImpl(const std::string& url);
  std::map<std::string, uint16_t> trie_paths_;  // every node path of the trie -> its value (0xFF on interior nodes)
  std::map<uint16_t, std::shared_ptr<DeviceTable>> tables_;
  int file_value_type_ = kFloat;
  mutable std::shared_mutex mutex_;  // Get* read the two maps shared, AddTable / Load replace them exclusively
};

}  // namespace store
}  // namespace blaze
