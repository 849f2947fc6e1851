// ref_driver.cc -- thin extern "C" driver around the REAL reference sources.
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile (target `ref`) in a
// container that has the reference tree; the output goes to oracle/_ref/ and
// is never committed.  It compiles, from where they lie in the reference tree,
//   blaze/store/quick_embedding/hashtable.cc, trie.cc, blaze/common/log.cc,
//   blaze/common/exception.cc
// and includes the header-only udf_processor.h and weight_blob.h.  Those are
// the pieces of the embedding path that build with g++ alone.
// QuickEmbeddingDict itself does not: quick_embedding_dict.h pulls in
// version_verifier.h -> common/types.h -> blaze/proto/blaze.pb.h, which is
// protoc-generated code that this image cannot generate.  Its per-sample loop
// (quick_embedding_dict.cc:105-141) is therefore re-walked below, but every
// arithmetic and lookup step inside the loop is the reference's own object code:
// UdfProcessorFactory<float,float>, HashTable::Lookup, WeightBlob::GetWeights.
#include <cstdint>
#include <cstring>
#include <sstream>
#include <string>
#include <vector>

#include "blaze/store/quick_embedding/hashtable.h"
#include "blaze/store/quick_embedding/trie.h"
#include "blaze/store/quick_embedding/udf_processor.h"
#include "blaze/store/quick_embedding/weight_blob.h"

using namespace blaze::store;

#define REF_API extern "C" __attribute__((visibility("default")))

struct RefTable {
  BulkLoadHashTable hash;
  WeightBlob<float> blob;
  int dim = 0;
};

// Build a one-table dict the way EmbeddingBuilder / the dict unit test do
// (test/store/quick_embedding/quick_embedding_dict_test.cc:30-79):
// InsertWeights -> byte offset -> hash value.
REF_API void* ref_table_build(const int64_t* keys, const float* rows, int64_t n, int dim) {
  RefTable* t = new RefTable();
  t->dim = dim;
  if (!t->blob.AllocateMemory((size_t)n * dim)) {
    delete t;
    return nullptr;
  }
  for (int64_t i = 0; i < n; ++i) {
    float* w = nullptr;
    uint64_t off = t->blob.InsertWeights(dim, &w);
    if (off == 0 || !w) {
      delete t;
      return nullptr;
    }
    memcpy(w, rows + i * dim, sizeof(float) * dim);
    t->hash.PreInsert((uint64_t)keys[i], off);
  }
  if (!t->hash.BulkLoad()) {
    delete t;
    return nullptr;
  }
  return t;
}

REF_API void ref_table_free(void* h) { delete static_cast<RefTable*>(h); }

// HashTable::Lookup on the table's index; value is the blob byte offset.
REF_API int ref_table_lookup(void* h, uint64_t key, uint64_t* value) {
  return static_cast<RefTable*>(h)->hash.Lookup(key, value) ? 1 : 0;
}

// Serialised HashTable image (HashTable::Dump); returns size, copies if dst.
REF_API uint64_t ref_table_hash_dump(void* h, unsigned char* dst) {
  std::ostringstream os(std::ios::binary);
  static_cast<RefTable*>(h)->hash.Dump(&os);
  std::string s = os.str();
  if (dst) memcpy(dst, s.data(), s.size());
  return s.size();
}

// Serialised WeightBlob image (WeightBlob::Dump).
REF_API uint64_t ref_table_blob_dump(void* h, unsigned char* dst) {
  std::ostringstream os(std::ios::binary);
  static_cast<RefTable*>(h)->blob.Dump(&os);
  std::string s = os.str();
  if (dst) memcpy(dst, s.data(), s.size());
  return s.size();
}

struct RefItem {
  int32_t udf;
  int32_t trunc_dir;
  int32_t trunc_num;
  int32_t pad_;
  float* out;
  int64_t stride;
};

// The per-feature-group walk of QuickEmbeddingDict::Get
// (quick_embedding_dict.cc:105-141) over the reference's own processors.
REF_API int ref_embed_get(void* h, const int64_t* ids, const float* values, const int32_t* segments, int64_t batch,
                          const RefItem* items, int32_t n_items) {
  RefTable* t = static_cast<RefTable*>(h);
  std::vector<SparsePullerInput::Param> params(n_items);
  std::vector<float*> out(n_items);
  for (int k = 0; k < n_items; ++k) {
    params[k].udf_type = static_cast<UDFType>(items[k].udf);
    params[k].trunc_direction = static_cast<TruncDirection>(items[k].trunc_dir);
    params[k].trunc_num = items[k].trunc_num;
    out[k] = items[k].out;
  }
  const int64_t* key = ids;
  const float* value = values;
  for (int64_t i = 0; i < batch; ++i) {
    size_t num = static_cast<size_t>(segments[i]);
    for (int k = 0; k < n_items; ++k)
      UdfProcessorFactory<float, float>::Create(params[k].udf_type)->InitProcess(t->dim, params[k], out[k]);
    for (size_t j = 0; j < num; ++j) {
      uint64_t off;
      if (!t->hash.Lookup((uint64_t)key[j], &off)) continue;
      float* w = t->blob.GetWeights(off);
      if (!w) continue;
      for (int k = 0; k < n_items; ++k)
        UdfProcessorFactory<float, float>::Create(params[k].udf_type)
            ->ElementProcess(value[j], w, t->dim, j, num, params[k], out[k]);
    }
    for (int k = 0; k < n_items; ++k) {
      UdfProcessorFactory<float, float>::Create(params[k].udf_type)->ReduceProcess(t->dim, num, params[k], out[k]);
      out[k] += items[k].stride;
    }
    key += num;
    value += num;
  }
  return 0;
}

// Trie: name -> gid, as QuickEmbeddingDict::GetGid uses it.
REF_API void* ref_trie_build(const char* const* names, const uint16_t* gids, int n) {
  BulkLoadTrie* t = new BulkLoadTrie();
  for (int i = 0; i < n; ++i) t->PreInsert(names[i], gids[i]);
  if (!t->BulkLoad()) {
    delete t;
    return nullptr;
  }
  return t;
}

REF_API void ref_trie_free(void* h) { delete static_cast<BulkLoadTrie*>(h); }

REF_API int ref_trie_lookup(void* h, const char* name, uint16_t* gid) {
  return static_cast<BulkLoadTrie*>(h)->Lookup(name, gid) ? 1 : 0;
}

REF_API uint64_t ref_trie_dump(void* h, unsigned char* dst) {
  std::ostringstream os(std::ios::binary);
  static_cast<BulkLoadTrie*>(h)->Dump(&os);
  std::string s = os.str();
  if (dst) memcpy(dst, s.data(), s.size());
  return s.size();
}
