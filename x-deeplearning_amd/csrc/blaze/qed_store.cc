#include "blaze/qed_store.h"

#include <algorithm>
#include <fstream>
#include <numeric>

#include "blaze/runtime.h"
#include "blaze_hip.h"

namespace blaze {
namespace store {

// ------------------------------------------------------------------------------------------ registry
SparsePullerCreationRegisterer* SparsePullerCreationRegisterer::Get() {
  static SparsePullerCreationRegisterer* inst = new SparsePullerCreationRegisterer();
  return inst;
}
bool SparsePullerCreationRegisterer::Register(const std::string& name, FCreateSparsePuller fcs) {
  if (fcs_map_.count(name)) BLAZE_THROW("sparse puller ", name, " is registered twice");
  fcs_map_[name] = fcs;
  return true;
}
SparsePuller* SparsePullerCreationRegisterer::CreateSparsePuller(const std::string& name) {
  auto it = fcs_map_.find(name);
  BLAZE_CONDITION_THROW(it != fcs_map_.end(), "sparse puller: ", name, " is not registered");
  return it->second();
}

static SparsePuller* CreateQedHipSparsePuller() { return new QedHipSparsePuller(); }
REGISTER_SPARSE_PULLER_CREATION("qed_hip_sparse_puller", CreateQedHipSparsePuller);
// the name existing callers pass (predictor.h:236 default); on this build it is the device store
REGISTER_SPARSE_PULLER_CREATION("qed_sparse_puller", CreateQedHipSparsePuller);

// ------------------------------------------------------------------------------------------ tables
DeviceTable::~DeviceTable() {
  if (!owns) return;
  if (data) (void)hipFree(data);
  if (row_scale && scale_pitch != pitch) (void)hipFree(row_scale);  // (a scale stored inside the rows is part of `data`)
  if (hash_buckets) (void)hipFree(hash_buckets);
  if (hash_pairs) (void)hipFree(hash_pairs);
}

namespace {

const char kMagic[] = "ALIMAMA_MODEL_SERVING_EMBEDDING";
const uint32_t kSteps[] = {53,       97,       193,       389,       769,       1543,     3079,     6151,     12289,
                           24593,    49157,    98317,     196613,    393241,    786433,   1572869,  3145739,  6291469,
                           12582917, 25165843, 50331653,  100663319, 201326611, 402653189, 805306457};

uint32_t BucketSize(uint64_t n) {  // CalculateBucketSize, hashtable.cc:23-32
  for (uint32_t s : kSteps)
    if (s > n) return s;
  return kSteps[sizeof(kSteps) / sizeof(kSteps[0]) - 1];
}

int ElemSize(int value_type) { return value_type == kFloat ? 4 : (value_type == kFloat16 ? 2 : 1); }

// upload rows (host, unpadded, in `order`) to a pitched device table
void UploadRows(DeviceTable* t, const unsigned char* rows_host, int64_t row_bytes, const std::vector<int64_t>* order) {
  t->pitch = bz_table_pitch(row_bytes, 0);  // rows never straddle the 128-byte lines the memory system fetches
  std::vector<unsigned char> staged((size_t)t->rows * t->pitch, 0);
  for (int64_t r = 0; r < t->rows; ++r) {
    const int64_t src = order ? (*order)[r] : r;
    memcpy(&staged[(size_t)r * t->pitch], rows_host + src * row_bytes, (size_t)row_bytes);
  }
  HIP_CHECK(hipMalloc(&t->data, staged.size() ? staged.size() : 16));
  HIP_CHECK(hipMemcpy(t->data, staged.data(), staged.size(), hipMemcpyHostToDevice));
}

// device image of the hash index: prime bucket count, pairs sorted by (bucket, key) (BulkLoadHashTable,
// hashtable.cc:144-187), the value being the row number in the repacked table
void UploadHash(DeviceTable* t, const std::vector<uint64_t>& keys, const std::vector<uint64_t>& row_of_key) {
  const uint64_t n = keys.size();
  t->hash_bucket_size = BucketSize(n);
  std::vector<uint64_t> idx(n);
  std::iota(idx.begin(), idx.end(), 0);
  const uint32_t nb = t->hash_bucket_size;
  std::sort(idx.begin(), idx.end(), [&](uint64_t a, uint64_t b) {
    const uint32_t ba = (uint32_t)keys[a] % nb, bb = (uint32_t)keys[b] % nb;
    if (ba != bb) return ba < bb;
    return keys[a] < keys[b];
  });
  std::vector<uint64_t> buckets(nb, 0), pairs(2 * n);
  std::vector<uint32_t> count(nb, 0);
  for (uint64_t i = 0; i < n; ++i) {
    const uint32_t b = (uint32_t)keys[idx[i]] % nb;
    if (count[b] == 0) buckets[b] = 16 * i;
    ++count[b];
    pairs[2 * i] = keys[idx[i]];
    pairs[2 * i + 1] = row_of_key[idx[i]];
  }
  for (uint32_t b = 0; b < nb; ++b) buckets[b] = (buckets[b] & 0xffffffffffull) | ((uint64_t)(count[b] & 0xffffffu) << 40);
  HIP_CHECK(hipMalloc((void**)&t->hash_buckets, nb * 8));
  HIP_CHECK(hipMemcpy(t->hash_buckets, buckets.data(), nb * 8, hipMemcpyHostToDevice));
  HIP_CHECK(hipMalloc((void**)&t->hash_pairs, n ? n * 16 : 16));
  HIP_CHECK(hipMemcpy(t->hash_pairs, pairs.data(), n * 16, hipMemcpyHostToDevice));
}

// keys are exactly {0..n-1}: rows can be ordered by key and addressed directly
bool DenseKeys(const std::vector<uint64_t>& keys, std::vector<int64_t>* pos_of_key) {
  const uint64_t n = keys.size();
  pos_of_key->assign(n, -1);
  for (uint64_t i = 0; i < n; ++i) {
    if (keys[i] >= n || (*pos_of_key)[keys[i]] >= 0) return false;
    (*pos_of_key)[keys[i]] = (int64_t)i;
  }
  return true;
}

struct SlotCache : SparsePuller::DeviceCache {
  std::vector<bz_embed_slot> host;
  std::vector<bz_embed_slot> scratch;  // this call's records, rebuilt in place every call
  bz_embed_slot* pinned = nullptr;
  bz_embed_slot* dev = nullptr;
  size_t cap = 0;
  bz_embed_launch launch;
  int64_t* offsets = nullptr;  // scratch for the separate scan, when the planner advises it
  size_t offsets_cap = 0;      // in elements
  // the tables the records point into: held so that a table replaced in the store (AddTable, Load) outlives the
  // launches that may still read it
  std::vector<std::shared_ptr<const DeviceTable>> tables;
  ~SlotCache() override {
    if (pinned) (void)hipHostFree(pinned);
    if (dev) (void)hipFree(dev);
    if (offsets) (void)hipFree(offsets);
  }
};

}  // namespace

Status QedHipSparsePuller::Load(const std::string& url) {
  try {
    return LoadImpl(url);
  } catch (std::exception& e) {
    LOG_ERROR("load quick embedding dict failed! url: %s: %s", url.c_str(), e.what());
    return kFail;
  }
}

Status QedHipSparsePuller::LoadImpl(const std::string& url) {
  std::ifstream is(url, std::ios::binary);
  if (!is.is_open()) {
    LOG_ERROR("load quick embedding dict failed! url: %s", url.c_str());
    return kFail;
  }
  is.seekg(0, std::ios::end);
  const uint64_t file_bytes = (uint64_t)is.tellg();
  is.seekg(0, std::ios::beg);
  // sizes read from the file are checked against what is left of it before anything is allocated for them
  auto left = [&]() -> uint64_t {
    const std::streamoff at = is.tellg();
    return at < 0 ? 0 : file_bytes - std::min<uint64_t>(file_bytes, (uint64_t)at);
  };
  // [1] header
  char magic[31];
  is.read(magic, 31);
  uint32_t version = 0;
  is.read((char*)&version, 4);
  if (!is.good() || memcmp(magic, kMagic, 31) != 0) {
    LOG_ERROR("load verifier failed! url: %s", url.c_str());
    return kFail;
  }
  switch (version % 1000) {
    case 0: file_value_type_ = kFloat; break;
    case 1: file_value_type_ = kFloat16; break;
    case 2: file_value_type_ = kInt8; break;
    default:
      LOG_ERROR("unknown value type of dict url: %s version: %u", url.c_str(), version);
      return kFail;
  }
  // [2] trie
  uint64_t trie_len = 0;
  is.read((char*)&trie_len, 8);
  if (!is.good() || trie_len > (1ull << 32) || trie_len > left()) {
    LOG_ERROR("load trie failed! url: %s", url.c_str());
    return kFail;
  }
  std::vector<unsigned char> trie(trie_len);
  is.read((char*)trie.data(), (std::streamsize)trie_len);
  if (!is.good()) {
    LOG_ERROR("load trie failed! url: %s", url.c_str());
    return kFail;
  }
  std::map<std::string, uint16_t> paths;
  {
    std::vector<std::pair<uint32_t, std::string>> stack = {{0u, std::string()}};
    while (!stack.empty()) {
      auto cur = stack.back();
      stack.pop_back();
      size_t pos = cur.first;
      BLAZE_CONDITION_THROW(pos + 3 <= trie.size(), "trie node offset ", pos, " outside the ", trie.size(), " trie bytes");
      uint16_t value;
      memcpy(&value, &trie[pos], 2);
      const uint8_t nbranch = trie[pos + 2];
      pos += 3;
      paths[cur.second] = value;
      BLAZE_CONDITION_THROW(pos + 5ull * nbranch <= trie.size(), "trie node at ", cur.first, " overruns the trie bytes");
      BLAZE_CONDITION_THROW(paths.size() <= (1u << 20), "trie has too many nodes");
      for (int b = 0; b < nbranch; ++b) {
        const uint8_t ch = trie[pos];
        uint32_t off;
        memcpy(&off, &trie[pos + 1], 4);
        pos += 5;
        BLAZE_CONDITION_THROW(off > cur.first, "trie child offset does not move forward (corrupt file)");
        stack.emplace_back(off, cur.second + (char)ch);
      }
    }
  }
  // [3] tables
  std::map<uint16_t, std::shared_ptr<DeviceTable>> tables;
  const int esz = ElemSize(file_value_type_);
  uint16_t gid;
  while (is.read((char*)&gid, 2)) {
    uint32_t nbucket = 0;
    is.read((char*)&nbucket, 4);
    if (!is.good() || (uint64_t)nbucket * 8 > left()) { LOG_ERROR("load hashtable failed! url: %s gid: %d", url.c_str(), gid); return kFail; }
    std::vector<uint64_t> buckets(nbucket);
    is.read((char*)buckets.data(), (std::streamsize)nbucket * 8);
    uint64_t pair_bytes = 0;
    is.read((char*)&pair_bytes, 8);
    if (!is.good() || pair_bytes % 16 != 0 || pair_bytes > left()) { LOG_ERROR("load hashtable failed! url: %s gid: %d", url.c_str(), gid); return kFail; }
    std::vector<uint64_t> pairs(pair_bytes / 8);
    is.read((char*)pairs.data(), (std::streamsize)pair_bytes);
    uint64_t blob_bytes = 0;
    is.read((char*)&blob_bytes, 8);
    if (!is.good() || blob_bytes == 0 || blob_bytes > left()) { LOG_ERROR("load weight blob failed! url: %s gid: %d", url.c_str(), gid); return kFail; }
    std::vector<unsigned char> blob(blob_bytes);
    is.read((char*)blob.data(), (std::streamsize)blob_bytes);
    if (!is.good()) { LOG_ERROR("load weight blob failed! url: %s gid: %d", url.c_str(), gid); return kFail; }

    const uint64_t n = pair_bytes / 16;
    std::shared_ptr<DeviceTable> t(new DeviceTable());
    t->value_type = file_value_type_;
    t->rows = (int64_t)n;
    if (n == 0) {
      tables[gid] = std::move(t);
      continue;
    }
    // the file does not record dim: every row has the same width, so it is (blob - pad byte) / rows
    BLAZE_CONDITION_THROW((blob_bytes - 1) % n == 0 && ((blob_bytes - 1) / n) % esz == 0,
                          "gid ", gid, ": blob of ", blob_bytes, " bytes does not hold ", n, " equal rows");
    const int64_t row_bytes = (int64_t)((blob_bytes - 1) / n);
    t->dim = (int)(row_bytes / esz);
    std::vector<uint64_t> keys(n), blob_row(n);
    for (uint64_t i = 0; i < n; ++i) {
      keys[i] = pairs[2 * i];
      const uint64_t off = pairs[2 * i + 1];
      BLAZE_CONDITION_THROW(off >= 1 && off < blob_bytes && (off - 1) % row_bytes == 0, "gid ", gid, ": key ", keys[i],
                            " points at blob offset ", off, " which is not a row start");
      blob_row[i] = (off - 1) / row_bytes;
    }
    std::vector<int64_t> pos_of_key;
    if (DenseKeys(keys, &pos_of_key)) {
      std::vector<int64_t> order(n);  // table row k <- blob row of key k
      for (uint64_t k = 0; k < n; ++k) order[k] = (int64_t)blob_row[pos_of_key[k]];
      UploadRows(t.get(), blob.data() + 1, row_bytes, &order);
    } else {
      UploadRows(t.get(), blob.data() + 1, row_bytes, nullptr);
      UploadHash(t.get(), keys, blob_row);
    }
    tables[gid] = std::move(t);
  }
  std::unique_lock<std::shared_mutex> lock(mutex_);
  trie_paths_ = std::move(paths);
  tables_ = std::move(tables);
  return kOK;
}

Status QedHipSparsePuller::AddTable(const std::string& table_name, int value_type, int64_t rows, int dim, const void* rows_ptr,
                                    bool on_device, const int64_t* keys, const float* scale) {
  try {
    BLAZE_CONDITION_THROW(value_type == kFloat || value_type == kFloat16 || value_type == kInt8, "Unsupported value type:", value_type);
    BLAZE_CONDITION_THROW(rows > 0 && dim > 0 && rows_ptr != nullptr, "AddTable: rows=", rows, " dim=", dim);
    BLAZE_CONDITION_THROW(value_type != kInt8 || scale != nullptr, "AddTable: int8 table needs a per-row scale");
    std::shared_ptr<DeviceTable> t(new DeviceTable());
    t->value_type = value_type;
    t->rows = rows;
    t->dim = dim;
    const int64_t row_bytes = (int64_t)dim * ElemSize(value_type);
    t->pitch = bz_table_pitch(row_bytes, scale ? 4 : 0);
    BLAZE_CONDITION_THROW(t->pitch > 0, "AddTable: row of ", row_bytes, " bytes");
    HIP_CHECK(hipMalloc(&t->data, (size_t)rows * t->pitch));
    if (t->pitch != row_bytes) HIP_CHECK(hipMemset(t->data, 0, (size_t)rows * t->pitch));
    HIP_CHECK(hipMemcpy2D(t->data, t->pitch, rows_ptr, row_bytes, row_bytes, rows,
                          on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice));
    if (scale) {
      // the scale travels with its row: one line fetch per id instead of two
      const int64_t at = (row_bytes + 3) / 4 * 4;
      t->row_scale = (float*)((char*)t->data + at);
      t->scale_pitch = t->pitch;
      HIP_CHECK(hipMemcpy2D(t->row_scale, t->pitch, scale, 4, 4, rows, on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice));
    }
    if (keys) {
      std::vector<uint64_t> k(rows), r(rows);
      for (int64_t i = 0; i < rows; ++i) {
        k[i] = (uint64_t)keys[i];
        r[i] = (uint64_t)i;
      }
      UploadHash(t.get(), k, r);
    }
    std::unique_lock<std::shared_mutex> lock(mutex_);
    uint16_t gid = 0;
    auto it = trie_paths_.find(table_name);
    if (it != trie_paths_.end() && it->second != 0xFF) {
      gid = it->second;
    } else {
      while (tables_.count(gid) || gid == 0xFF) ++gid;
      for (size_t len = 0; len < table_name.size(); ++len)
        if (!trie_paths_.count(table_name.substr(0, len))) trie_paths_[table_name.substr(0, len)] = 0xFF;
      trie_paths_[table_name] = gid;
    }
    tables_[gid] = std::move(t);
    return kOK;
  } catch (std::exception& e) {
    LOG_ERROR("AddTable %s failed: %s", table_name.c_str(), e.what());
    return kFail;
  }
}

bool QedHipSparsePuller::LookupGid(const std::string& name, uint16_t* gid) const {
  std::shared_lock<std::shared_mutex> lock(mutex_);
  auto it = trie_paths_.find(name);
  if (it == trie_paths_.end()) return false;
  *gid = it->second;
  return true;
}

std::shared_ptr<const DeviceTable> QedHipSparsePuller::table(uint16_t gid) const {
  std::shared_lock<std::shared_mutex> lock(mutex_);
  auto it = tables_.find(gid);
  return it == tables_.end() ? nullptr : it->second;
}

namespace {

// What one thread needs to serve host-memory Get calls: a stream, one growing device arena for the staged inputs and
// output columns, and the launch cache GetOnStream keeps.  Lives until the thread ends.
struct HostStage {
  int device = -1;
  hipStream_t stream = nullptr;
  char* arena = nullptr;
  size_t cap = 0;
  std::unique_ptr<SparsePuller::DeviceCache> cache;
  ~HostStage() {
    if (arena) (void)hipFree(arena);
    if (stream) (void)hipStreamDestroy(stream);
  }
};

size_t Align256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace

// SparsePuller::Get as the reference declares it (blaze/store/sparse_puller.h:77-83) and as its host Embedding operator
// calls it (embedding_op.cc:87): every pointer is HOST memory.  The tables live on the device, so the ids, counts and
// values are copied there, the pooling kernel runs, and each item's columns are copied back into the caller's block:
// two PCIe crossings and a wait per call.  The lookup itself is the same kernel GetOnStream launches; nothing is
// computed on the host.  Columns of the block that belong to no item, and the columns of an unknown table's items,
// are left as the caller had them (quick_embedding_dict.cc:95).  Re-entrant: the staging state is per thread.
Status QedHipSparsePuller::Get(const std::vector<SparsePullerInput>& input, std::vector<SparsePullerOutput>& output) {
  if (input.size() != output.size()) return kFail;
  thread_local HostStage hs;
  int device = 0;
  HIP_CHECK(hipGetDevice(&device));
  if (hs.device != device) {
    BLAZE_CONDITION_THROW(hs.device < 0, "a thread's host-memory Get calls must stay on one device");
    HIP_CHECK(hipStreamCreateWithFlags(&hs.stream, hipStreamNonBlocking));
    hs.device = device;
  }
  struct ItemPlan {
    size_t at = 0, span = 0;  // arena offset; elements per sample on the device copy
    bool copy_back = false;
  };
  struct GroupPlan {
    size_t key_at = 0, num_at = 0, value_at = 0, nkeys = 0;
    int esz = 4;
    std::vector<ItemPlan> items;
  };
  std::vector<GroupPlan> plan(input.size());
  size_t need = 0;
  for (size_t i = 0; i < input.size(); ++i) {
    const SparsePullerInput& in = input[i];
    const SparsePullerOutput& out = output[i];
    if (in.in_item.size() != out.out_item.size()) return kFail;
    if (in.in_item.empty()) continue;
    BLAZE_CONDITION_THROW(in.key_type == kInt64, "Unsupported key type:", in.key_type);
    BLAZE_CONDITION_THROW(in.value_type == kFloat, "Unsupported value type:", in.value_type);
    BLAZE_CONDITION_THROW(in.num_type == kInt32, "Unsupported num type:", in.num_type);
    const int out_type = out.out_type ? out.out_type : in.value_type;
    BLAZE_CONDITION_THROW(out_type == kFloat || out_type == kFloat16, "Unsupported block type:", out_type);
    BLAZE_CONDITION_THROW(in.dim > 0, "dim ", in.dim);
    GroupPlan& g = plan[i];
    g.esz = out_type == kFloat ? 4 : 2;
    // the reference's structure carries no id count: it is the sum of the per-sample counts
    const int32_t* counts = (const int32_t*)in.key_num;
    BLAZE_CONDITION_THROW(in.key_num_size == 0 || counts != nullptr, "key_num is null");
    size_t nkeys = 0;
    for (size_t b = 0; b < in.key_num_size; ++b) nkeys += counts[b] > 0 ? (size_t)counts[b] : 0;
    BLAZE_CONDITION_THROW(in.key_size == 0 || in.key_size == nkeys, "key_size ", in.key_size, " but the counts add up to ", nkeys);
    BLAZE_CONDITION_THROW(nkeys == 0 || in.key != nullptr, "key is null");
    g.nkeys = nkeys;
    g.key_at = need;
    need += Align256(nkeys * 8);
    g.num_at = need;
    need += Align256(in.key_num_size * 4);
    g.value_at = need;
    if (in.value != nullptr) need += Align256(nkeys * 4);
    uint16_t gid = 0;
    std::shared_ptr<const DeviceTable> t;
    if (LookupGid(in.name, &gid)) t = table(gid);
    const bool known = t != nullptr && t->rows > 0;
    g.items.resize(in.in_item.size());
    for (size_t k = 0; k < in.in_item.size(); ++k) {
      ItemPlan& it = g.items[k];
      const size_t pitch = out.out_item[k].assign_pitch ? out.out_item[k].assign_pitch : (size_t)in.dim;
      const size_t positions = in.in_item[k].udf_type == kAssign ? (size_t)std::max(1, in.in_item[k].trunc_num) : 1;
      it.span = (positions - 1) * pitch + (size_t)in.dim;
      BLAZE_CONDITION_THROW(out.out_item[k].out != nullptr && out.out_item[k].stride >= it.span, "item ", k, " of ", in.name,
                            ": ", it.span, " elements a sample do not fit a stride of ", out.out_item[k].stride);
      it.copy_back = known && in.key_num_size > 0;
      it.at = need;
      need += Align256(in.key_num_size * it.span * g.esz);
    }
  }
  if (need == 0) return kOK;
  if (hs.cap < need) {
    if (hs.arena) HIP_CHECK(hipFree(hs.arena));  // (the previous call waited for its stream before it returned)
    hs.arena = nullptr;
    hs.cap = 0;
    ++AllocationCount();
    HIP_CHECK(hipMalloc((void**)&hs.arena, need + need / 2));
    hs.cap = need + need / 2;
  }
  std::vector<SparsePullerInput> dev_in(input);
  std::vector<SparsePullerOutput> dev_out(output);
  for (size_t i = 0; i < input.size(); ++i) {
    const SparsePullerInput& in = input[i];
    if (in.in_item.empty()) continue;
    const GroupPlan& g = plan[i];
    if (g.nkeys) HIP_CHECK(hipMemcpyAsync(hs.arena + g.key_at, in.key, g.nkeys * 8, hipMemcpyHostToDevice, hs.stream));
    if (in.key_num_size) HIP_CHECK(hipMemcpyAsync(hs.arena + g.num_at, in.key_num, in.key_num_size * 4, hipMemcpyHostToDevice, hs.stream));
    if (in.value != nullptr && g.nkeys) HIP_CHECK(hipMemcpyAsync(hs.arena + g.value_at, in.value, g.nkeys * 4, hipMemcpyHostToDevice, hs.stream));
    dev_in[i].key = hs.arena + g.key_at;
    dev_in[i].key_num = hs.arena + g.num_at;
    dev_in[i].value = in.value != nullptr ? hs.arena + g.value_at : nullptr;
    dev_in[i].key_size = g.nkeys;
    for (size_t k = 0; k < g.items.size(); ++k) {
      dev_out[i].out_item[k].out = hs.arena + g.items[k].at;
      dev_out[i].out_item[k].stride = g.items[k].span;
    }
  }
  Status st = GetOnStream(dev_in, dev_out, hs.stream, &hs.cache);
  if (st == kOK) {
    for (size_t i = 0; i < input.size(); ++i) {
      const GroupPlan& g = plan[i];
      for (size_t k = 0; k < g.items.size(); ++k) {
        if (!g.items[k].copy_back) continue;
        const size_t row_bytes = g.items[k].span * g.esz;
        HIP_CHECK(hipMemcpy2DAsync(output[i].out_item[k].out, output[i].out_item[k].stride * g.esz, hs.arena + g.items[k].at,
                                   row_bytes, row_bytes, input[i].key_num_size, hipMemcpyDeviceToHost, hs.stream));
      }
    }
  }
  HIP_CHECK(hipStreamSynchronize(hs.stream));
  return st;
}

Status QedHipSparsePuller::GetOnStream(const std::vector<SparsePullerInput>& input, std::vector<SparsePullerOutput>& output,
                                       void* stream, std::unique_ptr<DeviceCache>* cache) {
  if (input.size() != output.size()) return kFail;
  if (!*cache) cache->reset(new SlotCache());
  SlotCache* sc = static_cast<SlotCache*>(cache->get());
  std::vector<bz_embed_slot>& slots = sc->scratch;
  slots.clear();
  std::vector<std::shared_ptr<const DeviceTable>> held;
  for (size_t i = 0; i < input.size(); ++i) {
    const SparsePullerInput& in = input[i];
    const SparsePullerOutput& out = output[i];
    if (in.in_item.size() != out.out_item.size()) return kFail;
    if (in.in_item.empty()) continue;  // feature group absent from the operator's inputs
    // the type switches of store/defines.h:12-67
    BLAZE_CONDITION_THROW(in.key_type == kInt64, "Unsupported key type:", in.key_type);
    BLAZE_CONDITION_THROW(in.value_type == kFloat, "Unsupported value type:", in.value_type);
    BLAZE_CONDITION_THROW(in.num_type == kInt32, "Unsupported num type:", in.num_type);
    const int out_type = out.out_type ? out.out_type : in.value_type;
    BLAZE_CONDITION_THROW(out_type == kFloat || out_type == kFloat16, "Unsupported block type:", out_type);
    uint16_t gid = 0;
    std::shared_ptr<const DeviceTable> t;
    if (LookupGid(in.name, &gid)) t = table(gid);  // table name miss: the block keeps its zeros
    if (t != nullptr && t->rows == 0) t = nullptr;
    if (t != nullptr) held.push_back(t);
    if (t != nullptr)
      BLAZE_CONDITION_THROW(t->dim == in.dim, "table ", in.name, " has dim ", t->dim, " but the embedding config says ", in.dim);
    for (size_t k = 0; k < in.in_item.size(); ++k) {
      bz_embed_slot s;
      memset(&s, 0, sizeof(s));
      if (t) {
        s.table = t->data;
        s.row_scale = t->row_scale;
        s.scale_pitch = t->scale_pitch;
        s.hash_buckets = t->hash_buckets;
        s.hash_pairs = t->hash_pairs;
        s.hash_bucket_size = t->hash_bucket_size;
        s.rows = t->rows;
        s.pitch = t->pitch;
        s.table_dtype = t->value_type == kFloat ? BZ_F32 : (t->value_type == kFloat16 ? BZ_F16 : BZ_I8);
      } else {
        s.table_dtype = BZ_F32;
      }
      s.dim = in.dim;
      s.ids = (const int64_t*)in.key;
      s.values = (const float*)in.value;
      s.segments = (const int32_t*)in.key_num;
      s.nnz = (int64_t)in.key_size;
      s.offsets = nullptr;  // fused scan
      s.out = out.out_item[k].out;
      s.out_stride = (int64_t)out.out_item[k].stride;
      s.assign_pitch = (int32_t)out.out_item[k].assign_pitch;
      s.out_dtype = out_type == kFloat ? BZ_F32 : BZ_F16;
      s.udf = (int)in.in_item[k].udf_type;
      s.trunc_dir = (int)in.in_item[k].trunc_direction;
      s.trunc_num = in.in_item[k].trunc_num;
      s.batch = (int32_t)in.key_num_size;
      slots.push_back(s);
    }
  }
  // (the previous call's tables are let go only now: its launch has been waited for before this predictor runs again)
  sc->tables.swap(held);
  if (slots.empty()) return kOK;
  BZ_CHECK(bz_embed_plan(slots.data(), (int)slots.size(), &sc->launch));
  hipStream_t st = (hipStream_t)stream;
  if (sc->launch.scan_first) {
    // many workgroups per slot: scan every slot's counts once into scratch instead of once per workgroup
    size_t need = 0;
    for (const auto& s : slots) need += (size_t)s.batch + 1;
    if (sc->offsets_cap < need) {
      if (sc->offsets) HIP_CHECK(hipFree(sc->offsets));  // (its last reader finished: a predictor is waited for before its next pass)
      ++AllocationCount();
      HIP_CHECK(hipMalloc((void**)&sc->offsets, need * sizeof(int64_t)));
      sc->offsets_cap = need;
    }
    size_t at = 0;
    for (auto& s : slots) {
      s.offsets = sc->offsets + at;
      at += (size_t)s.batch + 1;
    }
    BZ_CHECK(bz_embed_plan(slots.data(), (int)slots.size(), &sc->launch));
  }
  // an operator of few slots: the records travel as kernel arguments, nothing to upload
  if (sc->launch.fused_scan && !sc->launch.scan_first && slots.size() <= (size_t)(sc->launch.variant != 0 ? BZ_EMBED_ARG_SLOTS : 16)) {
    BZ_CHECK(bz_embed_pool_args(slots.data(), &sc->launch, st));
    return kOK;
  }
  const size_t bytes = slots.size() * sizeof(bz_embed_slot);
  const bool changed = sc->host.size() != slots.size() || memcmp(sc->host.data(), slots.data(), bytes) != 0;
  if (changed) {
    if (sc->cap < slots.size()) {
      // the previous launch that read the old buffers has completed: the net waits for its stream after every run
      if (sc->pinned) HIP_CHECK(hipHostFree(sc->pinned));
      if (sc->dev) HIP_CHECK(hipFree(sc->dev));
      sc->cap = slots.size();
      AllocationCount() += 2;
      HIP_CHECK(hipHostMalloc((void**)&sc->pinned, sc->cap * sizeof(bz_embed_slot), hipHostMallocDefault));
      HIP_CHECK(hipMalloc((void**)&sc->dev, sc->cap * sizeof(bz_embed_slot)));
    }
    memcpy(sc->pinned, slots.data(), bytes);
    HIP_CHECK(hipMemcpyAsync(sc->dev, sc->pinned, bytes, hipMemcpyHostToDevice, st));
    sc->host = slots;
  }
  if (!sc->launch.fused_scan) BZ_CHECK(bz_segments_to_offsets_slots(sc->dev, (int)slots.size(), st));
  BZ_CHECK(bz_embed_pool(sc->dev, &sc->launch, st));
  return kOK;
}

}  // namespace store
}  // namespace blaze
