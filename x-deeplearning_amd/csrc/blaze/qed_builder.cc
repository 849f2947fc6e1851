#include "blaze/qed_builder.h"

#include <algorithm>
#include <fstream>
#include <map>
#include <queue>
#include <vector>

#include "blaze/common.h"

namespace blaze {
namespace store {

namespace {

const uint32_t kSteps[] = {53,       97,       193,       389,       769,       1543,     3079,     6151,     12289,
                           24593,    49157,    98317,     196613,    393241,    786433,   1572869,  3145739,  6291469,
                           12582917, 25165843, 50331653,  100663319, 201326611, 402653189, 805306457};

std::vector<std::string> Split(const std::string& s, char delim) {
  std::vector<std::string> out;
  size_t b = 0;
  while (true) {
    size_t e = s.find(delim, b);
    if (e == std::string::npos) {
      out.push_back(s.substr(b));
      return out;
    }
    out.push_back(s.substr(b, e - b));
    b = e + 1;
  }
}

// trie bytes: BFS order, node = {u16 value, u8 nbranch, (u8 char, u32 child offset)*} (trie.cc:155-200)
std::string TrieBytes(const std::vector<std::pair<std::string, uint16_t>>& names) {
  struct Node {
    uint16_t value = 0xFF;
    std::map<unsigned char, int> next;
  };
  std::vector<Node> nodes(1);
  for (const auto& kv : names) {
    int cur = 0;
    for (unsigned char c : kv.first) {
      BLAZE_CONDITION_THROW(c < 128, "key has invalid charactor: ", kv.first);
      auto it = nodes[cur].next.find(c);
      if (it == nodes[cur].next.end()) {
        nodes.emplace_back();
        nodes[cur].next[c] = (int)nodes.size() - 1;
        cur = (int)nodes.size() - 1;
      } else {
        cur = it->second;
      }
    }
    if (nodes[cur].value != 0xFF)
      BLAZE_CONDITION_THROW(nodes[cur].value == kv.second, "conflict value with same key=", kv.first);
    nodes[cur].value = kv.second;
  }
  auto node_size = [&](int n) { return 3 + 5 * nodes[n].next.size(); };
  std::string bytes;
  std::queue<int> q;
  q.push(0);
  size_t allocated = node_size(0);
  while (!q.empty()) {
    const int n = q.front();
    q.pop();
    const uint16_t v = nodes[n].value;
    const uint8_t nb = (uint8_t)nodes[n].next.size();
    bytes.append((const char*)&v, 2);
    bytes.append((const char*)&nb, 1);
    for (const auto& kv : nodes[n].next) {
      const uint8_t ch = kv.first;
      const uint32_t off = (uint32_t)allocated;
      bytes.append((const char*)&ch, 1);
      bytes.append((const char*)&off, 4);
      allocated += node_size(kv.second);
      q.push(kv.second);
    }
  }
  return bytes;
}

}  // namespace

bool BuildQuickEmbedding(const std::string& path, const std::string& meta, const std::string& output_file, int value_type, int,
                         std::string* err) {
  try {
    BLAZE_CONDITION_THROW(value_type == kFloat || value_type == kFloat16, "Unsupported value type:", value_type);
    std::vector<std::string> fg_list;
    {
      std::ifstream fin(path + '/' + meta);
      BLAZE_CONDITION_THROW(fin.is_open(), "can not open meta file: ", path + '/' + meta);
      std::string buff;
      getline(fin, buff);
      while (!fin.eof()) {
        if (!buff.empty()) fg_list.push_back(buff);
        getline(fin, buff);
      }
    }
    BLAZE_CONDITION_THROW(!fg_list.empty(), "empty fg list!");
    std::ofstream os(output_file, std::ios::binary);
    BLAZE_CONDITION_THROW(os.is_open(), "can not open file: ", output_file);
    os.write("ALIMAMA_MODEL_SERVING_EMBEDDING", 31);
    const uint32_t version = 2000 + (value_type == kFloat ? 0 : 1);
    os.write((const char*)&version, 4);
    std::vector<std::pair<std::string, uint16_t>> names;
    for (size_t i = 0; i < fg_list.size(); ++i) names.emplace_back(fg_list[i], (uint16_t)i);
    const std::string trie = TrieBytes(names);
    const uint64_t trie_len = trie.size();
    os.write((const char*)&trie_len, 8);
    os.write(trie.data(), (std::streamsize)trie.size());
    const int esz = value_type == kFloat ? 4 : 2;
    for (size_t t = 0; t < fg_list.size(); ++t) {
      const std::string file = path + '/' + fg_list[t];
      std::ifstream fin(file);
      BLAZE_CONDITION_THROW(fin.is_open(), "can not open file: ", file);
      std::string buff;
      getline(fin, buff);
      BLAZE_CONDITION_THROW((bool)fin, "can not read first line, file: ", file);
      const int dim = (int)Split(buff, ',').size() - 1;
      BLAZE_CONDITION_THROW(dim >= 0, "invalid field size");
      struct Item {
        uint64_t key, value;
        uint32_t bucket;
      };
      std::vector<Item> items;
      std::string blob(1, '\0');  // byte 0 is the pad: offset 0 means "none"
      while (fin) {
        std::vector<std::string> fields = Split(buff, ',');
        if ((int)fields.size() == dim + 1) {
          try {
            const uint64_t key = (uint64_t)std::stoll(fields[0]);
            std::vector<float> w(dim);
            for (int i = 0; i < dim; ++i) w[i] = std::stof(fields[i + 1]);
            const uint64_t offset = blob.size();
            if (value_type == kFloat) {
              blob.append((const char*)w.data(), (size_t)dim * 4);
            } else {
              for (int i = 0; i < dim; ++i) {
                const uint16_t h = FloatToHalf(w[i]);
                blob.append((const char*)&h, 2);
              }
            }
            items.push_back({key, offset, (uint32_t)key});
          } catch (std::exception&) {
            LOG_ERROR("lexical cast failed! %s", buff.c_str());
          }
        } else {
          LOG_ERROR("string buff fields num error! %s", buff.c_str());
        }
        getline(fin, buff);
      }
      (void)esz;
      // BulkLoadHashTable: prime bucket count, sort by (bucket, key), bucket records {offset:40, size:24}
      uint32_t nbucket = kSteps[sizeof(kSteps) / sizeof(kSteps[0]) - 1];
      for (uint32_t s : kSteps)
        if (s > items.size()) {
          nbucket = s;
          break;
        }
      for (auto& it : items) it.bucket %= nbucket;
      std::sort(items.begin(), items.end(), [](const Item& a, const Item& b) {
        if (a.bucket != b.bucket) return a.bucket < b.bucket;
        return a.key < b.key;
      });
      std::vector<uint64_t> first(nbucket, 0), count(nbucket, 0), pairs(2 * items.size());
      for (size_t i = 0; i < items.size(); ++i) {
        if (count[items[i].bucket]++ == 0) first[items[i].bucket] = 16 * i;
        pairs[2 * i] = items[i].key;
        pairs[2 * i + 1] = items[i].value;
      }
      const uint16_t gid = (uint16_t)t;
      os.write((const char*)&gid, 2);
      os.write((const char*)&nbucket, 4);
      for (uint32_t b = 0; b < nbucket; ++b) {
        const uint64_t rec = (first[b] & 0xffffffffffull) | ((count[b] & 0xffffffull) << 40);
        os.write((const char*)&rec, 8);
      }
      const uint64_t pair_bytes = 16 * items.size();
      os.write((const char*)&pair_bytes, 8);
      os.write((const char*)pairs.data(), (std::streamsize)pair_bytes);
      const uint64_t blob_bytes = blob.size();
      os.write((const char*)&blob_bytes, 8);
      os.write(blob.data(), (std::streamsize)blob.size());
      BLAZE_CONDITION_THROW(os.good(), "export binary file failed!");
    }
    return true;
  } catch (std::exception& e) {
    if (err) *err = e.what();
    return false;
  }
}

}  // namespace store
}  // namespace blaze
