// registry.h -- string-keyed factories, the mechanism behind REGISTER_*_OPERATOR, REGISTER_NET and
// REGISTER_SPARSE_PULLER_CREATION.  Same contract as the reference's blaze/common/registry.h:23-83:
// duplicate keys throw at static-initialisation time, an unknown key creates nullptr.
#pragma once

#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "blaze/common.h"

namespace blaze {

template <class ObjectPtrType, class... Args>
class Registry {
 public:
  typedef std::function<ObjectPtrType(Args...)> Creator;

  void Register(const std::string& key, Creator creator) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (creators_.count(key)) BLAZE_THROW("key ", key, " is duplicate registered");
    creators_[key] = creator;
  }
  bool Has(const std::string& key) const { return creators_.count(key) != 0; }
  ObjectPtrType Create(const std::string& key, Args... args) {
    auto it = creators_.find(key);
    if (it == creators_.end()) {
      LOG_ERROR("key=%s not exist", key.c_str());
      return nullptr;
    }
    return it->second(args...);
  }
  std::vector<std::string> Keys() const {
    std::vector<std::string> keys;
    for (const auto& it : creators_) keys.push_back(it.first);
    return keys;
  }

 private:
  std::mutex mutex_;
  std::map<std::string, Creator> creators_;
};

template <class ObjectPtrType, class... Args>
struct Registerer {
  Registerer(const std::string& key, Registry<ObjectPtrType, Args...>* registry,
             typename Registry<ObjectPtrType, Args...>::Creator creator) {
    registry->Register(key, creator);
  }
  template <class Derived>
  static ObjectPtrType DefaultCreator(Args... args) {
    return ObjectPtrType(new Derived(args...));
  }
};

#define BLAZE_CONCAT_IMPL(a, b) a##b
#define BLAZE_CONCAT(a, b) BLAZE_CONCAT_IMPL(a, b)
#define ANONYMOUS_VARIABLE(str) BLAZE_CONCAT(str, __COUNTER__)

}  // namespace blaze
