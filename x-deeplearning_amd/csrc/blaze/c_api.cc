// c_api.cc -- the Blaze_* C ABI over Predictor / PredictorManager (include/blaze_c_api.h).
#include "blaze_c_api.h"

#include <hip/hip_runtime.h>

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <mutex>
#include <thread>

#include "blaze/optimizer.h"
#include "blaze/predictor.h"
#include "blaze/qed_builder.h"
#include "blaze/qed_store.h"
#include "blaze_hip.h"

using blaze::Predictor;
using blaze::PredictorManager;

namespace {

// thread-local message buffer (the reference keeps 4 MB per thread; messages here are short)
struct ErrorEntry {
  char last_string[16384];
};
ErrorEntry* ErrorStore() {
  static thread_local ErrorEntry e = {{0}};
  return &e;
}

// thread-local storage behind the string arrays the List*/Param*/DumpObservers calls hand out
struct StringVectorEntry {
  std::vector<std::string> strings, values;
  std::vector<const char*> names, keys, vals;
};
StringVectorEntry* StringStore() {
  static thread_local StringVectorEntry e;
  return &e;
}

int Fail(const char* what) {
  const std::string& why = blaze::last_error_for_thread();
  if (why.empty())
    Blaze_SetLastErrorString("%s", what);
  else
    Blaze_SetLastErrorString("%s: %s", what, why.c_str());
  blaze::last_error_for_thread().clear();
  return -1;
}

int ReturnNames(const std::vector<std::string>& src, size_t* ndim, const char*** names) {
  StringVectorEntry* e = StringStore();
  e->strings = src;
  e->names.clear();
  for (const auto& s : e->strings) e->names.push_back(s.c_str());
  *ndim = e->names.size();
  *names = e->names.data();
  return 0;
}

}  // namespace

extern "C" {

void Blaze_GetLastErrorString(const char** msg) { *msg = ErrorStore()->last_string; }

void Blaze_SetLastErrorString(const char* format, ...) {
  va_list ap;
  va_start(ap, format);
  vsnprintf(ErrorStore()->last_string, sizeof(ErrorStore()->last_string), format, ap);
  va_end(ap);
}

int Blaze_InitScheduler(int enable_batching, int max_batch_size, int batch_timeout_micros, int num_threads_for_cpu,
                        int num_threads_for_cuda, int num_threads_for_pipe) {
  if (!blaze::InitScheduler(enable_batching, max_batch_size, batch_timeout_micros, num_threads_for_cpu, num_threads_for_cuda,
                            num_threads_for_pipe))
    return Fail("InitScheduler Failed");
  return 0;
}

int Blaze_PredictorManagerCreate(PredictorManagerHandle* handle) {
  if (handle == nullptr) return Fail("Create PredictorManager Failed");
  *handle = new PredictorManager();
  return 0;
}
int Blaze_PredictorManagerDelete(PredictorManagerHandle handle) {
  delete reinterpret_cast<PredictorManager*>(handle);
  (void)hipGetLastError();  // teardown ignores the runtime's return codes; none may surface in the caller's next call
  return 0;
}
int Blaze_PredictorManagerSetDataType(PredictorManagerHandle handle, int data_type) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr) return Fail("SetDataType: the predict manager is nullptr");
  pm->SetDataType(static_cast<blaze::PredictDataType>(data_type));
  return 0;
}
int Blaze_PredictorManagerSetRunMode(PredictorManagerHandle handle, const char* run_mode) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr) return Fail("SetRunMode: the predict manager is nullptr");
  pm->SetRunMode(run_mode);
  return 0;
}
int Blaze_LoadSparseModelWeight(PredictorManagerHandle handle, const char* file) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr || file == nullptr) return Fail("Load sparse model weight failed");
  if (!pm->LoadSparseModelWeight(file)) return Fail("Load sparse model weight failed");
  return 0;
}
int Blaze_PredictorManagerLoadModel(PredictorManagerHandle handle, const char* file, int optimization_pass) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr || file == nullptr) return Fail("Load blaze model failed");
  if (!pm->LoadModel(file, optimization_pass != 0)) return Fail("Load blaze model failed");
  return 0;
}
int Blaze_PredcitorManagerLoadModel(PredictorManagerHandle handle, const char* file, int optimization_pass) {
  return Blaze_PredictorManagerLoadModel(handle, file, optimization_pass);
}
int Blaze_PredictorManagerLoadDeepNetModel(PredictorManagerHandle handle, const char* conf, const char* param, int optimization_pass) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr) return Fail("The predict manager is nullptr");
  if (!pm->LoadDeepNetModel(conf, param, optimization_pass != 0)) return Fail("Load deepnet model failed");
  return 0;
}
int Blaze_PredictorManagerLoadModelFromString(PredictorManagerHandle handle, const char* data, size_t len, int is_text) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr || data == nullptr) return Fail("The predict manager is nullptr");
  try {
    blaze::NetDef def;
    if (is_text) {
      blaze::ParseNetDefText(std::string(data, len), &def);
    } else if (!blaze::ParseNetDefBinary(data, len, &def)) {
      return Fail("malformed NetDef");
    }
    if (!pm->LoadNetDef(def)) return Fail("LoadNetDef failed");
  } catch (std::exception& e) {
    blaze::last_error_for_thread() = e.what();
    return Fail("Load model from string failed");
  }
  return 0;
}

int Blaze_PredictorCreate(PredictorManagerHandle mgr, int device_type, int device_id, PredictorHandle* handle) {
  auto* pm = reinterpret_cast<PredictorManager*>(mgr);
  if (pm == nullptr || handle == nullptr) return Fail("Create Predictor Failed");
  Predictor* p = pm->CreatePredictor(static_cast<blaze::PredictDeviceType>(device_type), device_id);
  if (p == nullptr) return Fail("Create Predictor Failed");
  *handle = p;
  return 0;
}
int Blaze_PredictorDelete(PredictorHandle handle) {
  if (handle == nullptr) return -1;
  delete reinterpret_cast<Predictor*>(handle);
  (void)hipGetLastError();
  return 0;
}

int Blaze_PredictorReshapeInput(PredictorHandle handle, const char* name, const int* data, int num) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return Fail("The predictor is nullptr");
  std::vector<size_t> shape;
  for (int i = 0; i < num; ++i) shape.push_back((size_t)data[i]);
  if (!p->ReshapeInput(name, shape)) {
    Blaze_SetLastErrorString("Reshape input: %s failed", name);
    return -1;
  }
  return 0;
}
int Blaze_PredictorFeed(PredictorHandle handle, const char* name, void* data, int len) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return Fail("The predictor is nullptr");
  if (!p->Feed(name, data, (size_t)len)) {
    Blaze_SetLastErrorString("Feed %s failed", name);
    return -1;
  }
  return 0;
}
int Blaze_PredictorFeedMany(PredictorHandle handle, int count, const char* const* names, const void* const* data, const size_t* lens) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr || count < 0 || (count > 0 && (names == nullptr || data == nullptr || lens == nullptr))) return -1;
  for (int i = 0; i < count; ++i)
    if (names[i] == nullptr || (data[i] == nullptr && lens[i] != 0)) return Fail("FeedMany: null name or data");
  if (!p->FeedMany(count, names, data, lens)) return Fail("FeedMany failed");
  return 0;
}
int Blaze_PredictorForward(PredictorHandle handle) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  if (!p->Forward()) return Fail("Forward failed");
  return 0;
}
int Blaze_PredictorForwardN(PredictorHandle handle, int count) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  for (int i = 0; i < count; ++i)
    if (!p->Forward()) return Fail("Forward failed");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Serving pool: n persistent threads, each driving its own predictors -- the reference's deployment model (one
// Predictor per thread, api/cpp_api/predictor.h:90-92; example/cpp/predictor_example.cc runs one loop per thread).
// ---------------------------------------------------------------------------------------------------------------
namespace {
struct ServePool {
  std::vector<std::thread> threads;
  std::mutex mu;
  std::condition_variable cv_work, cv_done;
  uint64_t generation = 0;
  std::atomic<uint64_t> generation_hint{0};  // copy of `generation` that idle threads poll without the mutex
  std::atomic<int> pending_hint{0};          // copy of `pending` that Run polls without the mutex
  int pending = 0;
  bool stop = false;
  // the job of the current generation
  Predictor** handles = nullptr;
  int n_handles = 0;
  int64_t steps = 0;
  int depth = 2;  // passes a thread keeps queued on its stream
  std::atomic<int> failed{0};
  std::string error;
  // what every pass of the last job took on its thread, launch to "the wait has returned" (milliseconds): the latency a
  // request sees under the load of that job, as the reference's example times each Forward inside its serving loop
  // (example/cpp/predictor_example.cc:129-140)
  std::vector<std::vector<float>> latency_ms;
  // The threads' streams, spread evenly over the hardware queues.  The runtime serves a handful of hardware queues (4 by
  // default) and gives a new stream the least used one, counting every stream of the process, idle ones included: eight
  // threads that each create a stream can end up 3-3-1-1 on the queues, and the threads that share a queue with two
  // others then set the pace of the whole pool.  So the pool creates the streams itself at its first job, finds out by
  // measurement which of them share a queue (ShareQueue), keeps an even selection and hands one to each thread.
  int streams_device = -1;
  std::vector<hipStream_t> assigned;  // stream of thread t (owned by the thread once it has adopted it)
  std::vector<int> queue_of;          // the queue group of thread t's stream, numbered in order of discovery
  std::vector<char> adopted;

  explicit ServePool(int n) : latency_ms(n), adopted(n, 0) {
    for (int t = 0; t < n; ++t) threads.emplace_back([this, t] { Loop(t); });
  }
  ~ServePool() {
    {
      std::lock_guard<std::mutex> lock(mu);
      stop = true;
    }
    cv_work.notify_all();
    for (auto& th : threads) th.join();
    for (size_t t = 0; t < assigned.size(); ++t)
      if (!adopted[t] && assigned[t]) (void)hipStreamDestroy(assigned[t]);
  }

  // Do two streams share a hardware queue?  A kernel queued on b while a is kept busy finishes at once when they do not,
  // and only after a's kernel when they do.  "At once" cannot be wrong; "late" can be the host's doing, so it is asked twice.
  static bool ShareQueue(hipStream_t a, hipStream_t b) {
    constexpr int kBusyUs = 300;
    for (int attempt = 0; attempt < 2; ++attempt) {
      BZ_CHECK(bz_spin(kBusyUs, a));
      const auto t0 = std::chrono::steady_clock::now();
      BZ_CHECK(bz_spin(0, b));
      HIP_CHECK(hipStreamSynchronize(b));
      const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
      HIP_CHECK(hipStreamSynchronize(a));
      if (us < kBusyUs / 2) return false;
    }
    return true;
  }

  void AssignStreams(int device) {
    const int n = (int)threads.size();
    int cur = 0;
    HIP_CHECK(hipGetDevice(&cur));
    if (cur != device) HIP_CHECK(hipSetDevice(device));
    std::vector<hipStream_t> cand;
    std::vector<int> group;               // of each candidate
    std::vector<hipStream_t> first_of;    // a member of each group
    std::vector<int> picked;              // candidates kept, in thread order
    const int per_round = std::max(n, 8);  // a few more than a small pool needs, so that every queue shows up
    for (int round = 0; round < 4 && (int)picked.size() < n; ++round) {
      for (int i = 0; i < per_round; ++i) {
        hipStream_t s = nullptr;
        HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
        BZ_CHECK(bz_spin(0, s));  // the runtime binds a stream to its queue at the first launch
        HIP_CHECK(hipStreamSynchronize(s));
        int g = -1;
        for (size_t k = 0; k < first_of.size() && g < 0; ++k)
          if (ShareQueue(first_of[k], s)) g = (int)k;
        if (g < 0) {
          g = (int)first_of.size();
          first_of.push_back(s);
        }
        cand.push_back(s);
        group.push_back(g);
      }
      // as even a share of the n threads for every queue seen as there can be, the fuller shares to the queues that
      // have the most candidates
      const int G = (int)first_of.size();
      std::vector<int> have(G, 0), order(G), cap(G, 0);
      for (int g : group) ++have[g];
      for (int g = 0; g < G; ++g) order[g] = g;
      std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return have[a] > have[b]; });
      for (int k = 0; k < G; ++k) cap[order[k]] = n / G + (k < n % G ? 1 : 0);
      picked.clear();
      std::vector<int> taken(G, 0);
      for (size_t c = 0; c < cand.size() && (int)picked.size() < n; ++c)
        if (taken[group[c]] < cap[group[c]]) {
          ++taken[group[c]];
          picked.push_back((int)c);
        }
    }
    // (queues that never offered enough candidates: fill up with what there is)
    std::vector<char> used(cand.size(), 0);
    for (int c : picked) used[c] = 1;
    for (size_t c = 0; c < cand.size() && (int)picked.size() < n; ++c)
      if (!used[c]) {
        used[c] = 1;
        picked.push_back((int)c);
      }
    // threads that follow each other take different queues
    std::vector<std::vector<int>> by_group(first_of.size());
    for (int c : picked) by_group[group[c]].push_back(c);
    assigned.clear();
    queue_of.clear();
    for (size_t k = 0; (int)assigned.size() < n; ++k)
      for (auto& members : by_group)
        if (k < members.size()) {
          assigned.push_back(cand[members[k]]);
          queue_of.push_back(group[members[k]]);
        }
    for (size_t c = 0; c < cand.size(); ++c)
      if (!used[c]) HIP_CHECK(hipStreamDestroy(cand[c]));
    streams_device = device;
    if (cur != device) HIP_CHECK(hipSetDevice(cur));
  }
  void Loop(int t) {
    uint64_t seen = 0;
    for (;;) {
      int n_threads;
      {
        // a job that follows the previous one at once (a warm-up run, then the timed one) should not pay a futex
        // wake-up per thread: poll for a short while before going to sleep
        const auto spin_until = std::chrono::steady_clock::now() + std::chrono::microseconds(2000);
        while (generation_hint.load(std::memory_order_acquire) == seen && std::chrono::steady_clock::now() < spin_until) {
        }
        std::unique_lock<std::mutex> lock(mu);
        cv_work.wait(lock, [&] { return stop || generation != seen; });
        if (stop) return;
        seen = generation;
        n_threads = (int)threads.size();
      }
      if (!adopted[t] && t < (int)assigned.size()) {
        try {
          blaze::HIPContext::AdoptThreadStream(streams_device, 0, assigned[t]);
          adopted[t] = 1;
        } catch (std::exception& e) {
          blaze::last_error_for_thread() = e.what();
          if (!failed.exchange(1)) {
            std::lock_guard<std::mutex> lock(mu);
            error = e.what();
          }
        }
      }
      // step i of the job runs predictor i % n_handles; thread t takes the steps i == t (mod n_threads), so a
      // predictor is only ever used by one thread when n_handles is a multiple of n_threads.  With at least `depth`
      // predictors per thread, the thread keeps `depth` passes queued on its stream: it launches step j + depth - 1
      // before it waits for step j, so the device does not idle while the host is woken up and launches again.
      const int per_thread = n_handles / n_threads;
      const int64_t d = std::max<int64_t>(1, std::min<int64_t>(depth, per_thread));
      auto fail = [&] {
        if (!failed.exchange(1)) {
          std::lock_guard<std::mutex> lock(mu);
          error = blaze::last_error_for_thread();
        }
      };
      using Clock = std::chrono::steady_clock;
      std::vector<float>& lat = latency_ms[t];
      lat.clear();
      lat.reserve((size_t)std::min<int64_t>(steps / n_threads + 1, 1 << 22));
      auto record = [&](Clock::time_point from) {
        if (lat.size() < lat.capacity()) lat.push_back(std::chrono::duration<float, std::milli>(Clock::now() - from).count());
      };
      if (d == 1) {
        for (int64_t i = t; i < steps && !failed.load(std::memory_order_relaxed); i += n_threads) {
          const auto t0 = Clock::now();
          if (!handles[i % n_handles]->Forward()) fail();
          record(t0);
        }
      } else {
        Clock::time_point began[64];  // launch times of the passes in flight (depth <= 64)
        int64_t launched = t, waited = t;  // next step to launch / to wait for
        while (waited < steps) {
          while (launched < steps && (launched - waited) / n_threads < d && !failed.load(std::memory_order_relaxed)) {
            began[(launched / n_threads) % 64] = Clock::now();
            if (!handles[launched % n_handles]->ForwardLaunch()) fail();
            launched += n_threads;
          }
          if (waited >= launched) break;  // a failure stopped the launches
          if (!handles[waited % n_handles]->ForwardWait()) fail();
          record(began[(waited / n_threads) % 64]);
          waited += n_threads;
        }
      }
      {
        std::lock_guard<std::mutex> lock(mu);
        pending_hint.store(--pending, std::memory_order_release);
        if (pending == 0) cv_done.notify_all();
      }
    }
  }
  bool Run(Predictor** h, int n, int64_t k) {
    if (streams_device < 0 && n > 0 && h[0] != nullptr && h[0]->device_id() >= 0) {
      try {
        AssignStreams(h[0]->device_id());
      } catch (std::exception& e) {
        error = e.what();
        return false;
      }
    }
    std::unique_lock<std::mutex> lock(mu);
    handles = h;
    n_handles = n;
    steps = k;
    failed = 0;
    error.clear();
    pending = (int)threads.size();
    pending_hint.store(pending, std::memory_order_release);
    ++generation;
    generation_hint.store(generation, std::memory_order_release);
    cv_work.notify_all();
    lock.unlock();
    // short jobs end before a sleeping caller could be woken: poll first, sleep only when the job is a long one
    const auto spin_until = std::chrono::steady_clock::now() + std::chrono::microseconds(5000);
    while (pending_hint.load(std::memory_order_acquire) != 0 && std::chrono::steady_clock::now() < spin_until) {
    }
    lock.lock();
    cv_done.wait(lock, [&] { return pending == 0; });
    return failed.load() == 0;
  }
};
}  // namespace

int Blaze_ServePoolCreate(int n_threads, ServePoolHandle* handle) {
  if (handle == nullptr || n_threads < 1 || n_threads > 256) return Fail("ServePoolCreate: bad arguments");
  *handle = new ServePool(n_threads);
  return 0;
}
int Blaze_ServePoolRun(ServePoolHandle handle, PredictorHandle* predictors, int n_predictors, int64_t steps) {
  auto* pool = reinterpret_cast<ServePool*>(handle);
  if (pool == nullptr || predictors == nullptr || n_predictors < 1 || steps < 0) return Fail("ServePoolRun: bad arguments");
  if (n_predictors % (int)pool->threads.size() != 0)
    return Fail("ServePoolRun: the number of predictors must be a multiple of the pool's threads (a predictor belongs to one thread)");
  if (!pool->Run(reinterpret_cast<Predictor**>(predictors), n_predictors, steps)) {
    Blaze_SetLastErrorString("Forward failed in the serving pool: %s", pool->error.c_str());
    return -1;
  }
  return 0;
}
int Blaze_ServePoolSetDepth(ServePoolHandle handle, int depth) {
  auto* pool = reinterpret_cast<ServePool*>(handle);
  if (pool == nullptr || depth < 1 || depth > 64) return Fail("ServePoolSetDepth: bad arguments");
  std::lock_guard<std::mutex> lock(pool->mu);
  pool->depth = depth;
  return 0;
}
int Blaze_ServePoolLatencies(ServePoolHandle handle, float* out_ms, int64_t capacity, int64_t* count) {
  auto* pool = reinterpret_cast<ServePool*>(handle);
  if (pool == nullptr || count == nullptr || capacity < 0 || (capacity > 0 && out_ms == nullptr))
    return Fail("ServePoolLatencies: bad arguments");
  std::lock_guard<std::mutex> lock(pool->mu);  // (no job is running: Run returns only when its threads are done)
  int64_t n = 0;
  for (const auto& v : pool->latency_ms)
    for (float x : v) {
      if (n < capacity) out_ms[n] = x;
      ++n;
    }
  *count = n;
  return 0;
}
int Blaze_PredictorForwardLaunch(PredictorHandle handle) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  if (!p->ForwardLaunch()) return Fail("ForwardLaunch failed");
  return 0;
}
int Blaze_PredictorForwardWait(PredictorHandle handle) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  if (!p->ForwardWait()) return Fail("ForwardWait failed");
  return 0;
}
int Blaze_ServePoolStreamQueues(ServePoolHandle handle, int* queue_of_thread, int capacity, int* count) {
  auto* pool = reinterpret_cast<ServePool*>(handle);
  if (pool == nullptr || count == nullptr || (capacity > 0 && queue_of_thread == nullptr)) return Fail("ServePoolStreamQueues: bad arguments");
  *count = (int)pool->queue_of.size();
  for (int t = 0; t < *count && t < capacity; ++t) queue_of_thread[t] = pool->queue_of[t];
  return 0;
}

int Blaze_ServePoolDelete(ServePoolHandle handle) {
  delete reinterpret_cast<ServePool*>(handle);
  (void)hipGetLastError();
  return 0;
}

int Blaze_PredictorOutputShape(PredictorHandle handle, const char* name, size_t* ndim, size_t** nshape) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  try {
    const std::vector<size_t>& shape = p->OutputShape(name);
    *ndim = shape.size();
    *nshape = const_cast<size_t*>(shape.data());
  } catch (std::exception& e) {
    Blaze_SetLastErrorString("%s", e.what());
    return -1;
  }
  return 0;
}
int Blaze_PredictorOutputDataType(PredictorHandle handle, const char* name, int* data_type) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  *data_type = p->OutputDataType(name);
  return *data_type < 0 ? Fail("not an output of the net") : 0;
}
int Blaze_PredictorOutput(PredictorHandle handle, const char* name, void* data, size_t len) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  size_t slen = 0;
  void* dptr = nullptr;
  if (!p->Output(name, &dptr, &slen)) {
    Blaze_SetLastErrorString("Output %s failed", name);
    return -1;
  }
  if (slen > len) {
    Blaze_SetLastErrorString("Output %s needs %zu bytes, caller gave %zu", name, slen, len);
    return -1;
  }
  memcpy(data, dptr, slen);
  return 0;
}

int Blaze_PredictorParamName(PredictorHandle handle, size_t* ndim, const char*** name) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  return ReturnNames(p->ListInternalName(), ndim, name);
}
int Blaze_PredictorParamShape(PredictorHandle handle, const char* name, size_t* ndim, size_t** nshape) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  try {
    const std::vector<size_t>& shape = p->InternalShape(name);
    *ndim = shape.size();
    *nshape = const_cast<size_t*>(shape.data());
  } catch (std::exception& e) {
    Blaze_SetLastErrorString("%s", e.what());
    return -1;
  }
  return 0;
}
int Blaze_PredictorParamDataType(PredictorHandle handle, const char* name, int* data_type) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  *data_type = p->InternalDataType(name);
  return *data_type < 0 ? Fail("not a parameter of the net") : 0;
}
int Blaze_PredictorParam(PredictorHandle handle, const char* name, void* data, size_t len) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  size_t slen = 0;
  void* dptr = nullptr;
  if (!p->InternalParam(name, &dptr, &slen) || slen > len) {
    Blaze_SetLastErrorString("Param %s failed", name);
    return -1;
  }
  memcpy(data, dptr, slen);
  return 0;
}

int Blaze_PredictorListInputNames(PredictorHandle handle, size_t* ndim, const char*** names) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  return ReturnNames(p->ListInputName(), ndim, names);
}
int Blaze_PredictorListOutputNames(PredictorHandle handle, size_t* ndim, const char*** names) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  return ReturnNames(p->ListOutputName(), ndim, names);
}

int Blaze_PredictorRegisterObservers(PredictorHandle handle, size_t ndim, const char** names) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  std::vector<std::string> v;
  for (size_t i = 0; i < ndim; ++i) v.push_back(names[i]);
  p->RegisterObservers(v);
  return 0;
}
int Blaze_PredictorDumpObservers(PredictorHandle handle, size_t* ndim, const char*** key, const char*** value) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr) return -1;
  std::unordered_map<std::string, std::string> dump;
  p->DumpObservers(&dump);
  StringVectorEntry* e = StringStore();
  e->strings.clear();
  e->values.clear();
  for (const auto& kv : dump) {
    e->strings.push_back(kv.first);
    e->values.push_back(kv.second);
  }
  e->keys.clear();
  e->vals.clear();
  for (size_t i = 0; i < e->strings.size(); ++i) {
    e->keys.push_back(e->strings[i].c_str());
    e->vals.push_back(e->values[i].c_str());
  }
  *ndim = e->keys.size();
  *key = e->keys.data();
  *value = e->vals.data();
  return 0;
}

int Blaze_ConvertBlaze(const char*, const char*, int, int, int, int, const char**, const int*, const char*, int) {
  Blaze_SetLastErrorString("Blaze_ConvertBlaze: the model importers are not part of this build");
  return -1;
}
// c_api_blaze_optimizer.cc: load the model, run the optimizer, store the result (binary != 0: wire format, else text).
// Of the reference's passes this build has the parallel-Gemm fusion (blaze/optimizer.h).
int Blaze_OptimizeBlaze(const char* raw_model_file, const char* optimized_model_file, int binary) {
  if (raw_model_file == nullptr || optimized_model_file == nullptr) return Fail("OptimizeBlaze: null argument");
  try {
    blaze::NetDef def;
    std::string err;
    if (!blaze::LoadNetDefFromFile(raw_model_file, &def, &err)) {
      Blaze_SetLastErrorString("OptimizeBlaze: %s", err.c_str());
      return -1;
    }
    blaze::FuseGemmChains(&def);
    blaze::FuseParallelGemms(&def);
    std::string s;
    if (binary)
      blaze::SerializeNetDefBinary(def, &s);
    else
      blaze::SerializeNetDefText(def, &s);
    FILE* f = fopen(optimized_model_file, "wb");
    if (f == nullptr || fwrite(s.data(), 1, s.size(), f) != s.size()) {
      if (f) fclose(f);
      Blaze_SetLastErrorString("OptimizeBlaze: cannot write %s", optimized_model_file);
      return -1;
    }
    fclose(f);
  } catch (std::exception& e) {
    Blaze_SetLastErrorString("OptimizeBlaze: %s", e.what());
    return -1;
  }
  return 0;
}
int Blaze_QuickEmbeddingBuildFp32(const char* path, const char* meta, const char* output_file, int thread_num) {
  std::string err;
  if (!blaze::store::BuildQuickEmbedding(path, meta, output_file, blaze::kFloat, thread_num, &err)) {
    Blaze_SetLastErrorString("QuickEmbeddingBuildFp32 failed: %s", err.c_str());
    return -1;
  }
  return 0;
}
int Blaze_QuickEmbeddingBuildFp16(const char* path, const char* meta, const char* output_file, int thread_num) {
  std::string err;
  if (!blaze::store::BuildQuickEmbedding(path, meta, output_file, blaze::kFloat16, thread_num, &err)) {
    Blaze_SetLastErrorString("QuickEmbeddingBuildFp16 failed: %s", err.c_str());
    return -1;
  }
  return 0;
}

int Blaze_HipStoreAddTable(PredictorManagerHandle handle, const char* table_name, int value_type, int64_t rows, int dim,
                           const void* rows_ptr, int on_device, const int64_t* keys, const float* scale) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr || table_name == nullptr) return Fail("The predict manager is nullptr");
  try {
    auto& puller = pm->EnsureSparsePuller("qed_hip_sparse_puller");
    auto* qed = dynamic_cast<blaze::store::QedHipSparsePuller*>(puller.get());
    if (qed == nullptr) return Fail("the manager's sparse puller is not the device store");
    if (qed->AddTable(table_name, value_type, rows, dim, rows_ptr, on_device != 0, keys, scale) != blaze::store::kOK)
      return Fail("AddTable failed");
  } catch (std::exception& e) {
    blaze::last_error_for_thread() = e.what();
    return Fail("AddTable failed");
  }
  return 0;
}

int Blaze_HipStoreGet(PredictorManagerHandle handle, const char* table_name, const int64_t* keys, const int32_t* key_num,
                      size_t batch, const float* values, int dim, int n_items, const int* udf_type, const int* trunc_direction,
                      const int* trunc_num, void* const* out, const size_t* stride, int out_type) {
  auto* pm = reinterpret_cast<PredictorManager*>(handle);
  if (pm == nullptr || table_name == nullptr) return Fail("The predict manager is nullptr");
  if (n_items < 0 || (n_items > 0 && (udf_type == nullptr || trunc_direction == nullptr || trunc_num == nullptr || out == nullptr ||
                                      stride == nullptr)))
    return Fail("null argument");
  try {
    auto& puller = pm->EnsureSparsePuller("qed_hip_sparse_puller");
    std::vector<blaze::store::SparsePullerInput> in(1);
    std::vector<blaze::store::SparsePullerOutput> o(1);
    in[0].name = table_name;
    in[0].key = const_cast<int64_t*>(keys);
    in[0].key_num = const_cast<int32_t*>(key_num);
    in[0].key_num_size = batch;
    in[0].value = const_cast<float*>(values);
    in[0].key_type = blaze::kInt64;
    in[0].value_type = blaze::kFloat;
    in[0].num_type = blaze::kInt32;
    in[0].dim = dim;
    o[0].out_type = out_type;
    for (int k = 0; k < n_items; ++k) {
      blaze::store::SparsePullerInput::Param p;
      p.udf_type = (blaze::store::UDFType)udf_type[k];
      p.trunc_direction = (blaze::store::TruncDirection)trunc_direction[k];
      p.trunc_num = trunc_num[k];
      in[0].in_item.push_back(p);
      blaze::store::SparsePullerOutput::OutItem item;
      item.out = out[k];
      item.stride = stride[k];
      o[0].out_item.push_back(item);
    }
    if (puller->Get(in, o) != blaze::store::kOK) return Fail("Get failed");
  } catch (std::exception& e) {
    blaze::last_error_for_thread() = e.what();
    return Fail("Get failed");
  }
  return 0;
}

int Blaze_ConvertNetDef(const char* in, size_t len, int in_is_text, int out_is_text, char* out, size_t cap, size_t* out_len) {
  if (in == nullptr || out_len == nullptr) return Fail("null argument");
  try {
    blaze::NetDef def;
    if (in_is_text) {
      blaze::ParseNetDefText(std::string(in, len), &def);
    } else if (!blaze::ParseNetDefBinary(in, len, &def)) {
      return Fail("malformed NetDef");
    }
    std::string s;
    if (out_is_text)
      blaze::SerializeNetDefText(def, &s);
    else
      blaze::SerializeNetDefBinary(def, &s);
    *out_len = s.size();
    if (out != nullptr) {
      if (cap < s.size()) return Fail("output buffer too small");
      memcpy(out, s.data(), s.size());
    }
  } catch (std::exception& e) {
    blaze::last_error_for_thread() = e.what();
    return Fail("convert failed");
  }
  return 0;
}

int Blaze_AllocationCount(int64_t* count) {
  if (count == nullptr) return Fail("AllocationCount: null argument");
  *count = blaze::AllocationCount().load();
  return 0;
}
int Blaze_PredictorInputDevicePtr(PredictorHandle handle, const char* name, void** ptr) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr || ptr == nullptr) return -1;
  *ptr = p->InputDevicePtr(name);
  return *ptr ? 0 : Fail("not an input of the net (or an input that lives inside a Concat output and has no plain buffer)");
}
int Blaze_PredictorOutputDevicePtr(PredictorHandle handle, const char* name, void** ptr) {
  auto* p = reinterpret_cast<Predictor*>(handle);
  if (p == nullptr || ptr == nullptr) return -1;
  *ptr = p->OutputDevicePtr(name);
  return *ptr ? 0 : Fail("not an output of the net");
}

}  // extern "C"
