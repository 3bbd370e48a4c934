// A stand-in for the HIP runtime, for ONE purpose: running the process-rank engine's HOST code (threads, queues, rings,
// hand-overs, done words: tandem_amd/csrc/engine.hip, engine_abi.hip) on a machine without a GPU and under the host's
// sanitizers, which cannot share a process with the real runtime. It is linked into tests/cpp/engine_host_test only;
// the library the package loads is never built from it, and nothing here computes a result anybody ships.
//
// What it models: "device" memory is POSIX shared memory (so that an IPC memory handle can be opened by another
// process). A stream is a thread with a queue: what is launched on it runs later, in order, so work on two streams
// overlaps unless an event or a value orders it, and the data-race sanitizer sees every pair of accesses that the
// engine left unordered. An event is complete once the stream has passed its record; a stream's write of a value is a
// store, its wait for a value a spin, both when the stream gets there. The null stream runs everything at once in
// the calling thread. With FAKE_HIP_JITTER_US=n in the environment every piece of work on a stream starts up to n
// microseconds late, a different amount each time: streams then lag behind the host by varying distances, and whatever
// the engine assumed about their progress without checking shows as a wrong number or a data race.

#include <fcntl.h>
#include <hip/hip_runtime_api.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>

#include "fake_hip.h"

namespace {

struct Block {
  std::string name;  // of the shared-memory object; empty for plain host memory
  size_t bytes;
};

std::mutex g_mu;
std::map<void*, Block> g_blocks;  // what this process allocated or opened
std::atomic<uint64_t> g_serial{0};

void* map_shared(const std::string& name, size_t bytes, bool create) {
  const int fd = ::shm_open(name.c_str(), create ? (O_CREAT | O_EXCL | O_RDWR) : O_RDWR, 0600);
  if (fd < 0) return nullptr;
  if (create && ::ftruncate(fd, static_cast<off_t>(bytes)) != 0) {
    ::close(fd);
    ::shm_unlink(name.c_str());
    return nullptr;
  }
  if (!create) {
    struct stat st;
    if (::fstat(fd, &st) != 0) {
      ::close(fd);
      return nullptr;
    }
    bytes = static_cast<size_t>(st.st_size);
  }
  void* p = ::mmap(nullptr, bytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  ::close(fd);
  if (p == MAP_FAILED) return nullptr;
  std::lock_guard<std::mutex> lock(g_mu);
  g_blocks[p] = Block{create ? name : std::string(), bytes};
  return p;
}

// A stream: a thread that runs what is queued, in order.
class Stream {
 public:
  Stream() : worker_([this] { run(); }) {}
  ~Stream() {
    {
      std::lock_guard<std::mutex> lock(mu_);
      stop_ = true;
    }
    cv_.notify_all();
    worker_.join();
  }
  void push(std::function<void()> work) {
    {
      std::lock_guard<std::mutex> lock(mu_);
      queue_.push_back(std::move(work));
      ++pending_;
    }
    cv_.notify_all();
  }
  bool idle() {
    std::lock_guard<std::mutex> lock(mu_);
    return pending_ == 0;
  }
  void drain() {
    std::unique_lock<std::mutex> lock(mu_);
    done_.wait(lock, [this] { return pending_ == 0; });
  }

 private:
  void run() {
    for (;;) {
      std::function<void()> work;
      {
        std::unique_lock<std::mutex> lock(mu_);
        cv_.wait(lock, [this] { return stop_ || !queue_.empty(); });
        if (queue_.empty()) return;  // stopping, and everything queued has run
        work = std::move(queue_.front());
        queue_.pop_front();
      }
      if (jitter_us_ > 0) {  // FAKE_HIP_JITTER_US: every piece of work starts up to that many microseconds late
        seed_ = seed_ * 6364136223846793005ull + 1442695040888963407ull;
        std::this_thread::sleep_for(std::chrono::microseconds((seed_ >> 33) % (static_cast<uint64_t>(jitter_us_) + 1)));
      }
      work();
      {
        std::lock_guard<std::mutex> lock(mu_);
        --pending_;
      }
      done_.notify_all();
    }
  }
  std::mutex mu_;
  std::condition_variable cv_, done_;
  std::deque<std::function<void()>> queue_;
  int pending_ = 0;  // queued or running
  bool stop_ = false;
  const int jitter_us_ = std::getenv("FAKE_HIP_JITTER_US") ? std::atoi(std::getenv("FAKE_HIP_JITTER_US")) : 0;
  uint64_t seed_ = static_cast<uint64_t>(::getpid()) * 2654435761u + reinterpret_cast<uintptr_t>(this);
  std::thread worker_;  // last: the others exist before it starts
};

// An event's state: records asked for, and the latest one a stream has passed. Two counters of atomics, so that an
// interprocess event (FAKE_HIP_IPC_EVENTS=1; refused otherwise, as on the machines the engine was built on) can keep them in
// shared memory, where the process that opened the handle waits for records of the process that made it.
struct EventState {
  std::atomic<uint64_t> recorded, completed;
};

struct Event {
  EventState* state = nullptr;
  std::string shared_name;  // of the shared-memory object of an interprocess event; empty: state is this process's own
  bool owner = false;
  ~Event() {
    if (shared_name.empty()) {
      delete state;
    } else {
      ::munmap(state, sizeof(EventState));
      if (owner) ::shm_unlink(shared_name.c_str());
    }
  }
  void wait_for(uint64_t ticket) const {
    while (state->completed.load(std::memory_order_acquire) < ticket) std::this_thread::yield();
  }
};

bool ipc_events() { return std::getenv("FAKE_HIP_IPC_EVENTS") != nullptr; }

EventState* map_event(const std::string& name, bool create) {
  const int fd = ::shm_open(name.c_str(), create ? (O_CREAT | O_EXCL | O_RDWR) : O_RDWR, 0600);
  if (fd < 0) return nullptr;
  if (create && ::ftruncate(fd, sizeof(EventState)) != 0) {
    ::close(fd);
    return nullptr;
  }
  void* p = ::mmap(nullptr, sizeof(EventState), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  ::close(fd);
  return p == MAP_FAILED ? nullptr : static_cast<EventState*>(p);  // a fresh object is all zeros: both counters at 0
}

Stream* as_stream(hipStream_t s) { return reinterpret_cast<Stream*>(s); }
std::shared_ptr<Event> as_event(hipEvent_t e) { return *reinterpret_cast<std::shared_ptr<Event>*>(e); }

}  // namespace

void fake_enqueue(hipStream_t stream, std::function<void()> work) {
  if (stream) as_stream(stream)->push(std::move(work));
  else work();
}

extern "C" {

hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipGetDevice(int* device) {
  *device = 0;
  return hipSuccess;
}
hipError_t hipGetLastError(void) { return hipSuccess; }
const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "an error of the stand-in runtime"; }

hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t attr, int) {
  *value = attr == hipDeviceAttributeCanUseStreamWaitValue ? 1 : 0;
  return hipSuccess;
}

hipError_t hipGetDeviceProperties(hipDeviceProp_t* prop, int) {
  std::memset(prop, 0, sizeof *prop);
  std::snprintf(prop->name, sizeof prop->name, "stand-in");
  prop->multiProcessorCount = 1;
  return hipSuccess;
}

hipError_t hipMalloc(void** ptr, size_t bytes) {
  const std::string name = "/tdmfake-" + std::to_string(::getpid()) + "-" + std::to_string(g_serial.fetch_add(1));
  *ptr = map_shared(name, bytes ? bytes : 1, true);
  return *ptr ? hipSuccess : hipErrorOutOfMemory;
}

hipError_t hipFree(void* ptr) {
  if (!ptr) return hipSuccess;
  Block b;
  {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_blocks.find(ptr);
    if (it == g_blocks.end()) return hipErrorInvalidValue;
    b = it->second;
    g_blocks.erase(it);
  }
  ::munmap(ptr, b.bytes);
  if (!b.name.empty()) ::shm_unlink(b.name.c_str());
  return hipSuccess;
}

hipError_t hipHostMalloc(void** ptr, size_t bytes, unsigned int) {
  *ptr = std::aligned_alloc(4096, (bytes + 4095) / 4096 * 4096);
  return *ptr ? hipSuccess : hipErrorOutOfMemory;
}

hipError_t hipHostFree(void* ptr) {
  std::free(ptr);
  return hipSuccess;
}

hipError_t hipIpcGetMemHandle(hipIpcMemHandle_t* handle, void* ptr) {
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_blocks.find(ptr);
  if (it == g_blocks.end() || it->second.name.empty() || it->second.name.size() >= sizeof handle->reserved) return hipErrorInvalidValue;
  std::memset(handle, 0, sizeof *handle);
  std::memcpy(handle->reserved, it->second.name.c_str(), it->second.name.size());
  return hipSuccess;
}

hipError_t hipIpcOpenMemHandle(void** ptr, hipIpcMemHandle_t handle, unsigned int) {
  char name[sizeof handle.reserved + 1] = {0};
  std::memcpy(name, handle.reserved, sizeof handle.reserved);
  *ptr = map_shared(name, 0, false);
  return *ptr ? hipSuccess : hipErrorInvalidValue;
}

hipError_t hipIpcCloseMemHandle(void* ptr) { return hipFree(ptr); }  // opened blocks carry no name: nothing is unlinked

hipError_t hipIpcGetEventHandle(hipIpcEventHandle_t* handle, hipEvent_t event) {
  std::shared_ptr<Event> e = as_event(event);
  if (!ipc_events() || e->shared_name.empty() || e->shared_name.size() >= sizeof handle->reserved) return hipErrorNotSupported;
  std::memset(handle, 0, sizeof *handle);
  std::memcpy(handle->reserved, e->shared_name.c_str(), e->shared_name.size());
  return hipSuccess;
}
hipError_t hipIpcOpenEventHandle(hipEvent_t* event, hipIpcEventHandle_t handle) {
  char name[sizeof handle.reserved + 1] = {0};
  std::memcpy(name, handle.reserved, sizeof handle.reserved);
  auto e = std::make_shared<Event>();
  e->state = map_event(name, false);
  if (!e->state) return hipErrorInvalidValue;
  e->shared_name = name;
  *event = reinterpret_cast<hipEvent_t>(new std::shared_ptr<Event>(std::move(e)));
  return hipSuccess;
}

hipError_t hipStreamCreateWithFlags(hipStream_t* stream, unsigned int) {
  *stream = reinterpret_cast<hipStream_t>(new Stream);
  return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t stream) {
  delete as_stream(stream);  // runs what is queued, then joins
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t stream) {
  if (stream) as_stream(stream)->drain();
  return hipSuccess;
}
hipError_t hipStreamQuery(hipStream_t stream) { return !stream || as_stream(stream)->idle() ? hipSuccess : hipErrorNotReady; }

hipError_t hipEventCreateWithFlags(hipEvent_t* event, unsigned flags) {
  auto e = std::make_shared<Event>();
  if ((flags & hipEventInterprocess) && ipc_events()) {
    e->shared_name = "/tdmfake-ev-" + std::to_string(::getpid()) + "-" + std::to_string(g_serial.fetch_add(1));
    e->state = map_event(e->shared_name, true);
    e->owner = true;
    if (!e->state) return hipErrorOutOfMemory;
  } else {
    e->state = new EventState{};
  }
  *event = reinterpret_cast<hipEvent_t>(new std::shared_ptr<Event>(std::move(e)));
  return hipSuccess;
}
hipError_t hipEventCreate(hipEvent_t* event) { return hipEventCreateWithFlags(event, 0); }
// As with the real runtime, an event may be destroyed while streams still have to pass or wait for it: what is queued keeps it alive.
hipError_t hipEventDestroy(hipEvent_t event) {
  delete reinterpret_cast<std::shared_ptr<Event>*>(event);
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) {
  std::shared_ptr<Event> e = as_event(event);
  const uint64_t ticket = e->state->recorded.fetch_add(1, std::memory_order_acq_rel) + 1;
  fake_enqueue(stream, [e, ticket] {
    uint64_t seen = e->state->completed.load(std::memory_order_relaxed);
    while (seen < ticket && !e->state->completed.compare_exchange_weak(seen, ticket, std::memory_order_release)) {
    }
  });
  return hipSuccess;
}
hipError_t hipEventQuery(hipEvent_t event) {
  std::shared_ptr<Event> e = as_event(event);
  return e->state->completed.load(std::memory_order_acquire) >= e->state->recorded.load(std::memory_order_acquire) ? hipSuccess : hipErrorNotReady;
}
hipError_t hipEventSynchronize(hipEvent_t event) {
  std::shared_ptr<Event> e = as_event(event);
  e->wait_for(e->state->recorded.load(std::memory_order_acquire));
  return hipSuccess;
}
hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) {
  *ms = 0;
  return hipSuccess;
}
// The stream waits for the record that was the event's latest when this was called (none: nothing to wait for).
hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned int) {
  std::shared_ptr<Event> e = as_event(event);
  const uint64_t ticket = e->state->recorded.load(std::memory_order_acquire);
  fake_enqueue(stream, [e, ticket] { e->wait_for(ticket); });
  return hipSuccess;
}

hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, hipMemcpyKind, hipStream_t stream) {
  fake_enqueue(stream, [dst, src, bytes] { std::memmove(dst, src, bytes); });
  return hipSuccess;
}

hipError_t hipStreamWriteValue32(hipStream_t stream, void* ptr, uint32_t value, unsigned int) {
  fake_enqueue(stream, [ptr, value] { reinterpret_cast<std::atomic<uint32_t>*>(ptr)->store(value, std::memory_order_release); });
  return hipSuccess;
}

// When the stream gets there it waits until the word has reached the value (at most twenty seconds: then it goes on,
// and whoever reads behind it finds the wrong numbers).
hipError_t hipStreamWaitValue32(hipStream_t stream, void* ptr, uint32_t value, unsigned int, uint32_t) {
  fake_enqueue(stream, [ptr, value] {
    const auto until = std::chrono::steady_clock::now() + std::chrono::seconds(20);
    while (reinterpret_cast<std::atomic<uint32_t>*>(ptr)->load(std::memory_order_acquire) < value) {
      if (std::chrono::steady_clock::now() > until) return;
      std::this_thread::yield();
    }
  });
  return hipSuccess;
}

hipError_t hipPointerGetAttributes(hipPointerAttribute_t* attr, const void*) {
  std::memset(attr, 0, sizeof *attr);
  attr->type = hipMemoryTypeDevice;  // every pointer counts as memory of device 0
  attr->device = 0;
  return hipSuccess;
}

}  // extern "C"
