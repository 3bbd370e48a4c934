// Shared-memory region, message rings and the waiting helpers of the process-rank engine.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "common.h"

namespace tandem_hip {


inline double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

inline int mod(int a, int n) { return ((a % n) + n) % n; }

constexpr int kBytesDtype = 6;  // TDM_U8 in spirit: copies only

// Messages: a piece's length in bytes, or (top bit set) a barrier with a tag in the low bits.
constexpr uint64_t kNoPiece = uint64_t(1) << 63;
constexpr uint64_t fence_tag(int kind, int dtype, int64_t numel) {
  return (static_cast<uint64_t>(kind) << 56) | (static_cast<uint64_t>(dtype) << 48) | (static_cast<uint64_t>(numel) & ((uint64_t(1) << 48) - 1));
}
// A piece's message carries, above its length (bits 0-39), what the sender is doing: the kind of collective, the element type
// and the tensor's length folded to 15 bits (bits 40-62). The reference's protocol has nothing of the kind: a rank that is
// in another collective, or in the same one with a tensor of another size, reads the pieces as if they were its own.
constexpr int kPieceTagShift = 40;
constexpr uint64_t kPieceLengthMask = (uint64_t(1) << kPieceTagShift) - 1;
constexpr uint64_t piece_tag(int kind, int dtype, int64_t numel) {
  const uint64_t n = static_cast<uint64_t>(numel);
  return ((static_cast<uint64_t>(kind & 15) << 19) | (static_cast<uint64_t>(dtype & 15) << 15) | ((n ^ (n >> 15) ^ (n >> 30) ^ (n >> 45)) & 0x7fff))
         << kPieceTagShift;
}

inline bool is_integer(int dtype) {
  return dtype == TDM_I64 || dtype == TDM_I32 || dtype == TDM_I16 || dtype == TDM_I8 || dtype == TDM_U8;
}

inline int elem_bytes(int dtype) {
  switch (dtype) {
    case TDM_F32: case TDM_I32: return 4;
    case TDM_F64: case TDM_I64: return 8;
    case TDM_F16: case TDM_BF16: case TDM_I16: return 2;
    case TDM_I8: case TDM_U8: case kBytesDtype: return 1;
    default: throw Invalid("unknown dtype " + std::to_string(dtype));
  }
}

// ---------------------------------------------------------------- shared region
constexpr uint64_t kRegionMagic = 0x74646d4849503032ull;  // "tdmHIP02"
constexpr size_t kLine = 64;
constexpr int kMaxSlots = 16;
// An arena is one exported allocation and stays under 2 GiB, a rank may share several. A byte of a rank's arenas is
// named by one number: the arena's index (in the order the rank shared them) in the bits from 31 up, the offset within it below.
constexpr int kMaxArenas = 64;
constexpr int kArenaShift = 31;
constexpr uint64_t kArenaLimit = uint64_t(1) << kArenaShift;

static_assert(std::atomic<uint64_t>::is_always_lock_free, "atomics shared between processes must be lock-free");

// One direction of one pair, written by the owner of the region (the sender):
// message k says slot k % slots holds `length[k % slots]` bytes.
struct alignas(kLine) Ring {
  alignas(kLine) std::atomic<uint64_t> head;  // messages published, advanced by the sender
  alignas(kLine) std::atomic<uint64_t> tail;  // messages released, advanced by the receiver
  alignas(kLine) uint64_t length[kMaxSlots];
};

struct alignas(kLine) PeerEntry {
  hipIpcMemHandle_t mem;               // the sender's slots for this peer
  hipIpcEventHandle_t full[kMaxSlots];  // sender recorded: slot j holds a piece
  hipIpcEventHandle_t free_[kMaxSlots]; // owner recorded: it finished reading THE PEER's slot j to the owner
  Ring ring;
};

struct alignas(kLine) RegionHeader {
  uint64_t magic;
  int32_t rank, size, device, slots;
  uint64_t slot_bytes;
  int64_t pid;
  int32_t use_events;
  int32_t reserved;
  // A rank's shared arenas (tdm_engine_share): device memory its peers may read and write directly.
  std::atomic<uint64_t> arena_bytes[kMaxArenas];  // 0 until published
  hipIpcMemHandle_t arena_mem[kMaxArenas];
  // The engine's own staging memory for the staged collectives (two halves, used in turn).
  std::atomic<uint64_t> staging_bytes;  // 0 until published
  hipIpcMemHandle_t staging_mem;
};

class Region {
 public:
  Region() = default;
  ~Region() { reset(); }
  Region(const Region&) = delete;
  Region& operator=(const Region&) = delete;

  static size_t bytes_for(int size) { return sizeof(RegionHeader) + static_cast<size_t>(size) * sizeof(PeerEntry); }

  void create(const std::string& name, int size) {
    reset();
    name_ = name;
    bytes_ = bytes_for(size);
    ::shm_unlink(name.c_str());  // a stale region from a crashed run with the same job name
    int fd = ::shm_open(name.c_str(), O_CREAT | O_EXCL | O_RDWR, 0600);
    if (fd < 0) throw std::runtime_error("shm_open(" + name + "): " + std::strerror(errno));
    if (::ftruncate(fd, static_cast<off_t>(bytes_)) != 0) {
      ::close(fd);
      ::shm_unlink(name.c_str());
      throw std::runtime_error("ftruncate(" + name + "): " + std::strerror(errno));
    }
    map(fd);
    owner_ = true;
    std::memset(data_, 0, bytes_);
    for (int p = 0; p < size; ++p) new (&entry(p)->ring) Ring();
  }

  void open(const std::string& name, int size) {
    reset();
    name_ = name;
    bytes_ = bytes_for(size);
    int fd = ::shm_open(name.c_str(), O_RDWR, 0600);
    if (fd < 0) throw std::runtime_error("shm_open(" + name + "): " + std::strerror(errno));
    struct stat st;
    if (::fstat(fd, &st) != 0 || static_cast<size_t>(st.st_size) < bytes_) {
      ::close(fd);
      throw std::runtime_error("region " + name + " is smaller than expected");
    }
    map(fd);
  }

  RegionHeader* header() const { return static_cast<RegionHeader*>(data_); }
  PeerEntry* entry(int peer) const {
    return reinterpret_cast<PeerEntry*>(static_cast<char*>(data_) + sizeof(RegionHeader)) + peer;
  }
  bool mapped() const { return data_ != nullptr; }

  void reset() {
    if (data_) ::munmap(data_, bytes_);
    if (owner_) ::shm_unlink(name_.c_str());
    data_ = nullptr;
    owner_ = false;
  }

 private:
  void map(int fd) {
    void* p = ::mmap(nullptr, bytes_, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    ::close(fd);
    if (p == MAP_FAILED) throw std::runtime_error("mmap(" + name_ + "): " + std::strerror(errno));
    data_ = p;
  }

  std::string name_;
  void* data_ = nullptr;
  size_t bytes_ = 0;
  bool owner_ = false;
};

// A wake-up through a condition variable costs 10-20 us; whoever expects news within
// that time polls for it first.
constexpr auto kSpinBeforeSleep = std::chrono::microseconds(100);

template <class Ready>
bool spin_for(Ready ready, std::chrono::microseconds limit = kSpinBeforeSleep) {
  const auto until = std::chrono::steady_clock::now() + limit;
  for (int i = 0;; ++i) {
    if (ready()) return true;
    if ((i & 15) == 15 && std::chrono::steady_clock::now() > until) return false;
    __builtin_ia32_pause();
  }
}

// Waiting for the GPU from a helper thread: poll (a query is cheap and takes no lock for
// long), first tightly, then every 50 us. The runtime's own blocking waits are avoided on
// purpose: while one thread sat in them for milliseconds, the training thread's kernel
// launches were seen to stall. `query` returns hipErrorNotReady until the work is done.
template <class Query>
hipError_t poll_gpu(Query query, double timeout_s) {
  hipError_t err = hipErrorNotReady;
  if (spin_for([&] { return (err = query()) != hipErrorNotReady; }, std::chrono::microseconds(300))) return err;
  const auto deadline = std::chrono::steady_clock::now() + std::chrono::duration<double>(timeout_s);
  for (;;) {
    std::this_thread::sleep_for(std::chrono::microseconds(50));
    if ((err = query()) != hipErrorNotReady) return err;
    if (std::chrono::steady_clock::now() > deadline) throw Timeout("timed out waiting for the GPU");
  }
}

// Spin, then yield, then short sleeps; throws Timeout.
template <class Ready>
void wait_until(Ready ready, double timeout_s, const char* what) {
  using clock = std::chrono::steady_clock;
  const auto start = clock::now();
  const auto deadline = start + std::chrono::duration<double>(timeout_s);
  for (uint64_t i = 0; !ready(); ++i) {
    if (i < 256) continue;
    if ((i & 63) != 0) {
      std::this_thread::yield();
      continue;
    }
    const auto t = clock::now();
    if (t > deadline) throw Timeout(what);
    if (t - start > std::chrono::milliseconds(2)) std::this_thread::sleep_for(std::chrono::microseconds(20));
  }
}

// ---------------------------------------------------------------- ring operations
// The sender publishes message k into length[k % slots] and advances head; the receiver
// reads messages in order and advances tail when it is done with one (possibly later,
// in the same order). Room for a new message: fewer than `slots` unreleased ones.
inline void ring_publish(Ring& r, int slots, uint64_t length) {
  const uint64_t head = r.head.load(std::memory_order_relaxed);
  r.length[head % slots] = length;
  r.head.store(head + 1, std::memory_order_release);  // the length is visible before the new head
}

inline bool ring_has_room(const Ring& r, uint64_t posted, int slots) {
  return posted - r.tail.load(std::memory_order_acquire) < static_cast<uint64_t>(slots);
}

inline void ring_wait_for_room(const Ring& r, uint64_t posted, int slots, double timeout_s, const char* what) {
  wait_until([&] { return ring_has_room(r, posted, slots); }, timeout_s, what);
}

// Message number `at` (0-based, the count of messages the receiver has read so far).
inline uint64_t ring_read(const Ring& r, uint64_t at, int slots, double timeout_s, const char* what) {
  wait_until([&] { return r.head.load(std::memory_order_acquire) > at; }, timeout_s, what);
  return r.length[at % slots];
}

inline void ring_release(Ring& r) {
  r.tail.store(r.tail.load(std::memory_order_relaxed) + 1, std::memory_order_release);
}

}  // namespace tandem_hip
