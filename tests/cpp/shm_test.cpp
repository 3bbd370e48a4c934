// Host-only checks of the process-rank engine's shared-memory layer (engine_shm.h):
// the region that a rank publishes and its peers open, and the message rings inside it.
// They follow what the reference tests of its own SharedMemory and Channel classes
// (tests/test_engine.py:27-178 there): create/open/unlink, errors that name the call,
// a ring that is full or empty until a time limit, many messages between two processes.
// No GPU call is made. Usage: shm_test <case> [args]; exit status 0 = passed.

#include <sys/wait.h>

#include <cstdio>
#include <string>

#include "../../tandem_amd/csrc/engine_shm.h"

namespace tandem_hip {
void set_last_error(const std::string&) {}  // common.h declares it; nothing here reports through it
}

using namespace tandem_hip;

#define CHECK(cond)                                                          \
  do {                                                                       \
    if (!(cond)) {                                                           \
      std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
      return 1;                                                              \
    }                                                                        \
  } while (0)

static std::string unique_name(const char* what) { return "/tandem-test-" + std::to_string(::getpid()) + "-" + what; }

static bool exists(const std::string& name) {
  int fd = ::shm_open(name.c_str(), O_RDONLY, 0600);
  if (fd >= 0) ::close(fd);
  return fd >= 0;
}

// create, write, open by name in the same process, read back; the creator unlinks the name
static int region_roundtrip() {
  const std::string name = unique_name("roundtrip");
  {
    Region mine;
    mine.create(name, 3);
    CHECK(mine.mapped() && exists(name));
    CHECK(mine.header()->magic == 0 && mine.entry(2)->ring.head.load() == 0);  // zero-filled
    mine.header()->rank = 7;
    mine.entry(1)->ring.length[5] = 1234;
    Region theirs;
    theirs.open(name, 3);
    CHECK(theirs.header()->rank == 7 && theirs.entry(1)->ring.length[5] == 1234);
    theirs.reset();
    CHECK(exists(name));  // a reader's reset leaves the name alone
  }
  CHECK(!exists(name));  // the creator's destructor unlinked it
  return 0;
}

// another process opens the region by name and sees what the creator wrote, and the other way round
static int region_two_processes() {
  const std::string name = unique_name("twoproc");
  Region mine;
  mine.create(name, 2);
  mine.header()->slot_bytes = 4096;
  const pid_t child = ::fork();
  if (child == 0) {
    Region theirs;
    try {
      theirs.open(name, 2);
    } catch (...) {
      ::_exit(2);
    }
    if (theirs.header()->slot_bytes != 4096) ::_exit(3);
    theirs.entry(0)->ring.length[0] = 99;
    std::atomic_thread_fence(std::memory_order_seq_cst);
    theirs.header()->pid = 42;
    ::_exit(0);
  }
  int status = 0;
  CHECK(::waitpid(child, &status, 0) == child && WIFEXITED(status) && WEXITSTATUS(status) == 0);
  CHECK(mine.header()->pid == 42 && mine.entry(0)->ring.length[0] == 99);
  return 0;
}

// errors name the call and the region; a stale name is replaced; a region that is too small is refused
static int region_errors() {
  const std::string missing = unique_name("missing");
  try {
    Region r;
    r.open(missing, 2);
    CHECK(false);
  } catch (const std::runtime_error& e) {
    CHECK(std::string(e.what()).find("shm_open(" + missing + ")") != std::string::npos);
  }
  CHECK(!exists(missing));  // a failed open leaves nothing behind
  try {
    Region r;
    r.create("/tandem/with/slashes", 2);
    CHECK(false);
  } catch (const std::runtime_error& e) {
    CHECK(std::string(e.what()).find("shm_open(/tandem/with/slashes)") != std::string::npos);
  }
  const std::string stale = unique_name("stale");
  int fd = ::shm_open(stale.c_str(), O_CREAT | O_EXCL | O_RDWR, 0600);  // what a crashed run leaves: the name, 16 bytes
  CHECK(fd >= 0 && ::ftruncate(fd, 16) == 0);
  ::close(fd);
  try {
    Region r;
    r.open(stale, 2);
    CHECK(false);
  } catch (const std::runtime_error& e) {
    CHECK(std::string(e.what()).find("smaller than expected") != std::string::npos);
  }
  {
    Region fresh;
    fresh.create(stale, 2);  // replaces the stale one
    Region again;
    again.open(stale, 2);
    CHECK(again.header()->magic == 0);
  }
  CHECK(!exists(stale));
  return 0;
}

// one process: publish up to `slots` messages, then no room; read in order; release makes room
static int ring_one_process() {
  const std::string name = unique_name("ring");
  Region mine;
  mine.create(name, 2);
  Ring& r = mine.entry(1)->ring;
  const int slots = 3;
  uint64_t posted = 0;
  for (int k = 0; k < slots; ++k) {
    CHECK(ring_has_room(r, posted, slots));
    ring_publish(r, slots, 100 + k);
    ++posted;
  }
  CHECK(!ring_has_room(r, posted, slots));
  try {  // full: blocks until the time limit, then says what it waited for
    ring_wait_for_room(r, posted, slots, 0.05, "no room in the ring");
    CHECK(false);
  } catch (const Timeout& e) {
    CHECK(std::string(e.what()) == "no room in the ring");
  }
  for (int k = 0; k < slots; ++k) CHECK(ring_read(r, k, slots, 1.0, "read") == 100u + k);
  const double t0 = now_s();
  try {  // empty: the same
    ring_read(r, slots, slots, 0.05, "nothing arrived");
    CHECK(false);
  } catch (const Timeout& e) {
    CHECK(std::string(e.what()) == "nothing arrived");
  }
  CHECK(now_s() - t0 >= 0.05 && now_s() - t0 < 1.0);
  ring_release(r);
  CHECK(ring_has_room(r, posted, slots));
  ring_publish(r, slots, 7);  // reuses the first slot
  CHECK(ring_read(r, slots, slots, 1.0, "read") == 7);
  return 0;
}

// two processes: the child sends `count` numbered messages under the ring's flow control,
// the parent reads, checks the order and releases, sometimes late (two at a time)
static int ring_two_processes(int slots, int count) {
  const std::string name = unique_name("ring2");
  Region mine;
  mine.create(name, 2);
  const pid_t child = ::fork();
  if (child == 0) {
    try {
      Region theirs;
      theirs.open(name, 2);
      Ring& r = theirs.entry(1)->ring;
      for (uint64_t k = 0; k < static_cast<uint64_t>(count); ++k) {
        ring_wait_for_room(r, k, slots, 20.0, "child: no room");
        ring_publish(r, slots, k * 3 + 1);
      }
    } catch (...) {
      ::_exit(2);
    }
    ::_exit(0);
  }
  Ring& r = mine.entry(1)->ring;
  uint64_t unreleased = 0;
  for (uint64_t k = 0; k < static_cast<uint64_t>(count); ++k) {
    CHECK(ring_read(r, k, slots, 20.0, "parent: nothing arrived") == k * 3 + 1);
    ++unreleased;
    if (slots == 1 || k % 2 == 1 || unreleased == static_cast<uint64_t>(slots)) {
      for (; unreleased; --unreleased) ring_release(r);
    }
  }
  int status = 0;
  CHECK(::waitpid(child, &status, 0) == child && WIFEXITED(status) && WEXITSTATUS(status) == 0);
  CHECK(r.head.load() == static_cast<uint64_t>(count));
  return 0;
}

// two threads, for the data-race sanitizer: the sender fills a payload slot with plain stores before it publishes, the
// receiver reads the slot after ring_read and then releases; a slot is rewritten only once the ring has room again.
// That is the engine's use of a ring (a message means the bytes have landed, a release that they have been read), and
// head's and tail's release/acquire pairs are all that orders the plain accesses.
static int ring_two_threads(int slots, int count) {
  const std::string name = unique_name("ring3");
  Region mine;
  mine.create(name, 2);
  Ring& r = mine.entry(1)->ring;
  constexpr int kWords = 8;
  std::vector<uint64_t> payload(static_cast<size_t>(slots) * kWords);
  std::atomic<int> sender_failed{0};
  std::thread sender([&] {
    try {
      for (uint64_t k = 0; k < static_cast<uint64_t>(count); ++k) {
        ring_wait_for_room(r, k, slots, 10.0, "sender: no room");
        for (int i = 0; i < kWords; ++i) payload[(k % slots) * kWords + i] = k * kWords + i;
        ring_publish(r, slots, k * 3 + 1);
      }
    } catch (...) {
      sender_failed.store(1);
    }
  });
  int bad = 0;
  try {
    for (uint64_t k = 0; k < static_cast<uint64_t>(count); ++k) {
      if (ring_read(r, k, slots, 10.0, "receiver: nothing arrived") != k * 3 + 1) ++bad;
      for (int i = 0; i < kWords; ++i) bad += payload[(k % slots) * kWords + i] != k * kWords + i;
      ring_release(r);
    }
  } catch (const Timeout&) {
    ++bad;
  }
  sender.join();
  CHECK(bad == 0 && sender_failed.load() == 0);
  CHECK(r.head.load() == static_cast<uint64_t>(count) && r.tail.load() == static_cast<uint64_t>(count));
  return 0;
}

// the waiting helpers: spin_for gives up after its limit; wait_until returns as soon as the condition holds
static int waiting() {
  const double t0 = now_s();
  CHECK(!spin_for([] { return false; }, std::chrono::microseconds(2000)));
  const double spun = now_s() - t0;
  CHECK(spun >= 0.002 && spun < 0.5);
  CHECK(spin_for([] { return true; }));
  int calls = 0;
  wait_until([&] { return ++calls > 1000; }, 5.0, "never");
  CHECK(calls == 1001);
  CHECK(mod(-1, 4) == 3 && mod(5, 4) == 1 && mod(-8, 4) == 0);
  CHECK((fence_tag(5, 1, 1000) & kNoPiece) == 0 && fence_tag(5, 1, 1000) != fence_tag(6, 1, 1000) &&
        fence_tag(5, 1, 1000) != fence_tag(5, 2, 1000) && fence_tag(5, 1, 1000) != fence_tag(5, 1, 1001));
  return 0;
}

int main(int argc, char** argv) {
  const std::string which = argc > 1 ? argv[1] : "";
  try {
    if (which == "region_roundtrip") return region_roundtrip();
    if (which == "region_two_processes") return region_two_processes();
    if (which == "region_errors") return region_errors();
    if (which == "ring_one_process") return ring_one_process();
    if (which == "ring_two_processes") return ring_two_processes(argc > 2 ? std::atoi(argv[2]) : 2, argc > 3 ? std::atoi(argv[3]) : 1000);
    if (which == "ring_two_threads") return ring_two_threads(argc > 2 ? std::atoi(argv[2]) : 2, argc > 3 ? std::atoi(argv[3]) : 1000);
    if (which == "waiting") return waiting();
  } catch (const std::exception& e) {
    std::fprintf(stderr, "unexpected exception: %s\n", e.what());
    return 3;
  }
  std::fprintf(stderr, "unknown case '%s'\n", which.c_str());
  return 64;
}
