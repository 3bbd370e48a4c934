// The process-rank engine's types: Work handles and the Engine itself (see engine.hip).
#pragma once

#include "engine_shm.h"

namespace tandem_hip {

// ---------------------------------------------------------------- Work
// A point that is known on both clocks: the event was recorded on the engine's
// stream and waited for, and `host` was read right after.
struct Anchor {
  hipEvent_t event = nullptr;
  double host = 0;
  ~Anchor() {
    if (event) (void)hipEventDestroy(event);
  }
};

// Words in pinned host memory that a GPU stream can wait on (hipStreamWaitValue32) and
// that either the engine's stream (hipStreamWriteValue32) or the host sets: how
// wait() can order the caller's stream behind a collective whose launches the progress
// thread has not even made yet. Shared by the engine and its Works, freed by the last.
struct FlagPool {
  static constexpr int kFlags = 1024;
  uint32_t* base = nullptr;
  std::mutex mu;
  std::vector<int> free_list;
  std::vector<int> pending;  // released by their Works, not yet written by the GPU
  std::vector<uint32_t> generation;  // a word only ever grows: a stream still parked on an earlier
                                     // generation of it is let go by every later one as well

  static std::shared_ptr<FlagPool> make() {
    auto p = std::make_shared<FlagPool>();
    check_hip(hipHostMalloc(reinterpret_cast<void**>(&p->base), (kFlags + 1) * sizeof(uint32_t), hipHostMallocDefault), "hipHostMalloc (flags)");
    std::memset(p->base, 0, (kFlags + 1) * sizeof(uint32_t));
    p->generation.assign(kFlags, 0);
    for (int i = kFlags - 1; i >= 0; --i) p->free_list.push_back(i);
    return p;
  }
  ~FlagPool() {
    if (base) (void)hipHostFree(base);
  }
  // A word and the value its owner will wait for; -1: none left (the Work then waits on the host as usual).
  int acquire(uint32_t* value) {
    std::lock_guard<std::mutex> lock(mu);
    for (size_t k = 0; k < pending.size();) {  // words given back before the engine's stream had written them
      if (reached(pending[k])) {
        free_list.push_back(pending[k]);
        pending[k] = pending.back();
        pending.pop_back();
      } else {
        ++k;
      }
    }
    if (free_list.empty()) return -1;
    const int i = free_list.back();
    free_list.pop_back();
    *value = ++generation[i];
    return i;
  }
  // A word whose write is still queued on the engine's stream is not handed out again until the write has landed:
  // the next owner's value, set early by the host after a failure, would otherwise be overwritten by the smaller one.
  void release(int i) {
    std::lock_guard<std::mutex> lock(mu);
    (reached(i) ? free_list : pending).push_back(i);
  }
  bool reached(int i) const { return reached(i, generation[i]); }  // its latest generation (callers hold mu)
  // The GPU writes these words too (hipStreamWriteValue32): the host reads and writes them as atomics.
  bool reached(int i, uint32_t value) const {  // as hipStreamWaitValueGte compares
    return __atomic_load_n(base + i, __ATOMIC_ACQUIRE) >= value;
  }
  void set(int i, uint32_t value) { __atomic_store_n(base + i, value, __ATOMIC_SEQ_CST); }
  // One more word behind the pool: a parked stream that gave up waiting (park_kernel) leaves 1 there.
  uint32_t* gave_up_word() const { return base + kFlags; }
  bool gave_up() const { return __atomic_load_n(base + kFlags, __ATOMIC_ACQUIRE) != 0; }
};

struct Work {
  std::mutex mu;
  std::condition_variable cv;
  bool finished = false;   // the job has run (all its GPU work is enqueued)
  std::atomic<bool> finished_hint{false};  // set after `finished`: lets a waiter poll before it sleeps
  int status = TDM_OK;
  std::string error;
  double t0 = 0, t1 = 0;
  hipEvent_t done_event = nullptr;  // recorded on the engine's stream after the job: jobs with GPU work that have no flag word, or are timed
  bool uses_gpu = false;
  bool on_callers_stream = false;  // its kernels were launched on the submitting stream itself:
  hipStream_t launched_on = nullptr;  // wait() from that stream has nothing to order
  bool drained = false;  // the job ends with a fence: the engine's stream is idle when it has run
  int device = -1;
  // Device timing (only while the engine's timing switch is on): start_event is
  // recorded on the engine's stream once the inputs are ready; both events carry
  // time stamps, placed on the host clock through the engine's anchor.
  hipEvent_t start_event = nullptr;
  std::shared_ptr<Anchor> anchor;
  // Stream-ordered waiting (tdm_work_wait_stream; TANDEM_HIP_WAIT=stream): the word the caller's stream waits for.
  std::shared_ptr<FlagPool> flags;
  bool defer_default = false;  // tdm_work_wait parks too
  bool may_park = true;        // false: tdm_work_wait_stream waits on the host as well (a process with one hardware queue)
  double park_limit_s = 0;     // how long a stream parked on this Work waits at most before it gives up
  int flag = -1;
  uint32_t flag_value = 0;  // the word reaches this value when the collective is over

  ~Work() {
    if (done_event) (void)hipEventDestroy(done_event);
    if (start_event) (void)hipEventDestroy(start_event);
    if (flags && flag >= 0) {
      if (!finished) flags->set(flag, flag_value);  // the job never ran: nobody may stay parked on the word
      flags->release(flag);
    }
  }
};


// ---------------------------------------------------------------- Engine
class Engine {
 public:
  Engine(const std::string& job, int rank, int size, int slots, size_t slot_bytes, double timeout_s, int device);
  ~Engine();
  void connect();
  void close();
  void set_timing(bool on) { timing_.store(on ? 1 : 0, std::memory_order_release); }

  struct Buf {
    char* ptr;
    int64_t numel;
    int dtype;
  };

  std::shared_ptr<Work> all_reduce(Buf t, bool average, hipStream_t caller);
  std::shared_ptr<Work> reduce_scatter(Buf t, std::vector<int64_t> sizes, bool average, bool owner_only, hipStream_t caller);
  std::shared_ptr<Work> all_gather(Buf t, std::vector<int64_t> sizes, hipStream_t caller);
  std::shared_ptr<Work> unit_gather(Buf full, const char* shard, std::vector<int64_t> sizes, hipStream_t caller);
  std::shared_ptr<Work> broadcast(Buf t, int root, hipStream_t caller);
  std::shared_ptr<Work> sendrecv(Buf send, int dst, Buf recv, int src, hipStream_t caller);
  std::shared_ptr<Work> barrier();
  std::shared_ptr<Work> fence(hipStream_t caller);
  void* share(size_t bytes);
  int64_t own_arena_offset(const char* ptr, size_t bytes);
  std::shared_ptr<Work> unit_gather_direct(Buf full, const char* shard, std::vector<int64_t> sizes,
                                           std::vector<int64_t> peer_offsets, hipStream_t caller);
  // kind 0: all_reduce, 1: reduce_scatter (the owner's chunk only), 2: all_gather
  std::shared_ptr<Work> direct(int kind, Buf t, std::vector<int64_t> sizes, bool average, std::vector<int64_t> peer_offsets,
                               hipStream_t caller);

  // The step's constants come as fp32 (`s`, for fp32 buffers) or as doubles (`h`, any of K3's shard types): exactly one is set.
  std::shared_ptr<Work> zero2_step_direct(Buf param, Buf grad, std::vector<int64_t> param_offsets, std::vector<int64_t> grad_offsets,
                                          char* exp_avg, char* exp_avg_sq, int64_t total, bool average, const tdm_adamw_scalars* s,
                                          const tdm_adamw_hyper* h, int order, hipStream_t caller);

  int device() const { return device_; }
  hipStream_t stream() const { return stream_; }
  int rank() const { return rank_; }
  int size() const { return size_; }

 private:
  struct Chunk {
    char* ptr;
    int64_t numel;
  };

  std::shared_ptr<Work> submit(std::function<void()> job, hipStream_t caller, bool uses_gpu, bool host_ready = false,
                               bool drained = false);
  void stamp_start(Work& w, hipStream_t on);
  char* staging_half();
  const char* peer_staging(int peer, int half);
  void copy_pairs(const tdm_pair* pairs, int np, int dtype);
  void staged_all_reduce(const Buf& t, bool average);
  void staged_all_reduce_small(const Buf& t, bool average);
  void staged_all_gather(const Buf& t, const std::vector<Chunk>& cs, const char* own);
  void staged_reduce_scatter(const Buf& t, const std::vector<Chunk>& cs, bool average, bool partial_sums);
  void direct_bases(const Buf& t, const std::vector<int64_t>& peer_offsets, const char** base);
  void direct_fold(const Buf& t, const std::vector<Chunk>& cs, const char* const* base, bool average, bool to_all);
  void direct_copies(const Buf& t, const std::vector<Chunk>& cs, const char* const* base);
  void start();
  void release_device();
  void loop();
  void check(const Buf& t, const char* what, bool reduce) const;
  std::vector<Chunk> chunks(const Buf& t, const std::vector<int64_t>& sizes) const;
  int64_t piece_elems(int dtype) const { return std::max<int64_t>(1, static_cast<int64_t>(slot_bytes_) / elem_bytes(dtype)); }

  void put(int dst, const char* src, int64_t numel, int dtype, int scale_world);
  void take(int src, char* into, int64_t numel, int dtype, bool reduce, int scale_world);
  void exchange(const Chunk* send, int dst, const Chunk* recv, int src, int dtype, bool reduce, int put_scale,
                int take_scale);
  void ring_reduce_scatter(const std::vector<Chunk>& c, int dtype, bool average, bool keep_sent);
  void ring_all_gather(const std::vector<Chunk>& c, int dtype);
  void signal(int dst, uint64_t length);
  uint64_t await(int src);
  void release(int src);
  void barrier_now(bool after_gpu = false, uint64_t tag = 0);
  const char* peer_arena(int peer, int64_t offset, size_t bytes);

  std::string region_name(int rank) const { return "/tandem-" + job_ + "-" + std::to_string(rank) + "-hip"; }

  std::string job_;
  int rank_, size_, slots_;
  size_t slot_bytes_;
  double timeout_s_;
  int device_;
  bool use_events_;
  hipStream_t stream_ = nullptr;
  hipStream_t gather_stream_ = nullptr;  // direct unit gathers, launched by the caller's thread
  uint64_t put_tag_ = 0, take_tag_ = 0;  // progress thread only: piece_tag() of the slot-ring collective that is running
  hipEvent_t gather_mark_ = nullptr;     // progress thread only: where gather_stream_ stood when the job it runs was submitted
  hipStream_t anchor_stream_ = nullptr;  // carries nothing but the timing anchors: always idle
  std::mutex anchor_mu_, arena_mu_;      // both threads time their work and map peers' arenas
  Region mine_;
  std::vector<std::unique_ptr<Region>> theirs_;
  std::vector<void*> out_mem_, peer_mem_;
  std::vector<void*> arenas_;                      // in the order they were shared
  std::vector<size_t> arena_sizes_;
  std::vector<std::vector<void*>> peer_arena_;     // [peer][arena]: mapped at first use
  std::vector<std::vector<size_t>> peer_arena_bytes_;
  std::vector<std::vector<hipEvent_t>> full_, free_, peer_full_, peer_free_;
  std::vector<uint64_t> sent_, got_;     // pieces, per peer: pick the slot
  std::vector<uint64_t> posted_;         // messages queued or published to each peer (flow control)
  std::vector<uint64_t> taken_;          // messages consumed from each peer
  bool connected_ = false, closed_ = false;
  // staged collectives
  bool staged_ = true;               // TANDEM_HIP_ALGO=ring switches them off
  bool gathers_on_side_stream_ = false;  // TANDEM_HIP_GATHER=stream (or stream-words, stream-events)
  enum class GatherReady { kRingEvent, kWord, kFreshEvent };
  GatherReady gather_ready_ = GatherReady::kRingEvent;  // what a side-stream gather waits for before its copies
  bool gather_done_word_ = true;         // its end is a value word of the pool (else an event)
  std::vector<hipEvent_t> ready_events_; // kRingEvent: made at start, used in turn by the callers' threads
  std::atomic<uint64_t> ready_next_{0};
  std::shared_ptr<FlagPool> flags_;      // the words that tdm_work_wait_stream parks streams on
  bool want_flags_ = false;              // the device can make a stream wait for a value
  bool defer_default_ = false;           // TANDEM_HIP_WAIT=stream: tdm_work_wait parks as well
  double park_limit_s_ = 0;              // the engine's time limit and a margin, or TANDEM_HIP_PARK_LIMIT_S
  bool may_park_ = true;                 // false with GPU_MAX_HW_QUEUES=1: no stream is parked on a collective that has not run
  std::string sticky_error_;             // under mu_: a collective failed after its wait() had already returned
  bool ready_on_host_ = true;        // TANDEM_HIP_READY=gpu: wait for the caller's stream on the GPU instead
  // bytes per half (TANDEM_HIP_STAGING_BYTES). Two ranks, all_reduce of 256 MiB / 1 GiB: 0.52 / 1.93 ms with 64 MiB halves,
  // 0.43-0.45 / 1.62-1.66 with 128 MiB, 0.42 / 1.60 with 256 MiB: the handshakes of a pass are what a larger half saves.
  size_t staging_half_ = 128u << 20;
  size_t small_bytes_ = 32u << 20;   // all_reduce up to this size takes the one-handshake form (TANDEM_HIP_SMALL_BYTES)
  void* staging_ = nullptr;
  std::vector<void*> peer_staging_;
  uint64_t staged_ops_ = 0;          // picks the half; the same count on every rank
  std::atomic<int> timing_{0};
  bool timing_seen_ = false;           // under anchor_mu_
  std::shared_ptr<Anchor> anchor_;     // under anchor_mu_

  // "host" ordering: what to publish once the GPU has passed an event.
  struct Completion {
    hipEvent_t after;  // nullptr: publish at once (still in order)
    bool is_release;
    int peer;
    uint64_t length;
  };
  void complete_later(bool is_release, int peer, uint64_t length, bool after_stream);
  void completion_loop();
  void drain_completions();
  std::mutex cmu_;
  std::condition_variable ccv_;
  std::deque<Completion> completions_;
  bool cstop_ = false;
  std::atomic<uint64_t> cqueued_{0};  // completions ever queued
  std::atomic<uint64_t> csettled_{0}; // completions published (or dropped after a failure): what a barrier waits for
  uint64_t cdone_ = 0;                // completions ever taken (completion thread, under cmu_)
  std::string cerror_;
  std::thread completer_;

  std::mutex mu_;
  std::condition_variable cv_;
  std::deque<std::pair<std::function<void()>, std::shared_ptr<Work>>> jobs_;
  std::atomic<uint64_t> submitted_{0};  // jobs ever queued
  uint64_t started_ = 0;                // jobs ever taken (progress thread only)
  bool stopping_ = false;
  std::thread thread_;
};

}  // namespace tandem_hip
