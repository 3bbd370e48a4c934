// The engine behind Group(backend="hip"): one rank's half of a group whose ranks
// are processes sharing one MI355X.
//
// Shape of the thing (what the reference's native plug-in also is,
// tandem/csrc/collectives.h:43-126, tandem/csrc/cuda_links.h:1-22): an Engine per
// rank, a progress thread that runs queued collectives in submission order and
// never touches Python, Work handles, and per ordered pair of ranks a ring of
// `slots` device buffers that the sender owns and the receiver maps through HIP
// IPC. What differs is what moves through it:
//   * a put is one launch of the copy kernel into the sender's slot (dividing by
//     the world size on the way when the collective averages), a take is one
//     launch of the fused ring-step kernel that reads the peer's slot in place;
//   * an 8-byte message per piece in a shared-memory ring says which slot and how
//     long. Two ways of ordering a slot's hand-over against the GPU work:
//       "host"  (default) the progress thread only enqueues; a completion thread
//               waits on an ordinary event recorded after each kernel and then
//               publishes the message (piece ready) or the release (slot free), so
//               a message always means "the bytes have landed" and neither the
//               progress thread nor the caller ever blocks on the GPU;
//       "event" (TANDEM_HIP_SYNC=event) interprocess events full[j] / free[j],
//               exported with hipIpcGetEventHandle and waited for on the stream,
//               as the reference's CUDA engine does. HIP implements these by
//               registering a shared host page with the GPU; where the platform
//               refuses that registration they cannot be recorded, hence the default;
//   * every rank publishes its handles in one POSIX shared-memory region,
//     "/tandem-<job>-<rank>-hip", which also holds the message rings it sends on.
//
// Streams: a collective starts on the engine's stream once the caller's stream
// has reached the point of submission (an event), and tdm_work_wait makes the
// caller's stream wait for the collective's last kernel, as in the reference
// (tandem/csrc/collectives.cpp:159-224). Submission never blocks the caller. With
// host ordering, however, the progress thread hands every piece (and every fence)
// over only once the GPU has produced it, so a job is not fully enqueued before its
// last hand-over has happened on the GPU, and tdm_work_wait, which waits for the
// job to be enqueued, returns about when the collective's last kernel starts.

#include "engine.h"

namespace tandem_hip {

Engine::Engine(const std::string& job, int rank, int size, int slots, size_t slot_bytes, double timeout_s, int device)
    : job_(job), rank_(rank), size_(size), slots_(slots), slot_bytes_(slot_bytes), timeout_s_(timeout_s),
      device_(device), theirs_(size), out_mem_(size, nullptr), peer_mem_(size, nullptr), full_(size), free_(size),
      peer_full_(size), peer_free_(size), sent_(size, 0), got_(size, 0), posted_(size, 0), taken_(size, 0) {
  peer_arena_.assign(size, std::vector<void*>(kMaxArenas, nullptr));
  peer_arena_bytes_.assign(size, std::vector<size_t>(kMaxArenas, 0));
  if (size < 1 || rank < 0 || rank >= size) throw Invalid("rank must be in [0, size)");
  if (slots < 1 || slots > kMaxSlots) throw Invalid("slots must be in [1, " + std::to_string(kMaxSlots) + "]");
  if (slot_bytes < 16 || slot_bytes % 16) throw Invalid("slot_bytes must be a positive multiple of 16");
  if (slot_bytes * static_cast<size_t>(slots) >= (size_t(2) << 30)) {
    throw Invalid("slots * slot_bytes must stay under 2 GiB per pair (one IPC allocation)");
  }
  if (device < 0) throw Invalid("the hip engine needs a GPU: device must be >= 0 (there is no CPU path)");
  if (job.empty() || job.size() > 64) throw Invalid("job name must have 1..64 characters");
  const char* mode = std::getenv("TANDEM_HIP_SYNC");
  use_events_ = mode && std::string(mode) == "event";
  const char* algo = std::getenv("TANDEM_HIP_ALGO");
  if (algo && std::string(algo) == "ring") staged_ = false;
  else if (algo && *algo && std::string(algo) != "staged") throw Invalid("TANDEM_HIP_ALGO must be \"staged\" or \"ring\"");
  if (const char* sb = std::getenv("TANDEM_HIP_STAGING_BYTES")) {
    const long long v = std::atoll(sb);
    if (v < 4096 || v >= (1ll << 30) || v % 4096) throw Invalid("TANDEM_HIP_STAGING_BYTES must be a multiple of 4096 in [4096, 1 GiB)");
    staging_half_ = static_cast<size_t>(v);
  }
  if (const char* sm = std::getenv("TANDEM_HIP_SMALL_BYTES")) {
    const long long v = std::atoll(sm);
    if (v < 0) throw Invalid("TANDEM_HIP_SMALL_BYTES must not be negative");
    small_bytes_ = static_cast<size_t>(v);
  }
  {
    // Every Work gets a word that streams can be parked on (tdm_work_wait_stream) where the device can do that;
    // TANDEM_HIP_WAIT=stream makes the plain tdm_work_wait park too.
    int can = 0;
    (void)hipDeviceGetAttribute(&can, hipDeviceAttributeCanUseStreamWaitValue, device);
    want_flags_ = can == 1;
    if (const char* wm = std::getenv("TANDEM_HIP_WAIT")) {
      if (std::string(wm) == "stream") {
        if (!want_flags_) throw Invalid("TANDEM_HIP_WAIT=stream: this device cannot make a stream wait for a value");
        defer_default_ = true;
      } else if (std::string(wm) != "host") {
        throw Invalid("TANDEM_HIP_WAIT must be \"host\" or \"stream\"");
      }
    }
    // Parking a stream on a collective that has not run yet queues the wait BEFORE the write that ends it. The two must
    // not share a hardware queue: the runtime's wait is a kernel that spins at the head of its queue, and a write queued
    // behind it never runs. A process told to use a single hardware queue (GPU_MAX_HW_QUEUES=1) has nowhere else to put
    // the engine's stream (seen: every parked wait timed out), and with fewer queues than the four streams such a
    // process has at least (the caller's, and the engine's three) two of them share one: there every wait is taken on
    // the host, whatever was asked for. HIP's default is four.
    if (const char* hq = std::getenv("GPU_MAX_HW_QUEUES")) {
      const int queues = std::atoi(hq);
      if (queues >= 1 && queues < 4) may_park_ = false;
    }
    // A parked stream gives up by itself after the engine's own time limit and a margin (by then the host has declared
    // the collective failed and set the word, unless the write cannot get past the wait): no wait on the GPU is without end.
    park_limit_s_ = timeout_s_ + 10.0;
    if (const char* pl = std::getenv("TANDEM_HIP_PARK_LIMIT_S")) {
      const double v = std::atof(pl);
      if (!(v > 0)) throw Invalid("TANDEM_HIP_PARK_LIMIT_S must be a positive number of seconds");
      park_limit_s_ = v;
    }
  }
  if (const char* gm = std::getenv("TANDEM_HIP_GATHER")) {
    // "stream": on the engine's side stream; it starts behind an event of the caller's stream (from a ring of events)
    // and ends with a value word that wait() parks the caller's stream on. "stream-words": value words for both;
    // "stream-events": a fresh event for each, created and destroyed per gather (what the path first did).
    const std::string mode(gm);
    gathers_on_side_stream_ = mode == "stream" || mode == "stream-words" || mode == "stream-events";
    gather_ready_ = mode == "stream-words" ? GatherReady::kWord : mode == "stream-events" ? GatherReady::kFreshEvent : GatherReady::kRingEvent;
    gather_done_word_ = mode != "stream-events";
  }
  if (const char* rd = std::getenv("TANDEM_HIP_READY")) ready_on_host_ = std::string(rd) != "gpu";
  peer_staging_.assign(size, nullptr);

  check_hip(hipSetDevice(device_), "hipSetDevice");
  try {
    start();
  } catch (...) {  // no destructor runs for a constructor that throws
    release_device();
    throw;
  }
}

void Engine::start() {
  check_hip(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking), "hipStreamCreateWithFlags");  // default priority, all three
  if (want_flags_) flags_ = FlagPool::make();
  check_hip(hipStreamCreateWithFlags(&gather_stream_, hipStreamNonBlocking), "hipStreamCreateWithFlags (gathers)");
  if (gathers_on_side_stream_ && gather_ready_ == GatherReady::kRingEvent) {
    ready_events_.assign(64, nullptr);
    for (hipEvent_t& ev : ready_events_) check_hip(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "hipEventCreateWithFlags (ready ring)");
  }
  check_hip(hipStreamCreateWithFlags(&anchor_stream_, hipStreamNonBlocking), "hipStreamCreateWithFlags (anchors)");

  mine_.create(region_name(rank_), size_);
  RegionHeader* h = mine_.header();
  h->rank = rank_;
  h->size = size_;
  h->device = device_;
  h->slots = slots_;
  h->slot_bytes = slot_bytes_;
  h->pid = static_cast<int64_t>(::getpid());
  h->use_events = use_events_;
  constexpr unsigned kFlags = hipEventDisableTiming | hipEventInterprocess;
  for (int p = 0; p < size_; ++p) {
    if (p == rank_) continue;
    PeerEntry* e = mine_.entry(p);
    check_hip(hipMalloc(&out_mem_[p], static_cast<size_t>(slots_) * slot_bytes_), "hipMalloc (slots)");
    check_hip(hipIpcGetMemHandle(&e->mem, out_mem_[p]), "hipIpcGetMemHandle");
    if (use_events_) {
      full_[p].resize(slots_);
      free_[p].resize(slots_);
      for (int j = 0; j < slots_; ++j) {
        check_hip(hipEventCreateWithFlags(&full_[p][j], kFlags), "hipEventCreateWithFlags (full)");
        if (hipIpcGetEventHandle(&e->full[j], full_[p][j]) != hipSuccess) {
          (void)hipGetLastError();
          throw std::runtime_error("TANDEM_HIP_SYNC=event: this platform cannot export interprocess events "
                                   "(hipIpcGetEventHandle failed); use the default host ordering");
        }
        check_hip(hipEventCreateWithFlags(&free_[p][j], kFlags), "hipEventCreateWithFlags (free)");
        check_hip(hipIpcGetEventHandle(&e->free_[j], free_[p][j]), "hipIpcGetEventHandle (free)");
      }
    }
  }
  std::atomic_thread_fence(std::memory_order_release);
  h->magic = kRegionMagic;  // published last
  if (!use_events_) completer_ = std::thread([this] { completion_loop(); });
  thread_ = std::thread([this] { loop(); });
}

void Engine::connect() {
  if (connected_) return;
  check_hip(hipSetDevice(device_), "hipSetDevice");
  for (int p = 0; p < size_; ++p) {
    if (p == rank_) continue;
    theirs_[p] = std::make_unique<Region>();
    theirs_[p]->open(region_name(p), size_);
    const RegionHeader* h = theirs_[p]->header();
    if (h->magic != kRegionMagic || h->size != size_ || h->slots != slots_ || h->slot_bytes != slot_bytes_ ||
        h->rank != p || h->use_events != static_cast<int32_t>(use_events_)) {
      throw std::runtime_error("rank " + std::to_string(p) + "'s region does not match ours (size, slots, slot_bytes or sync mode)");
    }
    if (h->pid == static_cast<int64_t>(::getpid())) {
      throw std::runtime_error("two ranks of one group in one process: HIP IPC handles cannot be opened by their exporter");
    }
    // In p's region, the entry for us: p's slots for sending to us, their full
    // events, and the free events p records after reading OUR slots.
    PeerEntry* e = theirs_[p]->entry(rank_);
    check_hip(hipIpcOpenMemHandle(&peer_mem_[p], e->mem, hipIpcMemLazyEnablePeerAccess), "hipIpcOpenMemHandle");
    if (use_events_) {
      peer_full_[p].resize(slots_);
      peer_free_[p].resize(slots_);
      for (int j = 0; j < slots_; ++j) {
        check_hip(hipIpcOpenEventHandle(&peer_full_[p][j], e->full[j]), "hipIpcOpenEventHandle (full)");
        check_hip(hipIpcOpenEventHandle(&peer_free_[p][j], e->free_[j]), "hipIpcOpenEventHandle (free)");
      }
    }
  }
  connected_ = true;
}

void Engine::close() {
  {
    std::lock_guard<std::mutex> lock(mu_);
    if (stopping_) return;
    stopping_ = true;
  }
  cv_.notify_all();
  if (thread_.joinable()) thread_.join();  // runs what was queued first
  if (closed_) return;
  closed_ = true;
  (void)hipSetDevice(device_);
  // Our GPU work must finish, and every peer's (they read our slots), before any
  // rank frees its slots and events.
  hipError_t sync_err = hipStreamSynchronize(stream_);
  if (sync_err == hipSuccess && gather_stream_) sync_err = hipStreamSynchronize(gather_stream_);
  std::string barrier_err;
  if (connected_) {
    try {
      barrier_now();
      drain_completions();
    } catch (const std::exception& e) {
      barrier_err = e.what();
    }
  }
  if (completer_.joinable()) {
    {
      std::lock_guard<std::mutex> lock(cmu_);
      cstop_ = true;
    }
    ccv_.notify_all();
    completer_.join();
  }
  release_device();  // after the closing barrier: no peer reads our slots or arena any more
  check_hip(sync_err, "hipStreamSynchronize (close)");
  if (!barrier_err.empty()) throw std::runtime_error("close: " + barrier_err);
}

// Mappings of the peers' memory, our slots, events, stream, arena and region.
void Engine::release_device() {
  for (int p = 0; p < size_; ++p) {
    if (p == rank_) continue;
    if (peer_mem_[p]) (void)hipIpcCloseMemHandle(peer_mem_[p]);
    for (hipEvent_t e : peer_full_[p]) (void)hipEventDestroy(e);
    for (hipEvent_t e : peer_free_[p]) (void)hipEventDestroy(e);
    for (hipEvent_t e : full_[p]) (void)hipEventDestroy(e);
    for (hipEvent_t e : free_[p]) (void)hipEventDestroy(e);
    if (out_mem_[p]) (void)hipFree(out_mem_[p]);
    for (void*& a : peer_arena_[p]) {
      if (a) (void)hipIpcCloseMemHandle(a);
      a = nullptr;
    }
    if (peer_staging_[p]) (void)hipIpcCloseMemHandle(peer_staging_[p]);
    peer_staging_[p] = nullptr;
    peer_mem_[p] = out_mem_[p] = nullptr;
    peer_full_[p].clear(); peer_free_[p].clear(); full_[p].clear(); free_[p].clear();
    theirs_[p].reset();
  }
  for (hipStream_t* st : {&stream_, &gather_stream_, &anchor_stream_}) {
    if (*st) (void)hipStreamDestroy(*st);
    *st = nullptr;
  }
  for (hipEvent_t ev : ready_events_)
    if (ev) (void)hipEventDestroy(ev);
  ready_events_.clear();
  for (void* a : arenas_) (void)hipFree(a);
  arenas_.clear();
  arena_sizes_.clear();
  if (staging_) (void)hipFree(staging_);
  staging_ = nullptr;
  mine_.reset();
}

Engine::~Engine() {
  try {
    close();
  } catch (...) {  // a destructor must not throw; call close() to see errors
  }
}

// ---------------------------------------------------------------- progress thread
// host_ready: the job begins with a handshake that needs the inputs complete, not
// merely ordered on the GPU, so the progress thread itself waits for them (polling:
// an idle stream passes the event within microseconds) and the engine's stream
// is spared a wait packet.
std::shared_ptr<Work> Engine::submit(std::function<void()> job, hipStream_t caller, bool uses_gpu, bool host_ready, bool drained) {
  auto work = std::make_shared<Work>();
  work->device = device_;
  work->uses_gpu = uses_gpu;
  work->drained = drained;
  if (flags_ && uses_gpu) {
    work->flag = flags_->acquire(&work->flag_value);
    if (work->flag >= 0) work->flags = flags_;
    work->defer_default = defer_default_ && may_park_;
    work->may_park = may_park_;
    work->park_limit_s = park_limit_s_;
  }
  hipEvent_t ready = nullptr;
  if (uses_gpu) {
    // Start once the caller's stream has produced the inputs.
    check_hip(hipEventCreateWithFlags(&ready, hipEventDisableTiming), "hipEventCreateWithFlags (ready)");
    hipError_t err = hipEventRecord(ready, caller);
    if (err != hipSuccess) {
      (void)hipEventDestroy(ready);
      check_hip(err, "hipEventRecord (ready)");
    }
    job = [this, ready, host_ready, w = work.get(), inner = std::move(job)] {
      hipError_t e;
      if (host_ready) {
        try {
          e = poll_gpu([&] { return hipEventQuery(ready); }, timeout_s_);
        } catch (...) {
          (void)hipGetLastError();
          (void)hipEventDestroy(ready);
          throw;
        }
        (void)hipGetLastError();  // the "not ready" left by the polls
      } else {
        e = hipStreamWaitEvent(stream_, ready, 0);
      }
      (void)hipEventDestroy(ready);  // released once the GPU is past it
      check_hip(e, "waiting for the caller's stream (ready)");
      stamp_start(*w, stream_);
      inner();
    };
  }
  hipEvent_t mark = nullptr;
  if (uses_gpu && gathers_on_side_stream_) {
    // What a fence inside this job waits for on the gather stream: the gathers launched (by callers' threads) BEFORE
    // this call. A later gather may itself wait, through the caller's stream, for this job's end (a wait() that parks
    // the stream, then the next unit's gather): a fence that waited for everything on that stream would wait for itself.
    hipError_t err = hipEventCreateWithFlags(&mark, hipEventDisableTiming);
    if (err == hipSuccess && (err = hipEventRecord(mark, gather_stream_)) != hipSuccess) {
      (void)hipEventDestroy(mark);
      mark = nullptr;
    }
    if (err != hipSuccess) {
      if (ready) (void)hipEventDestroy(ready);
      check_hip(err, "marking the gather stream");
    }
    job = [this, mark, inner = std::move(job)] {
      struct Scope {  // the progress thread's alone; the event goes when the job has run or failed
        Engine* self;
        hipEvent_t mark;
        ~Scope() {
          self->gather_mark_ = nullptr;
          (void)hipEventDestroy(mark);
        }
      } scope{this, mark};
      gather_mark_ = mark;
      inner();
    };
  }
  {
    std::lock_guard<std::mutex> lock(mu_);
    if (sticky_error_.empty() && flags_ && flags_->gave_up()) {
      sticky_error_ = "a stream parked on a collective gave up waiting for its end (do the waiting stream and the engine's share a hardware queue?)";
    }
    if (stopping_ || !sticky_error_.empty()) {
      if (ready) (void)hipEventDestroy(ready);  // the job that would have released it never runs
      if (mark) (void)hipEventDestroy(mark);
      throw std::runtime_error(stopping_ ? "the engine is closed" : "an earlier collective failed: " + sticky_error_);
    }
    jobs_.emplace_back(std::move(job), work);
    submitted_.fetch_add(1, std::memory_order_release);
  }
  cv_.notify_one();
  return work;
}

// With timing on: a time-stamped event on the engine's stream, after the wait for
// the inputs and before the collective's first kernel. A fresh anchor is taken
// each time the switch goes on, so the two clocks cannot drift far apart.
void Engine::stamp_start(Work& w, hipStream_t on) {
  std::lock_guard<std::mutex> lock(anchor_mu_);
  if (timing_.load(std::memory_order_acquire) == 0) {
    timing_seen_ = false;
    return;
  }
  if (!timing_seen_ || !anchor_) {
    auto a = std::make_shared<Anchor>();
    check_hip(hipEventCreateWithFlags(&a->event, hipEventDefault), "hipEventCreate (anchor)");
    check_hip(hipEventRecord(a->event, anchor_stream_), "hipEventRecord (anchor)");
    check_hip(hipEventSynchronize(a->event), "hipEventSynchronize (anchor)");
    a->host = now_s();
    anchor_ = std::move(a);
    timing_seen_ = true;
  }
  check_hip(hipEventCreateWithFlags(&w.start_event, hipEventDefault), "hipEventCreate (start)");
  check_hip(hipEventRecord(w.start_event, on), "hipEventRecord (start)");
  w.anchor = anchor_;
}

void Engine::loop() {
  (void)hipSetDevice(device_);
  for (;;) {
    std::pair<std::function<void()>, std::shared_ptr<Work>> next;
    spin_for([this] { return submitted_.load(std::memory_order_acquire) != started_; });
    {
      std::unique_lock<std::mutex> lock(mu_);
      cv_.wait(lock, [this] { return stopping_ || !jobs_.empty(); });
      if (jobs_.empty()) return;  // stopping, and everything queued has run
      ++started_;
      next = std::move(jobs_.front());
      jobs_.pop_front();
    }
    Work& w = *next.second;
    int status = TDM_OK;
    std::string error;
    const double t0 = now_s();
    try {
      next.first();
    } catch (const Invalid& e) {
      status = TDM_EINVAL; error = e.what();
    } catch (const Timeout& e) {
      status = TDM_ETIMEOUT; error = e.what();
    } catch (const std::exception& e) {
      status = TDM_ERUNTIME; error = e.what();
    } catch (...) {
      status = TDM_ERUNTIME; error = "unknown error";
    }
    // Its end on the GPU: the flag word where the job has one (written by the engine's stream below), an event
    // where it has none, and for the time stamps.
    if (status == TDM_OK && w.uses_gpu && (w.start_event || (w.flag < 0 && !w.drained))) {
      if (hipEventCreateWithFlags(&w.done_event, w.start_event ? hipEventDefault : hipEventDisableTiming) != hipSuccess ||
          hipEventRecord(w.done_event, stream_) != hipSuccess) {
        status = TDM_ERUNTIME;
        error = "could not record the collective's completion event";
      }
    }
    if (w.flag >= 0) {
      // Whoever waits for the word on the GPU is let go behind the job's last kernel, by the
      // engine's own stream; after a failure (or with that stream idle anyway) at once, by the host.
      uint32_t* word = w.flags->base + w.flag;
      if (status == TDM_OK && !w.drained && hipStreamWriteValue32(stream_, word, w.flag_value, 0) != hipSuccess) {
        // The stream cannot say so itself: the host does, once the stream has run dry.
        (void)hipGetLastError();
        try {
          const hipError_t err = poll_gpu([this] { return hipStreamQuery(stream_); }, timeout_s_);
          if (err != hipSuccess) throw std::runtime_error(hipGetErrorString(err));
        } catch (const std::exception& e) {
          status = TDM_ERUNTIME;
          error = std::string("could not signal the collective's end: ") + e.what();
        }
        (void)hipGetLastError();
        w.flags->set(w.flag, w.flag_value);
      } else if (status != TDM_OK || w.drained) {
        w.flags->set(w.flag, w.flag_value);
      }
      if (status != TDM_OK) {  // its wait() may have returned long ago: the next call reports it
        std::lock_guard<std::mutex> lock(mu_);
        if (sticky_error_.empty()) sticky_error_ = error;
      }
    }
    {
      std::lock_guard<std::mutex> lock(w.mu);
      w.status = status;
      w.error = std::move(error);
      w.t0 = t0;
      w.t1 = now_s();
      w.finished = true;
    }
    w.finished_hint.store(true, std::memory_order_release);
    w.cv.notify_all();
  }
}

// ---------------------------------------------------------------- messages
void Engine::signal(int dst, uint64_t length) {
  ring_publish(mine_.entry(dst)->ring, slots_, length);
}

// The next message from src. Messages are consumed in order by the progress
// thread (taken_), and released, possibly later, in the same order (tail).
uint64_t Engine::await(int src) {
  const uint64_t at = taken_[src];
  const uint64_t length = ring_read(theirs_[src]->entry(rank_)->ring, at, slots_, timeout_s_,
                                    "timed out waiting for a message from a peer rank");
  taken_[src] = at + 1;
  return length;
}

void Engine::release(int src) {
  ring_release(theirs_[src]->entry(rank_)->ring);
}

// "host" ordering. Completions are published strictly in the order they were
// queued, which is the order of the kernels on the engine's stream.
void Engine::complete_later(bool is_release, int peer, uint64_t length, bool after_stream) {
  Completion c{nullptr, is_release, peer, length};
  if (after_stream) {
    check_hip(hipEventCreateWithFlags(&c.after, hipEventDisableTiming), "hipEventCreateWithFlags (completion)");
    hipError_t err = hipEventRecord(c.after, stream_);
    if (err != hipSuccess) {
      (void)hipEventDestroy(c.after);
      check_hip(err, "hipEventRecord (completion)");
    }
  }
  {
    std::lock_guard<std::mutex> lock(cmu_);
    if (!cerror_.empty()) throw std::runtime_error("completion thread failed: " + cerror_);
    completions_.push_back(c);
    cqueued_.fetch_add(1, std::memory_order_release);
  }
  ccv_.notify_one();
}

void Engine::completion_loop() {
  (void)hipSetDevice(device_);
  for (;;) {
    Completion c;
    spin_for([this] { return cqueued_.load(std::memory_order_acquire) != cdone_; });
    {
      std::unique_lock<std::mutex> lock(cmu_);
      ccv_.wait(lock, [this] { return cstop_ || !completions_.empty(); });
      if (completions_.empty()) return;
      c = completions_.front();
      completions_.pop_front();
      ++cdone_;
    }
    if (c.after) {
      hipError_t err;
      try {
        err = poll_gpu([&] { return hipEventQuery(c.after); }, timeout_s_);
      } catch (const Timeout&) {
        err = hipErrorNotReady;
      }
      (void)hipGetLastError();
      (void)hipEventDestroy(c.after);
      if (err != hipSuccess) {
        std::lock_guard<std::mutex> lock(cmu_);
        if (cerror_.empty()) cerror_ = std::string("waiting for a piece's kernel: ") + hipGetErrorString(err);
      }
    }
    bool failed;
    {
      // After a failure nothing more is published, this message or any later one:
      // the peers time out rather than read bad bytes or reuse a slot still in use.
      std::lock_guard<std::mutex> lock(cmu_);
      failed = !cerror_.empty();
    }
    if (!failed) {
      if (c.is_release) release(c.peer); else signal(c.peer, c.length);
    }
    csettled_.fetch_add(1, std::memory_order_release);
  }
}

void Engine::drain_completions() {
  if (use_events_) return;
  // Everything this thread has queued (it alone queues) has been published, or dropped after a failure.
  const uint64_t queued = cqueued_.load(std::memory_order_acquire);
  wait_until([&] { return csettled_.load(std::memory_order_acquire) >= queued; }, timeout_s_,
             "timed out waiting for the GPU to finish the queued pieces");
  std::lock_guard<std::mutex> lock(cmu_);
  if (!cerror_.empty()) throw std::runtime_error("completion thread failed: " + cerror_);
}

// after_gpu: the empty messages are published only once the GPU has finished what
// the engine's stream holds so far (a fence), not merely when it has been enqueued.
// tag: what the ranks must agree on at this point (0 for a plain barrier; the staged and
// direct collectives send the kind of operation and the tensor's size). A rank that is
// somewhere else in its program, or has a tensor of another size, is found out here
// instead of reading stale bytes: the slot ring finds such a rank by its piece lengths.
void Engine::barrier_now(bool after_gpu, uint64_t tag) {
  // Messages are published in order: everything queued for the completion thread
  // goes first. After that this thread publishes by itself; it has to wait for the
  // peers anyway, and handing over to the completion thread would cost two wake-ups.
  drain_completions();
  if (after_gpu) {
    hipError_t err = poll_gpu([this] { return hipStreamQuery(stream_); }, timeout_s_);
    (void)hipGetLastError();
    check_hip(err, "hipStreamQuery (fence)");
    // the gather stream: up to where it stood when this job was submitted (gather_mark_), or all of it
    hipEvent_t mark = gather_mark_;
    err = mark ? poll_gpu([mark] { return hipEventQuery(mark); }, timeout_s_)
               : poll_gpu([this] { return hipStreamQuery(gather_stream_); }, timeout_s_);
    (void)hipGetLastError();
    check_hip(err, "waiting for the gather stream (fence)");
  }
  // An empty message to every peer, then one from each. Rings are first in,
  // first out, so this also orders the barrier after every piece queued before.
  const uint64_t kEmpty = kNoPiece | (tag & ~kNoPiece);
  for (int p = 0; p < size_; ++p) {
    if (p == rank_) continue;
    Ring& r = mine_.entry(p)->ring;
    const uint64_t posted = posted_[p];
    ring_wait_for_room(r, posted, slots_, timeout_s_, "barrier: a peer rank never drained its messages");
    posted_[p] = posted + 1;
    signal(p, kEmpty);
  }
  for (int p = 0; p < size_; ++p) {
    if (p == rank_) continue;
    const uint64_t got = await(p);
    if (!(got & kNoPiece)) throw std::runtime_error("barrier out of step: expected an empty message, got a piece");
    if (got != kEmpty) {
      throw std::runtime_error("collectives out of step: rank " + std::to_string(p) + " is in another collective, or in the same "
                               "one with a tensor of another size");
    }
    release(p);
  }
}

// ---------------------------------------------------------------- pieces
void Engine::put(int dst, const char* src, int64_t numel, int dtype, int scale_world) {
  const size_t nbytes = static_cast<size_t>(numel) * elem_bytes(dtype);
  if (nbytes > slot_bytes_) throw Invalid("piece larger than a slot");
  const uint64_t k = sent_[dst];  // pieces so far: picks the slot
  const int j = static_cast<int>(k % slots_);
  Ring& r = mine_.entry(dst)->ring;
  // Room in the message ring means fewer than `slots` messages are unreleased, so
  // fewer than `slots` pieces are: dst has released slot j's previous piece ...
  const uint64_t posted = posted_[dst];
  ring_wait_for_room(r, posted, slots_, timeout_s_, "put: the peer never freed a slot");
  if (use_events_ && k >= static_cast<uint64_t>(slots_)) {
    // ... and enqueued its reads of it before recording free[j]: wait for those reads.
    check_hip(hipStreamWaitEvent(stream_, peer_free_[dst][j], 0), "hipStreamWaitEvent (free)");
  }
  char* slot = static_cast<char*>(out_mem_[dst]) + static_cast<size_t>(j) * slot_bytes_;
  if (dtype == kBytesDtype) {
    check_hip(hipMemcpyAsync(slot, src, nbytes, hipMemcpyDeviceToDevice, stream_), "hipMemcpyAsync (put)");
  } else {
    tdm_pair pr{slot, src, numel};
    copy_step(&pr, 1, dtype, scale_world, stream_);
  }
  posted_[dst] = posted + 1;
  sent_[dst] = k + 1;
  if (use_events_) {
    check_hip(hipEventRecord(full_[dst][j], stream_), "hipEventRecord (full)");
    signal(dst, nbytes | put_tag_);
  } else {
    complete_later(false, dst, nbytes | put_tag_, true);  // published once the copy has landed
  }
}

void Engine::take(int src, char* into, int64_t numel, int dtype, bool reduce, int scale_world) {
  const size_t nbytes = static_cast<size_t>(numel) * elem_bytes(dtype);
  const uint64_t message = await(src);
  if (message & kNoPiece) throw std::runtime_error("collectives out of step: expected a piece, got a barrier");
  if ((message & ~kPieceLengthMask) != take_tag_) {
    throw std::runtime_error("collectives out of step: rank " + std::to_string(src) + " is in another collective, or in the same "
                             "one with a tensor of another size or type");
  }
  if ((message & kPieceLengthMask) != nbytes) throw std::runtime_error("a piece arrived with the wrong length");
  const int j = static_cast<int>(got_[src] % slots_);
  if (use_events_) check_hip(hipStreamWaitEvent(stream_, peer_full_[src][j], 0), "hipStreamWaitEvent (full)");
  const char* slot = static_cast<const char*>(peer_mem_[src]) + static_cast<size_t>(j) * slot_bytes_;
  if (reduce) {
    // The kernel reads the peer's slot in place. The slot already holds x / world
    // when averaging; our own chunk is divided here, as part of the add.
    tdm_pair pr{into, slot, numel};
    reduce_step(&pr, 1, dtype, scale_world, scale_world > 1, false, false, stream_);
  } else if (dtype == kBytesDtype) {
    check_hip(hipMemcpyAsync(into, slot, nbytes, hipMemcpyDeviceToDevice, stream_), "hipMemcpyAsync (take)");
  } else {
    tdm_pair pr{into, slot, numel};
    copy_step(&pr, 1, dtype, 0, stream_);
  }
  got_[src] += 1;
  if (use_events_) {
    check_hip(hipEventRecord(free_[src][j], stream_), "hipEventRecord (free)");
    release(src);
  } else {
    complete_later(true, src, 0, true);  // the slot is free once our kernel has read it
  }
}

// Sends `send` to dst while receiving `recv` from src, one piece of each at a
// time, so a ring of ranks all sending at once never waits on itself.
void Engine::exchange(const Chunk* send, int dst, const Chunk* recv, int src, int dtype, bool reduce, int put_scale,
                      int take_scale) {
  const int64_t pe = piece_elems(dtype);
  const int es = elem_bytes(dtype);
  const int64_t ns = send ? (send->numel + pe - 1) / pe : 0;
  const int64_t nr = recv ? (recv->numel + pe - 1) / pe : 0;
  for (int64_t k = 0; k < std::max(ns, nr); ++k) {
    if (k < ns) put(dst, send->ptr + k * pe * es, std::min(pe, send->numel - k * pe), dtype, put_scale);
    if (k < nr) take(src, recv->ptr + k * pe * es, std::min(pe, recv->numel - k * pe), dtype, reduce, take_scale);
  }
}

// Step s: send chunk (r-s-1) to r+1, add chunk (r-s-2) from r-1 (tandem/comm.py:301-305).
// Averaging is fused: the chunk sent on the first step leaves as x / n (and, for a
// bare reduce_scatter, is divided in place first, because the reference's div_ of
// the whole tensor is observable there); every receiving chunk is divided as part
// of its add; later steps send partial sums, already divided.
void Engine::ring_reduce_scatter(const std::vector<Chunk>& c, int dtype, bool average, bool keep_sent) {
  const int n = size_, r = rank_;
  const int w = average ? n : 0;
  for (int s = 0; s < n - 1; ++s) {
    const Chunk& out = c[mod(r - s - 1, n)];
    int put_scale = 0;
    if (s == 0 && w > 1) {
      if (keep_sent && out.numel > 0) {
        tdm_pair pr{out.ptr, out.ptr, out.numel};
        copy_step(&pr, 1, dtype, w, stream_);  // in place: x / n
      } else {
        put_scale = w;
      }
    }
    exchange(&out, mod(r + 1, n), &c[mod(r - s - 2, n)], mod(r - 1, n), dtype, true, put_scale, w);
  }
}

void Engine::ring_all_gather(const std::vector<Chunk>& c, int dtype) {
  const int n = size_, r = rank_;
  for (int s = 0; s < n - 1; ++s) {
    exchange(&c[mod(r - s, n)], mod(r + 1, n), &c[mod(r - s - 1, n)], mod(r - 1, n), dtype, false, 0, 0);
  }
}

// ---------------------------------------------------------------- staged collectives
// all_reduce and all_gather of any tensor without the slots' piece-by-piece
// handshakes. Every rank owns staging memory that its peers map once: two halves,
// used in turn by successive staged operations.
//   all_reduce, per pass over at most half/W bytes of every ring chunk:
//     copy my tensor's part of every chunk I do not own into my staging; fence;
//     fold my own chunk's part out of my tensor and the peers' stagings, in the
//     ring's order for that chunk, into my tensor AND my staging; fence; copy the
//     other chunks' parts from their owners' stagings.
//   all_gather, per pass over at most half bytes of every chunk:
//     copy my chunk's part into my staging; fence; copy the others' from theirs.
// Two handshakes (one) per pass where the slot ring makes 2(W-1) per 4 MiB piece, and
// the bits are the ring's: the fold adds in the ring's order.
// Why two halves are enough without a closing fence: an operation writes a half that
// the peers last read two staged operations ago; every staged operation contains a
// fence that a rank enters only when its engine stream has drained, so when this rank
// has passed the fence of the operation in between, those reads are over.
char* Engine::staging_half() {
  if (!staging_) {
    check_hip(hipMalloc(&staging_, 2 * staging_half_), "hipMalloc (staging)");
    RegionHeader* h = mine_.header();
    check_hip(hipIpcGetMemHandle(&h->staging_mem, staging_), "hipIpcGetMemHandle (staging)");
    h->staging_bytes.store(2 * staging_half_, std::memory_order_release);  // the handle is visible before the size
  }
  return static_cast<char*>(staging_) + (staged_ops_++ % 2) * staging_half_;
}

// Only after a fence of the same operation: every rank publishes before it enters one.
const char* Engine::peer_staging(int peer, int half) {
  if (!peer_staging_[peer]) {
    RegionHeader* h = theirs_[peer]->header();
    if (h->staging_bytes.load(std::memory_order_acquire) != 2 * staging_half_) {
      throw std::runtime_error("rank " + std::to_string(peer) + " has no staging memory of our size (TANDEM_HIP_STAGING_BYTES, TANDEM_HIP_ALGO differ?)");
    }
    check_hip(hipIpcOpenMemHandle(&peer_staging_[peer], h->staging_mem, hipIpcMemLazyEnablePeerAccess), "hipIpcOpenMemHandle (staging)");
  }
  return static_cast<const char*>(peer_staging_[peer]) + static_cast<size_t>(half) * staging_half_;
}

void Engine::copy_pairs(const tdm_pair* pairs, int np, int dtype) {
  if (np == 0) return;
  if (dtype != kBytesDtype) {
    copy_step(pairs, np, dtype, 0, stream_);
    return;
  }
  for (int i = 0; i < np; ++i) {
    check_hip(hipMemcpyAsync(pairs[i].dst, pairs[i].src, static_cast<size_t>(pairs[i].count), hipMemcpyDeviceToDevice, stream_),
              "hipMemcpyAsync (staged copy)");
  }
}

// Tensors up to 32 MiB, where a handshake costs more than the extra traffic: every rank
// puts its whole tensor into its staging; fence; every rank folds every chunk by itself,
// each in the ring's order for that chunk, out of its own tensor and the peers' stagings.
// One handshake and two launches; (W+3) instead of about 4.5 passes over the tensor.
// Measured (barrier, all_reduce, device sync): 2 ranks 0.074 vs 0.115 ms up to 4 MiB,
// 0.097 vs 0.121 at 32 MiB; 4 ranks 0.17 vs 0.26 and 0.265 vs 0.296; at 64 MiB and
// 4 ranks the two-handshake passes win (0.37 vs 0.41).
void Engine::staged_all_reduce_small(const Buf& t, bool average) {
  const auto cs = chunks(t, {});
  const int n = size_, r = rank_;
  char* mine = staging_half();
  const int half = static_cast<int>((staged_ops_ - 1) % 2);
  tdm_pair whole{mine, t.ptr, t.numel};
  copy_pairs(&whole, 1, t.dtype);
  barrier_now(true, fence_tag(1, t.dtype, t.numel));  // every rank's tensor is in its staging
  tdm_fold_seg segs[TDM_MAX_WORLD];
  std::memset(segs, 0, sizeof segs);
  int ns = 0;
  for (int c = 0; c < n; ++c) {
    if (cs[c].numel == 0) continue;
    const size_t lo = static_cast<size_t>(cs[c].ptr - t.ptr);
    for (int q = 0; q < n; ++q) segs[ns].src[q] = q == r ? cs[c].ptr : peer_staging(q, half) + lo;
    segs[ns].dst[r] = cs[c].ptr;
    segs[ns].count = cs[c].numel;
    segs[ns].chunk = c;
    ++ns;
  }
  fold_step(segs, ns, n, t.dtype, average, stream_);
}

void Engine::staged_all_reduce(const Buf& t, bool average) {
  if (static_cast<size_t>(t.numel) * elem_bytes(t.dtype) <= std::min(small_bytes_, staging_half_)) {
    if (t.numel > 0) staged_all_reduce_small(t, average);
    return;
  }
  const auto cs = chunks(t, {});
  const int es = elem_bytes(t.dtype), n = size_, r = rank_;
  const size_t sub_bytes = staging_half_ / n / 256 * 256;  // one sub-slab per ring chunk
  const int64_t sub = static_cast<int64_t>(sub_bytes) / es;
  if (sub == 0) throw Invalid("all_reduce: the staging memory is too small for this world size");
  int64_t longest = 0;
  for (const Chunk& c : cs) longest = std::max(longest, c.numel);
  for (int64_t at = 0; at < longest; at += sub) {
    char* mine = staging_half();
    const int half = static_cast<int>((staged_ops_ - 1) % 2);
    auto part = [&](int c) { return std::max<int64_t>(0, std::min(sub, cs[c].numel - at)); };
    tdm_pair pairs[TDM_MAX_PAIRS];
    int np = 0;
    for (int c = 0; c < n; ++c) {
      if (c == r || part(c) == 0) continue;
      pairs[np++] = tdm_pair{mine + c * sub_bytes, cs[c].ptr + at * es, part(c)};
    }
    copy_pairs(pairs, np, t.dtype);
    barrier_now(true, fence_tag(2, t.dtype, t.numel));  // every rank's parts are in its staging
    if (part(r) > 0) {
      tdm_fold_seg seg;
      std::memset(&seg, 0, sizeof seg);
      char* own = cs[r].ptr + at * es;
      for (int q = 0; q < n; ++q) seg.src[q] = q == r ? own : peer_staging(q, half) + r * sub_bytes;
      seg.dst[r] = own;
      seg.dst[(r + 1) % n] = mine + r * sub_bytes;  // a second copy of the result, for the peers to fetch
      seg.count = part(r);
      seg.chunk = r;
      fold_step(&seg, 1, n, t.dtype, average, stream_);
    }
    barrier_now(true);  // every chunk's part is folded
    np = 0;
    for (int c = 0; c < n; ++c) {
      if (c == r || part(c) == 0) continue;
      pairs[np++] = tdm_pair{cs[c].ptr + at * es, peer_staging(c, half) + c * sub_bytes, part(c)};
    }
    copy_pairs(pairs, np, t.dtype);
  }
}

// reduce_scatter through the stagings. Per pass over a window of `half` bytes of the tensor: copy the
// window's parts of the chunks I do not own into my staging, at the same offsets; fence; fold my chunk's
// part out of my tensor and the peers' stagings. partial_sums: the ring also leaves, in chunk c of rank
// c + k, the sum after k terms (tandem/comm.py:350-352 in the reference; ZeRO drops them and asks for
// the owner's chunk only). Every rank then folds those too, each out of the stagings of the ranks the
// ring would have passed before it, in the ring's order, and with the whole group's divisor: k - 1
// staged copies and its own, written over its own. One handshake per pass instead of two per 4 MiB piece.
void Engine::staged_reduce_scatter(const Buf& t, const std::vector<Chunk>& cs, bool average, bool partial_sums) {
  const int es = elem_bytes(t.dtype), n = size_, r = rank_;
  const int64_t cap = static_cast<int64_t>(staging_half_) / es;
  for (int64_t at = 0; at < t.numel; at += cap) {
    char* mine = staging_half();
    const int half = static_cast<int>((staged_ops_ - 1) % 2);
    const int64_t end = std::min(t.numel, at + cap);
    // chunk c within the window, as element offsets of the tensor
    auto lo = [&](int c) { return std::max<int64_t>(at, (cs[c].ptr - t.ptr) / es); };
    auto hi = [&](int c) { return std::min<int64_t>(end, (cs[c].ptr - t.ptr) / es + cs[c].numel); };
    tdm_pair pairs[TDM_MAX_PAIRS];
    int np = 0;
    for (int c = 0; c < n; ++c) {
      if (c == r || hi(c) <= lo(c)) continue;
      pairs[np++] = tdm_pair{mine + (lo(c) - at) * es, t.ptr + lo(c) * es, hi(c) - lo(c)};
      if (np == TDM_MAX_PAIRS) {
        copy_pairs(pairs, np, t.dtype);
        np = 0;
      }
    }
    copy_pairs(pairs, np, t.dtype);
    barrier_now(true, fence_tag(3, t.dtype, t.numel));  // every rank's parts are in its staging
    if (hi(r) > lo(r)) {
      tdm_fold_seg seg;
      std::memset(&seg, 0, sizeof seg);
      char* own = t.ptr + lo(r) * es;
      for (int q = 0; q < n; ++q) seg.src[q] = q == r ? own : peer_staging(q, half) + (lo(r) - at) * es;
      seg.dst[r] = own;
      seg.count = hi(r) - lo(r);
      seg.chunk = r;
      fold_step(&seg, 1, n, t.dtype, average, stream_);
    }
    if (!partial_sums) continue;
    for (int k = 1; k < n; ++k) {  // chunk c = r - k: I am the k-th rank the ring passes with it
      const int c = mod(r - k, n);
      if (hi(c) <= lo(c)) continue;
      char* own = t.ptr + lo(c) * es;
      if (k == 1) {  // the first sender's own term, divided when averaging (the reference divides the whole tensor first)
        if (average) {
          tdm_pair pr{own, own, hi(c) - lo(c)};
          copy_step(&pr, 1, t.dtype, n, stream_);
        }
        continue;
      }
      tdm_fold_seg seg;
      std::memset(&seg, 0, sizeof seg);
      for (int j = 0; j < k - 1; ++j) seg.src[j] = peer_staging(mod(c + 1 + j, n), half) + (lo(c) - at) * es;
      seg.src[k - 1] = own;  // my term is added last
      seg.dst[0] = own;
      seg.count = hi(c) - lo(c);
      seg.chunk = k - 1;  // a fold over k sources starts at source (chunk + 1) % k = 0
      fold_step(&seg, 1, k, t.dtype, average, stream_, n);
    }
  }
}

// `own`: where this rank's chunk is read from (the chunk itself, or ZeRO-3's shard).
void Engine::staged_all_gather(const Buf& t, const std::vector<Chunk>& cs, const char* own) {
  const int es = elem_bytes(t.dtype), n = size_, r = rank_;
  const int64_t cap = static_cast<int64_t>(staging_half_) / es;
  int64_t longest = 0;
  for (const Chunk& c : cs) longest = std::max(longest, c.numel);
  for (int64_t at = 0; at < longest; at += cap) {
    char* mine = staging_half();
    const int half = static_cast<int>((staged_ops_ - 1) % 2);
    auto part = [&](int c) { return std::max<int64_t>(0, std::min(cap, cs[c].numel - at)); };
    tdm_pair pairs[TDM_MAX_PAIRS];
    int np = 0;
    if (part(r) > 0) {
      pairs[np++] = tdm_pair{mine, own + at * es, part(r)};
      if (own != cs[r].ptr) pairs[np++] = tdm_pair{cs[r].ptr + at * es, own + at * es, part(r)};
    }
    copy_pairs(pairs, np, t.dtype);
    barrier_now(true, fence_tag(4, t.dtype, t.numel));  // every rank's part is in its staging
    np = 0;
    for (int c = 0; c < n; ++c) {
      if (c == r || part(c) == 0) continue;
      pairs[np++] = tdm_pair{cs[c].ptr + at * es, peer_staging(c, half), part(c)};
      if (np == TDM_MAX_PAIRS) {
        copy_pairs(pairs, np, t.dtype);
        np = 0;
      }
    }
    copy_pairs(pairs, np, t.dtype);
  }
}

// ---------------------------------------------------------------- collectives
void Engine::check(const Buf& t, const char* what, bool reduce) const {
  if (t.numel < 0) throw Invalid(std::string(what) + ": negative element count");
  if (t.numel > 0 && t.ptr == nullptr) throw Invalid(std::string(what) + ": NULL tensor");
  const int es = elem_bytes(t.dtype);
  if (reinterpret_cast<uintptr_t>(t.ptr) % es) throw Invalid(std::string(what) + ": pointer not aligned to the element size");
  if (reduce && t.dtype == kBytesDtype) throw Invalid(std::string(what) + ": this dtype can be copied but not reduced");
  if (!connected_) throw std::runtime_error(std::string(what) + ": the engine is not connected");
  if (t.numel > 0) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, t.ptr) != hipSuccess || attr.type != hipMemoryTypeDevice || attr.device != device_) {
      (void)hipGetLastError();
      throw Invalid(std::string(what) + ": the tensor is not in the engine's GPU memory");
    }
  }
}

std::vector<Engine::Chunk> Engine::chunks(const Buf& t, const std::vector<int64_t>& sizes) const {
  std::vector<Chunk> out(size_);
  const int es = elem_bytes(t.dtype);
  if (sizes.empty()) {  // as even as possible, as torch.tensor_split cuts
    const int64_t base = t.numel / size_, extra = t.numel % size_;
    int64_t lo = 0;
    for (int q = 0; q < size_; ++q) {
      const int64_t n = base + (q < extra ? 1 : 0);
      out[q] = Chunk{t.ptr + lo * es, n};
      lo += n;
    }
    return out;
  }
  int64_t total = 0;
  for (int64_t s : sizes) {
    if (s < 0) throw Invalid("chunk sizes do not partition the tensor");
    total += s;
  }
  if (static_cast<int>(sizes.size()) != size_ || total != t.numel) throw Invalid("chunk sizes do not partition the tensor");
  int64_t lo = 0;
  for (int q = 0; q < size_; ++q) {
    out[q] = Chunk{t.ptr + lo * es, sizes[q]};
    lo += sizes[q];
  }
  return out;
}

std::shared_ptr<Work> Engine::all_reduce(Buf t, bool average, hipStream_t caller) {
  check(t, "all_reduce", true);
  if (average && is_integer(t.dtype)) throw Invalid("all_reduce: integer tensors cannot be averaged in place");
  return submit([this, t, average] {
    if (size_ == 1) return;
    if (staged_ && size_ <= TDM_MAX_WORLD) {
      staged_all_reduce(t, average);
      return;
    }
    auto c = chunks(t, {});
    put_tag_ = take_tag_ = piece_tag(1, t.dtype, t.numel);
    ring_reduce_scatter(c, t.dtype, average, false);
    ring_all_gather(c, t.dtype);
  }, caller, true, ready_on_host_);
}

std::shared_ptr<Work> Engine::reduce_scatter(Buf t, std::vector<int64_t> sizes, bool average, bool owner_only,
                                             hipStream_t caller) {
  check(t, "reduce_scatter", true);
  if (average && is_integer(t.dtype)) throw Invalid("reduce_scatter: integer tensors cannot be averaged in place");
  chunks(t, sizes);  // validate now, in the caller's thread
  return submit([this, t, sizes, average, owner_only] {
    if (size_ == 1) return;
    const auto cs = chunks(t, sizes);
    if (staged_ && size_ <= TDM_MAX_WORLD) {
      staged_reduce_scatter(t, cs, average, !owner_only);
    } else {
      put_tag_ = take_tag_ = piece_tag(2, t.dtype, t.numel);
      ring_reduce_scatter(cs, t.dtype, average, true);
    }
  }, caller, true, ready_on_host_);
}

std::shared_ptr<Work> Engine::all_gather(Buf t, std::vector<int64_t> sizes, hipStream_t caller) {
  check(t, "all_gather", false);
  chunks(t, sizes);
  return submit([this, t, sizes] {
    if (size_ == 1) return;
    const auto cs = chunks(t, sizes);
    if (staged_ && size_ < TDM_MAX_PAIRS) {
      staged_all_gather(t, cs, cs[rank_].ptr);
    } else {
      put_tag_ = take_tag_ = piece_tag(3, t.dtype, t.numel);
      ring_all_gather(cs, t.dtype);
    }
  }, caller, true, ready_on_host_);
}

// ZeRO-3's gather of one unit: this rank's shard is placed into its chunk of the
// (so far uninitialised) full buffer and the ring all-gather fills in the rest, all
// on the engine's stream, so the unit arrives while the caller's stream computes
// the previous one (tandem/zero.py:238-245 in the reference).
std::shared_ptr<Work> Engine::unit_gather(Buf full, const char* shard, std::vector<int64_t> sizes, hipStream_t caller) {
  check(full, "unit_gather", false);
  const auto c = chunks(full, sizes);
  if (c[rank_].numel > 0) {
    if (shard == nullptr) throw Invalid("unit_gather: NULL shard");
    check(Buf{const_cast<char*>(shard), c[rank_].numel, full.dtype}, "unit_gather (shard)", false);
  }
  return submit([this, full, shard, sizes] {
    const auto cs = chunks(full, sizes);
    const Chunk& mine = cs[rank_];
    if (size_ > 1 && staged_ && size_ < TDM_MAX_PAIRS) {
      staged_all_gather(full, cs, mine.numel > 0 ? shard : mine.ptr);
      return;
    }
    if (mine.numel > 0 && shard != mine.ptr) {
      if (full.dtype == kBytesDtype) {
        check_hip(hipMemcpyAsync(mine.ptr, shard, static_cast<size_t>(mine.numel), hipMemcpyDeviceToDevice, stream_),
                  "hipMemcpyAsync (unit_gather)");
      } else {
        tdm_pair pr{mine.ptr, shard, mine.numel};
        copy_step(&pr, 1, full.dtype, 0, stream_);
      }
    }
    put_tag_ = take_tag_ = piece_tag(4, full.dtype, full.numel);
    if (size_ > 1) ring_all_gather(cs, full.dtype);
  }, caller, true, ready_on_host_);
}

// Pipelined along the ring from the root: each rank forwards each piece as soon
// as it has it (tandem/comm.py:387-409).
std::shared_ptr<Work> Engine::broadcast(Buf t, int root, hipStream_t caller) {
  check(t, "broadcast", false);
  if (root < 0 || root >= size_) throw Invalid("broadcast: root outside [0, size)");
  return submit([this, t, root] {
    const int n = size_, pos = mod(rank_ - root, n);
    const int nxt = mod(rank_ + 1, n), prv = mod(rank_ - 1, n);
    const int64_t pe = piece_elems(t.dtype);
    const int es = elem_bytes(t.dtype);
    // copies carry bytes: their tags say how many, not of what type (the reference copies a float32 tensor into a uint8 one)
    put_tag_ = take_tag_ = piece_tag(5, 0, (t.numel * es) ^ (static_cast<int64_t>(root) << 40));
    for (int64_t k = 0; k * pe < t.numel; ++k) {
      char* piece = t.ptr + k * pe * es;
      const int64_t m = std::min(pe, t.numel - k * pe);
      if (pos > 0) take(prv, piece, m, t.dtype, false, 0);
      if (pos < n - 1) put(nxt, piece, m, t.dtype, 0);
    }
  }, caller, true, ready_on_host_);
}

std::shared_ptr<Work> Engine::sendrecv(Buf send, int dst, Buf recv, int src, hipStream_t caller) {
  const bool has_send = dst >= 0, has_recv = src >= 0;
  if (has_send) check(send, "send", false);
  if (has_recv) check(recv, "recv", false);
  if (has_send && (dst >= size_ || dst == rank_)) throw Invalid("send: bad destination rank");
  if (has_recv && (src >= size_ || src == rank_)) throw Invalid("recv: bad source rank");
  if (has_send && has_recv && send.dtype != recv.dtype) throw Invalid("sendrecv: the two tensors differ in dtype");
  return submit([this, send, dst, recv, src, has_send, has_recv] {
    Chunk s{send.ptr, send.numel}, r{recv.ptr, recv.numel};
    if (has_send) put_tag_ = piece_tag(6, 0, send.numel * elem_bytes(send.dtype));  // bytes, as for broadcast
    if (has_recv) take_tag_ = piece_tag(6, 0, recv.numel * elem_bytes(recv.dtype));
    exchange(has_send ? &s : nullptr, dst, has_recv ? &r : nullptr, src, has_send ? send.dtype : recv.dtype, false, 0, 0);
  }, caller, true, ready_on_host_);
}

// ---------------------------------------------------------------- shared arena, direct gather
// A rank may keep long-lived data (ZeRO-3's parameter shards) in an arena that its
// peers map once and then read directly: a unit gather is then W-1 copy kernels from
// the peers' arenas on this rank's engine stream, with no staging copy and no
// handshake per gather. The caller brackets every modification of the arena with
// fence(): before (every peer has finished reading) and after (the new contents are
// complete) -- ZeRO-3 changes its shards once per step, and gathers them 27 times.
void* Engine::share(size_t bytes) {
  std::lock_guard<std::mutex> lock(arena_mu_);
  if (arenas_.size() == static_cast<size_t>(kMaxArenas)) throw std::runtime_error("share: this engine already has " + std::to_string(kMaxArenas) + " arenas");
  if (bytes == 0 || bytes >= kArenaLimit) throw Invalid("share: an arena must be between 1 byte and 2 GiB (one IPC allocation)");
  check_hip(hipSetDevice(device_), "hipSetDevice");
  void* arena = nullptr;
  check_hip(hipMalloc(&arena, bytes), "hipMalloc (arena)");
  RegionHeader* h = mine_.header();
  const size_t k = arenas_.size();
  hipError_t err = hipIpcGetMemHandle(&h->arena_mem[k], arena);
  if (err != hipSuccess) {
    (void)hipFree(arena);
    check_hip(err, "hipIpcGetMemHandle (arena)");
  }
  arenas_.push_back(arena);
  arena_sizes_.push_back(bytes);
  h->arena_bytes[k].store(bytes, std::memory_order_release);  // the handle is visible before the size
  return arena;
}

// Where `bytes` bytes at `ptr` lie in this rank's arenas, as the one number its peers name them by; -1: not in any.
int64_t Engine::own_arena_offset(const char* ptr, size_t bytes) {
  std::lock_guard<std::mutex> lock(arena_mu_);
  for (size_t k = 0; k < arenas_.size(); ++k) {
    const char* a = static_cast<const char*>(arenas_[k]);
    if (ptr >= a && ptr + bytes <= a + arena_sizes_[k]) return static_cast<int64_t>((static_cast<uint64_t>(k) << kArenaShift) | static_cast<uint64_t>(ptr - a));
  }
  return -1;
}

// `bytes` bytes at `offset` of the peer's arenas (index and offset in one number), mapped at first use.
const char* Engine::peer_arena(int peer, int64_t offset, size_t bytes) {
  if (offset < 0) throw Invalid("direct: negative arena offset");
  const uint64_t k = static_cast<uint64_t>(offset) >> kArenaShift, at = static_cast<uint64_t>(offset) & (kArenaLimit - 1);
  if (k >= static_cast<uint64_t>(kMaxArenas)) throw Invalid("direct: no such arena");
  std::lock_guard<std::mutex> lock(arena_mu_);
  if (!peer_arena_[peer][k]) {
    RegionHeader* h = theirs_[peer]->header();
    const uint64_t size = h->arena_bytes[k].load(std::memory_order_acquire);
    if (size == 0) throw std::runtime_error("direct: rank " + std::to_string(peer) + " has not shared arena " + std::to_string(k));
    check_hip(hipIpcOpenMemHandle(&peer_arena_[peer][k], h->arena_mem[k], hipIpcMemLazyEnablePeerAccess), "hipIpcOpenMemHandle (arena)");
    peer_arena_bytes_[peer][k] = size;
  }
  if (at + bytes > peer_arena_bytes_[peer][k]) throw Invalid("direct: the range lies outside rank " + std::to_string(peer) + "'s arena");
  return static_cast<const char*>(peer_arena_[peer][k]) + at;
}

// Launched by the caller's thread: a direct gather exchanges no message with any
// rank, so it need not take its turn behind collectives whose hand-overs the progress
// thread is waiting for, and the caller never blocks on it. By default the copies go
// onto the caller's own stream, in order with its kernels: the copy of a 28 MB unit
// takes tens of microseconds at HBM speed, while running it on a side stream (the
// reference's design, TANDEM_HIP_GATHER=stream) costs two cross-queue waits per gather,
// which on a GPU shared by several processes were measured to cost more than they hide
// (85.8M GPT, 2 ranks: 26.7 ms per step in order, 29-34 ms on the side stream).
std::shared_ptr<Work> Engine::unit_gather_direct(Buf full, const char* shard, std::vector<int64_t> sizes,
                                                 std::vector<int64_t> peer_offsets, hipStream_t caller) {
  check(full, "unit_gather", false);
  if (full.dtype == kBytesDtype) throw Invalid("unit_gather: direct gathers need a typed tensor");
  const auto cs = chunks(full, sizes);
  if (static_cast<int>(peer_offsets.size()) != size_) throw Invalid("unit_gather: one arena offset per rank");
  if (cs[rank_].numel > 0 && shard == nullptr) throw Invalid("unit_gather: NULL shard");
  {
    std::lock_guard<std::mutex> lock(mu_);
    if (stopping_) throw std::runtime_error("the engine is closed");
  }
  const int es = elem_bytes(full.dtype);
  tdm_pair pairs[TDM_MAX_PAIRS * 2];
  int np = 0;
  for (int q = 0; q < size_; ++q) {
    if (cs[q].numel == 0) continue;
    const char* from;
    if (q == rank_) {
      if (shard == cs[q].ptr) continue;
      from = shard;
    } else {
      if (peer_offsets[q] < 0 || peer_offsets[q] % es) throw Invalid("unit_gather: bad arena offset");
      from = peer_arena(q, peer_offsets[q], static_cast<size_t>(cs[q].numel) * es);
    }
    if (np == TDM_MAX_PAIRS * 2) throw Invalid("unit_gather: too many ranks");
    pairs[np++] = tdm_pair{cs[q].ptr, from, cs[q].numel};
  }
  auto work = std::make_shared<Work>();
  work->device = device_;
  work->uses_gpu = true;
  work->t0 = now_s();
  check_hip(hipSetDevice(device_), "hipSetDevice");
  hipStream_t on = caller;
  if (gathers_on_side_stream_) {
    // Start once the caller's stream has produced the buffer (and finished with its last use): the side stream waits
    // for an event recorded on the caller's stream, taken from a ring made at start-up (no create and destroy per
    // gather). A value word would do too (TANDEM_HIP_GATHER=stream-words: the caller's stream writes it, the side
    // stream waits for it), but on this runtime a stream waits for a value with a kernel that spins, and with prefetch
    // the side stream waits for most of a block's compute: twelve milliseconds of spinning per step, during which the
    // matrix kernels beside it ran 11 % slower. The END of a gather is a value word either way (below): by the time the
    // caller needs the unit the word is usually there and no wait is queued at all.
    on = gather_stream_;
    bool ordered = false;
    if (flags_ && gather_ready_ == GatherReady::kWord) {
      uint32_t value = 0;
      const int word = flags_->acquire(&value);
      if (word >= 0) {
        hipError_t err = hipStreamWriteValue32(caller, flags_->base + word, value, 0);
        if (err == hipSuccess) {
          err = hipStreamWaitValue32(gather_stream_, flags_->base + word, value, hipStreamWaitValueGte, 0xffffffffu);
        } else {
          flags_->set(word, value);  // nothing will write it: it must not be handed out as pending for ever
        }
        flags_->release(word);  // stays out of circulation until the caller's stream has written it
        check_hip(err, "ordering a gather after the caller's stream (value)");
        ordered = true;
      }
    }
    if (!ordered && gather_ready_ != GatherReady::kFreshEvent && !ready_events_.empty()) {
      // An event out of a ring made at start-up: a wait takes the event's latest record at the time of the call, so
      // recording it again for a later gather does not disturb a wait still queued (and the ring is far longer than
      // the two or three gathers that are ever in flight).
      hipEvent_t ready = ready_events_[ready_next_.fetch_add(1, std::memory_order_relaxed) % ready_events_.size()];
      hipError_t err = hipEventRecord(ready, caller);
      if (err == hipSuccess) err = hipStreamWaitEvent(gather_stream_, ready, 0);
      check_hip(err, "ordering a gather after the caller's stream (event)");
      ordered = true;
    }
    if (!ordered) {
      hipEvent_t ready;
      check_hip(hipEventCreateWithFlags(&ready, hipEventDisableTiming), "hipEventCreateWithFlags (ready)");
      hipError_t err = hipEventRecord(ready, caller);
      if (err == hipSuccess) err = hipStreamWaitEvent(gather_stream_, ready, 0);
      (void)hipEventDestroy(ready);
      check_hip(err, "ordering a gather after the caller's stream");
    }
  }
  stamp_start(*work, on);
  for (int at = 0; at < np; at += TDM_MAX_PAIRS) {
    copy_step(pairs + at, std::min<int>(TDM_MAX_PAIRS, np - at), full.dtype, 0, on);
  }
  // Its end. On the side stream: the Work's own word, written by that stream behind the last copy, which wait() parks
  // the caller's stream on and done() reads (as for every collective of the progress thread). On the caller's own
  // stream nothing needs ordering afterwards: wait() finds the Work on the stream it would wait on. An event is
  // recorded only where there is no word, for done() on the caller's own stream, and for the time stamps.
  if (gathers_on_side_stream_ && flags_ && gather_done_word_) {
    work->flag = flags_->acquire(&work->flag_value);
    if (work->flag >= 0) {
      work->flags = flags_;
      const hipError_t err = hipStreamWriteValue32(gather_stream_, flags_->base + work->flag, work->flag_value, 0);
      if (err != hipSuccess) {  // no word after all (the Work gives it back); the event below takes its place
        flags_->set(work->flag, work->flag_value);
        flags_->release(work->flag);
        work->flag = -1;
        work->flags.reset();
        (void)hipGetLastError();
      }
    }
  }
  if (work->flag < 0 || work->start_event) {
    check_hip(hipEventCreateWithFlags(&work->done_event, work->start_event ? hipEventDefault : hipEventDisableTiming),
              "hipEventCreateWithFlags (done)");
    check_hip(hipEventRecord(work->done_event, on), "hipEventRecord (done)");
  }
  work->on_callers_stream = !gathers_on_side_stream_;
  work->launched_on = on;
  work->t1 = now_s();
  work->finished = true;
  work->finished_hint.store(true, std::memory_order_release);
  return work;
}

// ---------------------------------------------------------------- direct collectives
// For tensors that live in the ranks' shared arenas. No slots and no per-piece
// messages: a rank reads its peers' tensors where they lie.
//   all_reduce      fence; fold my chunk out of all ranks' tensors, in the ring's order
//                   for that chunk, into every rank's tensor (one kernel, W reads and W
//                   writes per element of the chunk); fence.
//   reduce_scatter  fence; the same fold into my tensor only; fence. Only the owner's
//                   chunk is produced.
//   all_gather      fence; copy every other chunk from its owner's tensor; fence.
// Per rank and element of the tensor that is 2 accesses for an all-reduce where the
// slot ring makes 9(W-1)/W, and two handshakes in all instead of two per piece. The
// first fence says every rank's input is complete, the last that nobody reads or
// writes a tensor any more, so the caller may change it again.
void Engine::direct_bases(const Buf& t, const std::vector<int64_t>& peer_offsets, const char** base) {
  const int es = elem_bytes(t.dtype);
  const size_t bytes = static_cast<size_t>(t.numel) * es;
  if (own_arena_offset(t.ptr, bytes) < 0) throw Invalid("direct collective: the tensor does not lie in one of this rank's shared arenas");
  for (int q = 0; q < size_; ++q) {
    if (q == rank_) {
      base[q] = t.ptr;
      continue;
    }
    if (peer_offsets[q] < 0 || peer_offsets[q] % es) throw Invalid("direct collective: bad arena offset");
    base[q] = peer_arena(q, peer_offsets[q], bytes);
  }
}

// to_all: the folded chunk is also written into every peer's tensor (their arenas are mapped writable). Chunk r of
// every rank's tensor is read and written by rank r's kernel alone, so the ranks' kernels need no order among them.
void Engine::direct_fold(const Buf& t, const std::vector<Chunk>& cs, const char* const* base, bool average, bool to_all) {
  const Chunk& mine = cs[rank_];
  if (mine.numel == 0) return;
  tdm_fold_seg seg;
  std::memset(&seg, 0, sizeof seg);
  const size_t lo = static_cast<size_t>(mine.ptr - t.ptr);
  for (int q = 0; q < size_; ++q) seg.src[q] = base[q] + lo;
  if (to_all) {
    for (int q = 0; q < size_; ++q) seg.dst[q] = const_cast<char*>(base[q]) + lo;
  }
  seg.dst[rank_] = mine.ptr;
  seg.count = mine.numel;
  seg.chunk = rank_;
  fold_step(&seg, 1, size_, t.dtype, average, stream_);
}

void Engine::direct_copies(const Buf& t, const std::vector<Chunk>& cs, const char* const* base) {
  tdm_pair pairs[TDM_MAX_PAIRS];
  int np = 0;
  for (int q = 0; q < size_; ++q) {
    if (q == rank_ || cs[q].numel == 0) continue;
    pairs[np++] = tdm_pair{cs[q].ptr, base[q] + (cs[q].ptr - t.ptr), cs[q].numel};
    if (np == TDM_MAX_PAIRS) {
      copy_step(pairs, np, t.dtype, 0, stream_);
      np = 0;
    }
  }
  if (np) copy_step(pairs, np, t.dtype, 0, stream_);
}

std::shared_ptr<Work> Engine::direct(int kind, Buf t, std::vector<int64_t> sizes, bool average,
                                     std::vector<int64_t> peer_offsets, hipStream_t caller) {
  const char* what = kind == 0 ? "all_reduce (direct)" : kind == 1 ? "reduce_scatter (direct)" : "all_gather (direct)";
  check(t, what, kind != 2);
  if (t.dtype == kBytesDtype) throw Invalid(std::string(what) + ": needs a typed tensor");
  if (kind != 2 && average && is_integer(t.dtype)) {
    throw Invalid(std::string(what) + ": integer tensors cannot be averaged in place");
  }
  if (kind != 2 && size_ > TDM_MAX_WORLD) throw Invalid(std::string(what) + ": the direct fold handles world sizes up to 8");
  if (static_cast<int>(peer_offsets.size()) != size_) throw Invalid(std::string(what) + ": one arena offset per rank");
  chunks(t, sizes);  // validate now, in the caller's thread
  return submit([this, kind, t, sizes, average, peer_offsets] {
    if (size_ == 1) return;
    const auto cs = chunks(t, sizes);
    const char* base[TDM_MAX_PAIRS > TDM_MAX_WORLD ? TDM_MAX_PAIRS : TDM_MAX_WORLD];
    if (size_ > static_cast<int>(sizeof base / sizeof base[0])) throw Invalid("direct collective: too many ranks");
    barrier_now(true, fence_tag(5 + kind, t.dtype, t.numel));  // every rank's input is complete
    // The peers' arenas are looked up behind the first fence: a rank that has reached it has shared its
    // arena, so the first direct collective of a group needs no barrier of the caller's before it.
    if (t.numel > 0) direct_bases(t, peer_offsets, base);  // an empty tensor still takes part in the fences
    if (kind == 2) direct_copies(t, cs, base);
    else direct_fold(t, cs, base, average, kind == 0);  // all_reduce: every rank's copy of my chunk written by my fold
    barrier_now(true);  // nobody reads or writes our tensor any more
  }, caller, true, true, true);
}

// ZeRO stage 2's communication and optimizer step in one launch per rank, for gradient
// and parameter buffers that live in the arenas: fence (every rank's gradients are
// complete, and no rank still computes with the old parameters); this rank folds its
// shard's gradients out of all ranks' buffers in the ring's order, takes the AdamW step
// and writes the new parameters into every rank's buffer; fence (every rank's writes have
// landed). Replaces a reduce_scatter per bucket, grad_shard.add_, the update and the
// all_gather (tandem/zero.py:141-163) with (8W + 20) bytes per element of the shard.
std::shared_ptr<Work> Engine::zero2_step_direct(Buf param, Buf grad, std::vector<int64_t> param_offsets,
                                                std::vector<int64_t> grad_offsets, char* exp_avg, char* exp_avg_sq,
                                                int64_t total, bool average, const tdm_adamw_scalars* s_in,
                                                const tdm_adamw_hyper* h_in, int order, hipStream_t caller) {
  const char* what = "zero2_step (direct)";
  check(param, what, true);
  check(grad, what, true);
  if ((s_in == nullptr) == (h_in == nullptr)) throw Invalid(std::string(what) + ": the step's constants as fp32 or as doubles, one of the two");
  const int dtype = param.dtype;
  if (dtype != grad.dtype) throw Invalid(std::string(what) + ": parameters and gradients differ in dtype");
  if (s_in != nullptr && dtype != TDM_F32) throw Invalid(std::string(what) + ": fp32 constants go with fp32 buffers");
  if (dtype != TDM_F32 && dtype != TDM_F64 && dtype != TDM_BF16 && dtype != TDM_F16) {
    throw Invalid(std::string(what) + ": fp32, fp64, bf16 or fp16 buffers");
  }
  if (param.numel != grad.numel) throw Invalid(std::string(what) + ": parameters and gradients differ in length");
  if (size_ > TDM_MAX_WORLD) throw Invalid(std::string(what) + ": world sizes up to 8");
  if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid(std::string(what) + ": unknown update order");
  if (dtype != TDM_F32 && order != TDM_ADAMW_HOST_ORDER) throw Invalid(std::string(what) + ": the device order is defined for fp32 shards only");
  if (static_cast<int>(param_offsets.size()) != size_ || static_cast<int>(grad_offsets.size()) != size_) {
    throw Invalid(std::string(what) + ": one arena offset per rank");
  }
  if (param.numel > 0) {
    if (!exp_avg || !exp_avg_sq) throw Invalid(std::string(what) + ": NULL optimizer state");
    check(Buf{exp_avg, param.numel, dtype}, what, false);
    check(Buf{exp_avg_sq, param.numel, dtype}, what, false);
  }
  const bool typed = h_in != nullptr;
  const tdm_adamw_scalars s = typed ? tdm_adamw_scalars{} : *s_in;
  const tdm_adamw_hyper h = typed ? *h_in : tdm_adamw_hyper{};
  return submit([this, param, grad, param_offsets, grad_offsets, exp_avg, exp_avg_sq, total, average, s, h, typed, dtype, order] {
    tdm_step_seg seg;
    std::memset(&seg, 0, sizeof seg);
    seg.dtype = dtype;
    if (size_ > 1) barrier_now(true, fence_tag(9, dtype, total));
    if (param.numel > 0) {  // a rank with an empty shard still takes part in the fences
      const char* base[TDM_MAX_WORLD];
      direct_bases(grad, grad_offsets, base);
      for (int q = 0; q < size_; ++q) seg.grad[q] = base[q];
      direct_bases(param, param_offsets, base);
      for (int q = 0; q < size_; ++q) seg.param[q] = const_cast<char*>(base[q]);  // the peers' arenas are mapped writable
      seg.exp_avg = exp_avg;
      seg.exp_avg_sq = exp_avg_sq;
      seg.count = param.numel;
      seg.chunk = rank_;
    }
    if (typed) zero2_step_segment_typed(seg, size_, average, h, order, stream_);
    else zero2_step_segment(seg, size_, average, s, order, stream_);
    if (size_ > 1) barrier_now(true);
  }, caller, true, true, true);
}

// A barrier that is also ordered against the GPU: it starts after the caller's
// stream has finished what it held at the call, and a rank's arrival is only
// announced once its engine stream has finished too.
std::shared_ptr<Work> Engine::fence(hipStream_t caller) {
  if (!connected_) throw std::runtime_error("fence: the engine is not connected");
  return submit([this] { barrier_now(true); }, caller, true, true, true);
}

std::shared_ptr<Work> Engine::barrier() {
  if (!connected_) throw std::runtime_error("barrier: the engine is not connected");
  return submit([this] { barrier_now(); }, nullptr, false);
}

}  // namespace tandem_hip
