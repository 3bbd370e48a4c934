// The C ABI of the process-rank engine (include/tandem_hip.h): argument checks, error codes, handles.

#include "engine.h"

// ---------------------------------------------------------------- C ABI
using namespace tandem_hip;

struct tdm_engine {
  std::unique_ptr<Engine> impl;
};

struct tdm_work {
  std::shared_ptr<Work> impl;
};

namespace {

int finish_submit(std::shared_ptr<Work> w, tdm_work** out) {
  auto* handle = new tdm_work{std::move(w)};
  *out = handle;
  return TDM_OK;
}

Engine& engine_of(tdm_engine* e) {
  if (e == nullptr || !e->impl) throw Invalid("NULL engine");
  return *e->impl;
}

}  // namespace

extern "C" {

int tdm_engine_create(const char* job, int rank, int size, int slots, int64_t slot_bytes, double timeout_s, int device,
                      tdm_engine** out) {
  return guard([&] {
    if (job == nullptr || out == nullptr) throw Invalid("NULL argument");
    if (slot_bytes <= 0) throw Invalid("slot_bytes must be positive");
    auto e = std::make_unique<Engine>(job, rank, size, slots, static_cast<size_t>(slot_bytes), timeout_s, device);
    *out = new tdm_engine{std::move(e)};
  });
}

int tdm_engine_connect(tdm_engine* e) {
  return guard([&] { engine_of(e).connect(); });
}

int tdm_engine_close(tdm_engine* e) {
  return guard([&] { engine_of(e).close(); });
}

int tdm_engine_destroy(tdm_engine* e) {
  return guard([&] { delete e; });
}

int tdm_all_reduce(tdm_engine* e, void* ptr, int64_t numel, int dtype, int average, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    finish_submit(engine_of(e).all_reduce(Engine::Buf{static_cast<char*>(ptr), numel, dtype}, average != 0,
                                          static_cast<hipStream_t>(caller)), out);
  });
}

namespace {
int reduce_scatter_call(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, int average,
                        bool owner_only, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    if (nsizes < 0 || (nsizes > 0 && sizes == nullptr)) throw Invalid("bad sizes");
    std::vector<int64_t> sz(sizes, sizes + nsizes);
    finish_submit(engine_of(e).reduce_scatter(Engine::Buf{static_cast<char*>(ptr), numel, dtype}, std::move(sz),
                                              average != 0, owner_only, static_cast<hipStream_t>(caller)), out);
  });
}
}  // namespace

int tdm_reduce_scatter(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, int average,
                       tdm_stream caller, tdm_work** out) {
  return reduce_scatter_call(e, ptr, numel, dtype, sizes, nsizes, average, false, caller, out);
}

int tdm_reduce_scatter_owner(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, int average,
                             tdm_stream caller, tdm_work** out) {
  return reduce_scatter_call(e, ptr, numel, dtype, sizes, nsizes, average, true, caller, out);
}

int tdm_all_gather(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, tdm_stream caller,
                   tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    if (nsizes < 0 || (nsizes > 0 && sizes == nullptr)) throw Invalid("bad sizes");
    std::vector<int64_t> sz(sizes, sizes + nsizes);
    finish_submit(engine_of(e).all_gather(Engine::Buf{static_cast<char*>(ptr), numel, dtype}, std::move(sz),
                                          static_cast<hipStream_t>(caller)), out);
  });
}

int tdm_unit_gather(tdm_engine* e, void* full, int64_t numel, int dtype, const void* shard, const int64_t* sizes, int nsizes,
                    tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    if (nsizes < 0 || (nsizes > 0 && sizes == nullptr)) throw Invalid("bad sizes");
    std::vector<int64_t> sz(sizes, sizes + nsizes);
    finish_submit(engine_of(e).unit_gather(Engine::Buf{static_cast<char*>(full), numel, dtype},
                                           static_cast<const char*>(shard), std::move(sz),
                                           static_cast<hipStream_t>(caller)), out);
  });
}

int tdm_broadcast(tdm_engine* e, void* ptr, int64_t numel, int dtype, int root, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    finish_submit(engine_of(e).broadcast(Engine::Buf{static_cast<char*>(ptr), numel, dtype}, root,
                                         static_cast<hipStream_t>(caller)), out);
  });
}

int tdm_sendrecv(tdm_engine* e, const void* send, int64_t send_numel, int dst, void* recv, int64_t recv_numel, int src,
                 int dtype, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    finish_submit(engine_of(e).sendrecv(Engine::Buf{static_cast<char*>(const_cast<void*>(send)), send_numel, dtype}, dst,
                                        Engine::Buf{static_cast<char*>(recv), recv_numel, dtype}, src,
                                        static_cast<hipStream_t>(caller)), out);
  });
}

int tdm_engine_share(tdm_engine* e, int64_t bytes, void** ptr) {
  return guard([&] {
    if (ptr == nullptr || bytes <= 0) throw Invalid("share: bad arguments");
    *ptr = engine_of(e).share(static_cast<size_t>(bytes));
  });
}

int tdm_engine_arena_offset(tdm_engine* e, const void* ptr, int64_t bytes, int64_t* offset) {
  return guard([&] {
    if (offset == nullptr || bytes < 0 || (ptr == nullptr && bytes > 0)) throw Invalid("arena_offset: bad arguments");
    *offset = engine_of(e).own_arena_offset(static_cast<const char*>(ptr), static_cast<size_t>(bytes));
  });
}

int tdm_unit_gather_direct(tdm_engine* e, void* full, int64_t numel, int dtype, const void* shard, const int64_t* sizes,
                           int nsizes, const int64_t* peer_offsets, int noffsets, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    if (nsizes < 0 || (nsizes > 0 && sizes == nullptr) || noffsets < 0 || (noffsets > 0 && peer_offsets == nullptr)) {
      throw Invalid("bad sizes or offsets");
    }
    std::vector<int64_t> sz(sizes, sizes + nsizes), off(peer_offsets, peer_offsets + noffsets);
    finish_submit(engine_of(e).unit_gather_direct(Engine::Buf{static_cast<char*>(full), numel, dtype},
                                                  static_cast<const char*>(shard), std::move(sz), std::move(off),
                                                  static_cast<hipStream_t>(caller)), out);
  });
}

namespace {
int direct_call(tdm_engine* e, int kind, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, int average,
                const int64_t* peer_offsets, int noffsets, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    if (nsizes < 0 || (nsizes > 0 && sizes == nullptr) || noffsets < 0 || (noffsets > 0 && peer_offsets == nullptr)) {
      throw Invalid("bad sizes or offsets");
    }
    std::vector<int64_t> sz(sizes, sizes + nsizes), off(peer_offsets, peer_offsets + noffsets);
    finish_submit(engine_of(e).direct(kind, Engine::Buf{static_cast<char*>(ptr), numel, dtype}, std::move(sz), average != 0,
                                      std::move(off), static_cast<hipStream_t>(caller)), out);
  });
}
}  // namespace

int tdm_direct_all_reduce(tdm_engine* e, void* ptr, int64_t numel, int dtype, int average, const int64_t* peer_offsets,
                          int noffsets, tdm_stream caller, tdm_work** out) {
  return direct_call(e, 0, ptr, numel, dtype, nullptr, 0, average, peer_offsets, noffsets, caller, out);
}

int tdm_direct_reduce_scatter(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                              int average, const int64_t* peer_offsets, int noffsets, tdm_stream caller, tdm_work** out) {
  return direct_call(e, 1, ptr, numel, dtype, sizes, nsizes, average, peer_offsets, noffsets, caller, out);
}

int tdm_direct_all_gather(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                          const int64_t* peer_offsets, int noffsets, tdm_stream caller, tdm_work** out) {
  return direct_call(e, 2, ptr, numel, dtype, sizes, nsizes, 0, peer_offsets, noffsets, caller, out);
}

namespace {
int direct_zero2_step(tdm_engine* e, void* param, const int64_t* param_offsets, const void* grad, const int64_t* grad_offsets,
                      int noffsets, void* exp_avg, void* exp_avg_sq, int64_t count, int64_t total, int average, int dtype,
                      const tdm_adamw_scalars* s, const tdm_adamw_hyper* h, int order, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    if (s == nullptr && h == nullptr) throw Invalid("NULL constants");
    if (noffsets < 0 || (noffsets > 0 && (param_offsets == nullptr || grad_offsets == nullptr))) throw Invalid("bad offsets argument");
    std::vector<int64_t> po(param_offsets, param_offsets + noffsets), go(grad_offsets, grad_offsets + noffsets);
    finish_submit(engine_of(e).zero2_step_direct(Engine::Buf{static_cast<char*>(param), count, dtype},
                                                 Engine::Buf{static_cast<char*>(const_cast<void*>(grad)), count, dtype},
                                                 std::move(po), std::move(go), static_cast<char*>(exp_avg),
                                                 static_cast<char*>(exp_avg_sq), total, average != 0, s, h, order,
                                                 static_cast<hipStream_t>(caller)),
                  out);
  });
}
}  // namespace

int tdm_direct_zero2_step(tdm_engine* e, void* param, const int64_t* param_offsets, const void* grad, const int64_t* grad_offsets,
                          int noffsets, void* exp_avg, void* exp_avg_sq, int64_t count, int64_t total, int average,
                          const tdm_adamw_scalars* s, int order, tdm_stream caller, tdm_work** out) {
  if (s == nullptr) return guard([] { throw Invalid("NULL scalars"); });
  return direct_zero2_step(e, param, param_offsets, grad, grad_offsets, noffsets, exp_avg, exp_avg_sq, count, total, average, TDM_F32, s,
                           nullptr, order, caller, out);
}

int tdm_direct_zero2_step_typed(tdm_engine* e, void* param, const int64_t* param_offsets, const void* grad, const int64_t* grad_offsets,
                                int noffsets, void* exp_avg, void* exp_avg_sq, int64_t count, int64_t total, int average, int dtype,
                                const tdm_adamw_hyper* h, int order, tdm_stream caller, tdm_work** out) {
  if (h == nullptr) return guard([] { throw Invalid("NULL constants"); });
  return direct_zero2_step(e, param, param_offsets, grad, grad_offsets, noffsets, exp_avg, exp_avg_sq, count, total, average, dtype,
                           nullptr, h, order, caller, out);
}

int tdm_fence(tdm_engine* e, tdm_stream caller, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    finish_submit(engine_of(e).fence(static_cast<hipStream_t>(caller)), out);
  });
}

int tdm_barrier(tdm_engine* e, tdm_work** out) {
  return guard([&] {
    if (out == nullptr) throw Invalid("NULL work pointer");
    finish_submit(engine_of(e).barrier(), out);
  });
}

static int wait_for(tdm_work* w, tdm_stream caller, bool may_park);

int tdm_work_wait(tdm_work* w, tdm_stream caller) { return wait_for(w, caller, w && w->impl && w->impl->defer_default); }

int tdm_work_wait_stream(tdm_work* w, tdm_stream caller) { return wait_for(w, caller, true); }

// may_park: a collective that has not run yet is not waited for on the host; the caller's stream is parked on its word.
static int wait_for(tdm_work* w, tdm_stream caller, bool may_park) {
  if (w == nullptr || !w->impl) {
    set_last_error("NULL work");
    return TDM_EINVAL;
  }
  Work& work = *w->impl;
  if (work.flags && work.flags->gave_up()) {
    set_last_error("a stream parked on a collective gave up waiting for its end: what that stream computed since is not to be trusted");
    return TDM_ERUNTIME;
  }
  if (may_park && work.may_park && work.flag >= 0 && !work.finished_hint.load(std::memory_order_acquire)) {
    // The job has not run yet: park the caller's stream on its word and return. The host
    // goes on queueing work behind the collective; a failure shows at the next call.
    // The wait is a kernel of the library's own with a time limit: it is queued before the write that ends it, and
    // should that write never run the stream goes on by itself and the next call on the engine says so.
    return guard([&] {
      int current = -1;  // a kernel launch wants the stream's device current; the caller's choice is put back
      check_hip(hipGetDevice(&current), "hipGetDevice");
      if (current != work.device) check_hip(hipSetDevice(work.device), "hipSetDevice");
      try {
        park_stream(static_cast<hipStream_t>(caller), work.flags->base + work.flag, work.flag_value, work.park_limit_s,
                    work.flags->gave_up_word());
      } catch (...) {
        if (current != work.device) (void)hipSetDevice(current);
        throw;
      }
      if (current != work.device) check_hip(hipSetDevice(current), "hipSetDevice");
    });
  }
  spin_for([&] { return work.finished_hint.load(std::memory_order_acquire); });
  {
    std::unique_lock<std::mutex> lock(work.mu);
    work.cv.wait(lock, [&] { return work.finished; });
    if (work.status != TDM_OK) {
      set_last_error(work.error);
      return work.status;
    }
  }
  if (work.on_callers_stream && work.launched_on == static_cast<hipStream_t>(caller)) return TDM_OK;
  if (work.flag >= 0) {
    if (work.flags->reached(work.flag, work.flag_value)) return TDM_OK;  // the GPU is past it already: nothing to order
    return guard([&] {
      check_hip(hipStreamWaitValue32(static_cast<hipStream_t>(caller), work.flags->base + work.flag, work.flag_value,
                                     hipStreamWaitValueGte, 0xffffffffu),
                "hipStreamWaitValue32 (wait)");
    });
  }
  if (work.done_event) {
    return guard([&] {
      const hipError_t q = hipEventQuery(work.done_event);
      if (q == hipSuccess) return;
      if (q == hipErrorNotReady) (void)hipGetLastError();
      check_hip(hipStreamWaitEvent(static_cast<hipStream_t>(caller), work.done_event, 0), "hipStreamWaitEvent (wait)");
    });
  }
  return TDM_OK;
}

int tdm_work_done(tdm_work* w) {
  if (w == nullptr || !w->impl) return 0;
  Work& work = *w->impl;
  // The word is written behind the job's last kernel (or by the host, after a failure): it may be there a moment before the
  // progress thread has marked the job as run, and a caller whose stream was let go by it must not be told "not yet".
  if (work.flag >= 0) return work.flags->reached(work.flag, work.flag_value) ? 1 : 0;
  std::lock_guard<std::mutex> lock(work.mu);
  if (!work.finished) return 0;
  if (work.status != TDM_OK) return 1;
  if (work.done_event) return hipEventQuery(work.done_event) == hipSuccess ? 1 : 0;
  return 1;
}

int tdm_work_times(tdm_work* w, double* started, double* finished) {
  if (w == nullptr || !w->impl) {
    set_last_error("NULL work");
    return TDM_EINVAL;
  }
  Work& work = *w->impl;
  {
    std::unique_lock<std::mutex> lock(work.mu);
    work.cv.wait(lock, [&] { return work.finished; });
    if (started) *started = work.t0;
    if (finished) *finished = work.t1;
    if (work.status != TDM_OK || !work.start_event || !work.done_event || !work.anchor) return TDM_OK;
  }
  // Timed on the device: wait for its last kernel, then place both stamps on the host clock.
  return guard([&] {
    check_hip(hipEventSynchronize(work.done_event), "hipEventSynchronize (times)");
    float ms0 = 0, ms1 = 0;
    check_hip(hipEventElapsedTime(&ms0, work.anchor->event, work.start_event), "hipEventElapsedTime (start)");
    check_hip(hipEventElapsedTime(&ms1, work.anchor->event, work.done_event), "hipEventElapsedTime (done)");
    if (started) *started = work.anchor->host + static_cast<double>(ms0) * 1e-3;
    if (finished) *finished = work.anchor->host + static_cast<double>(ms1) * 1e-3;
  });
}

int tdm_engine_set_timing(tdm_engine* e, int on) {
  if (e == nullptr || !e->impl) {
    set_last_error("NULL engine");
    return TDM_EINVAL;
  }
  e->impl->set_timing(on != 0);
  return TDM_OK;
}

int tdm_work_free(tdm_work* w) {
  delete w;
  return TDM_OK;
}

}  // extern "C"
