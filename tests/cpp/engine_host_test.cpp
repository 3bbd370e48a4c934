// The process-rank engine's host side on a machine without a GPU: W processes, each with an engine built from the very
// sources of the library (engine.hip, engine_abi.hip, abi.hip) against a stand-in runtime (fake_hip.cpp) and stand-in
// kernels (fake_kernels.cpp), run the collectives through the C ABI and check where every element ended up. What this
// sees that the GPU tests do not: the engine's threads (caller, progress, completion) and the stand-in's stream threads
// under the host's sanitizers for data races, addresses and undefined behaviour. A dependency between two streams that
// the engine forgot (the collective on the caller's producer, the caller's consumer on the collective) is a data race
// between those threads and is reported as one. Numbers are integer-valued, so sums are exact in any order; the
// order of the sums is the GPU tests' business.
//
// usage: engine_host_test <world> <staged|ring> [staging_bytes|0] [-|dies|out_of_step|no_ipc_events] [NAME=VALUE,...]
//   the last argument: environment variables the engine reads (TANDEM_HIP_GATHER=stream and the like)
//   dies:        the last rank leaves right after connecting; the others' collective must time out, later calls must fail
//                at once, close must come back
//   out_of_step: rank 0 brings a tensor of another length than the others; every rank must be told

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/wait.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../include/tandem_hip.h"
#include "fake_hip.h"

#define REQUIRE(cond)                                                                                     \
  do {                                                                                                    \
    if (!(cond)) {                                                                                        \
      std::fprintf(stderr, "rank %d: %s:%d: %s failed (%s)\n", g_rank, __FILE__, __LINE__, #cond, tdm_last_error()); \
      return 1;                                                                                           \
    }                                                                                                     \
  } while (0)

static int g_rank = -1;

static float value(int rank, int64_t i, int salt) { return static_cast<float>((rank + 1) * ((i + salt) % 13) - salt % 5); }

static std::vector<int64_t> split(int64_t n, int w, bool uneven) {
  std::vector<int64_t> s(w);
  for (int q = 0; q < w; ++q) s[q] = n / w + (q < n % w ? 1 : 0);
  if (uneven && w > 1) {  // one empty chunk, its elements given to the next rank
    s[1 % w] += s[0];
    s[0] = 0;
  }
  return s;
}

// What must happen when the group falls apart: an error with a message on every rank that is still there, no hang.
static int run_broken(tdm_engine* e, int rank, int world, const std::string& scenario) {
  if (scenario == "dies" && rank == world - 1) ::_exit(0);  // without closing: its peers find nobody
  std::vector<float> x(scenario == "out_of_step" && rank == 0 ? 1000 : 1001, 1.0f);
  tdm_work* w = nullptr;
  REQUIRE(tdm_all_reduce(e, x.data(), static_cast<int64_t>(x.size()), TDM_F32, 0, nullptr, &w) == TDM_OK);
  const int rc = tdm_work_wait(w, nullptr);
  const std::string said = tdm_last_error();
  REQUIRE(rc != TDM_OK && !said.empty());
  // a neighbour of the rank that left times out; a rank further along the ring may instead be reached by the closing
  // barrier of one that already has, where it expected a piece
  if (scenario == "dies") REQUIRE(rc == TDM_ETIMEOUT || said.find("out of step") != std::string::npos);
  REQUIRE(tdm_work_done(w) == 1 && tdm_work_free(w) == TDM_OK);
  REQUIRE(tdm_all_reduce(e, x.data(), static_cast<int64_t>(x.size()), TDM_F32, 0, nullptr, &w) != TDM_OK);  // the engine remembers
  REQUIRE(std::string(tdm_last_error()).find("earlier collective failed") != std::string::npos);
  (void)tdm_engine_close(e);  // its barrier may fail as well; it must return
  REQUIRE(tdm_engine_destroy(e) == TDM_OK);
  return 0;
}

// A stream parked on a collective whose end does not come in time gives up by itself (TANDEM_HIP_PARK_LIMIT_S, here a
// twentieth of a second; the peers come 300 ms late), and the next call on the engine says so. The collective itself
// still runs when the peers arrive: they are not to be left waiting for this rank.
static int run_park_gives_up(tdm_engine* e, int rank, int world) {
  hipStream_t caller = nullptr;
  REQUIRE(hipStreamCreateWithFlags(&caller, hipStreamNonBlocking) == hipSuccess);
  std::vector<float> x(1000, static_cast<float>(rank + 1));
  tdm_work* w = nullptr;
  if (rank != 0) std::this_thread::sleep_for(std::chrono::milliseconds(300));
  REQUIRE(tdm_all_reduce(e, x.data(), 1000, TDM_F32, 0, caller, &w) == TDM_OK);
  if (rank == 0) {
    const auto began = std::chrono::steady_clock::now();
    REQUIRE(tdm_work_wait_stream(w, caller) == TDM_OK);  // parked: the collective cannot have run
    REQUIRE(hipStreamSynchronize(caller) == hipSuccess);
    const auto took = std::chrono::steady_clock::now() - began;
    REQUIRE(took >= std::chrono::milliseconds(40) && took < std::chrono::milliseconds(250));  // let go by its own limit, not by the peers
    tdm_work* again = nullptr;
    REQUIRE(tdm_all_reduce(e, x.data(), 1000, TDM_F32, 0, caller, &again) != TDM_OK);
    REQUIRE(std::string(tdm_last_error()).find("gave up") != std::string::npos);
    REQUIRE(tdm_work_wait(w, caller) != TDM_OK && std::string(tdm_last_error()).find("gave up") != std::string::npos);
  } else {
    REQUIRE(tdm_work_wait(w, caller) == TDM_OK && hipStreamSynchronize(caller) == hipSuccess);
    REQUIRE(x[0] == static_cast<float>(world * (world + 1) / 2));
  }
  REQUIRE(tdm_work_free(w) == TDM_OK);
  (void)tdm_engine_close(e);
  REQUIRE(tdm_engine_destroy(e) == TDM_OK);
  return 0;
}

static int run_rank(int rank, int world, const std::string& job, std::atomic<int>* arrived, const std::string& scenario) {
  g_rank = rank;
  tdm_engine* e = nullptr;
  if (scenario == "no_ipc_events") {  // a platform without interprocess events: the engine says so by name and leaves nothing behind
    ::setenv("TANDEM_HIP_SYNC", "event", 1);
    REQUIRE(tdm_engine_create(job.c_str(), rank, world, 2, 4096, 1.0, 0, &e) != TDM_OK && e == nullptr);
    REQUIRE(std::string(tdm_last_error()).find("cannot export interprocess events") != std::string::npos);
    REQUIRE(tdm_engine_create(job.c_str(), rank, world, 0, 4096, 1.0, 0, &e) == TDM_EINVAL);
    REQUIRE(tdm_engine_create(job.c_str(), rank, world, 2, 100, 1.0, 0, &e) == TDM_EINVAL);
    REQUIRE(tdm_engine_create(job.c_str(), world, world, 2, 4096, 1.0, 0, &e) == TDM_EINVAL);
    REQUIRE(tdm_engine_create(job.c_str(), rank, world, 2, 4096, 1.0, -1, &e) == TDM_EINVAL);
    return 0;
  }
  REQUIRE(tdm_engine_create(job.c_str(), rank, world, 2, 4096, scenario.empty() ? 20.0 : 1.0, 0, &e) == TDM_OK);
  arrived->fetch_add(1);  // the launcher's barrier: every rank has published its region
  while (arrived->load() < world) std::this_thread::yield();
  REQUIRE(tdm_engine_connect(e) == TDM_OK);
  if (scenario == "park_gives_up") return run_park_gives_up(e, rank, world);
  if (!scenario.empty()) return run_broken(e, rank, world, scenario);

  hipStream_t caller = nullptr;
  REQUIRE(hipStreamCreateWithFlags(&caller, hipStreamNonBlocking) == hipSuccess);
  const int64_t lengths[] = {0, 1, 5, 1000, 4099, 40000};
  int salt = 0;
  for (int64_t n : lengths) {
    for (int uneven = 0; uneven < 2; ++uneven) {
      const std::vector<int64_t> sizes = split(n, world, uneven != 0);
      int64_t lo = 0;
      for (int q = 0; q < rank; ++q) lo += sizes[q];
      ++salt;
      auto total = [&](int64_t i, int s) {
        float t = 0;
        for (int q = 0; q < world; ++q) t += value(q, i, s);
        return t;
      };
      // several collectives in flight at once, waited for in order; done() polled meanwhile
      std::vector<float> a(n), b(n), c(n), d(n);
      // Every other round the tensors are produced and consumed on a stream of the caller's: the producer is slow,
      // so an engine that did not wait for it would fold what was there before, and the consumer runs right behind
      // the waits, so a wait that did not order the stream would let it read too early.
      hipStream_t st = salt % 2 ? caller : nullptr;
      std::vector<float> b2(n);
      fake_enqueue(st, [&, lo] {
        if (st) std::this_thread::sleep_for(std::chrono::microseconds(300));
        for (int64_t i = 0; i < n; ++i) {
          a[i] = value(rank, i, salt);
          b[i] = b2[i] = value(rank, i, salt + 100);
          c[i] = i >= lo && i < lo + sizes[rank] ? value(rank, i, salt + 200) : -1.0f;
          d[i] = rank == world - 1 ? value(rank, i, salt + 300) : -2.0f;
        }
      });
      tdm_work *wa, *wb, *wb2, *wc, *wd;
      REQUIRE(tdm_all_reduce(e, a.data(), n, TDM_F32, 0, st, &wa) == TDM_OK);
      REQUIRE(tdm_reduce_scatter(e, b.data(), n, TDM_F32, sizes.data(), world, 0, st, &wb) == TDM_OK);
      REQUIRE(tdm_reduce_scatter_owner(e, b2.data(), n, TDM_F32, uneven ? sizes.data() : nullptr, uneven ? world : 0, 0, st, &wb2) == TDM_OK);
      REQUIRE(tdm_all_gather(e, c.data(), n, TDM_F32, sizes.data(), world, st, &wc) == TDM_OK);
      REQUIRE(tdm_broadcast(e, d.data(), n, TDM_F32, world - 1, st, &wd) == TDM_OK);
      (void)tdm_work_done(wd);
      REQUIRE(tdm_work_wait(wa, st) == TDM_OK);
      REQUIRE(tdm_work_wait_stream(wb, st) == TDM_OK);
      REQUIRE(tdm_work_wait(wb2, st) == TDM_OK);
      REQUIRE(tdm_work_wait_stream(wc, st) == TDM_OK);
      REQUIRE(tdm_work_wait(wd, st) == TDM_OK);
      std::atomic<int64_t> early{0};
      fake_enqueue(st, [&] {  // the consumer: sums what the collectives left, behind the waits
        double sum = 0;
        for (int64_t i = 0; i < n; ++i) sum += a[i] + c[i] + d[i];
        double want = 0;
        for (int64_t i = 0; i < n; ++i) {
          for (int q = 0; q < world; ++q) want += value(q, i, salt);
          want += value(world - 1, i, salt + 300);
        }
        int owner = 0;
        int64_t end = sizes[0];
        for (int64_t i = 0; i < n; ++i) {
          while (i >= end) end += sizes[++owner];
          want += value(owner, i, salt + 200);
        }
        if (sum != want) early.fetch_add(1);
      });
      REQUIRE(hipStreamSynchronize(st) == hipSuccess && early.load() == 0);
      REQUIRE(tdm_work_done(wa) == 1 && tdm_work_done(wd) == 1);
      double t0 = 0, t1 = 0;
      REQUIRE(tdm_work_times(wa, &t0, &t1) == TDM_OK && t1 >= t0);
      for (tdm_work* w : {wa, wb, wb2, wc, wd}) REQUIRE(tdm_work_free(w) == TDM_OK);
      const std::vector<int64_t> even = split(n, world, false);
      const std::vector<int64_t>& owner_sizes = uneven ? sizes : even;
      int64_t olo = 0;
      for (int q = 0; q < rank; ++q) olo += owner_sizes[q];
      for (int64_t i = 0; i < n; ++i) {
        REQUIRE(a[i] == total(i, salt));
        if (i >= lo && i < lo + sizes[rank]) REQUIRE(b[i] == total(i, salt + 100));
        if (i >= olo && i < olo + owner_sizes[rank]) REQUIRE(b2[i] == total(i, salt + 100));
        int owner = 0;
        for (int64_t at = sizes[0]; i >= at; at += sizes[++owner]) {
        }
        REQUIRE(c[i] == value(owner, i, salt + 200));
        REQUIRE(d[i] == value(world - 1, i, salt + 300));
      }
      // an average, a ring of sendrecvs, a barrier and a fence
      std::vector<float> m(n), out(n, 0.0f), in(n, -3.0f);
      for (int64_t i = 0; i < n; ++i) {
        m[i] = static_cast<float>(world) * value(rank, i, salt + 400);
        out[i] = value(rank, i, salt + 500);
      }
      tdm_work *wm, *ws, *wbar, *wf;
      REQUIRE(tdm_all_reduce(e, m.data(), n, TDM_F32, 1, nullptr, &wm) == TDM_OK);
      REQUIRE(tdm_sendrecv(e, out.data(), n, (rank + 1) % world, in.data(), n, (rank + world - 1) % world, TDM_F32, nullptr, &ws) == TDM_OK);
      REQUIRE(tdm_barrier(e, &wbar) == TDM_OK);
      REQUIRE(tdm_fence(e, nullptr, &wf) == TDM_OK);
      for (tdm_work* w : {wm, ws, wbar, wf}) REQUIRE(tdm_work_wait(w, nullptr) == TDM_OK && tdm_work_free(w) == TDM_OK);
      for (int64_t i = 0; i < n; ++i) {
        REQUIRE(m[i] == total(i, salt + 400));
        REQUIRE(in[i] == value((rank + world - 1) % world, i, salt + 500));
      }
    }
  }

  // arenas: two of them; the direct collectives and a direct unit gather reach into the peers' second one
  void *first = nullptr, *second = nullptr;
  REQUIRE(tdm_engine_share(e, 1 << 16, &first) == TDM_OK && tdm_engine_share(e, 1 << 20, &second) == TDM_OK);
  const int64_t n = 30011;
  const std::vector<int64_t> sizes = split(n, world, false);
  int64_t lo = 0;
  for (int q = 0; q < rank; ++q) lo += sizes[q];
  float* t = reinterpret_cast<float*>(static_cast<char*>(second) + 256 * (rank + 1));
  std::vector<int64_t> offs(world);
  for (int q = 0; q < world; ++q) offs[q] = (int64_t(1) << 31) + 256 * (q + 1);
  int64_t mine = -2;
  REQUIRE(tdm_engine_arena_offset(e, t, n * 4, &mine) == TDM_OK && mine == offs[rank]);
  REQUIRE(tdm_engine_arena_offset(e, &mine, 8, &mine) == TDM_OK && mine == -1);
  for (int64_t i = 0; i < n; ++i) t[i] = value(rank, i, 900);
  tdm_work* w = nullptr;
  REQUIRE(tdm_direct_all_reduce(e, t, n, TDM_F32, 0, offs.data(), world, nullptr, &w) == TDM_OK);
  REQUIRE(tdm_work_wait(w, nullptr) == TDM_OK && tdm_work_free(w) == TDM_OK);
  for (int64_t i = 0; i < n; ++i) {
    float want = 0;
    for (int q = 0; q < world; ++q) want += value(q, i, 900);
    REQUIRE(t[i] == want);
  }
  for (int64_t i = 0; i < n; ++i) t[i] = i >= lo && i < lo + sizes[rank] ? value(rank, i, 901) : -4.0f;
  REQUIRE(tdm_direct_all_gather(e, t, n, TDM_F32, sizes.data(), world, offs.data(), world, nullptr, &w) == TDM_OK);
  REQUIRE(tdm_work_wait(w, nullptr) == TDM_OK && tdm_work_free(w) == TDM_OK);
  std::vector<float> full(n, -5.0f);
  std::vector<int64_t> shard_offs(world);
  int64_t at = 0;
  for (int q = 0; q < world; ++q) {
    shard_offs[q] = offs[q] + at * 4;  // rank q's own chunk, where the all-gather left it
    at += sizes[q];
  }
  REQUIRE(tdm_unit_gather_direct(e, full.data(), n, TDM_F32, t + lo, sizes.data(), world, shard_offs.data(), world, caller, &w) == TDM_OK);
  REQUIRE(tdm_work_wait(w, caller) == TDM_OK && tdm_work_free(w) == TDM_OK);
  REQUIRE(hipStreamSynchronize(caller) == hipSuccess);
  for (int64_t i = 0, owner = 0, end = sizes[0]; i < n; ++i) {
    while (i >= end) end += sizes[++owner];
    REQUIRE(t[i] == value(static_cast<int>(owner), i, 901) && full[i] == t[i]);
  }
  REQUIRE(tdm_fence(e, nullptr, &w) == TDM_OK && tdm_work_wait(w, nullptr) == TDM_OK && tdm_work_free(w) == TDM_OK);

  // A fence whose wait only parks the caller's stream, and behind it a gather that is launched (by this thread, on the
  // side stream when gathers run there) before the progress thread has got to the fence: the fence is held back by a slow
  // producer on the caller's stream. The gather waits for the caller's stream, which waits for the fence's end, so a
  // fence that waited for EVERYTHING on the side stream would wait for itself. It waits for what was launched before it.
  {
    std::fill(full.begin(), full.end(), -5.0f);
    tdm_work *wf, *wg;
    const auto began = std::chrono::steady_clock::now();
    fake_enqueue(caller, [] { std::this_thread::sleep_for(std::chrono::microseconds(400)); });
    REQUIRE(tdm_fence(e, caller, &wf) == TDM_OK);
    REQUIRE(tdm_work_wait_stream(wf, caller) == TDM_OK);
    REQUIRE(tdm_unit_gather_direct(e, full.data(), n, TDM_F32, t + lo, sizes.data(), world, shard_offs.data(), world, caller, &wg) == TDM_OK);
    REQUIRE(tdm_work_wait(wg, caller) == TDM_OK && tdm_work_free(wg) == TDM_OK);
    REQUIRE(tdm_work_wait(wf, caller) == TDM_OK && tdm_work_free(wf) == TDM_OK);
    REQUIRE(hipStreamSynchronize(caller) == hipSuccess);
    for (int64_t i = 0; i < n; ++i) REQUIRE(full[i] == t[i]);
    // (the stand-in's parked stream gives up after twenty seconds, so the cycle would show as a stall, not as a hang)
    REQUIRE(std::chrono::steady_clock::now() - began < std::chrono::seconds(5));
    REQUIRE(tdm_fence(e, nullptr, &w) == TDM_OK && tdm_work_wait(w, nullptr) == TDM_OK && tdm_work_free(w) == TDM_OK);
  }

  // A process with a single hardware queue (GPU_MAX_HW_QUEUES=1): no stream is parked on a collective that has not run,
  // tdm_work_wait_stream waits on the host like tdm_work_wait. Parked (any other setting), it returns at once: the
  // collective cannot start before the slow producer on the caller's stream has finished.
  {
    const char* hq = std::getenv("GPU_MAX_HW_QUEUES");
    const bool single = hq && std::atoi(hq) == 1;
    std::vector<float> x(1000, static_cast<float>(rank + 1));
    const auto began = std::chrono::steady_clock::now();
    fake_enqueue(caller, [] { std::this_thread::sleep_for(std::chrono::milliseconds(40)); });
    REQUIRE(tdm_all_reduce(e, x.data(), 1000, TDM_F32, 0, caller, &w) == TDM_OK);
    REQUIRE(tdm_work_wait_stream(w, caller) == TDM_OK);
    const auto took = std::chrono::steady_clock::now() - began;
    REQUIRE(single ? took >= std::chrono::milliseconds(35) : took < std::chrono::milliseconds(25));
    REQUIRE(hipStreamSynchronize(caller) == hipSuccess && tdm_work_free(w) == TDM_OK);
    REQUIRE(x[0] == static_cast<float>(world * (world + 1) / 2));
  }

  // ZeRO-2's step as one launch per rank: gradients and parameters in the second arena, every rank updates its own shard
  // and writes it into every rank's parameters (the stand-in's "step" is parameter - averaged gradient)
  {
    float* grads = t;                                            // n floats at offs[q]
    float* params = t + (n + 63) / 64 * 64;                      // behind them, on every rank at the same distance
    std::vector<int64_t> goffs(world), poffs(world);
    for (int q = 0; q < world; ++q) {
      goffs[q] = offs[q] + lo * 4;
      poffs[q] = offs[q] + ((n + 63) / 64 * 64 + lo) * 4;
    }
    for (int64_t i = 0; i < n; ++i) {
      grads[i] = static_cast<float>(world) * value(rank, i, 903);
      params[i] = value(0, i, 904);  // the same on every rank
    }
    std::vector<float> m(sizes[rank], 0.0f), v(sizes[rank], 0.0f);
    tdm_adamw_scalars sc;
    std::memset(&sc, 0, sizeof sc);
    REQUIRE(tdm_direct_zero2_step(e, params + lo, poffs.data(), grads + lo, goffs.data(), world, m.data(), v.data(), sizes[rank], n, 1,
                                  &sc, TDM_ADAMW_HOST_ORDER, nullptr, &w) == TDM_OK);
    REQUIRE(tdm_work_wait(w, nullptr) == TDM_OK && tdm_work_free(w) == TDM_OK);
    for (int64_t i = 0; i < n; ++i) {
      float g = 0;
      for (int q = 0; q < world; ++q) g += value(q, i, 903);
      REQUIRE(params[i] == value(0, i, 904) - g);
      if (i >= lo && i < lo + sizes[rank]) REQUIRE(m[i - lo] == g && v[i - lo] == g * g);
    }
  }

  // the same step over float64 buffers, its constants as doubles: the typed entry point, the element size in the arena offsets
  {
    double* grads = reinterpret_cast<double*>(t);
    double* params = grads + (n + 63) / 64 * 64;
    std::vector<int64_t> goffs(world), poffs(world);
    for (int q = 0; q < world; ++q) {
      goffs[q] = offs[q] + lo * 8;
      poffs[q] = offs[q] + ((n + 63) / 64 * 64 + lo) * 8;
    }
    for (int64_t i = 0; i < n; ++i) {
      grads[i] = static_cast<double>(world) * value(rank, i, 905);
      params[i] = value(0, i, 906);
    }
    std::vector<double> m(sizes[rank], 0.0), v(sizes[rank], 0.0);
    tdm_adamw_hyper hy;
    std::memset(&hy, 0, sizeof hy);
    REQUIRE(tdm_direct_zero2_step_typed(e, params + lo, poffs.data(), grads + lo, goffs.data(), world, m.data(), v.data(), sizes[rank], n, 1,
                                        TDM_F64, &hy, TDM_ADAMW_DEVICE_ORDER, nullptr, &w) == TDM_EINVAL);  // fp32 only
    REQUIRE(tdm_direct_zero2_step_typed(e, params + lo, poffs.data(), grads + lo, goffs.data(), world, m.data(), v.data(), sizes[rank], n, 1,
                                        TDM_I32, &hy, TDM_ADAMW_HOST_ORDER, nullptr, &w) == TDM_EINVAL);
    REQUIRE(tdm_direct_zero2_step_typed(e, params + lo, poffs.data(), grads + lo, goffs.data(), world, m.data(), v.data(), sizes[rank], n, 1,
                                        TDM_F64, nullptr, TDM_ADAMW_HOST_ORDER, nullptr, &w) == TDM_EINVAL);
    REQUIRE(tdm_direct_zero2_step_typed(e, params + lo, poffs.data(), grads + lo, goffs.data(), world, m.data(), v.data(), sizes[rank], n, 1,
                                        TDM_F64, &hy, TDM_ADAMW_HOST_ORDER, nullptr, &w) == TDM_OK);
    REQUIRE(tdm_work_wait(w, nullptr) == TDM_OK && tdm_work_free(w) == TDM_OK);
    for (int64_t i = 0; i < n; ++i) {
      double g = 0;
      for (int q = 0; q < world; ++q) g += value(q, i, 905);
      REQUIRE(params[i] == value(0, i, 906) - g);
      if (i >= lo && i < lo + sizes[rank]) REQUIRE(m[i - lo] == g && v[i - lo] == g * g);
    }
  }

  // the same gather through the engine's own path (no arenas), produced and consumed on the caller's stream, with device
  // time stamps on
  REQUIRE(tdm_engine_set_timing(e, 1) == TDM_OK);
  std::vector<float> shard(sizes[rank]), whole(n, -6.0f);
  std::atomic<int64_t> wrong{0};
  fake_enqueue(caller, [&] {
    std::this_thread::sleep_for(std::chrono::microseconds(300));
    for (int64_t i = 0; i < sizes[rank]; ++i) shard[i] = value(rank, lo + i, 902);
  });
  REQUIRE(tdm_unit_gather(e, whole.data(), n, TDM_F32, shard.data(), sizes.data(), world, caller, &w) == TDM_OK);
  REQUIRE(tdm_work_wait_stream(w, caller) == TDM_OK);
  fake_enqueue(caller, [&] {
    for (int64_t i = 0, owner = 0, end = sizes[0]; i < n; ++i) {
      while (i >= end) end += sizes[++owner];
      if (whole[i] != value(static_cast<int>(owner), i, 902)) wrong.fetch_add(1);
    }
  });
  REQUIRE(hipStreamSynchronize(caller) == hipSuccess && wrong.load() == 0);
  double started = 0, finished = 0;
  REQUIRE(tdm_work_times(w, &started, &finished) == TDM_OK && finished >= started && tdm_work_free(w) == TDM_OK);
  REQUIRE(tdm_engine_set_timing(e, 0) == TDM_OK);

  // more collectives in flight than the engine has done words
  const int many = 1100;
  std::vector<float> rows(static_cast<size_t>(many) * 3);
  std::vector<tdm_work*> works(many);
  for (int k = 0; k < many; ++k) {
    for (int j = 0; j < 3; ++j) rows[k * 3 + j] = static_cast<float>(k + rank);
    REQUIRE(tdm_all_reduce(e, &rows[k * 3], 3, TDM_F32, 0, nullptr, &works[k]) == TDM_OK);
  }
  for (int k = 0; k < many; ++k) {
    REQUIRE(tdm_work_wait(works[k], nullptr) == TDM_OK && tdm_work_free(works[k]) == TDM_OK);
    REQUIRE(rows[k * 3 + 2] == static_cast<float>(world * k + world * (world - 1) / 2));
  }

  // refusals come back as codes with a message, from the calling thread
  REQUIRE(tdm_all_reduce(e, rows.data(), 3, TDM_I32, 1, nullptr, &w) == TDM_EINVAL && std::strlen(tdm_last_error()) > 0);
  REQUIRE(tdm_all_reduce(e, nullptr, 3, TDM_F32, 0, nullptr, &w) == TDM_EINVAL);
  const int64_t bad[2] = {1, 1};
  REQUIRE(tdm_all_gather(e, rows.data(), 3, TDM_F32, bad, 2, nullptr, &w) == TDM_EINVAL);
  REQUIRE(hipStreamDestroy(caller) == hipSuccess);
  REQUIRE(tdm_engine_close(e) == TDM_OK);
  REQUIRE(tdm_all_reduce(e, rows.data(), 3, TDM_F32, 0, nullptr, &w) != TDM_OK);
  REQUIRE(tdm_engine_destroy(e) == TDM_OK);
  return 0;
}

int main(int argc, char** argv) {
  const int world = argc > 1 ? std::atoi(argv[1]) : 2;
  const std::string algo = argc > 2 ? argv[2] : "staged";
  if (world < 2 || world > 8) return 64;
  ::setenv("TANDEM_HIP_ALGO", algo.c_str(), 1);
  if (argc > 3 && std::atoll(argv[3]) > 0) ::setenv("TANDEM_HIP_STAGING_BYTES", argv[3], 1);
  const std::string scenario = argc > 4 && std::string(argv[4]) != "-" ? argv[4] : "";
  for (std::string rest = argc > 5 ? argv[5] : ""; !rest.empty();) {
    const size_t comma = rest.find(','), eq = rest.find('=');
    if (eq == std::string::npos || eq > comma) return 64;
    ::setenv(rest.substr(0, eq).c_str(), rest.substr(eq + 1, comma == std::string::npos ? comma : comma - eq - 1).c_str(), 1);
    rest = comma == std::string::npos ? "" : rest.substr(comma + 1);
  }
  const std::string job = "host" + std::to_string(::getpid());
  void* shared = ::mmap(nullptr, 4096, PROT_READ | PROT_WRITE, MAP_SHARED | MAP_ANONYMOUS, -1, 0);
  if (shared == MAP_FAILED) return 65;
  auto* arrived = new (shared) std::atomic<int>(0);
  std::vector<pid_t> children;
  for (int r = 0; r < world; ++r) {  // forked before any thread exists
    const pid_t pid = ::fork();
    if (pid < 0) return 66;
    if (pid == 0) {
      std::exit(run_rank(r, world, job, arrived, scenario));  // through the exit handlers: the leak check runs there
    }
    children.push_back(pid);
  }
  int failed = 0;
  for (pid_t pid : children) {
    int status = 0;
    if (::waitpid(pid, &status, 0) != pid || !WIFEXITED(status) || WEXITSTATUS(status) != 0) ++failed;
  }
  if (failed) std::fprintf(stderr, "%d of %d ranks failed\n", failed, world);
  if (failed || !scenario.empty()) {  // what a rank that did not close left in /dev/shm
    for (int r = 0; r < world; ++r) {
      ::shm_unlink(("/tandem-" + job + "-" + std::to_string(r) + "-hip").c_str());
      for (int k = 0; k < 64; ++k) ::shm_unlink(("/tdmfake-" + std::to_string(children[r]) + "-" + std::to_string(k)).c_str());
    }
  }
  return failed ? 1 : 0;
}
