// The four launchers the engine calls (tandem_amd/csrc/common.h), as plain loops on the host: the other half of the
// stand-in that tests/cpp/fake_hip.cpp describes, linked into tests/cpp/engine_host_test only. fp32, fp64, int32 and
// int64; the sums are formed in the order the kernels form them, which for the integer-valued numbers the test
// sends does not matter. Like a launch, each returns at once: the loop runs when the stream gets to it.

#include <chrono>
#include <cstring>
#include <string>
#include <thread>

#include <vector>

#include "../../tandem_amd/csrc/common.h"
#include "fake_hip.h"

namespace tandem_hip {

namespace {

int size_of(int dtype) {
  switch (dtype) {
    case TDM_F32: case TDM_I32: return 4;
    case TDM_F64: case TDM_I64: return 8;
    case TDM_F16: case TDM_BF16: case TDM_I16: return 2;
    case TDM_I8: case TDM_U8: return 1;
    default: throw Invalid("unknown dtype " + std::to_string(dtype));
  }
}

template <typename F>
void dispatch(int dtype, F&& f) {
  switch (dtype) {
    case TDM_F32: f(static_cast<float*>(nullptr)); break;
    case TDM_F64: f(static_cast<double*>(nullptr)); break;
    case TDM_I32: f(static_cast<int32_t*>(nullptr)); break;
    case TDM_I64: f(static_cast<int64_t*>(nullptr)); break;
    default: throw Invalid("the stand-in kernels know fp32, fp64, int32 and int64");
  }
}

template <typename T>
T divided(T x, int world) {
  return world > 1 ? static_cast<T>(x / static_cast<T>(world)) : x;
}

}  // namespace

void reduce_step(const tdm_pair* pairs, int npairs, int dtype, int world, bool scale_dst, bool scale_src, bool writeback_src,
                 hipStream_t stream, int) {
  (void)size_of(dtype);
  const std::vector<tdm_pair> ps(pairs, pairs + npairs);
  fake_enqueue(stream, [=] {
    dispatch(dtype, [&](auto* tag) {
      using T = std::remove_pointer_t<decltype(tag)>;
      for (const tdm_pair& p : ps) {
        T* d = static_cast<T*>(p.dst);
        T* s = const_cast<T*>(static_cast<const T*>(p.src));
        for (int64_t k = 0; k < p.count; ++k) {
          const T x = scale_dst ? divided(d[k], world) : d[k], y = scale_src ? divided(s[k], world) : s[k];
          if (scale_src && writeback_src) s[k] = y;
          d[k] = static_cast<T>(x + y);
        }
      }
    });
  });
}

void copy_step(const tdm_pair* pairs, int npairs, int dtype, int world, hipStream_t stream, int) {
  const int es = size_of(dtype);
  const std::vector<tdm_pair> ps(pairs, pairs + npairs);
  fake_enqueue(stream, [=] {
    if (world <= 1) {
      for (const tdm_pair& p : ps) std::memmove(p.dst, p.src, static_cast<size_t>(p.count) * es);
      return;
    }
    dispatch(dtype, [&](auto* tag) {
      using T = std::remove_pointer_t<decltype(tag)>;
      for (const tdm_pair& p : ps) {
        T* d = static_cast<T*>(p.dst);
        const T* s = static_cast<const T*>(p.src);
        for (int64_t k = 0; k < p.count; ++k) d[k] = divided(s[k], world);
      }
    });
  });
}

void fold_step(const tdm_fold_seg* segs, int nseg, int world, int dtype, bool average, hipStream_t stream, int divide_by) {
  if (world < 2 || world > TDM_MAX_WORLD) throw Invalid("the direct fold handles world sizes 2..8");
  (void)size_of(dtype);
  const int by = average ? (divide_by ? divide_by : world) : 1;
  const std::vector<tdm_fold_seg> sgs(segs, segs + nseg);
  fake_enqueue(stream, [=] {
    dispatch(dtype, [&](auto* tag) {
      using T = std::remove_pointer_t<decltype(tag)>;
      for (const tdm_fold_seg& sg : sgs) {
        for (int64_t k = 0; k < sg.count; ++k) {
          T acc = divided(static_cast<const T*>(sg.src[(sg.chunk + 1) % world])[k], by);
          for (int j = 2; j <= world; ++j) acc = static_cast<T>(divided(static_cast<const T*>(sg.src[(sg.chunk + j) % world])[k], by) + acc);
          for (int r = 0; r < world; ++r)
            if (sg.dst[r]) static_cast<T*>(sg.dst[r])[k] = acc;
        }
      }
    });
  });
}

// The data flow of ZeRO-2's step, not its arithmetic: the shard's gradients folded in the ring's order and averaged, the
// moments bumped, and "parameter - gradient" written into every rank's parameter buffer. (AdamW itself is the kernels'
// and the GPU tests' business.)
// A stream parked on a word, as park_kernel parks it: until the word has reached the value, or the time is up.
void park_stream(hipStream_t stream, const uint32_t* word, uint32_t value, double limit_s, uint32_t* gave_up) {
  fake_enqueue(stream, [=] {
    const auto until = std::chrono::steady_clock::now() + std::chrono::duration<double>(limit_s);
    while (__atomic_load_n(word, __ATOMIC_ACQUIRE) < value) {
      if (std::chrono::steady_clock::now() > until) {
        __atomic_store_n(gave_up, 1u, __ATOMIC_RELEASE);
        return;
      }
      std::this_thread::yield();
    }
  });
}

namespace {
template <typename T>
void step_data_flow(const tdm_step_seg& sg, int world, bool average, hipStream_t stream) {
  if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
  const tdm_step_seg seg = sg;
  fake_enqueue(stream, [=] {
    T* m = static_cast<T*>(seg.exp_avg);
    T* v = static_cast<T*>(seg.exp_avg_sq);
    for (int64_t k = 0; k < seg.count; ++k) {
      T g = divided(static_cast<const T*>(seg.grad[(seg.chunk + 1) % world])[k], average ? world : 1);
      for (int j = 2; j <= world; ++j) g = divided(static_cast<const T*>(seg.grad[(seg.chunk + j) % world])[k], average ? world : 1) + g;
      m[k] += g;
      v[k] += g * g;
      const T p = static_cast<const T*>(seg.param[seg.chunk])[k] - g;
      for (int r = 0; r < world; ++r) static_cast<T*>(seg.param[r])[k] = p;
    }
  });
}
}  // namespace

void zero2_step_segment(const tdm_step_seg& sg, int world, bool average, const tdm_adamw_scalars&, int, hipStream_t stream) {
  if (sg.dtype != TDM_F32) throw Invalid("fp32 constants go with fp32 shards");
  step_data_flow<float>(sg, world, average, stream);
}

// The same for the shard types that take their constants as doubles; the stand-in knows fp32 and float64.
void zero2_step_segment_typed(const tdm_step_seg& sg, int world, bool average, const tdm_adamw_hyper&, int, hipStream_t stream) {
  if (sg.dtype == TDM_F32) step_data_flow<float>(sg, world, average, stream);
  else if (sg.dtype == TDM_F64) step_data_flow<double>(sg, world, average, stream);
  else throw Invalid("the stand-in steps fp32 and float64 shards");
}

}  // namespace tandem_hip
