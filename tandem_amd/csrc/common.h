// Error plumbing shared by the kernels and the engine: C++ exceptions inside,
// status codes and a thread-local message at the C boundary.
#pragma once

#include <hip/hip_runtime.h>

#include <stdexcept>
#include <string>

#include "../../include/tandem_hip.h"

namespace tandem_hip {

struct Invalid : std::invalid_argument {
  using std::invalid_argument::invalid_argument;
};

struct Timeout : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline void check_hip(hipError_t err, const char* what) {
  if (err != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(err));
}

void set_last_error(const std::string& message);

template <class F>
int guard(F&& body) {
  try {
    body();
    return TDM_OK;
  } catch (const Invalid& e) {
    set_last_error(e.what());
    return TDM_EINVAL;
  } catch (const Timeout& e) {
    set_last_error(e.what());
    return TDM_ETIMEOUT;
  } catch (const std::exception& e) {
    set_last_error(e.what());
    return TDM_ERUNTIME;
  } catch (...) {
    set_last_error("unknown error");
    return TDM_ERUNTIME;
  }
}

// kernels.hip
// policy: which accesses are non-temporal (2, 5 or 7; see kernels.hip); 2 suits a launch on its own
void reduce_step(const tdm_pair* pairs, int npairs, int dtype, int world, bool scale_dst, bool scale_src,
                 bool writeback_src, hipStream_t stream, int policy = 2);
void copy_step(const tdm_pair* pairs, int npairs, int dtype, int world, hipStream_t stream, int policy = 2);
void fold_step(const tdm_fold_seg* segs, int nseg, int world, int dtype, bool average, hipStream_t stream);
// kernels_chain.hip: the ring reduce-scatter of a whole group in one launch (rank q's buffer at base[q], chunk c =
// elements [lo[c], lo[c] + len[c])); world sizes 2..kChainMaxWorld
constexpr int kChainMaxWorld = 4;
bool chain_handles(int world);
void chain_reduce_scatter(char* const* base, const int64_t* lo, const int64_t* len, int world, int dtype, int es, bool average,
                          bool keep_sent, int max_grid, hipStream_t stream);
void zero2_step_segment(const tdm_step_seg& seg, int world, bool average, const tdm_adamw_scalars& s, int order, hipStream_t stream);

}  // namespace tandem_hip
