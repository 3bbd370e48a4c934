// Error plumbing shared by the kernels and the engine: C++ exceptions inside,
// status codes and a thread-local message at the C boundary.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
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

// How a segment of `count` elements whose streams start at ptrs[0..n) is walked. When every stream starts at
// the same distance from a 16-byte boundary, the first `head` elements (fewer than a vector) are peeled off,
// the remaining `body` elements start aligned and take the dwordx4 path (vec), in `tiles` tiles of tile_elems.
// Otherwise (or when the segment is shorter than its head) everything goes element by element: head 0, body = count.
struct SegPlan {
  bool vec;
  int head;
  int64_t body, tiles;
};

inline SegPlan plan_segment(const uintptr_t* ptrs, int n, int64_t count, int es, int64_t tile_elems) {
  SegPlan p{false, 0, count, count > 0 ? (count + tile_elems - 1) / tile_elems : 0};
  if (count <= 0 || n <= 0) return p;
  const uintptr_t phase = ptrs[0] % 16;
  for (int i = 1; i < n; ++i)
    if (ptrs[i] % 16 != phase) return p;
  const int64_t head = static_cast<int64_t>((16 - phase) % 16) / es;
  if (head >= count) return p;
  p.vec = true;
  p.head = static_cast<int>(head);
  p.body = count - head;
  p.tiles = (p.body + tile_elems - 1) / tile_elems;
  return p;
}

// kernels.hip
// policy: which accesses are non-temporal (2, 5 or 7; see kernels.hip); 2 suits a launch on its own
void reduce_step(const tdm_pair* pairs, int npairs, int dtype, int world, bool scale_dst, bool scale_src,
                 bool writeback_src, hipStream_t stream, int policy = 2);
void copy_step(const tdm_pair* pairs, int npairs, int dtype, int world, hipStream_t stream, int policy = 2);
// divide_by: what averaging divides by when that is not `world` (a partial sum of a larger ring: world = the terms folded)
void fold_step(const tdm_fold_seg* segs, int nseg, int world, int dtype, bool average, hipStream_t stream, int divide_by = 0);
// kernels_chain.hip: the ring reduce-scatter of a whole group in one launch (rank q's buffer at base[q], chunk c =
// elements [lo[c], lo[c] + len[c])); world sizes 2..kChainMaxWorld. Returns false, with nothing launched, when the ranks'
// copies of some chunk disagree within 16 bytes: the kernel has no element-by-element path (it would set its register
// count), and the caller takes the ring's steps.
constexpr int kChainMaxWorld = 8;
bool chain_handles(int world);
bool chain_reduce_scatter(char* const* base, const int64_t* lo, const int64_t* len, int world, int dtype, int es, bool average,
                          bool keep_sent, bool cold, unsigned occupancy_pad, int xcd_shift, int max_grid, hipStream_t stream);
// the ring all-gather of a whole group in one launch: every chunk read once from its owner and stored into the
// other ranks' buffers; world sizes 2..8; `cold`: the footprint is beyond the caches (non-temporal accesses)
bool gather_handles(int world);
void gather_multicast(char* const* base, const int64_t* lo, const int64_t* len, int world, int es, bool cold, unsigned occupancy_pad,
                      int xcd_shift, int vectors_per_lane, int max_grid, hipStream_t stream);
// ZeRO-3's unit gather for every rank in one launch (world sizes 1..8): shard q read once, stored into all the full buffers
void unit_gather_multicast(char* const* fulls, const char* const* shards, const int64_t* sizes, int world, int es, bool cold,
                           unsigned occupancy_pad, int xcd_shift, int vectors_per_lane, int max_grid, hipStream_t stream);
void zero2_step_segment(const tdm_step_seg& seg, int world, bool average, const tdm_adamw_scalars& s, int order, hipStream_t stream);
void park_stream(hipStream_t stream, const uint32_t* word, uint32_t value, double limit_s, uint32_t* gave_up);
void zero2_step_segment_typed(const tdm_step_seg& seg, int world, bool average, const tdm_adamw_hyper& h, int order, hipStream_t stream);

}  // namespace tandem_hip
