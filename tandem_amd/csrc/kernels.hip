// Streaming kernels of tandem's data-parallel reduction path for gfx950 (MI355X):
// K1 ring-step reduce / copy, K2 bucket fold, K3 sharded AdamW, K4 unit gather.
//
// All four are HBM-bound element-wise passes, so they share one shape: a launch
// covers a small table of streams, the work is cut into tiles of 2 to 4 KiB per
// stream, workgroups walk the tiles grid-stride (consecutive workgroups touch
// consecutive tiles, so a sweep of the grid is one contiguous multi-MiB slot of
// every stream), and each lane keeps several independent 16-byte loads in flight
// before its first use. No LDS. Arithmetic is exact IEEE in the tensor's own
// precision: built with -ffp-contract=off, true division, correctly rounded
// sqrt; the only fused multiply-adds are the explicit ones in K3.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <type_traits>

#include "../../include/tandem_hip.h"
#include "common.h"

#include "kernels_device.h"

// The table of tdm_k2_bucket_fold_static: records for up to kStaticTiles tiles, in every GPU's
// memory for as long as the library is loaded (2.25 MiB). Host code reaches it through
// static_table() only.
constexpr int64_t kStaticTiles = 16384;
static __device__ __align__(256) unsigned char scratch[kStaticTiles * sizeof(tandem_hip::FoldSegDev)];

namespace tandem_hip {

namespace {

// ---------------------------------------------------------------- host side
int elem_size(int dtype) {
  switch (dtype) {
    case TDM_F32: case TDM_I32: return 4;
    case TDM_F64: case TDM_I64: return 8;
    case TDM_F16: case TDM_BF16: case TDM_I16: return 2;
    case TDM_I8: case TDM_U8: return 1;
    default: return 0;
  }
}

// How the fold and step kernels walk a segment (plan_segment), over the pointers that exist: entries of
// ranks beyond the world size are NULL by contract, so the plan does not need the world size.
SegPlan plan_fold(const tdm_fold_seg& s, int es) {
  uintptr_t ptrs[2 * TDM_MAX_WORLD];
  int n = 0;
  for (int r = 0; r < TDM_MAX_WORLD; ++r) {
    if (s.src[r]) ptrs[n++] = reinterpret_cast<uintptr_t>(s.src[r]);
    if (s.dst[r]) ptrs[n++] = reinterpret_cast<uintptr_t>(s.dst[r]);
  }
  return plan_segment(ptrs, n, s.count, es, static_cast<int64_t>(kTileVecs) * (16 / es));
}

// The element size of a step segment: its dtype field names TDM_F32 (0, what a caller that knows nothing of the field
// leaves there), TDM_F64, TDM_BF16 or TDM_F16; 0 for anything else.
int step_elem_size(const tdm_step_seg& s) {
  return s.dtype == TDM_F32 ? 4 : s.dtype == TDM_F64 ? 8 : (s.dtype == TDM_BF16 || s.dtype == TDM_F16) ? 2 : 0;
}

SegPlan plan_step(const tdm_step_seg& s) {
  uintptr_t ptrs[2 * TDM_MAX_WORLD + 2];
  int n = 0;
  for (int r = 0; r < TDM_MAX_WORLD; ++r) {
    if (s.grad[r]) ptrs[n++] = reinterpret_cast<uintptr_t>(s.grad[r]);
    if (s.param[r]) ptrs[n++] = reinterpret_cast<uintptr_t>(s.param[r]);
  }
  if (s.exp_avg) ptrs[n++] = reinterpret_cast<uintptr_t>(s.exp_avg);
  if (s.exp_avg_sq) ptrs[n++] = reinterpret_cast<uintptr_t>(s.exp_avg_sq);
  const int es = step_elem_size(s);
  if (es == 0) throw Invalid("a step segment's dtype must be TDM_F32, TDM_F64, TDM_BF16 or TDM_F16");
  return plan_segment(ptrs, n, s.count, es, static_cast<int64_t>(kTileVecs) * (16 / es));
}

bool is_floating(int dtype) { return dtype == TDM_F32 || dtype == TDM_F64 || dtype == TDM_F16 || dtype == TDM_BF16; }

// Compute units of the current device: asked of the runtime once per device, and looked up once per
// entry-point call (a collective of several launches asks hipGetDevice once, not per launch).
int compute_units() {
  static std::atomic<int> cus[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

thread_local int t_call_cus = 0;  // set while a collective of several launches runs on this thread

struct CallScope {
  bool outer;
  CallScope() : outer(t_call_cus == 0) { if (outer) t_call_cus = compute_units(); }
  ~CallScope() { if (outer) t_call_cus = 0; }
};

// tile_of()'s shift per kernel family (TDM_XCD_*), settable through tdm_set_xcd_group.
constexpr int kXcdKinds = TDM_XCD_STEP + 1;
std::atomic<int> g_xcd_shift[kXcdKinds] = {{-1}, {-1}, {-1}, {-1}, {-1}, {-1}};  // -1: the measured default below (launches may come from several threads)

// Defaults, from sweeps of the shift (0..9) on MI355X at the 85.8M-parameter and 64-256 MiB
// workloads. The unit is what one workgroup takes: 4 KiB for K1, the copy step and a fold within
// the caches, 2 KiB for the table-driven folds, the one-launch step, AdamW and a fold beyond the
// caches. Launches with one or two write streams want the plain order (K1, the copy step and the
// two-rank bucket fold lose 1-8 % with any grouping); the many-stream launches gain: the one-launch
// ZeRO-2 step 1-3 % at 64 parts per XCD, ZeRO-2's fold into the shards 3 % at 256, AdamW 0.5-1 %
// at 128, the single-launch all-reduce 2-8 % (runs of 128 KiB per XCD beyond the Infinity Cache,
// 1 MiB within). Differences of 1-2 % between neighbouring shifts do not repeat from one machine
// to the next; the defaults are the choices that were never behind the plain order.
int xcd_shift(int kind, int world, bool cold) {
  const int set = g_xcd_shift[kind].load(std::memory_order_relaxed);
  if (set >= 0) return set;
  switch (kind) {
    // cold: the one-launch reduce-scatter beyond the caches. Runs of 256 KiB per XCD, 256 MiB / 1 GiB per rank: world 3
    // 221 -> 211 / 922 -> 890 us, world 5 432 -> 413 / 1865 -> 1704, world 8 667 -> 678 / 3097 -> 2631; world 4 loses (287 -> 299).
    case TDM_XCD_REDUCE: return cold && world >= 3 && world != 4 ? 6 : 0;
    case TDM_XCD_STEP: return 6;
    case TDM_XCD_ADAMW: return 7;
    case TDM_XCD_FOLD_TABLE: return world >= 4 ? 8 : 0;
    case TDM_XCD_FOLD: return cold ? (world == 3 ? 8 : world >= 4 ? 6 : 5) : (world >= 3 ? 8 : 0);
    default: return 0;
  }
}

// Occupancy cap per kernel family: bytes of LDS that a launch asks for per workgroup and never
// touches, so that fewer workgroups fit a compute unit (160 KiB of LDS each). The many-stream
// kernels keep far more loads in flight than the memory system needs (13 KiB per wave for the
// one-launch step, thousands of waves), and what waits there only widens the set of DRAM rows
// open at once. Measured on MI355X at the 85.8M-parameter step, 24 KiB per workgroup (6 workgroups
// = 3 waves per SIMD): one-launch step 0.780 -> 0.745 ms, AdamW on four shards 0.385 -> 0.377 ms,
// AdamW writing every rank's copy 0.587 -> 0.569 ms; 16 KiB and 32-40 KiB give less, 64 KiB
// (one wave per SIMD) is 30 % slower. Launches with few streams lose with any cap (two-rank bucket
// fold 0.212 -> 0.25 ms at 24 KiB, ZeRO-2's fold into the shards 0.36 -> 0.39).
std::atomic<int> g_occupancy_pad[kXcdKinds] = {{-1}, {-1}, {-1}, {-1}, {-1}, {-1}};

unsigned occupancy_pad(int kind, bool cold = true, int world = 0) {
  const int set = g_occupancy_pad[kind].load(std::memory_order_relaxed);
  if (set >= 0) return static_cast<unsigned>(set);
  switch (kind) {
    // the one-launch reduce-scatter (the ring's reduce step takes no pad): 2 W - 1 streams per workgroup. Beyond the caches,
    // 256 MiB per rank, no pad against this one: world 3 221 -> 211 us, world 4 295 -> 287, world 5 437 -> 405, world 8 697 -> 667.
    case TDM_XCD_REDUCE: return !cold ? 0 : world <= 4 ? 16384 : world <= 6 ? 24576 : 32768;
    case TDM_XCD_STEP: return 24576;
    case TDM_XCD_ADAMW: return 24576;
    case TDM_XCD_COPY: return cold ? 16384 : 0;  // the one-launch all-gather (the ring's copy step takes no pad)
    case TDM_XCD_FOLD: return cold ? 24576 : 0;  // 256 MiB per rank at world 4: 0.350 -> 0.343 ms; 64 MiB: 0.078 -> 0.081
    default: return 0;
  }
}

int grid_for(int64_t tiles) {
  const int64_t cap = static_cast<int64_t>(t_call_cus ? t_call_cus : compute_units()) * g_blocks_per_cu;
  return static_cast<int>(std::max<int64_t>(1, std::min(tiles, cap)));
}

// Validates the pairs and lays out the by-value table. Returns the tile count (0: nothing to do).
int64_t build_pairs(const tdm_pair* pairs, int npairs, int esize, bool ranges_must_not_overlap, int tile_vecs, PairTable* tab) {
  if (npairs < 0 || npairs > TDM_MAX_PAIRS) throw Invalid("npairs must be in [0, " + std::to_string(TDM_MAX_PAIRS) + "]");
  if (npairs > 0 && pairs == nullptr) throw Invalid("pairs is NULL");
  std::memset(tab, 0, sizeof *tab);
  const int64_t tile_elems = static_cast<int64_t>(tile_vecs) * (16 / esize);
  int64_t tiles = 0;
  int k = 0;
  for (int i = 0; i < npairs; ++i) {
    const tdm_pair& p = pairs[i];
    if (p.count < 0) throw Invalid("pair " + std::to_string(i) + ": negative count");
    if (p.count == 0) continue;  // an empty chunk exchanges nothing (tandem/comm.py:292-294)
    if (p.dst == nullptr || p.src == nullptr) throw Invalid("pair " + std::to_string(i) + ": NULL pointer");
    const uintptr_t d = reinterpret_cast<uintptr_t>(p.dst), s = reinterpret_cast<uintptr_t>(p.src);
    if (d % esize || s % esize) throw Invalid("pair " + std::to_string(i) + ": pointer not aligned to the element size");
    const uintptr_t bytes = static_cast<uintptr_t>(p.count) * esize;
    if (ranges_must_not_overlap && d < s + bytes && s < d + bytes) {
      throw Invalid("pair " + std::to_string(i) + ": destination and source overlap");
    }
    tab->dst[k] = static_cast<char*>(p.dst);
    tab->src[k] = static_cast<char*>(const_cast<void*>(p.src));
    tab->count[k] = p.count;
    tab->vec_ok[k] = (d % 16) == (s % 16);
    int64_t head = ((16 - d % 16) % 16) / esize;
    tab->head[k] = static_cast<int32_t>(std::min<int64_t>(head, p.count));
    tiles += (p.count + tile_elems - 1) / tile_elems;
    tab->tile_end[k] = tiles;
    ++k;
  }
  tab->npairs = k;
  return tiles;
}

template <typename T>
Divisor<T> make_divisor(int world) {
  using A = typename Elem<T>::acc;
  Divisor<T> d;
  d.divisor = static_cast<A>(world > 0 ? world : 1);
  if constexpr (Elem<T>::floating) d.reciprocal = static_cast<A>(1) / d.divisor; else d.reciprocal = 1;
  return d;
}

// 0: no division, 1: power of two (exact reciprocal), 2: true division
int div_kind(int world, bool any_scale) {
  if (world <= 1 || !any_scale) return 0;
  return (world & (world - 1)) == 0 ? 1 : 2;
}

// The four cache policies K1 is built with (bit 0: loads of the stream that is read,
// modified and written back; bit 1: loads of the read-once stream; bit 2: stores are
// non-temporal): 2 for a launch on its own; 7, 5 and 0 for particular steps of a ring.
template <typename T, int kMask>
void launch_reduce_m(const PairTable& tab, int64_t tiles, int world, bool any_scale, hipStream_t stream) {
  const Divisor<T> dv = make_divisor<T>(world);
  const dim3 grid(grid_for(tiles)), block(kThreads);
  if constexpr (!Elem<T>::floating) {  // integers are never divided: only this kernel is built for them
    hipLaunchKernelGGL((k1_reduce_kernel<T, 0, kMask>), grid, block, 0, stream, tab, dv);
  } else {
    switch (div_kind(world, any_scale)) {
      case 0: hipLaunchKernelGGL((k1_reduce_kernel<T, 0, kMask>), grid, block, 0, stream, tab, dv); break;
      case 1: hipLaunchKernelGGL((k1_reduce_kernel<T, 1, kMask>), grid, block, 0, stream, tab, dv); break;
      default: hipLaunchKernelGGL((k1_reduce_kernel<T, 2, kMask>), grid, block, 0, stream, tab, dv); break;
    }
  }
}

template <typename T>
void launch_reduce(const PairTable& tab, int64_t tiles, int world, bool any_scale, int policy, hipStream_t stream) {
#ifdef TDM_ALL_POLICIES  // search builds: every policy, fp32 only
  if constexpr (std::is_same<T, float>::value) {
    switch (policy) {
      case 1: launch_reduce_m<T, 1>(tab, tiles, world, any_scale, stream); return;
      case 3: launch_reduce_m<T, 3>(tab, tiles, world, any_scale, stream); return;
      case 4: launch_reduce_m<T, 4>(tab, tiles, world, any_scale, stream); return;
      case 6: launch_reduce_m<T, 6>(tab, tiles, world, any_scale, stream); return;
      default: break;
    }
  }
#endif
  switch (policy) {
    case 7: launch_reduce_m<T, 7>(tab, tiles, world, any_scale, stream); break;
    case 5: launch_reduce_m<T, 5>(tab, tiles, world, any_scale, stream); break;
    case 0: launch_reduce_m<T, 0>(tab, tiles, world, any_scale, stream); break;
    default: launch_reduce_m<T, TDM_NT_MASK>(tab, tiles, world, any_scale, stream); break;
  }
}

template <typename T, int kMask>
void launch_copy_m(const PairTable& tab, int64_t tiles, int world, hipStream_t stream) {
  const Divisor<T> dv = make_divisor<T>(world);
  const dim3 grid(grid_for(tiles)), block(kCopyThreads);
  if constexpr (!Elem<T>::floating) {
    hipLaunchKernelGGL((k1_copy_kernel<T, 0, kMask>), grid, block, 0, stream, tab, dv);
  } else {
    switch (div_kind(world, true)) {
      case 0: hipLaunchKernelGGL((k1_copy_kernel<T, 0, kMask>), grid, block, 0, stream, tab, dv); break;
      case 1: hipLaunchKernelGGL((k1_copy_kernel<T, 1, kMask>), grid, block, 0, stream, tab, dv); break;
      default: hipLaunchKernelGGL((k1_copy_kernel<T, 2, kMask>), grid, block, 0, stream, tab, dv); break;
    }
  }
}

template <typename T>
void launch_copy(const PairTable& tab, int64_t tiles, int world, int policy, hipStream_t stream) {
#ifdef TDM_ALL_POLICIES
  if constexpr (std::is_same<T, float>::value) {
    switch (policy) {
      case 4: launch_copy_m<T, 4>(tab, tiles, world, stream); return;
      case 6: launch_copy_m<T, 6>(tab, tiles, world, stream); return;
      default: break;
    }
  }
#endif
  switch (policy) {
    case 7: launch_copy_m<T, 7>(tab, tiles, world, stream); break;
    case 5: launch_copy_m<T, 5>(tab, tiles, world, stream); break;  // (a copy has no read-modify-write stream: 5 is 4)
    case 0: launch_copy_m<T, 0>(tab, tiles, world, stream); break;
    default: launch_copy_m<T, TDM_NT_MASK>(tab, tiles, world, stream); break;
  }
}

template <typename T, int kWorld, bool kAcc>
void launch_fold_w(const void* image, int64_t tiles, int average, hipStream_t stream) {
  const Divisor<T> dv = make_divisor<T>(kWorld);
  const dim3 grid(grid_for(tiles * FoldShape<kWorld>::kParts)), block(FoldShape<kWorld>::kT);
  const FoldSegDev* img = static_cast<const FoldSegDev*>(image);
  if constexpr (!Elem<T>::floating) {
    hipLaunchKernelGGL((k2_fold_kernel<T, kWorld, 0, kAcc>), grid, block, occupancy_pad(TDM_XCD_FOLD_TABLE), stream, img, tiles, dv, xcd_shift(TDM_XCD_FOLD_TABLE, kWorld, true));
  } else {
    switch (div_kind(kWorld, average != 0)) {
      case 0: hipLaunchKernelGGL((k2_fold_kernel<T, kWorld, 0, kAcc>), grid, block, occupancy_pad(TDM_XCD_FOLD_TABLE), stream, img, tiles, dv, xcd_shift(TDM_XCD_FOLD_TABLE, kWorld, true)); break;
      case 1: hipLaunchKernelGGL((k2_fold_kernel<T, kWorld, 1, kAcc>), grid, block, occupancy_pad(TDM_XCD_FOLD_TABLE), stream, img, tiles, dv, xcd_shift(TDM_XCD_FOLD_TABLE, kWorld, true)); break;
      default: hipLaunchKernelGGL((k2_fold_kernel<T, kWorld, 2, kAcc>), grid, block, occupancy_pad(TDM_XCD_FOLD_TABLE), stream, img, tiles, dv, xcd_shift(TDM_XCD_FOLD_TABLE, kWorld, true)); break;
    }
  }
}

template <typename T, int kWorld>
void launch_fold_small_w(const FoldSmall& table, int average, hipStream_t stream, int divide_by) {
  const int divisor = divide_by > 0 ? divide_by : kWorld;
  const Divisor<T> dv = make_divisor<T>(divisor);
  // bytes touched: every tile is read from kWorld ranks (and written back to most of them)
  const bool cold = table.tile_end[table.nseg - 1] * static_cast<int64_t>(kTileVecs) * 16 * kWorld >= cold_footprint(kWorld);
  const dim3 grid(grid_for(table.tile_end[table.nseg - 1] * (cold ? fold_small_parts<kWorld>() : 1))), block(kThreads);
  FoldSmall tab = table;
  tab.shift = xcd_shift(TDM_XCD_FOLD, kWorld, cold);
  if constexpr (!Elem<T>::floating) {
    if (cold) hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 0, true>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv);
    else hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 0, false>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv);
  } else {
    switch (div_kind(divisor, average != 0) * 2 + (cold ? 1 : 0)) {
      case 0: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 0, false>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv); break;
      case 1: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 0, true>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv); break;
      case 2: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 1, false>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv); break;
      case 3: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 1, true>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv); break;
      case 4: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 2, false>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv); break;
      default: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 2, true>), grid, block, occupancy_pad(TDM_XCD_FOLD, cold), stream, tab, dv); break;
    }
  }
}

template <typename T>
void launch_fold_small(const FoldSmall& tab, int world, int average, hipStream_t stream, int divide_by = 0) {
  switch (world) {
    case 2: launch_fold_small_w<T, 2>(tab, average, stream, divide_by); break;
    case 3: launch_fold_small_w<T, 3>(tab, average, stream, divide_by); break;
    case 4: launch_fold_small_w<T, 4>(tab, average, stream, divide_by); break;
    case 5: launch_fold_small_w<T, 5>(tab, average, stream, divide_by); break;
    case 6: launch_fold_small_w<T, 6>(tab, average, stream, divide_by); break;
    case 7: launch_fold_small_w<T, 7>(tab, average, stream, divide_by); break;
    case 8: launch_fold_small_w<T, 8>(tab, average, stream, divide_by); break;
    default: throw Invalid("the direct fold handles world sizes 2..8");
  }
}

template <typename T, bool kAcc>
void launch_fold_a(const void* image, int64_t tiles, int world, int average, hipStream_t stream) {
  switch (world) {
    case 1: launch_fold_w<T, 1, kAcc>(image, tiles, average, stream); break;
    case 2: launch_fold_w<T, 2, kAcc>(image, tiles, average, stream); break;
    case 3: launch_fold_w<T, 3, kAcc>(image, tiles, average, stream); break;
    case 4: launch_fold_w<T, 4, kAcc>(image, tiles, average, stream); break;
    case 5: launch_fold_w<T, 5, kAcc>(image, tiles, average, stream); break;
    case 6: launch_fold_w<T, 6, kAcc>(image, tiles, average, stream); break;
    case 7: launch_fold_w<T, 7, kAcc>(image, tiles, average, stream); break;
    case 8: launch_fold_w<T, 8, kAcc>(image, tiles, average, stream); break;
    default: throw Invalid("world must be in [1, 8]");
  }
}

template <typename T>
void launch_fold(const void* image, int64_t tiles, int world, int average, bool accumulate, hipStream_t stream) {
  if (accumulate) launch_fold_a<T, true>(image, tiles, world, average, stream);
  else launch_fold_a<T, false>(image, tiles, world, average, stream);
}

template <int kWorld, int kOrder>
void launch_step_o(const void* image, int64_t tiles, int average, const tdm_adamw_scalars& s, hipStream_t stream) {
  const Divisor<float> dv = make_divisor<float>(kWorld);
  const StepSegDev* t = static_cast<const StepSegDev*>(image);
  const dim3 grid(grid_for(tiles * kStepParts)), block(kThreads);
  switch (div_kind(kWorld, average != 0)) {
    case 0: hipLaunchKernelGGL((k23_zero2_step_kernel<kWorld, 0, kOrder>), grid, block, occupancy_pad(TDM_XCD_STEP), stream, t, tiles, dv, s, xcd_shift(TDM_XCD_STEP, kWorld, true)); break;
    case 1: hipLaunchKernelGGL((k23_zero2_step_kernel<kWorld, 1, kOrder>), grid, block, occupancy_pad(TDM_XCD_STEP), stream, t, tiles, dv, s, xcd_shift(TDM_XCD_STEP, kWorld, true)); break;
    default: hipLaunchKernelGGL((k23_zero2_step_kernel<kWorld, 2, kOrder>), grid, block, occupancy_pad(TDM_XCD_STEP), stream, t, tiles, dv, s, xcd_shift(TDM_XCD_STEP, kWorld, true)); break;
  }
}

template <int kWorld>
void launch_step_w(const void* image, int64_t tiles, int average, const tdm_adamw_scalars& s, int order, hipStream_t stream) {
  if (order == TDM_ADAMW_HOST_ORDER) launch_step_o<kWorld, TDM_ADAMW_HOST_ORDER>(image, tiles, average, s, stream);
  else launch_step_o<kWorld, TDM_ADAMW_DEVICE_ORDER>(image, tiles, average, s, stream);
}

template <int kWorld, int kOrder>
void launch_step_one_o(const StepSegDev& whole, int64_t tiles, int average, const tdm_adamw_scalars& s, hipStream_t stream) {
  const Divisor<float> dv = make_divisor<float>(kWorld);
  const dim3 grid(grid_for(tiles * kStepParts)), block(kThreads);
  switch (div_kind(kWorld, average != 0)) {
    case 0: hipLaunchKernelGGL((k23_zero2_step_one_kernel<kWorld, 0, kOrder>), grid, block, occupancy_pad(TDM_XCD_STEP), stream, whole, tiles, dv, s, xcd_shift(TDM_XCD_STEP, kWorld, true)); break;
    case 1: hipLaunchKernelGGL((k23_zero2_step_one_kernel<kWorld, 1, kOrder>), grid, block, occupancy_pad(TDM_XCD_STEP), stream, whole, tiles, dv, s, xcd_shift(TDM_XCD_STEP, kWorld, true)); break;
    default: hipLaunchKernelGGL((k23_zero2_step_one_kernel<kWorld, 2, kOrder>), grid, block, occupancy_pad(TDM_XCD_STEP), stream, whole, tiles, dv, s, xcd_shift(TDM_XCD_STEP, kWorld, true)); break;
  }
}

template <int kWorld>
void launch_step_one_w(const StepSegDev& whole, int64_t tiles, int average, const tdm_adamw_scalars& s, int order, hipStream_t stream) {
  if (order == TDM_ADAMW_HOST_ORDER) launch_step_one_o<kWorld, TDM_ADAMW_HOST_ORDER>(whole, tiles, average, s, stream);
  else launch_step_one_o<kWorld, TDM_ADAMW_DEVICE_ORDER>(whole, tiles, average, s, stream);
}

int64_t step_tiles(const tdm_step_seg* segs, int nseg) {
  int64_t tiles = 0;
  for (int i = 0; i < nseg; ++i) tiles += plan_step(segs[i]).tiles;
  return tiles;
}

}  // namespace

namespace {
// One segment as the record the one-segment kernels take in their arguments; *tiles: how many tiles it spans.
StepSegDev whole_segment(const tdm_step_seg& sg, int world, int64_t* tiles) {
  if (sg.chunk < 0 || sg.chunk >= world) throw Invalid("chunk outside [0, world)");
  if (!sg.exp_avg || !sg.exp_avg_sq) throw Invalid("NULL optimizer state");
  const int es = step_elem_size(sg);
  if (es == 0) throw Invalid("a step segment's dtype must be TDM_F32, TDM_F64, TDM_BF16 or TDM_F16");
  StepSegDev whole;
  std::memset(&whole, 0, sizeof whole);
  if (reinterpret_cast<uintptr_t>(sg.exp_avg) % es || reinterpret_cast<uintptr_t>(sg.exp_avg_sq) % es) throw Invalid("pointer not aligned to the element size");
  for (int r = 0; r < world; ++r) {
    if (!sg.grad[r] || !sg.param[r]) throw Invalid("NULL gradient or parameter");
    const uintptr_t a = reinterpret_cast<uintptr_t>(sg.grad[r]), b = reinterpret_cast<uintptr_t>(sg.param[r]);
    if (a % es || b % es) throw Invalid("pointer not aligned to the element size");
  }
  for (int r = world; r < TDM_MAX_WORLD; ++r)
    if (sg.grad[r] || sg.param[r]) throw Invalid("pointers of ranks beyond the world size must be NULL");
  const SegPlan plan = plan_step(sg);
  const int64_t skip = static_cast<int64_t>(plan.head) * es;  // the kernel reaches back for the head
  for (int r = 0; r < world; ++r) {
    whole.g[r] = static_cast<const char*>(sg.grad[r]) + skip;
    whole.p[r] = static_cast<char*>(sg.param[r]) + skip;
  }
  whole.m = static_cast<char*>(sg.exp_avg) + skip;
  whole.v = static_cast<char*>(sg.exp_avg_sq) + skip;
  whole.count = plan.body;
  whole.chunk = sg.chunk;
  whole.vec_ok = plan.vec ? 1 + plan.head : 0;
  *tiles = plan.tiles;
  return whole;
}
}  // namespace

// Used by the engine too: ZeRO-2's step over one segment (a rank's shard), see tdm_k23_zero2_step_segment.
void zero2_step_segment(const tdm_step_seg& sg, int world, bool average, const tdm_adamw_scalars& s, int order, hipStream_t stream) {
  if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
  if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid("unknown update order");
  if (sg.count < 0) throw Invalid("negative count");
  if (sg.count == 0) return;
  if (sg.dtype != TDM_F32) throw Invalid("the step with fp32 constants handles fp32 shards (dtype " + std::to_string(sg.dtype) + "): tdm_k23_zero2_step_segment_typed takes the others");
  int64_t tiles = 0;
  const StepSegDev whole = whole_segment(sg, world, &tiles);
  switch (world) {
    case 1: launch_step_one_w<1>(whole, tiles, average, s, order, stream); break;
    case 2: launch_step_one_w<2>(whole, tiles, average, s, order, stream); break;
    case 3: launch_step_one_w<3>(whole, tiles, average, s, order, stream); break;
    case 4: launch_step_one_w<4>(whole, tiles, average, s, order, stream); break;
    case 5: launch_step_one_w<5>(whole, tiles, average, s, order, stream); break;
    case 6: launch_step_one_w<6>(whole, tiles, average, s, order, stream); break;
    case 7: launch_step_one_w<7>(whole, tiles, average, s, order, stream); break;
    default: launch_step_one_w<8>(whole, tiles, average, s, order, stream); break;
  }
  check_hip(hipGetLastError(), "k23_zero2_step_one launch");
}

namespace {
// A stream parked on a word until a collective that has not run yet has ended: one lane polls the word (pinned host
// memory, written by the engine's stream or, after a failure, by the host) until it has reached `value`, and gives up
// after `limit_ticks` of the device's wall clock, leaving 1 in *gave_up for the host to find: whatever goes wrong with
// the write that should end the wait, the kernel ends.
__global__ void park_kernel(const uint32_t* word, uint32_t value, long long limit_ticks, uint32_t* gave_up) {
  const long long began = wall_clock64();
  for (;;) {
    if (__hip_atomic_load(word, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) >= value) return;
    if (wall_clock64() - began > limit_ticks) {
      __hip_atomic_store(gave_up, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
      return;
    }
    __builtin_amdgcn_s_sleep(16);
  }
}
}  // namespace

// Used by the engine: `stream` waits until *word >= value, for at most limit_s seconds (then *gave_up becomes 1).
void park_stream(hipStream_t stream, const uint32_t* word, uint32_t value, double limit_s, uint32_t* gave_up) {
  if (word == nullptr || gave_up == nullptr) throw Invalid("park_stream: NULL word");
  int device = 0, khz = 0;
  check_hip(hipGetDevice(&device), "hipGetDevice");
  check_hip(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device), "hipDeviceGetAttribute (wall clock rate)");
  if (khz <= 0) throw std::runtime_error("the device reports no wall clock rate");
  const double ticks = std::min(std::max(limit_s, 0.0), 86400.0) * 1e3 * khz;
  hipLaunchKernelGGL(park_kernel, dim3(1), dim3(1), 0, stream, word, value, static_cast<long long>(ticks), gave_up);
  check_hip(hipGetLastError(), "park_kernel launch");
}

// Used by the engine too.
void reduce_step(const tdm_pair* pairs, int npairs, int dtype, int world, bool scale_dst, bool scale_src,
                 bool writeback_src, hipStream_t stream, int policy) {
  const int es = elem_size(dtype);
  if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
  const bool any_scale = (scale_dst || scale_src) && world > 1;
  if (any_scale && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
  PairTable tab;
  const int64_t tiles = build_pairs(pairs, npairs, es, true, kK1TileVecs, &tab);
  if (tiles == 0) return;
  tab.flags = (any_scale && scale_dst ? 1 : 0) | (any_scale && scale_src ? 2 : 0) | (any_scale && scale_src && writeback_src ? 4 : 0) |
              (xcd_shift(TDM_XCD_REDUCE, world, false) << 8);
  switch (dtype) {
    case TDM_F32: launch_reduce<float>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_F64: launch_reduce<double>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_F16: launch_reduce<f16_t>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_BF16: launch_reduce<bf16_t>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_I64: launch_reduce<int64_t>(tab, tiles, 1, false, policy, stream); break;
    case TDM_I32: launch_reduce<int32_t>(tab, tiles, 1, false, policy, stream); break;
    case TDM_I16: launch_reduce<int16_t>(tab, tiles, 1, false, policy, stream); break;
    default: launch_reduce<int8_t>(tab, tiles, 1, false, policy, stream); break;  // TDM_I8 and TDM_U8: the same bits
  }
  check_hip(hipGetLastError(), "k1_reduce launch");
}

void copy_step(const tdm_pair* pairs, int npairs, int dtype, int world, hipStream_t stream, int policy) {
  const int es = elem_size(dtype);
  if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
  if (world > 1 && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
  PairTable tab;
  // dst == src is allowed when scaling in place (div_ of a chunk); partial overlap never is
  if (npairs > 0 && pairs == nullptr) throw Invalid("pairs is NULL");
  if (npairs < 0 || npairs > TDM_MAX_PAIRS) throw Invalid("npairs must be in [0, " + std::to_string(TDM_MAX_PAIRS) + "]");
  tdm_pair kept[TDM_MAX_PAIRS];
  int nkept = 0;
  for (int i = 0; i < npairs; ++i) {
    const tdm_pair& p = pairs[i];
    if (p.dst == p.src && p.count > 0 && world <= 1) continue;  // copying onto itself
    if (p.count > 0 && p.dst != p.src && p.dst != nullptr && p.src != nullptr) {
      const uintptr_t d = reinterpret_cast<uintptr_t>(p.dst), s = reinterpret_cast<uintptr_t>(p.src);
      const uintptr_t bytes = static_cast<uintptr_t>(p.count) * es;
      if (d < s + bytes && s < d + bytes) throw Invalid("copy: destination and source overlap");
    }
    kept[nkept++] = p;
  }
  const int64_t tiles = build_pairs(kept, nkept, es, false, kCopyTileVecs, &tab);
  tab.flags = xcd_shift(TDM_XCD_COPY, world, false) << 8;
  if (tiles == 0) return;
  switch (dtype) {
    case TDM_F32: launch_copy<float>(tab, tiles, world, policy, stream); break;
    case TDM_F64: launch_copy<double>(tab, tiles, world, policy, stream); break;
    case TDM_F16: launch_copy<f16_t>(tab, tiles, world, policy, stream); break;
    case TDM_BF16: launch_copy<bf16_t>(tab, tiles, world, policy, stream); break;
    case TDM_I64: launch_copy<int64_t>(tab, tiles, 1, policy, stream); break;
    case TDM_I32: launch_copy<int32_t>(tab, tiles, 1, policy, stream); break;
    case TDM_I16: launch_copy<int16_t>(tab, tiles, 1, policy, stream); break;
    default: launch_copy<int8_t>(tab, tiles, 1, policy, stream); break;
  }
  check_hip(hipGetLastError(), "k1_copy launch");
}

// ---------------------------------------------------------------- a whole group in one process
// Rank r is bufs[r]; a ring step is ONE launch carrying every rank's pair.
namespace {

struct LocalRanks {
  char* base[TDM_MAX_PAIRS];
  int64_t lo[TDM_MAX_PAIRS], len[TDM_MAX_PAIRS];  // chunk bounds, in elements
  int world, es, dtype;
  int64_t footprint;  // bytes of all ranks' tensors together
};

LocalRanks local_ranks(void* const* bufs, int world, int64_t numel, int dtype, const int64_t* sizes, int nsizes) {
  LocalRanks lr;
  lr.es = elem_size(dtype);
  if (lr.es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
  if (world < 1 || world > TDM_MAX_PAIRS) throw Invalid("world must be in [1, " + std::to_string(TDM_MAX_PAIRS) + "]");
  if (numel < 0) throw Invalid("negative element count");
  if (bufs == nullptr) throw Invalid("NULL rank buffers");
  lr.world = world;
  lr.dtype = dtype;
  lr.footprint = numel * lr.es * world;
  for (int r = 0; r < world; ++r) {
    if (numel > 0 && bufs[r] == nullptr) throw Invalid("rank " + std::to_string(r) + ": NULL buffer");
    lr.base[r] = static_cast<char*>(bufs[r]);
  }
  for (int a = 0; a < world && numel > 0; ++a)
    for (int b = a + 1; b < world; ++b) {
      const uintptr_t x = reinterpret_cast<uintptr_t>(bufs[a]), y = reinterpret_cast<uintptr_t>(bufs[b]);
      const uintptr_t bytes = static_cast<uintptr_t>(numel) * lr.es;
      if (x < y + bytes && y < x + bytes) throw Invalid("rank buffers overlap");
    }
  if (nsizes == 0) {  // as torch.tensor_split cuts
    const int64_t base = numel / world, extra = numel % world;
    int64_t at = 0;
    for (int q = 0; q < world; ++q) {
      lr.lo[q] = at;
      lr.len[q] = base + (q < extra ? 1 : 0);
      at += lr.len[q];
    }
  } else {
    if (nsizes != world || sizes == nullptr) throw Invalid("chunk sizes do not partition the tensor");
    int64_t at = 0;
    for (int q = 0; q < world; ++q) {
      if (sizes[q] < 0) throw Invalid("chunk sizes do not partition the tensor");
      lr.lo[q] = at;
      lr.len[q] = sizes[q];
      at += sizes[q];
    }
    if (at != numel) throw Invalid("chunk sizes do not partition the tensor");
  }
  return lr;
}

int wrap(int a, int n) { return ((a % n) + n) % n; }

// Step s: rank r adds chunk (r-s-2) of rank r-1 into its own (tandem/comm.py:301-305).
// Every receiving chunk is still undivided; the sender's only on the first step.
// Cache policy of each step of a ring on one GPU, from searches over the policies of
// every step at 8 MiB - 1 GiB per rank (TB/s over the whole reduce-scatter + all-gather
// at 256 MiB per rank, against policy 2 throughout): W=2: 7.07 vs 6.90 (64 MiB: 6.77 vs
// 6.33); W=3: 6.85 vs 6.47; W=4: 7.04 vs 6.59; W=8: nothing gained.
// What the winners at W=4 share. Footprint beyond the 256 MB Infinity Cache: the first
// reduce step, which touches everything for the first time, loads and stores non-
// temporally; the last step of either phase stores non-temporally and loads plainly
// what the step before it has just written. Footprint that fits (up to 80 MiB per rank;
// 64 MiB: 6.76 vs 6.57, 16 MiB: 5.99 vs 5.75): after the first touch everything stays
// cached, only the very last stores are non-temporal. At W=2 and W=3 a footprint that
// fits with room to spare does best with everything cached.
int ring_policy(int world, int step, bool gather, int64_t footprint_bytes) {
  // Measurement knob: TDM_RING_POLICY="r0,r1,...,g0,g1,..." (one digit per step; reduce steps, then gather steps).
  static const std::string knob = [] { const char* e = std::getenv("TDM_RING_POLICY"); return std::string(e ? e : ""); }();  // read once
  if (!knob.empty()) {
    const char* env = knob.c_str();
    const size_t at = static_cast<size_t>(2 * ((gather ? world - 1 : 0) + step));
#ifdef TDM_ALL_POLICIES
    if (std::strlen(env) > at && env[at] >= '0' && env[at] <= '7') return env[at] - '0';
#else
    if (std::strlen(env) > at && (env[at] == '0' || env[at] == '5' || env[at] == '7')) return env[at] - '0';
#endif
    return TDM_NT_MASK;
  }
  const bool first = step == 0, last = step == world - 2;
  switch (world) {
    case 2:
      if (footprint_bytes <= (int64_t(80) << 20)) return 0;  // 32 MiB per rank: 6.94 vs 6.56
      return gather ? 7 : TDM_NT_MASK;
    case 3:
      if (footprint_bytes <= (int64_t(224) << 20)) return 0;  // 64 MiB per rank: 6.54 vs 6.11; 16 MiB: 5.20 vs 4.03
      return last ? 5 : TDM_NT_MASK;
    case 4:
      if (footprint_bytes <= (int64_t(352) << 20)) return gather ? (last ? 5 : 0) : (first ? 7 : last ? TDM_NT_MASK : 0);
      return gather ? (last ? 5 : TDM_NT_MASK) : (first ? 7 : last ? 5 : TDM_NT_MASK);
    default: return TDM_NT_MASK;
  }
}

int64_t footprint(const LocalRanks& lr) { return lr.footprint; }

// Which form a ring collective of buffer ranks takes: its W-1 steps, one launch each, or the
// whole reduce-scatter (all-gather) as ONE launch. -1: by world size. The one-launch forms read
// every rank's copy of a chunk once and write the W-1 partial sums (read the owner's chunk once
// and write the W-1 copies), 4 (2W-1) (4 W) bytes per element where the steps move 12 (W-1)
// (8 (W-1)), and leave no gaps between launches. Measured on MI355X, reduce-scatter, steps
// against one launch: world 4 at 4 MiB per rank 15.3 against 10.4 us, 16 MiB 25.8 / 21.6, 64 MiB
// 88 / 70, 96 MiB 132 / 120, 128 MiB 175 / 152, 256 MiB 337 / 291 (once the ranks' tensors together
// exceed 320 MiB: non-temporal accesses, 2 KiB per workgroup and stream and an occupancy cap; with
// everything cached and 4 KiB the one launch loses there, 343); world 3 at 64 MiB 65 / 55,
// 96 MiB 94 / 79, 256 MiB 235 / 211; world 5 at 16 MiB 45 / 31, 256 MiB 514 / 405; world 8 at 4 MiB
// 29.5 / 14, 16 MiB 64 / 41, 256 MiB 861 / 667, 1 GiB 3690 / 2630.
// At world 2 a collective is one step anyway and the step kernels' policies do better (64 MiB
// 49 / 51 us, 256 MiB 186 / 236).
std::atomic<int> g_ring_form{-1};
constexpr int64_t kOneLaunchFootprint = int64_t(296) << 20;  // beyond: nothing written is found in the caches again (world 4, reduce-scatter at 320 MiB: 112 us with the cached kernel, 99 with the other)

bool one_launch_form(const LocalRanks& lr) {
  if (!chain_handles(lr.world)) return false;
  const int set = g_ring_form.load(std::memory_order_relaxed);
  return set >= 0 ? set == 1 : lr.world >= 3;
}

// The all-gather as one launch wins at every size from world 3 on (world 4, 256 MiB per rank: 236 -> 191 us;
// 16 MiB: 22.5 -> 13.5; world 8, 256 MiB: 556 -> 383): it moves 4 W instead of 8 (W-1) bytes per element. At
// world 2 both forms are one launch and the step kernel's policy does better (74 against 80 us at 256 MiB).
bool gather_in_one_launch(const LocalRanks& lr) {
  if (!gather_handles(lr.world)) return false;
  const int set = g_ring_form.load(std::memory_order_relaxed);
  return set >= 0 ? set == 1 : lr.world >= 3;
}

void local_reduce_scatter(const LocalRanks& lr, bool average, bool keep_sent, hipStream_t stream) {
  const int n = lr.world;
  if (one_launch_form(lr)) {
    const int64_t cap = static_cast<int64_t>(t_call_cus ? t_call_cus : compute_units()) * g_blocks_per_cu;
    const bool cold = lr.footprint > kOneLaunchFootprint;
    if (chain_reduce_scatter(lr.base, lr.lo, lr.len, n, lr.dtype, lr.es, average, keep_sent, cold,
                             occupancy_pad(TDM_XCD_REDUCE, cold, n), xcd_shift(TDM_XCD_REDUCE, n, cold),
                             static_cast<int>(std::min<int64_t>(cap, int64_t(1) << 30)), stream)) {
      return;
    }
  }
  for (int s = 0; s < n - 1; ++s) {
    tdm_pair pairs[TDM_MAX_PAIRS];
    int np = 0;
    for (int r = 0; r < n; ++r) {
      const int c = wrap(r - s - 2, n);
      if (lr.len[c] == 0) continue;
      pairs[np++] = tdm_pair{lr.base[r] + lr.lo[c] * lr.es, lr.base[wrap(r - 1, n)] + lr.lo[c] * lr.es, lr.len[c]};
    }
    if (np) reduce_step(pairs, np, lr.dtype, average ? n : 1, true, s == 0, s == 0 && keep_sent, stream, ring_policy(n, s, false, footprint(lr)));
  }
}

// Step s: rank r copies chunk (r-s-1) from rank r-1 (tandem/comm.py:307-311).
void local_all_gather(const LocalRanks& lr, hipStream_t stream) {
  const int n = lr.world;
  if (gather_in_one_launch(lr)) {
    // every chunk is read once from its owner and stored into the other ranks' buffers: the ring's W-1
    // forwarding steps leave the same bytes
    const int64_t cap = static_cast<int64_t>(t_call_cus ? t_call_cus : compute_units()) * g_blocks_per_cu;
    const bool cold = lr.footprint > kOneLaunchFootprint;
    // beyond the caches: 2 KiB per workgroup and stream and 16 KiB of occupancy pad (world 4, 256 MiB per rank: 189 us with
    // 4 KiB and no pad, 174 with the pad, 168 with both; 32 KiB: 202-232)
    gather_multicast(lr.base, lr.lo, lr.len, n, lr.es, cold, occupancy_pad(TDM_XCD_COPY, cold), xcd_shift(TDM_XCD_COPY, n, cold),
                     cold ? 1 : kWarmVecs, static_cast<int>(std::min<int64_t>(cap, int64_t(1) << 30)), stream);
    return;
  }
  for (int s = 0; s < n - 1; ++s) {
    tdm_pair pairs[TDM_MAX_PAIRS];
    int np = 0;
    for (int r = 0; r < n; ++r) {
      const int c = wrap(r - s - 1, n);
      if (lr.len[c] == 0) continue;
      pairs[np++] = tdm_pair{lr.base[r] + lr.lo[c] * lr.es, lr.base[wrap(r - 1, n)] + lr.lo[c] * lr.es, lr.len[c]};
    }
    if (np) copy_step(pairs, np, lr.dtype, 0, stream, ring_policy(n, s, true, footprint(lr)));
  }
}

// The whole all-reduce as one launch: every element is read from all ranks,
// folded in the ring's order for its chunk and written to all ranks.
void local_all_reduce_fold(const LocalRanks& lr, bool average, hipStream_t stream) {
  const int n = lr.world;
  tdm_fold_seg segs[TDM_MAX_WORLD];
  std::memset(segs, 0, sizeof segs);
  for (int c = 0; c < n; ++c) {
    for (int r = 0; r < n; ++r) {
      char* p = lr.base[r] + lr.lo[c] * lr.es;
      segs[c].src[r] = p;
      segs[c].dst[r] = p;
    }
    segs[c].count = lr.len[c];
    segs[c].chunk = c;
  }
  fold_step(segs, n, n, lr.dtype, average, stream);
}

}  // namespace

// Up to 8 segments folded in one launch, the table passed by value. Used by the
// engine too (a rank folding its own chunk out of its peers' shared arenas).
void fold_step(const tdm_fold_seg* segs, int nseg, int world, int dtype, bool average, hipStream_t stream, int divide_by) {
  const int es = elem_size(dtype);
  if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
  if (world < 2 || world > TDM_MAX_WORLD) throw Invalid("the direct fold handles world sizes 2..8");
  if (nseg < 0 || nseg > TDM_MAX_WORLD || (nseg > 0 && segs == nullptr)) throw Invalid("the direct fold takes up to 8 segments");
  if (average && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
  FoldSmall tab;
  std::memset(&tab, 0, sizeof tab);
  int64_t tiles = 0;
  int k = 0;
  for (int i = 0; i < nseg; ++i) {
    const tdm_fold_seg& s = segs[i];
    if (s.count < 0) throw Invalid("fold: negative count");
    if (s.count == 0) continue;
    if (s.chunk < 0 || s.chunk >= world) throw Invalid("fold: chunk outside [0, world)");
    for (int r = 0; r < world; ++r) {
      if (s.src[r] == nullptr) throw Invalid("fold: NULL source");
      const uintptr_t a = reinterpret_cast<uintptr_t>(s.src[r]), b = reinterpret_cast<uintptr_t>(s.dst[r]);
      if (a % es || b % es) throw Invalid("fold: pointer not aligned to the element size");
    }
    for (int r = world; r < TDM_MAX_WORLD; ++r)
      if (s.src[r] || s.dst[r]) throw Invalid("fold: pointers of ranks beyond the world size must be NULL");
    const SegPlan plan = plan_fold(s, es);
    const int64_t skip = static_cast<int64_t>(plan.head) * es;  // the kernel reaches back for the head
    for (int r = 0; r < world; ++r) {
      tab.seg[k].src[r] = static_cast<const char*>(s.src[r]) + skip;
      tab.seg[k].dst[r] = s.dst[r] ? static_cast<char*>(s.dst[r]) + skip : nullptr;
    }
    tab.seg[k].count = plan.body;
    tab.seg[k].chunk = s.chunk;
    tab.seg[k].vec_ok = plan.vec ? 1 + plan.head : 0;
    tiles += plan.tiles;
    tab.tile_end[k] = tiles;
    ++k;
  }
  tab.nseg = k;
  if (k == 0) return;
  switch (dtype) {
    case TDM_F32: launch_fold_small<float>(tab, world, average, stream, divide_by); break;
    case TDM_F64: launch_fold_small<double>(tab, world, average, stream, divide_by); break;
    case TDM_F16: launch_fold_small<f16_t>(tab, world, average, stream, divide_by); break;
    case TDM_BF16: launch_fold_small<bf16_t>(tab, world, average, stream, divide_by); break;
    case TDM_I64: launch_fold_small<int64_t>(tab, world, 0, stream); break;
    case TDM_I32: launch_fold_small<int32_t>(tab, world, 0, stream); break;
    case TDM_I16: launch_fold_small<int16_t>(tab, world, 0, stream); break;
    default: launch_fold_small<int8_t>(tab, world, 0, stream); break;
  }
  check_hip(hipGetLastError(), "k2_fold_small launch");
}

}  // namespace tandem_hip

using namespace tandem_hip;

extern "C" {

int tdm_local_reduce_scatter(void* const* bufs, int world, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                             int average, int keep_sent, tdm_stream stream) {
  return guard([&] {
    CallScope scope;
    if (average && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
    const LocalRanks lr = local_ranks(bufs, world, numel, dtype, sizes, nsizes);
    if (world > 1) local_reduce_scatter(lr, average != 0, keep_sent != 0, static_cast<hipStream_t>(stream));
  });
}

int tdm_local_all_gather(void* const* bufs, int world, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                         tdm_stream stream) {
  return guard([&] {
    CallScope scope;
    const LocalRanks lr = local_ranks(bufs, world, numel, dtype, sizes, nsizes);
    if (world > 1) local_all_gather(lr, static_cast<hipStream_t>(stream));
  });
}

int tdm_local_all_reduce(void* const* bufs, int world, int64_t numel, int dtype, int average, int algorithm,
                         tdm_stream stream) {
  return guard([&] {
    CallScope scope;
    if (average && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
    if (algorithm != TDM_ALLREDUCE_RING && algorithm != TDM_ALLREDUCE_FOLD) throw Invalid("unknown all-reduce algorithm");
    const LocalRanks lr = local_ranks(bufs, world, numel, dtype, nullptr, 0);
    if (world == 1) return;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (algorithm == TDM_ALLREDUCE_FOLD) {
      if (world > TDM_MAX_WORLD) throw Invalid("the direct fold handles world sizes up to 8");
      local_all_reduce_fold(lr, average != 0, st);
    } else {
      local_reduce_scatter(lr, average != 0, false, st);
      local_all_gather(lr, st);
    }
  });
}

int tdm_table_tile_bytes(void) { return kTileVecs * 16; }

int tdm_build_geometry(int* k1_tile_bytes, int* workgroup_lanes, int* table_tile_bytes) {
  return guard([&] {
    if (!k1_tile_bytes || !workgroup_lanes || !table_tile_bytes) throw Invalid("NULL argument");
    *k1_tile_bytes = kK1TileVecs * 16;
    *workgroup_lanes = kThreads;
    *table_tile_bytes = kTileVecs * 16;
  });
}

int tdm_set_blocks_per_cu(int blocks) {
  return guard([&] {
    if (blocks < 0 || blocks > kDefaultBlocksPerCu) throw Invalid("blocks per compute unit must be in [0, " + std::to_string(kDefaultBlocksPerCu) + "]");
    g_blocks_per_cu = blocks == 0 ? kDefaultBlocksPerCu : blocks;
  });
}

int tdm_set_ring_form(int form) {
  return guard([&] {
    if (form < -1 || form > 1) throw Invalid("the ring form is 0 (steps), 1 (one launch) or -1 (by footprint)");
    g_ring_form.store(form, std::memory_order_relaxed);
  });
}

int tdm_set_occupancy_pad(int kind, int bytes) {
  return guard([&] {
    if (kind < -1 || kind >= kXcdKinds) throw Invalid("unknown kernel family");
    if (bytes < -1 || bytes > 65536) throw Invalid("the pad must be in [0, 65536] bytes, or -1 for the default");
    for (int k = 0; k < kXcdKinds; ++k)
      if (kind == -1 || kind == k) g_occupancy_pad[k].store(bytes, std::memory_order_relaxed);
  });
}

int tdm_set_xcd_group(int kind, int shift) {
  return guard([&] {
    if (kind < -1 || kind >= kXcdKinds) throw Invalid("unknown kernel family");
    if (shift < -1 || shift > 12) throw Invalid("the group shift must be in [0, 12], or -1 for the default");
    for (int k = 0; k < kXcdKinds; ++k)
      if (kind == -1 || kind == k) g_xcd_shift[k].store(shift, std::memory_order_relaxed);
  });
}

int64_t tdm_tile_of(int64_t index, int64_t total, int shift) {
  if (index < 0 || index >= total || shift < 0 || shift > 12) return -1;
  return tile_of(index, total, shift);
}

int tdm_k1_reduce_step(const tdm_pair* pairs, int npairs, int dtype, int world, int scale_dst, int scale_src,
                       int writeback_src, tdm_stream stream) {
  return guard([&] {
    reduce_step(pairs, npairs, dtype, world, scale_dst != 0, scale_src != 0, writeback_src != 0,
                static_cast<hipStream_t>(stream));
  });
}

int tdm_k1_copy_step(const tdm_pair* pairs, int npairs, int dtype, int world, tdm_stream stream) {
  return guard([&] { copy_step(pairs, npairs, dtype, world, static_cast<hipStream_t>(stream)); });
}

namespace {
int64_t fold_tiles(const tdm_fold_seg* segs, int nseg, int es) {
  int64_t tiles = 0;
  for (int i = 0; i < nseg; ++i) tiles += plan_fold(segs[i], es).tiles;
  return tiles;
}
}  // namespace

int64_t tdm_k2_table_tiles(const tdm_fold_seg* segs, int nseg, int dtype) {
  const int es = elem_size(dtype);
  if (nseg < 0 || es == 0 || (nseg > 0 && segs == nullptr)) return -1;
  return fold_tiles(segs, nseg, es);
}

int64_t tdm_k2_table_bytes(const tdm_fold_seg* segs, int nseg, int dtype) {
  const int64_t tiles = tdm_k2_table_tiles(segs, nseg, dtype);
  if (tiles < 0) return -1;
  return std::max<int64_t>(16, tiles * static_cast<int64_t>(sizeof(FoldSegDev)));
}

namespace {
// Checks segment i of a K2 table and says how it is walked.
SegPlan fold_seg_check(const tdm_fold_seg& s, int i, int world, int es) {
  if (s.count < 0) throw Invalid("segment " + std::to_string(i) + ": negative count");
  if (s.chunk < 0 || s.chunk >= world) throw Invalid("segment " + std::to_string(i) + ": chunk outside [0, world)");
  for (int r = 0; r < TDM_MAX_WORLD; ++r) {
    if (r >= world) {
      if (s.src[r] || s.dst[r]) throw Invalid("segment " + std::to_string(i) + ": pointers of ranks beyond the world size must be NULL");
      continue;
    }
    if (s.count > 0 && s.src[r] == nullptr) throw Invalid("segment " + std::to_string(i) + ": NULL source");
    const uintptr_t a = reinterpret_cast<uintptr_t>(s.src[r]), b = reinterpret_cast<uintptr_t>(s.dst[r]);
    if (a % es || b % es) throw Invalid("segment " + std::to_string(i) + ": pointer not aligned to the element size");
  }
  return plan_fold(s, es);
}
}  // namespace

int tdm_k2_table_build(const tdm_fold_seg* segs, int nseg, int world, int dtype, void* image) {
  return guard([&] {
    const int es = elem_size(dtype);
    if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
    if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
    if (nseg < 0 || (nseg > 0 && segs == nullptr) || image == nullptr) throw Invalid("bad table arguments");
    std::memset(image, 0, static_cast<size_t>(tdm_k2_table_bytes(segs, nseg, dtype)));
    FoldSegDev* out = static_cast<FoldSegDev*>(image);
    const int64_t tile_elems = static_cast<int64_t>(kTileVecs) * (16 / es);
    int64_t tiles = 0;
    for (int i = 0; i < nseg; ++i) {
      const tdm_fold_seg& s = segs[i];
      const SegPlan plan = fold_seg_check(s, i, world, es);
      // records describe the body (the segment without its peeled head): a record's byte offset within it is a
      // multiple of 4 KiB; the first record also carries the head
      for (int64_t at = 0; at < plan.body && s.count > 0; at += tile_elems) {
        FoldSegDev& rec = out[tiles++];
        for (int r = 0; r < world; ++r) {
          rec.src[r] = static_cast<const char*>(s.src[r]) + (plan.head + at) * es;
          rec.dst[r] = s.dst[r] ? static_cast<char*>(s.dst[r]) + (plan.head + at) * es : nullptr;
        }
        rec.count = std::min<int64_t>(tile_elems, plan.body - at);
        rec.chunk = s.chunk;
        rec.vec_ok = plan.vec ? (at == 0 ? 1 + plan.head : 1) : 0;
      }
    }
  });
}

namespace {
void bucket_fold(const void* table_dev, int64_t ntiles, int dtype, int world, int average, int accumulate, hipStream_t st) {
  if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
  if (ntiles < 0) throw Invalid("ntiles is negative");
  if (ntiles == 0) return;
  if (table_dev == nullptr) throw Invalid("table is NULL");
  if (average && world > 1 && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
  switch (dtype) {
    case TDM_F32: launch_fold<float>(table_dev, ntiles, world, average, accumulate != 0, st); break;
    case TDM_F64: launch_fold<double>(table_dev, ntiles, world, average, accumulate != 0, st); break;
    case TDM_F16: launch_fold<f16_t>(table_dev, ntiles, world, average, accumulate != 0, st); break;
    case TDM_BF16: launch_fold<bf16_t>(table_dev, ntiles, world, average, accumulate != 0, st); break;
    case TDM_I64: launch_fold<int64_t>(table_dev, ntiles, world, 0, accumulate != 0, st); break;
    case TDM_I32: launch_fold<int32_t>(table_dev, ntiles, world, 0, accumulate != 0, st); break;
    case TDM_I16: launch_fold<int16_t>(table_dev, ntiles, world, 0, accumulate != 0, st); break;
    case TDM_I8: case TDM_U8: launch_fold<int8_t>(table_dev, ntiles, world, 0, accumulate != 0, st); break;
    default: throw Invalid("unknown dtype " + std::to_string(dtype));
  }
  check_hip(hipGetLastError(), "k2_fold launch");
}
}  // namespace

int tdm_k2_bucket_fold(const void* table_dev, int64_t ntiles, int dtype, int world, int average, int accumulate,
                       tdm_stream stream) {
  return guard([&] { bucket_fold(table_dev, ntiles, dtype, world, average, accumulate, static_cast<hipStream_t>(stream)); });
}

// ---- the same fold for callers that cannot allocate: the table lives in a fixed device array
namespace {
// This GPU's copy of `scratch`, looked up once per device with that device current. The array's
// name is only a host-side handle: everything below uses the address kept here. With it, what orders
// the calls that share the table: a mutex held while a call enqueues its launches, the stream of the
// last call, and an event recorded behind that call's fold (created once, at the same set-up).
struct StaticTable {
  std::mutex mu;
  FoldSegDev* table = nullptr;
  hipEvent_t folded = nullptr;   // recorded after the last call's fold kernel
  hipStream_t last = nullptr;    // the stream of that call
  bool pending = false;          // `folded` has been recorded at least once
};

StaticTable* static_table() {
  constexpr int kMaxDevices = 64;
  static std::mutex setup;
  static StaticTable per_device[kMaxDevices];
  int dev = 0;
  check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) throw std::runtime_error("device index beyond 63");
  StaticTable& t = per_device[dev];
  std::lock_guard<std::mutex> lock(setup);
  if (t.table == nullptr) {
    void* p = nullptr;
    check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (p == nullptr) throw std::runtime_error("hipGetSymbolAddress(scratch) returned NULL");
    check_hip(hipEventCreateWithFlags(&t.folded, hipEventDisableTiming), "hipEventCreate");
    t.table = static_cast<FoldSegDev*>(p);
  }
  return &t;
}
}  // namespace

int64_t tdm_k2_static_max_tiles(void) { return kStaticTiles; }

int tdm_k2_bucket_fold_static(const tdm_fold_seg* segs, int nseg, int world, int dtype, int average, int accumulate,
                              tdm_stream stream) {
  return guard([&] {
    const int es = elem_size(dtype);
    if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
    if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
    if (nseg < 0 || (nseg > 0 && segs == nullptr)) throw Invalid("bad table arguments");
    if (average && world > 1 && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
    const int64_t tile_elems = static_cast<int64_t>(kTileVecs) * (16 / es);
    // every segment is checked, and the size known, before the first launch
    int64_t tiles = 0;
    for (int i = 0; i < nseg; ++i) {
      tiles += fold_seg_check(segs[i], i, world, es).tiles;
      if (tiles > kStaticTiles) {
        throw Invalid("the segments need more than " + std::to_string(kStaticTiles) + " table records (" +
                      std::to_string(kStaticTiles * static_cast<int64_t>(kTileVecs) * 16) +
                      " bytes of every rank's stream): beyond the fixed table of tdm_k2_bucket_fold_static; "
                      "split the call or use tdm_k2_table_build + tdm_k2_bucket_fold");
      }
    }
    if (tiles == 0) return;
    hipStream_t st = static_cast<hipStream_t>(stream);
    StaticTable& shared = *static_table();
    FoldSegDev* table = shared.table;
    // One call at a time enqueues its launches, and a call on another stream than the last one first waits, on the
    // GPU, for that call's fold: the records it is about to overwrite may still be in use there. A stream under
    // capture takes no part in this (a wait or a record would become nodes of the caller's graph).
    std::lock_guard<std::mutex> turn(shared.mu);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    check_hip(hipStreamIsCapturing(st, &capture), "hipStreamIsCapturing");
    const bool eager = capture == hipStreamCaptureStatusNone;
    if (eager && shared.pending && shared.last != st) check_hip(hipStreamWaitEvent(st, shared.folded, 0), "hipStreamWaitEvent");
    FillBatch batch;
    std::memset(&batch, 0, sizeof batch);
    batch.world = world;
    batch.es = es;
    batch.tile_elems = tile_elems;
    int64_t at = 0;  // records written by the batches before this one
    auto flush = [&] {
      if (batch.nseg == 0) return;
      const int64_t n = batch.first[batch.nseg] - batch.first[0];
      hipLaunchKernelGGL(k2_table_fill_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, batch, table);
      check_hip(hipGetLastError(), "k2_table_fill launch");
      batch.nseg = 0;
    };
    for (int i = 0; i < nseg; ++i) {
      const tdm_fold_seg& s = segs[i];
      if (s.count == 0) continue;
      const int k = batch.nseg;
      const SegPlan plan = plan_fold(s, es);
      batch.first[k] = at;
      at += plan.tiles;
      batch.first[k + 1] = at;
      batch.vec_ok[k] = plan.vec ? 1 + plan.head : 0;
      batch.seg[k] = s;  // the fill kernel sees the body: the segment without its peeled head
      for (int r = 0; r < world; ++r) {
        batch.seg[k].src[r] = static_cast<const char*>(s.src[r]) + static_cast<int64_t>(plan.head) * es;
        if (s.dst[r]) batch.seg[k].dst[r] = static_cast<char*>(s.dst[r]) + static_cast<int64_t>(plan.head) * es;
      }
      batch.seg[k].count = plan.body;
      if (++batch.nseg == kFillSegs) flush();
    }
    flush();
    bucket_fold(table, tiles, dtype, world, average, accumulate, st);
    if (eager) {
      check_hip(hipEventRecord(shared.folded, st), "hipEventRecord");
      shared.last = st;
      shared.pending = true;
    }
  });
}

namespace {
void adamw_launch(float* p, const float* g, float* m, float* v, int64_t n, const tdm_adamw_scalars* s, int order,
                  float* const* copies, int ncopies, hipStream_t st) {
  if (n < 0) throw Invalid("n is negative");
  if (ncopies < 0 || ncopies > TDM_MAX_WORLD - 1) throw Invalid("at most 7 further copies of the parameters");
  if (n == 0) return;
  if (!p || !g || !m || !v || !s || (ncopies > 0 && !copies)) throw Invalid("NULL argument");
  if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid("unknown update order");
  uintptr_t ptrs[4 + TDM_MAX_WORLD - 1] = {reinterpret_cast<uintptr_t>(p), reinterpret_cast<uintptr_t>(g),
                                           reinterpret_cast<uintptr_t>(m), reinterpret_cast<uintptr_t>(v)};
  AdamwArgs a{p, g, m, v, n, *s, ncopies, xcd_shift(TDM_XCD_ADAMW, 1, true), 0, {}};
  for (int c = 0; c < ncopies; ++c) {
    if (!copies[c]) throw Invalid("NULL copy of the parameters");
    a.copy[c] = copies[c];
    ptrs[4 + c] = reinterpret_cast<uintptr_t>(copies[c]);
  }
  for (int i = 0; i < 4 + ncopies; ++i)
    if (ptrs[i] % 4) throw Invalid("pointer not aligned to 4 bytes");
  for (int i = 0; i < 4 + ncopies; ++i)
    for (int j = i + 1; j < 4 + ncopies; ++j) {
      const uintptr_t bytes = static_cast<uintptr_t>(n) * 4;
      if (ptrs[i] < ptrs[j] + bytes && ptrs[j] < ptrs[i] + bytes) throw Invalid("p, g, m, v and the copies must not overlap");
    }
  // A shard cut out of a flat buffer starts anywhere (tensor_split). When all the streams start at the same distance
  // from a 16-byte boundary, the few elements before it are peeled off and the rest runs on vectors ...
  const SegPlan plan = plan_segment(ptrs, 4 + ncopies, n, 4, static_cast<int64_t>(kAdamwThreads) * kAdamwUnroll * 4);
  const bool vec = plan.vec;
  if (vec) {
    // ... and when the streams also agree on their distance from a 128-byte boundary, the head is stretched to it
    // (up to 31 elements): every wave then writes whole cache lines, which no other wave touches.
    int64_t head = plan.head;
    const uintptr_t line = (ptrs[0] + head * 4) % 128;
    bool same = true;
    for (int i = 1; i < 4 + ncopies; ++i) same = same && (ptrs[i] + head * 4) % 128 == line;
    const int64_t more = static_cast<int64_t>((128 - line) % 128) / 4;
    if (same && more < plan.body) head += more;
    if (head) {
      a.p += head, a.g += head, a.m += head, a.v += head;
      for (int c = 0; c < ncopies; ++c) a.copy[c] += head;
      a.n = n - head;
      a.head = static_cast<int>(head);
    }
  }
  const dim3 block(kAdamwThreads);
  const int64_t tiles = vec ? (a.n / 4 + kAdamwThreads * kAdamwUnroll - 1) / (kAdamwThreads * kAdamwUnroll) : (n + kAdamwThreads - 1) / kAdamwThreads;
  const dim3 grid(grid_for(std::max<int64_t>(tiles, 1)));
  const int which = (order == TDM_ADAMW_HOST_ORDER ? 0 : 4) + (vec ? 2 : 0) + (ncopies > 0 ? 1 : 0);
  const unsigned pad = occupancy_pad(TDM_XCD_ADAMW);
  switch (which) {
    case 0: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, false, false>), grid, block, pad, st, a); break;
    case 1: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, false, true>), grid, block, pad, st, a); break;
    case 2: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, true, false>), grid, block, pad, st, a); break;
    case 3: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, true, true>), grid, block, pad, st, a); break;
    case 4: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, false, false>), grid, block, pad, st, a); break;
    case 5: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, false, true>), grid, block, pad, st, a); break;
    case 6: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, true, false>), grid, block, pad, st, a); break;
    default: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, true, true>), grid, block, pad, st, a); break;
  }
  check_hip(hipGetLastError(), "k3_adamw launch");
}
}  // namespace

int tdm_k3_adamw(float* p, const float* g, float* m, float* v, int64_t n, const tdm_adamw_scalars* s, int order,
                 tdm_stream stream) {
  return guard([&] { adamw_launch(p, g, m, v, n, s, order, nullptr, 0, static_cast<hipStream_t>(stream)); });
}

int tdm_k3_adamw_gather(float* p, const float* g, float* m, float* v, int64_t n, const tdm_adamw_scalars* s, int order,
                        float* const* copies, int ncopies, tdm_stream stream) {
  return guard([&] { adamw_launch(p, g, m, v, n, s, order, copies, ncopies, static_cast<hipStream_t>(stream)); });
}

extern "C++" {
namespace {
// eps as add_(eps) applies it to a 16-bit tensor: rounded to the tensor's type (nearest even), as a float again.
template <typename T>
float eps_as_applied(double eps) {
  const float e = static_cast<float>(eps);
  if constexpr (std::is_same_v<T, bf16_t>) {
    uint32_t u;
    std::memcpy(&u, &e, 4);
    u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
    float rounded;
    std::memcpy(&rounded, &u, 4);
    return rounded;
  } else if constexpr (std::is_same_v<T, f16_t>) {
    return static_cast<float>(static_cast<_Float16>(e));
  } else {
    return e;
  }
}

// The step's constants as the kernels for T take them.
template <typename T>
AdamwHyper<typename AdamwMath<T>::S> typed_hyper(const tdm_adamw_hyper& h) {
  using S = typename AdamwMath<T>::S;
  AdamwHyper<S> s{};
  s.use_decay = h.use_decay;
  s.decay = static_cast<S>(h.decay), s.w1 = static_cast<S>(h.w1), s.beta2 = static_cast<S>(h.beta2);
  s.one_m_b2 = static_cast<S>(h.one_m_b2), s.bc2_sqrt = static_cast<S>(h.bc2_sqrt), s.neg_step = static_cast<S>(h.neg_step);
  s.eps = static_cast<S>(h.eps);
  if constexpr (sizeof(T) == 2) s.eps = eps_as_applied<T>(h.eps);
  // bfloat16's way round the division by bc2_sqrt: a product with the reciprocal, redone as a division where the low
  // 16 bits of the product come within 6 of a rounding tie (0x8000); the product is within 2.5 ulps of the quotient
  // as long as neither leaves the normal floats, which a divisor within [2^-30, 2^30] guarantees for every square
  // root of a bfloat16. Any other divisor: every element by division.
  s.inv_bc2 = static_cast<S>(1.0 / static_cast<double>(s.bc2_sqrt));
  constexpr uint32_t kWindow = 6;
  const bool usual = s.bc2_sqrt >= S(0x1p-30) && s.bc2_sqrt <= S(0x1p30);
  s.tie_bias = usual ? (kWindow - 0x8000u) & 0xffffu : 0u;
  s.tie_span = usual ? 2 * kWindow : 0xffffu;
  return s;
}

template <typename T>
void adamw_typed_launch(void* p_, const void* g_, void* m_, void* v_, int64_t n, const tdm_adamw_hyper& h, void* const* copies,
                        int ncopies, hipStream_t st) {
  constexpr int es = static_cast<int>(sizeof(T));
  uintptr_t ptrs[4 + TDM_MAX_WORLD - 1] = {reinterpret_cast<uintptr_t>(p_), reinterpret_cast<uintptr_t>(g_),
                                           reinterpret_cast<uintptr_t>(m_), reinterpret_cast<uintptr_t>(v_)};
  AdamwArgsT<T> a{};
  a.p = static_cast<T*>(p_), a.g = static_cast<const T*>(g_), a.m = static_cast<T*>(m_), a.v = static_cast<T*>(v_);
  a.n = n;
  a.s = typed_hyper<T>(h);
  a.ncopies = ncopies;
  a.shift = xcd_shift(TDM_XCD_ADAMW, 1, true);
  for (int c = 0; c < ncopies; ++c) {
    if (!copies[c]) throw Invalid("NULL copy of the parameters");
    a.copy[c] = static_cast<T*>(copies[c]);
    ptrs[4 + c] = reinterpret_cast<uintptr_t>(copies[c]);
  }
  for (int i = 0; i < 4 + ncopies; ++i)
    if (ptrs[i] % es) throw Invalid("pointer not aligned to the element size");
  for (int i = 0; i < 4 + ncopies; ++i)
    for (int j = i + 1; j < 4 + ncopies; ++j) {
      const uintptr_t bytes = static_cast<uintptr_t>(n) * es;
      if (ptrs[i] < ptrs[j] + bytes && ptrs[j] < ptrs[i] + bytes) throw Invalid("p, g, m, v and the copies must not overlap");
    }
  const SegPlan plan = plan_segment(ptrs, 4 + ncopies, n, es, static_cast<int64_t>(kAdamwThreads) * (16 / es));
  const bool vec = plan.vec;
  if (vec) {  // as for fp32: the head is stretched to the cache line when every stream agrees on it
    int64_t head = plan.head;
    const uintptr_t line = (ptrs[0] + head * es) % 128;
    bool same = true;
    for (int i = 1; i < 4 + ncopies; ++i) same = same && (ptrs[i] + head * es) % 128 == line;
    const int64_t more = static_cast<int64_t>((128 - line) % 128) / es;
    if (same && more < plan.body) head += more;
    a.p += head, a.g += head, a.m += head, a.v += head;
    for (int c = 0; c < ncopies; ++c) a.copy[c] += head;
    a.n = n - head;
    a.head = static_cast<int>(head);
  }
  const int64_t per = vec ? static_cast<int64_t>(kAdamwThreads) * (16 / es) : kAdamwThreads;
  const dim3 grid(grid_for(std::max<int64_t>((a.n + per - 1) / per, 1))), block(kAdamwThreads);
  // The 16-bit types round eight times per element and carry far more arithmetic per byte than fp32 and fp64, whose cap of three
  // waves per SIMD costs them 5-10 %: four 21.46M-element shards take 0.200-0.212 ms with 8 KiB, 0.22 with 16 or 24 KiB.
  const int set = g_occupancy_pad[TDM_XCD_ADAMW].load(std::memory_order_relaxed);
  const unsigned pad = set >= 0 ? static_cast<unsigned>(set) : sizeof(T) == 2 ? 8192u : occupancy_pad(TDM_XCD_ADAMW);
  switch ((vec ? 2 : 0) + (ncopies > 0 ? 1 : 0)) {
    case 0: hipLaunchKernelGGL((k3_adamw_typed_kernel<T, false, false>), grid, block, pad, st, a); break;
    case 1: hipLaunchKernelGGL((k3_adamw_typed_kernel<T, false, true>), grid, block, pad, st, a); break;
    case 2: hipLaunchKernelGGL((k3_adamw_typed_kernel<T, true, false>), grid, block, pad, st, a); break;
    default: hipLaunchKernelGGL((k3_adamw_typed_kernel<T, true, true>), grid, block, pad, st, a); break;
  }
  check_hip(hipGetLastError(), "k3_adamw (typed) launch");
}
}  // namespace
}  // extern "C++"

int tdm_k3_adamw_typed(void* p, const void* g, void* m, void* v, int64_t n, int dtype, const tdm_adamw_hyper* h, int order,
                       void* const* copies, int ncopies, tdm_stream stream) {
  return guard([&] {
    if (n < 0) throw Invalid("n is negative");
    if (ncopies < 0 || ncopies > TDM_MAX_WORLD - 1) throw Invalid("at most 7 further copies of the parameters");
    if (dtype != TDM_F32 && dtype != TDM_F64 && dtype != TDM_BF16 && dtype != TDM_F16) throw Invalid("AdamW handles fp32, fp64, bf16 and fp16 shards (dtype " + std::to_string(dtype) + ")");
    if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid("unknown update order");
    if (n == 0) return;
    if (!p || !g || !m || !v || !h || (ncopies > 0 && !copies)) throw Invalid("NULL argument");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == TDM_F32) {  // a Python double applied to a float tensor is rounded to fp32 once
      tdm_adamw_scalars s{h->use_decay, static_cast<float>(h->decay), static_cast<float>(h->w1), static_cast<float>(h->beta2),
                          static_cast<float>(h->one_m_b2), static_cast<float>(h->bc2_sqrt), static_cast<float>(h->eps),
                          static_cast<float>(h->neg_step), static_cast<float>(1.0 / h->bc2_sqrt)};
      adamw_launch(static_cast<float*>(p), static_cast<const float*>(g), static_cast<float*>(m), static_cast<float*>(v), n, &s, order,
                   reinterpret_cast<float* const*>(copies), ncopies, st);
      return;
    }
    if (order != TDM_ADAMW_HOST_ORDER) throw Invalid("the device order is defined for fp32 shards only");
    if (dtype == TDM_F64) adamw_typed_launch<double>(p, g, m, v, n, *h, copies, ncopies, st);
    else if (dtype == TDM_BF16) adamw_typed_launch<bf16_t>(p, g, m, v, n, *h, copies, ncopies, st);
    else adamw_typed_launch<f16_t>(p, g, m, v, n, *h, copies, ncopies, st);
  });
}

int64_t tdm_k23_table_tiles(const tdm_step_seg* segs, int nseg) {
  if (nseg < 0 || (nseg > 0 && segs == nullptr)) return -1;
  for (int i = 0; i < nseg; ++i)
    if (step_elem_size(segs[i]) == 0) return -1;
  return step_tiles(segs, nseg);
}

int64_t tdm_k23_table_bytes(const tdm_step_seg* segs, int nseg) {
  const int64_t tiles = tdm_k23_table_tiles(segs, nseg);
  if (tiles < 0) return -1;
  return std::max<int64_t>(16, tiles * static_cast<int64_t>(sizeof(StepSegDev)));
}

int tdm_k23_table_build(const tdm_step_seg* segs, int nseg, int world, void* image) {
  return guard([&] {
    if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
    if (nseg < 0 || (nseg > 0 && segs == nullptr) || image == nullptr) throw Invalid("bad table arguments");
    const int es = nseg > 0 ? step_elem_size(segs[0]) : 4;
    for (int i = 0; i < nseg; ++i) {  // before anything is sized by them
      if (step_elem_size(segs[i]) == 0) throw Invalid("segment " + std::to_string(i) + ": a step segment's dtype must be TDM_F32, TDM_F64, TDM_BF16 or TDM_F16");
      if (segs[i].dtype != segs[0].dtype) throw Invalid("segment " + std::to_string(i) + ": the segments of one table share one dtype");
    }
    std::memset(image, 0, static_cast<size_t>(tdm_k23_table_bytes(segs, nseg)));
    StepSegDev* out = static_cast<StepSegDev*>(image);
    const int64_t tile_elems = static_cast<int64_t>(kTileVecs) * (16 / es);
    int64_t tiles = 0;
    for (int i = 0; i < nseg; ++i) {
      const tdm_step_seg& sg = segs[i];
      if (sg.count < 0) throw Invalid("segment " + std::to_string(i) + ": negative count");
      if (sg.count == 0) continue;
      if (sg.chunk < 0 || sg.chunk >= world) throw Invalid("segment " + std::to_string(i) + ": chunk outside [0, world)");
      if (!sg.exp_avg || !sg.exp_avg_sq) throw Invalid("segment " + std::to_string(i) + ": NULL optimizer state");
      if (reinterpret_cast<uintptr_t>(sg.exp_avg) % es || reinterpret_cast<uintptr_t>(sg.exp_avg_sq) % es) {
        throw Invalid("segment " + std::to_string(i) + ": pointer not aligned to the element size");
      }
      for (int r = 0; r < TDM_MAX_WORLD; ++r) {
        if (r >= world) {
          if (sg.grad[r] || sg.param[r]) throw Invalid("segment " + std::to_string(i) + ": pointers of ranks beyond the world size must be NULL");
          continue;
        }
        if (!sg.grad[r] || !sg.param[r]) throw Invalid("segment " + std::to_string(i) + ": NULL gradient or parameter");
        const uintptr_t a = reinterpret_cast<uintptr_t>(sg.grad[r]), b = reinterpret_cast<uintptr_t>(sg.param[r]);
        if (a % es || b % es) throw Invalid("segment " + std::to_string(i) + ": pointer not aligned to the element size");
      }
      const SegPlan plan = plan_step(sg);
      for (int64_t at = 0; at < plan.body; at += tile_elems) {  // records describe the body; the first one carries the head
        StepSegDev& rec = out[tiles++];
        const int64_t off = (plan.head + at) * es;
        for (int r = 0; r < world; ++r) {
          rec.g[r] = static_cast<const char*>(sg.grad[r]) + off;
          rec.p[r] = static_cast<char*>(sg.param[r]) + off;
        }
        rec.m = static_cast<char*>(sg.exp_avg) + off;
        rec.v = static_cast<char*>(sg.exp_avg_sq) + off;
        rec.count = std::min<int64_t>(tile_elems, plan.body - at);
        rec.chunk = sg.chunk;
        rec.vec_ok = plan.vec ? (at == 0 ? 1 + plan.head : 1) : 0;
      }
    }
  });
}

int tdm_k23_zero2_step(const void* table_dev, int64_t ntiles, int world, int average, const tdm_adamw_scalars* s, int order,
                       tdm_stream stream) {
  return guard([&] {
    if (ntiles < 0) throw Invalid("ntiles is negative");
    if (ntiles == 0) return;
    if (table_dev == nullptr || s == nullptr) throw Invalid("NULL argument");
    if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid("unknown update order");
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (world) {
      case 1: launch_step_w<1>(table_dev, ntiles, average, *s, order, st); break;
      case 2: launch_step_w<2>(table_dev, ntiles, average, *s, order, st); break;
      case 3: launch_step_w<3>(table_dev, ntiles, average, *s, order, st); break;
      case 4: launch_step_w<4>(table_dev, ntiles, average, *s, order, st); break;
      case 5: launch_step_w<5>(table_dev, ntiles, average, *s, order, st); break;
      case 6: launch_step_w<6>(table_dev, ntiles, average, *s, order, st); break;
      case 7: launch_step_w<7>(table_dev, ntiles, average, *s, order, st); break;
      case 8: launch_step_w<8>(table_dev, ntiles, average, *s, order, st); break;
      default: throw Invalid("world must be in [1, 8]");
    }
    check_hip(hipGetLastError(), "k23_zero2_step launch");
  });
}

extern "C++" {
namespace {
template <typename T, int kWorld>
void launch_step_typed_w(const void* image, const StepSegDev* whole, int64_t tiles, int average, const tdm_adamw_hyper& h, hipStream_t stream) {
  const AdamwHyper<typename AdamwMath<T>::S> s = typed_hyper<T>(h);
  const Divisor<T> dv = make_divisor<T>(kWorld);
  const StepSegDev* t = static_cast<const StepSegDev*>(image);
  const dim3 grid(grid_for(tiles * kStepParts)), block(kThreads);
  // bf16 carries more arithmetic per byte and does better with more waves than the fp32 and fp64 steps: the 85.8M-parameter
  // step at world 4 takes 0.357-0.360 ms with a pad of 0-16 KiB and 0.399 with the family's 24 KiB.
  const int set = g_occupancy_pad[TDM_XCD_STEP].load(std::memory_order_relaxed);
  const unsigned pad = set >= 0 ? static_cast<unsigned>(set) : sizeof(T) == 2 ? 16384u : occupancy_pad(TDM_XCD_STEP);
  const int shift = xcd_shift(TDM_XCD_STEP, kWorld, true);
  if (whole != nullptr) {  // one segment, described in the kernel's arguments
    switch (div_kind(kWorld, average != 0)) {
      case 0: hipLaunchKernelGGL((k23_zero2_step_one_typed_kernel<T, kWorld, 0>), grid, block, pad, stream, *whole, tiles, dv, s, shift); break;
      case 1: hipLaunchKernelGGL((k23_zero2_step_one_typed_kernel<T, kWorld, 1>), grid, block, pad, stream, *whole, tiles, dv, s, shift); break;
      default: hipLaunchKernelGGL((k23_zero2_step_one_typed_kernel<T, kWorld, 2>), grid, block, pad, stream, *whole, tiles, dv, s, shift); break;
    }
    return;
  }
  switch (div_kind(kWorld, average != 0)) {
    case 0: hipLaunchKernelGGL((k23_zero2_step_typed_kernel<T, kWorld, 0>), grid, block, pad, stream, t, tiles, dv, s, shift); break;
    case 1: hipLaunchKernelGGL((k23_zero2_step_typed_kernel<T, kWorld, 1>), grid, block, pad, stream, t, tiles, dv, s, shift); break;
    default: hipLaunchKernelGGL((k23_zero2_step_typed_kernel<T, kWorld, 2>), grid, block, pad, stream, t, tiles, dv, s, shift); break;
  }
}

template <typename T>
void launch_step_typed(const void* image, const StepSegDev* whole, int64_t tiles, int world, int average, const tdm_adamw_hyper& h, hipStream_t stream) {
  switch (world) {
    case 1: launch_step_typed_w<T, 1>(image, whole, tiles, average, h, stream); break;
    case 2: launch_step_typed_w<T, 2>(image, whole, tiles, average, h, stream); break;
    case 3: launch_step_typed_w<T, 3>(image, whole, tiles, average, h, stream); break;
    case 4: launch_step_typed_w<T, 4>(image, whole, tiles, average, h, stream); break;
    case 5: launch_step_typed_w<T, 5>(image, whole, tiles, average, h, stream); break;
    case 6: launch_step_typed_w<T, 6>(image, whole, tiles, average, h, stream); break;
    case 7: launch_step_typed_w<T, 7>(image, whole, tiles, average, h, stream); break;
    case 8: launch_step_typed_w<T, 8>(image, whole, tiles, average, h, stream); break;
    default: throw Invalid("world must be in [1, 8]");
  }
}
}  // namespace
}  // extern "C++"

int tdm_k23_zero2_step_typed(const void* table_dev, int64_t ntiles, int world, int average, int dtype, const tdm_adamw_hyper* h,
                             int order, tdm_stream stream) {
  return guard([&] {
    if (ntiles < 0) throw Invalid("ntiles is negative");
    if (dtype != TDM_F32 && dtype != TDM_F64 && dtype != TDM_BF16 && dtype != TDM_F16) throw Invalid("the step handles fp32, fp64, bf16 and fp16 shards (dtype " + std::to_string(dtype) + ")");
    if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid("unknown update order");
    if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
    if (ntiles == 0) return;
    if (table_dev == nullptr || h == nullptr) throw Invalid("NULL argument");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == TDM_F32) {  // a Python double applied to a float tensor is rounded to fp32 once
      const tdm_adamw_scalars s{h->use_decay, static_cast<float>(h->decay), static_cast<float>(h->w1), static_cast<float>(h->beta2),
                                static_cast<float>(h->one_m_b2), static_cast<float>(h->bc2_sqrt), static_cast<float>(h->eps),
                                static_cast<float>(h->neg_step), static_cast<float>(1.0 / h->bc2_sqrt)};
      const int status = tdm_k23_zero2_step(table_dev, ntiles, world, average, &s, order, stream);
      if (status != TDM_OK) throw std::runtime_error(tdm_last_error());
      return;
    }
    if (order != TDM_ADAMW_HOST_ORDER) throw Invalid("the device order is defined for fp32 shards only");
    if (dtype == TDM_F64) launch_step_typed<double>(table_dev, nullptr, ntiles, world, average, *h, st);
    else if (dtype == TDM_BF16) launch_step_typed<bf16_t>(table_dev, nullptr, ntiles, world, average, *h, st);
    else launch_step_typed<f16_t>(table_dev, nullptr, ntiles, world, average, *h, st);
    check_hip(hipGetLastError(), "k23_zero2_step (typed) launch");
  });
}

extern "C++" {
namespace tandem_hip {
// Used by the engine too: the same over a segment of any of K3's shard types (seg.dtype), constants as Python doubles.
void zero2_step_segment_typed(const tdm_step_seg& sg, int world, bool average, const tdm_adamw_hyper& h, int order, hipStream_t stream) {
  if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
  if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid("unknown update order");
  if (sg.count < 0) throw Invalid("negative count");
  if (step_elem_size(sg) == 0) throw Invalid("a step segment's dtype must be TDM_F32, TDM_F64, TDM_BF16 or TDM_F16");
  if (sg.dtype == TDM_F32) {  // a Python double applied to a float tensor is rounded to fp32 once
    const tdm_adamw_scalars s{h.use_decay, static_cast<float>(h.decay), static_cast<float>(h.w1), static_cast<float>(h.beta2),
                              static_cast<float>(h.one_m_b2), static_cast<float>(h.bc2_sqrt), static_cast<float>(h.eps),
                              static_cast<float>(h.neg_step), static_cast<float>(1.0 / h.bc2_sqrt)};
    zero2_step_segment(sg, world, average, s, order, stream);
    return;
  }
  if (order != TDM_ADAMW_HOST_ORDER) throw Invalid("the device order is defined for fp32 shards only");
  if (sg.count == 0) return;
  int64_t tiles = 0;
  const StepSegDev whole = whole_segment(sg, world, &tiles);
  if (sg.dtype == TDM_F64) launch_step_typed<double>(nullptr, &whole, tiles, world, average, h, stream);
  else if (sg.dtype == TDM_BF16) launch_step_typed<bf16_t>(nullptr, &whole, tiles, world, average, h, stream);
  else launch_step_typed<f16_t>(nullptr, &whole, tiles, world, average, h, stream);
  check_hip(hipGetLastError(), "k23_zero2_step_one (typed) launch");
}
}  // namespace tandem_hip
}  // extern "C++"

int tdm_k23_zero2_step_segment_typed(const tdm_step_seg* seg, int world, int average, const tdm_adamw_hyper* h, int order,
                                     tdm_stream stream) {
  return guard([&] {
    if (seg == nullptr || h == nullptr) throw Invalid("NULL argument");
    zero2_step_segment_typed(*seg, world, average != 0, *h, order, static_cast<hipStream_t>(stream));
  });
}

int tdm_k23_zero2_step_segment(const tdm_step_seg* seg, int world, int average, const tdm_adamw_scalars* s, int order,
                               tdm_stream stream) {
  return guard([&] {
    if (seg == nullptr || s == nullptr) throw Invalid("NULL argument");
    zero2_step_segment(*seg, world, average != 0, *s, order, static_cast<hipStream_t>(stream));
  });
}

int tdm_k4_unit_gather(void* full, const void* const* shards, const int64_t* sizes, int world, int dtype,
                       tdm_stream stream) {
  return guard([&] {
    const int es = elem_size(dtype);
    if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
    if (world < 1 || world > TDM_MAX_PAIRS) throw Invalid("world must be in [1, 16]");
    if (!full || !shards || !sizes) throw Invalid("NULL argument");
    tdm_pair pairs[TDM_MAX_PAIRS];
    int np = 0;
    int64_t lo = 0;
    for (int q = 0; q < world; ++q) {
      if (sizes[q] < 0) throw Invalid("negative shard size");
      char* dst = static_cast<char*>(full) + lo * es;
      if (sizes[q] > 0) {
        if (shards[q] == nullptr) throw Invalid("NULL shard");
        if (shards[q] != dst) pairs[np++] = tdm_pair{dst, shards[q], sizes[q]};
      }
      lo += sizes[q];
    }
    copy_step(pairs, np, dtype, 0, static_cast<hipStream_t>(stream));
  });
}

int tdm_k4_unit_gather_all(void* const* fulls, const void* const* shards, const int64_t* sizes, int world, int dtype,
                           tdm_stream stream) {
  return guard([&] {
    CallScope scope;
    const int es = elem_size(dtype);
    if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
    if (world < 1 || world > TDM_MAX_PAIRS) throw Invalid("world must be in [1, 16]");
    if (!fulls || !shards || !sizes) throw Invalid("NULL argument");
    int64_t total = 0;
    for (int q = 0; q < world; ++q) {
      if (sizes[q] < 0) throw Invalid("negative shard size");
      total += sizes[q];
    }
    if (total == 0) return;  // an empty unit has no buffers to speak of
    for (int q = 0; q < world; ++q) {
      if (fulls[q] == nullptr) throw Invalid("NULL full buffer");
      if (sizes[q] > 0 && shards[q] == nullptr) throw Invalid("NULL shard");
      if (reinterpret_cast<uintptr_t>(fulls[q]) % es || reinterpret_cast<uintptr_t>(shards[q]) % es) throw Invalid("pointer not aligned to the element size");
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (world > TDM_MAX_WORLD) {  // beyond the one launch's table: rank by rank
      for (int r = 0; r < world; ++r) {
        tdm_pair pairs[TDM_MAX_PAIRS];
        int np = 0;
        int64_t lo = 0;
        for (int q = 0; q < world; ++q) {
          char* dst = static_cast<char*>(fulls[r]) + lo * es;
          if (sizes[q] > 0 && shards[q] != dst) pairs[np++] = tdm_pair{dst, shards[q], sizes[q]};
          lo += sizes[q];
        }
        copy_step(pairs, np, dtype, 0, st);
      }
      return;
    }
    char* f[TDM_MAX_WORLD];
    const char* s[TDM_MAX_WORLD];
    for (int q = 0; q < world; ++q) {
      f[q] = static_cast<char*>(fulls[q]);
      s[q] = static_cast<const char*>(shards[q]);
    }
    const int64_t cap = static_cast<int64_t>(t_call_cus ? t_call_cus : compute_units()) * g_blocks_per_cu;
    // Everything cached: what a gather writes is read by the unit's forward or backward straight away. (Twelve block units of
    // the 85.8M GPT gathered in turn at world 2: 19.4 us per unit with two vectors per lane, 18.8 with one; 17.6-18.0 with
    // non-temporal accesses, which would leave the consumer to fetch the unit from HBM.)
    // Tile order: runs of 8 tiles (16 KiB) per XCD unless the family's shift is set by hand. In the same sweep of 0..6 the plain
    // order gave 18.8 us per block unit, every grouping from 4 tiles up 18.0-18.2.
    const int set = g_xcd_shift[TDM_XCD_COPY].load(std::memory_order_relaxed);
    unit_gather_multicast(f, s, sizes, world, es, false, occupancy_pad(TDM_XCD_COPY, false), set >= 0 ? set : 3, 1,
                          static_cast<int>(std::min<int64_t>(cap, int64_t(1) << 30)), st);
  });
}

}  // extern "C"
