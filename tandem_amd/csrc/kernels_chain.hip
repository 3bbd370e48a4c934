// The ring reduce-scatter of a whole group in ONE launch, and its all-gather in one more, for ranks
// that are buffers of one process.
//
// The ring's W-1 steps (tandem/comm.py:301-305 in the reference) pass chunk c round the ring:
// rank c+1 sends it, rank c+2 adds its own and sends the sum on, ..., rank c adds last. Every
// element of chunk c is therefore a chain
//     acc = y[c+1];   acc = y[c+k] + acc   (k = 2 .. W),      y_q = x_q / W when averaging,
// and after the last step rank c+k's copy of chunk c holds the chain's value after k terms
// (observable: tandem/comm.py:350-352). One workgroup can run the whole chain for its tile: it
// reads the W ranks' copies once, and stores the partial sum after k terms into rank c+k's copy,
// which leaves memory bit for bit as the W-1 launches of the step kernel do, with W reads and
// W-1 (keep_sent: W) writes of 4 bytes per element instead of 3 (W-1) (+1) accesses.
// Within the caches everything is loaded and stored plainly, 4 KiB of every stream per workgroup;
// beyond them non-temporally, 2 KiB per workgroup (the caller says which).

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <string>

#include "../../include/tandem_hip.h"
#include "common.h"

#include "kernels_device.h"

namespace tandem_hip {

namespace {

// One chunk per segment: rank q's copy of the chunk at ptr[q].
struct ChainTable {
  int nseg;
  int keep_sent;  // the first sender's copy is left holding y (x / W), as div_ of the whole tensor does
  int shift;      // of tile_of()
  int64_t tile_end[TDM_MAX_WORLD];
  char* ptr[TDM_MAX_WORLD][TDM_MAX_WORLD];  // [segment][rank]
  int64_t count[TDM_MAX_WORLD];
  int32_t chunk[TDM_MAX_WORLD];
  int32_t vec_ok[TDM_MAX_WORLD];  // 1 + h: ptr 16-byte aligned with h more elements directly before it
};

template <typename T, int kWorld, int kDiv>
__device__ __forceinline__ void chain_elem(const T (&in)[kWorld], T (&out)[kWorld], const Divisor<T>& dv) {
  // in[k]: rank (c+1+k) % W's element; out[k]: what that rank holds afterwards
  using A = typename Elem<T>::acc;
  A acc = scaled<T, kDiv>(Elem<T>::widen(in[0]), dv.divisor, dv.reciprocal);
  out[0] = Elem<T>::narrow(acc);
#pragma unroll
  for (int k = 1; k < kWorld; ++k) {
    const A y = scaled<T, kDiv>(Elem<T>::widen(in[k]), dv.divisor, dv.reciprocal);
    acc = Elem<T>::widen(Elem<T>::narrow(static_cast<A>(y + acc)));
    out[k] = Elem<T>::narrow(acc);
  }
}

// kMask: the cache policy (kernels_device.h): 0 everything cached, for footprints that stay in the caches; 7 non-temporal
// loads and stores, for footprints beyond them.
// A workgroup takes kU vectors per lane and stream: 2 (4 KiB of every stream) within the caches, 1 beyond them
// and from five ranks on (a lane holds kU vectors of every rank at once).
constexpr int chain_vecs(int world, bool cold) { return !cold && world <= 4 ? kWarmVecs : 1; }

template <typename T, int kWorld, int kDiv, int kMask, int kU = chain_vecs(kWorld, kMask != 0)>
__global__ __launch_bounds__(kThreads) void k1_chain_kernel(ChainTable tab, Divisor<T> dv) {
  constexpr int L = lanes<T>();
  constexpr int kVecs = kThreads * kU;  // vectors of every stream per workgroup
  const int64_t total = tab.tile_end[tab.nseg - 1];
  for (int64_t at = blockIdx.x; at < total; at += gridDim.x) {
    const int64_t tile = tile_of(at, total, tab.shift);
    int sg = 0;
    while (tile >= tab.tile_end[sg]) ++sg;
    const int64_t t = tile - (sg ? tab.tile_end[sg - 1] : 0);
    const int c = tab.chunk[sg];
    const int64_t n = tab.count[sg];
    char* p[kWorld];  // in ring order: p[k] is rank (c+1+k) % W's copy
#pragma unroll
    for (int k = 0; k < kWorld; ++k) p[k] = tab.ptr[sg][(c + 1 + k) % kWorld];
    const bool keep = tab.keep_sent != 0;
    {  // every segment is vectorisable: the host sends chunks whose copies disagree within 16 bytes through the ring's steps
      const int64_t nv = n / L;
      vec16 raw[kWorld][kU];
#pragma unroll
      for (int k = 0; k < kWorld; ++k)
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int64_t v = t * kVecs + threadIdx.x + static_cast<int64_t>(u) * kThreads;
          if (v < nv) raw[k][u] = load_rmw<kMask>(p[k] + v * 16);
        }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t v = t * kVecs + threadIdx.x + static_cast<int64_t>(u) * kThreads;
        if (v < nv) {
          // the chain rank by rank over the vector's lanes (chain_elem's arithmetic): a rank's partial sums are
          // stored as soon as they exist, so a lane holds one accumulator per element and never all W results
          if constexpr (!Elem<T>::floating) {  // integers: never divided (the first sender's copy stays), whole vectors added
            vec16 sum = raw[0][u];
#pragma unroll
            for (int k = 1; k < kWorld; ++k) {
              sum = add_vec<T>(raw[k][u], sum);
              store16<kMask>(p[k] + v * 16, sum);
            }
          } else {
            using A = typename Elem<T>::acc;
            A acc[L];
#pragma unroll
            for (int k = 0; k < kWorld; ++k) {
              const Lanes<T> x = unpack<T>(raw[k][u]);
              Lanes<T> o;
#pragma unroll
              for (int l = 0; l < L; ++l) {
                const A y = scaled<T, kDiv>(Elem<T>::widen(x.v[l]), dv.divisor, dv.reciprocal);
                acc[l] = k == 0 ? y : Elem<T>::widen(Elem<T>::narrow(static_cast<A>(y + acc[l])));
                o.v[l] = Elem<T>::narrow(acc[l]);
              }
              if (k > 0 || keep) store16<kMask>(p[k] + v * 16, pack<T>(o));
            }
          }
        }
      }
      const int head = tab.vec_ok[sg] - 1;
      // the chunk's last few elements (lanes 0..) and the few before its first whole vector (lanes 32..)
      if (t == 0 && (threadIdx.x < n - nv * L || (threadIdx.x >= 32 && static_cast<int>(threadIdx.x) - 32 < head))) {
        const int64_t i = threadIdx.x < 32 ? nv * L + threadIdx.x : -1 - (static_cast<int64_t>(threadIdx.x) - 32);
        T in[kWorld], out[kWorld];
#pragma unroll
        for (int k = 0; k < kWorld; ++k) in[k] = reinterpret_cast<const T*>(p[k])[i];
        chain_elem<T, kWorld, kDiv>(in, out, dv);
        if (keep) reinterpret_cast<T*>(p[0])[i] = out[0];
#pragma unroll
        for (int k = 1; k < kWorld; ++k) reinterpret_cast<T*>(p[k])[i] = out[k];
      }
    }
  }
}

template <typename T, int kWorld, int kMask>
void launch_chain_m(const ChainTable& tab, bool average, int grid, unsigned pad, hipStream_t stream) {
  Divisor<T> dv;
  using A = typename Elem<T>::acc;
  dv.divisor = static_cast<A>(kWorld);
  if constexpr (Elem<T>::floating) dv.reciprocal = static_cast<A>(1) / dv.divisor; else dv.reciprocal = 1;
  const dim3 g(grid), b(kThreads);
  if constexpr (Elem<T>::floating) {
    if (average && (kWorld & (kWorld - 1)) == 0) {
      hipLaunchKernelGGL((k1_chain_kernel<T, kWorld, 1, kMask>), g, b, pad, stream, tab, dv);
      return;
    }
    if (average) {
      hipLaunchKernelGGL((k1_chain_kernel<T, kWorld, 2, kMask>), g, b, pad, stream, tab, dv);
      return;
    }
  }
  hipLaunchKernelGGL((k1_chain_kernel<T, kWorld, 0, kMask>), g, b, pad, stream, tab, dv);
}

template <typename T>
void launch_chain(const ChainTable& tab, int world, bool average, int grid, bool cold, unsigned pad, hipStream_t stream) {
  switch (world * 2 + (cold ? 1 : 0)) {
    case 4: launch_chain_m<T, 2, 0>(tab, average, grid, pad, stream); break;
    case 5: launch_chain_m<T, 2, 7>(tab, average, grid, pad, stream); break;
    case 6: launch_chain_m<T, 3, 0>(tab, average, grid, pad, stream); break;
    case 7: launch_chain_m<T, 3, 7>(tab, average, grid, pad, stream); break;
    case 8: launch_chain_m<T, 4, 0>(tab, average, grid, pad, stream); break;
    case 9: launch_chain_m<T, 4, 7>(tab, average, grid, pad, stream); break;
    case 10: launch_chain_m<T, 5, 0>(tab, average, grid, pad, stream); break;
    case 11: launch_chain_m<T, 5, 7>(tab, average, grid, pad, stream); break;
    case 12: launch_chain_m<T, 6, 0>(tab, average, grid, pad, stream); break;
    case 13: launch_chain_m<T, 6, 7>(tab, average, grid, pad, stream); break;
    case 14: launch_chain_m<T, 7, 0>(tab, average, grid, pad, stream); break;
    case 15: launch_chain_m<T, 7, 7>(tab, average, grid, pad, stream); break;
    case 16: launch_chain_m<T, 8, 0>(tab, average, grid, pad, stream); break;
    default: launch_chain_m<T, 8, 7>(tab, average, grid, pad, stream); break;
  }
}

// ---------------------------------------------------------------- the all-gather in one launch
// The ring forwards every chunk W-1 times, one neighbour at a time: W-1 launches that each read and write a
// chunk's worth per rank, 8 (W-1) bytes per element of the tensor. With every rank's buffer in reach, a
// workgroup reads its tile of chunk c ONCE from the owner and stores it into the W-1 other ranks' copies:
// 4 W bytes per element, the same bytes in memory afterwards (copies have no order to preserve).
// The same kernel gathers a ZeRO-3 unit for every rank at once: a segment is then one rank's shard, read once and stored
// into its slice of all W ranks' full buffers.
struct GatherTable {
  int nseg;
  int shift;  // of tile_of()
  int32_t ndst[TDM_MAX_WORLD];  // destinations of every segment (W - 1 for the all-gather, up to W for a unit gather)
  int64_t tile_end[TDM_MAX_WORLD];
  const char* src[TDM_MAX_WORLD];
  char* dst[TDM_MAX_WORLD][TDM_MAX_WORLD];
  int64_t bytes[TDM_MAX_WORLD];
  int32_t vec_ok[TDM_MAX_WORLD];  // as the other tables': 0 byte by byte, 1 + h with h bytes before the pointers
};

template <int kMask, int kU>
__global__ __launch_bounds__(kThreads) void k1_gather_kernel(GatherTable tab) {
  constexpr int kVecs = kThreads * kU;  // vectors of every stream per workgroup
  constexpr int64_t kTileBytes = static_cast<int64_t>(kVecs) * 16;
  const int64_t total = tab.tile_end[tab.nseg - 1];
  for (int64_t at = blockIdx.x; at < total; at += gridDim.x) {
    const int64_t tile = tile_of(at, total, tab.shift);
    int sg = 0;
    while (tile >= tab.tile_end[sg]) ++sg;
    const int64_t t = tile - (sg ? tab.tile_end[sg - 1] : 0);
    const char* __restrict__ from = tab.src[sg];
    const int64_t n = tab.bytes[sg];
    const int ndst = tab.ndst[sg];
    if (tab.vec_ok[sg]) {
      const int64_t nv = n / 16;
      vec16 raw[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t v = t * kVecs + threadIdx.x + static_cast<int64_t>(u) * kThreads;
        if (v < nv) raw[u] = load_stream<kMask>(from + v * 16);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t v = t * kVecs + threadIdx.x + static_cast<int64_t>(u) * kThreads;
        if (v < nv)
          for (int k = 0; k < ndst; ++k) store16<kMask>(tab.dst[sg][k] + v * 16, raw[u]);
      }
      const int head = tab.vec_ok[sg] - 1;
      // the bytes after the last whole vector (lanes 0..15) and before the first (lanes 32..47)
      if (t == 0 && (threadIdx.x < n - nv * 16 || (threadIdx.x >= 32 && static_cast<int>(threadIdx.x) - 32 < head))) {
        const int64_t i = threadIdx.x < 32 ? nv * 16 + threadIdx.x : -1 - (static_cast<int64_t>(threadIdx.x) - 32);
        const char byte = from[i];
        for (int k = 0; k < ndst; ++k) tab.dst[sg][k][i] = byte;
      }
    } else {  // the copies disagree within 16 bytes: byte by byte, still coalesced
      const int64_t b0 = t * kTileBytes + threadIdx.x;
      for (int64_t i = b0; i < n && i < (t + 1) * kTileBytes; i += kThreads) {
        const char byte = from[i];
        for (int k = 0; k < ndst; ++k) tab.dst[sg][k][i] = byte;
      }
    }
  }
}

}  // namespace

namespace {
void launch_gather(const GatherTable& tab, int64_t tiles, bool cold, unsigned pad, int per_lane, int max_grid, hipStream_t stream) {
  if (tab.nseg == 0) return;
  if (per_lane != 1 && per_lane != 2) throw Invalid("1 or 2 vectors per lane");
  const dim3 grid(static_cast<unsigned>(tiles < max_grid ? tiles : max_grid)), block(kThreads);
  switch ((cold ? 2 : 0) + (per_lane == 2 ? 1 : 0)) {
    case 0: hipLaunchKernelGGL((k1_gather_kernel<0, 1>), grid, block, pad, stream, tab); break;
    case 1: hipLaunchKernelGGL((k1_gather_kernel<0, 2>), grid, block, pad, stream, tab); break;
    case 2: hipLaunchKernelGGL((k1_gather_kernel<7, 1>), grid, block, pad, stream, tab); break;
    default: hipLaunchKernelGGL((k1_gather_kernel<7, 2>), grid, block, pad, stream, tab); break;
  }
  check_hip(hipGetLastError(), "k1_gather launch");
}
}  // namespace

bool gather_handles(int world) { return world >= 2 && world <= TDM_MAX_WORLD; }

void gather_multicast(char* const* base, const int64_t* lo, const int64_t* len, int world, int es, bool cold, unsigned pad,
                      int shift, int per_lane, int max_grid, hipStream_t stream) {
  if (!gather_handles(world)) throw Invalid("the one-launch all-gather handles world sizes 2..8");
  GatherTable tab;
  std::memset(&tab, 0, sizeof tab);
  tab.shift = shift;
  const int64_t tile_bytes = static_cast<int64_t>(kThreads) * per_lane * 16;
  int64_t tiles = 0;
  int k = 0;
  for (int c = 0; c < world; ++c) {
    if (len[c] == 0) continue;
    uintptr_t at[TDM_MAX_WORLD];
    for (int q = 0; q < world; ++q) at[q] = reinterpret_cast<uintptr_t>(base[q] + lo[c] * es);
    const SegPlan plan = plan_segment(at, world, len[c] * es, 1, tile_bytes);  // in bytes: copies have no element type
    tab.src[k] = base[c] + lo[c] * es + plan.head;
    int d = 0;
    for (int q = 0; q < world; ++q)
      if (q != c) tab.dst[k][d++] = base[q] + lo[c] * es + plan.head;
    tab.ndst[k] = d;
    tab.bytes[k] = plan.body;
    tab.vec_ok[k] = plan.vec ? 1 + plan.head : 0;
    tiles += plan.tiles;
    tab.tile_end[k] = tiles;
    ++k;
  }
  tab.nseg = k;
  launch_gather(tab, tiles, cold, pad, per_lane, max_grid, stream);
}

// ZeRO-3's gather of one unit for EVERY rank in one launch: rank q's shard is read once and stored into elements
// [lo_q, lo_q + sizes[q]) of all `world` full buffers (a full buffer whose slice IS the shard is skipped).
void unit_gather_multicast(char* const* fulls, const char* const* shards, const int64_t* sizes, int world, int es, bool cold,
                           unsigned pad, int shift, int per_lane, int max_grid, hipStream_t stream) {
  if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("the one-launch unit gather handles world sizes 1..8");
  GatherTable tab;
  std::memset(&tab, 0, sizeof tab);
  tab.shift = shift;
  const int64_t tile_bytes = static_cast<int64_t>(kThreads) * per_lane * 16;
  int64_t tiles = 0, lo = 0;
  int k = 0;
  for (int q = 0; q < world; ++q) {
    const int64_t bytes = sizes[q] * es;
    const int64_t at_bytes = lo * es;
    lo += sizes[q];
    if (bytes == 0) continue;
    uintptr_t at[TDM_MAX_WORLD + 1];
    int np = 0, d = 0;
    at[np++] = reinterpret_cast<uintptr_t>(shards[q]);
    char* dsts[TDM_MAX_WORLD];
    for (int r = 0; r < world; ++r) {
      char* dst = fulls[r] + at_bytes;
      if (dst == shards[q]) continue;  // the shard already lies in this rank's full buffer
      const uintptr_t a = reinterpret_cast<uintptr_t>(dst), b = reinterpret_cast<uintptr_t>(shards[q]);
      if (a < b + static_cast<uintptr_t>(bytes) && b < a + static_cast<uintptr_t>(bytes)) throw Invalid("unit gather: a full buffer overlaps a shard");
      dsts[d++] = dst;
      at[np++] = a;
    }
    if (d == 0) continue;
    const SegPlan plan = plan_segment(at, np, bytes, 1, tile_bytes);
    tab.src[k] = shards[q] + plan.head;
    for (int i = 0; i < d; ++i) tab.dst[k][i] = dsts[i] + plan.head;
    tab.ndst[k] = d;
    tab.bytes[k] = plan.body;
    tab.vec_ok[k] = plan.vec ? 1 + plan.head : 0;
    tiles += plan.tiles;
    tab.tile_end[k] = tiles;
    ++k;
  }
  tab.nseg = k;
  launch_gather(tab, tiles, cold, pad, per_lane, max_grid, stream);
}

bool chain_handles(int world) { return world >= 2 && world <= kChainMaxWorld; }

bool chain_reduce_scatter(char* const* base, const int64_t* lo, const int64_t* len, int world, int dtype, int es, bool average,
                          bool keep_sent, bool cold, unsigned pad, int shift, int max_grid, hipStream_t stream) {
  if (!chain_handles(world)) throw Invalid("the one-launch reduce-scatter handles world sizes 2..8");
  ChainTable tab;
  std::memset(&tab, 0, sizeof tab);
  tab.keep_sent = keep_sent && average ? 1 : 0;  // without a division the first sender's copy is x already
  tab.shift = shift;
  const int64_t tile_elems = static_cast<int64_t>(kThreads) * chain_vecs(world, cold) * (16 / es);  // as the kernel's kU
  int64_t tiles = 0;
  int k = 0;
  for (int c = 0; c < world; ++c) {
    if (len[c] == 0) continue;  // an empty chunk travels nowhere (tandem/comm.py:292-294)
    uintptr_t at[TDM_MAX_WORLD];
    for (int q = 0; q < world; ++q) at[q] = reinterpret_cast<uintptr_t>(base[q] + lo[c] * es);
    const SegPlan plan = plan_segment(at, world, len[c], es, tile_elems);
    if (!plan.vec) return false;  // the ranks' copies disagree within 16 bytes: nothing launched, the caller takes the ring's steps
    for (int q = 0; q < world; ++q) tab.ptr[k][q] = base[q] + (lo[c] + plan.head) * es;
    tab.count[k] = plan.body;
    tab.chunk[k] = c;
    tab.vec_ok[k] = 1 + plan.head;
    tiles += plan.tiles;
    tab.tile_end[k] = tiles;
    ++k;
  }
  tab.nseg = k;
  if (k == 0) return true;
  const int grid = static_cast<int>(tiles < max_grid ? tiles : max_grid);
  switch (dtype) {
    case TDM_F32: launch_chain<float>(tab, world, average, grid, cold, pad, stream); break;
    case TDM_F64: launch_chain<double>(tab, world, average, grid, cold, pad, stream); break;
    case TDM_F16: launch_chain<f16_t>(tab, world, average, grid, cold, pad, stream); break;
    case TDM_BF16: launch_chain<bf16_t>(tab, world, average, grid, cold, pad, stream); break;
    case TDM_I64: launch_chain<int64_t>(tab, world, false, grid, cold, pad, stream); break;
    case TDM_I32: launch_chain<int32_t>(tab, world, false, grid, cold, pad, stream); break;
    case TDM_I16: launch_chain<int16_t>(tab, world, false, grid, cold, pad, stream); break;
    case TDM_I8: case TDM_U8: launch_chain<int8_t>(tab, world, false, grid, cold, pad, stream); break;
    default: throw Invalid("unknown dtype " + std::to_string(dtype));
  }
  check_hip(hipGetLastError(), "k1_chain launch");
  return true;
}

}  // namespace tandem_hip
