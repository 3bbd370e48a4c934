// libtandem_probe.so (include/tandem_probe.h): a library of its own, not linked into the plug-in.
// A measurement kernel, not part of the reduction path: R streams read and W streams written in
// the geometry the streaming kernels use (workgroups of 128 lanes, 16-byte vectors, one tile per
// workgroup, the tile order of tile_of(), non-temporal loads and stores), with no table and no
// arithmetic worth the name. What it reaches for a given (R, W) over buffers far larger than the
// caches is what the memory system gives that mix of streams; bench.py reports the fused kernels
// against it.

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "../../include/tandem_probe.h"
#include "common.h"

#include "kernels_device.h"

namespace tandem_hip {

namespace {
thread_local std::string probe_error;
}

// common.h's guard() reports through this; the plug-in has its own in abi.hip
void set_last_error(const std::string& message) { probe_error = message; }

namespace {

struct MixArgs {
  const char* rd[TDM_MAX_WORLD];
  char* wr[TDM_MAX_WORLD];
  int64_t vecs;  // 16-byte vectors per stream
  int shift;     // of tile_of()
};

template <int R, int W, int U>
__global__ __launch_bounds__(kThreads) void mix_probe_kernel(MixArgs a) {
  const int64_t tiles = (a.vecs + kThreads * U - 1) / (kThreads * U);
  for (int64_t at = blockIdx.x; at < tiles; at += gridDim.x) {
    const int64_t v0 = tile_of(at, tiles, a.shift) * (kThreads * U) + threadIdx.x;
    vec16 acc[U];
#pragma unroll
    for (int u = 0; u < U; ++u) acc[u] = vec16{static_cast<uint32_t>(v0), 1u, 2u, 3u};
    if constexpr (R > 0) {
      vec16 in[R][U];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int64_t v = v0 + u * kThreads;
          if (v < a.vecs) in[r][u] = load_stream<7>(a.rd[r] + v * 16);
        }
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int u = 0; u < U; ++u) acc[u] += in[r][u];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t v = v0 + u * kThreads;
      if (v < a.vecs) {
        if constexpr (W > 0) {
#pragma unroll
          for (int w = 0; w < W; ++w) store16<7>(a.wr[w] + v * 16, acc[u]);
        } else {
          // read-only: the loads must not be dropped; this store never happens with the probe's inputs
          if (acc[u].x == 0xfeedbeefu && acc[u].y == 0xfeedbeefu) store16<7>(const_cast<char*>(a.rd[0]) + v * 16, acc[u]);
        }
      }
    }
  }
}

template <int R, int W>
void launch_u(const MixArgs& a, int per_lane, dim3 grid, unsigned pad, hipStream_t st) {
  if (per_lane == 1) hipLaunchKernelGGL((mix_probe_kernel<R, W, 1>), grid, dim3(kThreads), pad, st, a);
  else hipLaunchKernelGGL((mix_probe_kernel<R, W, 2>), grid, dim3(kThreads), pad, st, a);
}

template <int R>
void launch_w(const MixArgs& a, int nwrites, int per_lane, dim3 grid, unsigned pad, hipStream_t st) {
  switch (nwrites) {
    case 0: if constexpr (R > 0) launch_u<R, 0>(a, per_lane, grid, pad, st); break;
    case 1: launch_u<R, 1>(a, per_lane, grid, pad, st); break;
    case 2: launch_u<R, 2>(a, per_lane, grid, pad, st); break;
    case 3: launch_u<R, 3>(a, per_lane, grid, pad, st); break;
    case 4: launch_u<R, 4>(a, per_lane, grid, pad, st); break;
    case 5: launch_u<R, 5>(a, per_lane, grid, pad, st); break;
    case 6: launch_u<R, 6>(a, per_lane, grid, pad, st); break;
    case 7: launch_u<R, 7>(a, per_lane, grid, pad, st); break;
    default: launch_u<R, 8>(a, per_lane, grid, pad, st); break;
  }
}

}  // namespace

}  // namespace tandem_hip

using namespace tandem_hip;

#define PROBE_EXPORT extern "C" __attribute__((visibility("default")))

PROBE_EXPORT const char* tdm_probe_last_error(void) { return probe_error.c_str(); }

PROBE_EXPORT int tdm_probe_stream_mix(const void* const* reads, int nreads, void* const* writes, int nwrites, int64_t bytes,
                                      int vectors_per_lane, int xcd_shift, int occupancy_pad, void* stream) {
  return guard([&] {
    if (nreads < 0 || nreads > TDM_MAX_WORLD || nwrites < 0 || nwrites > TDM_MAX_WORLD || nreads + nwrites == 0) {
      throw Invalid("the probe takes 0..8 streams to read and 0..8 to write, at least one in all");
    }
    if ((nreads > 0 && reads == nullptr) || (nwrites > 0 && writes == nullptr)) throw Invalid("NULL stream table");
    if (bytes < 0 || bytes % 16) throw Invalid("bytes per stream must be a multiple of 16");
    if (vectors_per_lane != 1 && vectors_per_lane != 2) throw Invalid("1 or 2 vectors per lane");
    if (xcd_shift < 0 || xcd_shift > 12) throw Invalid("the group shift must be in [0, 12]");
    if (occupancy_pad < 0 || occupancy_pad > 65536) throw Invalid("the pad must be in [0, 65536] bytes");
    if (bytes == 0) return;
    MixArgs a{};
    for (int r = 0; r < nreads; ++r) {
      if (!reads[r] || reinterpret_cast<uintptr_t>(reads[r]) % 16) throw Invalid("streams must be 16-byte aligned and not NULL");
      a.rd[r] = static_cast<const char*>(reads[r]);
    }
    for (int w = 0; w < nwrites; ++w) {
      if (!writes[w] || reinterpret_cast<uintptr_t>(writes[w]) % 16) throw Invalid("streams must be 16-byte aligned and not NULL");
      a.wr[w] = static_cast<char*>(writes[w]);
    }
    a.vecs = bytes / 16;
    a.shift = xcd_shift;
    const int64_t per_tile = static_cast<int64_t>(kThreads) * vectors_per_lane;
    const int64_t tiles = (a.vecs + per_tile - 1) / per_tile;
    const dim3 grid(static_cast<unsigned>(tiles < (int64_t(1) << 30) ? tiles : (int64_t(1) << 30)));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const unsigned pad = static_cast<unsigned>(occupancy_pad);
    switch (nreads) {
      case 0: launch_w<0>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      case 1: launch_w<1>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      case 2: launch_w<2>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      case 3: launch_w<3>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      case 4: launch_w<4>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      case 5: launch_w<5>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      case 6: launch_w<6>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      case 7: launch_w<7>(a, nwrites, vectors_per_lane, grid, pad, st); break;
      default: launch_w<8>(a, nwrites, vectors_per_lane, grid, pad, st); break;
    }
    check_hip(hipGetLastError(), "mix_probe launch");
  });
}
