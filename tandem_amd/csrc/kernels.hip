// Streaming kernels of tandem's data-parallel reduction path for gfx950 (MI355X):
// K1 ring-step reduce / copy, K2 bucket fold, K3 sharded AdamW, K4 unit gather.
//
// All four are HBM-bound element-wise passes, so they share one shape: a launch
// covers a small table of streams, the work is cut into tiles of 16 KiB per
// stream, workgroups walk the tiles grid-stride (consecutive workgroups touch
// consecutive tiles, so a sweep of the grid is one contiguous multi-MiB slot of
// every stream), and each lane keeps several independent 16-byte loads in flight
// before its first use. No LDS. Arithmetic is exact IEEE in the tensor's own
// precision: built with -ffp-contract=off, true division, correctly rounded
// sqrt; the only fused multiply-adds are the explicit ones in K3.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "../../include/tandem_hip.h"
#include "common.h"

namespace tandem_hip {

namespace {

#ifndef TDM_THREADS
#define TDM_THREADS 256
#endif
#ifndef TDM_UNROLL
#define TDM_UNROLL 4
#endif
constexpr int kThreads = TDM_THREADS;
constexpr int kUnroll = TDM_UNROLL;             // 16-byte vectors per lane per tile and stream
#ifndef TDM_K1_UNROLL
#define TDM_K1_UNROLL 2
#endif
// K1 and the copy kernel cut their pairs into tiles of their own, 8 KiB per stream: against 16 KiB the
// ring (reduce-scatter + all-gather, world 4) runs 3 % faster at 64 MiB per rank (6.95 vs 6.74 TB/s), 2 %
// at 16 MiB and equally fast at 256 MiB; different tile sizes for the two kernels are worse than either.
constexpr int kK1Unroll = TDM_K1_UNROLL;
constexpr int kK1TileVecs = kThreads * kK1Unroll;
#ifndef TDM_COPY_UNROLL
#define TDM_COPY_UNROLL TDM_K1_UNROLL
#endif
constexpr int kCopyUnroll = TDM_COPY_UNROLL;
constexpr int kCopyTileVecs = kThreads * kCopyUnroll;
constexpr int kTileVecs = kThreads * kUnroll;   // 1024 vectors = 16 KiB of every stream
// Measured on MI355X: one 16 KiB tile per workgroup beats a persistent grid-stride
// loop by 5-8% (the hardware dispatcher balances 8 XCDs better than a fixed stride),
// so the grid covers the tiles one to one up to 256 Ki workgroups (4 GiB per stream)
// and strides only beyond that.
constexpr int kDefaultBlocksPerCu = 1024;

int g_blocks_per_cu = kDefaultBlocksPerCu;
constexpr int64_t kColdFootprint = int64_t(512) << 20;  // twice the Infinity Cache

typedef uint32_t vec16 __attribute__((ext_vector_type(4)));  // one dwordx4 access

// ---------------------------------------------------------------- element types
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };

template <typename T> struct Elem;

template <> struct Elem<float> {
  using acc = float;
  static constexpr bool floating = true;
  static __device__ __forceinline__ acc widen(float x) { return x; }
  static __device__ __forceinline__ float narrow(acc x) { return x; }
};
template <> struct Elem<double> {
  using acc = double;
  static constexpr bool floating = true;
  static __device__ __forceinline__ acc widen(double x) { return x; }
  static __device__ __forceinline__ double narrow(acc x) { return x; }
};
template <> struct Elem<int64_t> {
  using acc = int64_t;
  static constexpr bool floating = false;
  static __device__ __forceinline__ acc widen(int64_t x) { return x; }
  static __device__ __forceinline__ int64_t narrow(acc x) { return x; }
};
template <> struct Elem<int32_t> {
  using acc = int32_t;
  static constexpr bool floating = false;
  static __device__ __forceinline__ acc widen(int32_t x) { return x; }
  static __device__ __forceinline__ int32_t narrow(acc x) { return x; }
};
template <> struct Elem<f16_t> {
  using acc = float;
  static constexpr bool floating = true;
  static __device__ __forceinline__ acc widen(f16_t x) {
    _Float16 h;
    __builtin_memcpy(&h, &x.bits, 2);
    return static_cast<float>(h);
  }
  static __device__ __forceinline__ f16_t narrow(acc x) {
    _Float16 h = static_cast<_Float16>(x);  // round to nearest even, once
    f16_t out;
    __builtin_memcpy(&out.bits, &h, 2);
    return out;
  }
};
template <> struct Elem<bf16_t> {
  using acc = float;
  static constexpr bool floating = true;
  static __device__ __forceinline__ acc widen(bf16_t x) { return __uint_as_float(static_cast<uint32_t>(x.bits) << 16); }
  static __device__ __forceinline__ bf16_t narrow(acc x) {
    uint32_t u = __float_as_uint(x);
    bf16_t out;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
      out.bits = 0x7fc0u;  // NaN
    } else {
      u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
      out.bits = static_cast<uint16_t>(u >> 16);
    }
    return out;
  }
};

// x / world as the element type would store it. kDiv: 0 none, 1 world is a power
// of two (multiplying by the exact reciprocal gives the same bits as dividing,
// denormal results included), 2 true division.
template <typename T, int kDiv>
__device__ __forceinline__ typename Elem<T>::acc scaled(typename Elem<T>::acc x, typename Elem<T>::acc divisor,
                                                        typename Elem<T>::acc reciprocal) {
  using A = typename Elem<T>::acc;
  if constexpr (kDiv == 0 || !Elem<T>::floating) {
    return x;
  } else if constexpr (kDiv == 1) {
    return Elem<T>::widen(Elem<T>::narrow(static_cast<A>(x * reciprocal)));
  } else {
    return Elem<T>::widen(Elem<T>::narrow(static_cast<A>(x / divisor)));
  }
}

template <typename T>
constexpr int lanes() { return 16 / static_cast<int>(sizeof(T)); }

template <typename T>
struct Lanes {
  T v[lanes<T>()];
};

template <typename T>
__device__ __forceinline__ Lanes<T> unpack(const vec16& raw) {
  Lanes<T> out;
  __builtin_memcpy(&out, &raw, 16);
  return out;
}
template <typename T>
__device__ __forceinline__ vec16 pack(const Lanes<T>& in) {
  vec16 out;
  __builtin_memcpy(&out, &in, 16);
  return out;
}

// Cache policy, measured on MI355X. K1 with 4 x 64 MiB chunk pairs per launch: a
// stream that is only read does best with non-temporal loads (it is not kept in
// L2 / Infinity Cache), a stream that is read, modified and written back does best
// with plain loads and plain stores (the store hits the line the load brought in).
// Both non-temporal: 6.4 TB/s; both plain: 5.4; this split: 7.0. The bucket fold
// and AdamW run once per training step over data that nothing has touched since
// the last step: there non-temporal stores pay as well (fold 0.260 -> 0.240 ms,
// AdamW on four shards 0.448 -> 0.415 ms), and for AdamW non-temporal loads of
// the streams it rewrites.
// -DTDM_NT_MASK=<0..7> (and _K2, _K3) build the other combinations for measurement.
#ifndef TDM_NT_MASK
#define TDM_NT_MASK 2  // bit0: read-modify-write loads, bit1: read-once loads, bit2: stores are non-temporal
#endif
#ifndef TDM_NT_MASK_K2
#define TDM_NT_MASK_K2 6  // the bucket fold over a device table (the by-value fold of one collective keeps TDM_NT_MASK)
#endif
#ifndef TDM_NT_MASK_K3
#define TDM_NT_MASK_K3 7  // AdamW
#endif
#ifndef TDM_NT_MASK_K3C
#define TDM_NT_MASK_K3C TDM_NT_MASK_K3  // AdamW's further copies of the parameters
#endif
template <int kMask = TDM_NT_MASK>
__device__ __forceinline__ vec16 load_stream(const void* p) {  // read once, never written here
  if constexpr (kMask & 2) return __builtin_nontemporal_load(static_cast<const vec16*>(p));
  else return *static_cast<const vec16*>(p);
}
template <int kMask = TDM_NT_MASK>
__device__ __forceinline__ vec16 load_rmw(const void* p) {  // about to be overwritten by this lane
  if constexpr (kMask & 1) return __builtin_nontemporal_load(static_cast<const vec16*>(p));
  else return *static_cast<const vec16*>(p);
}
template <int kMask = TDM_NT_MASK>
__device__ __forceinline__ void store16(void* p, const vec16& v) {
  if constexpr (kMask & 4) __builtin_nontemporal_store(v, static_cast<vec16*>(p));
  else *static_cast<vec16*>(p) = v;
}

// ---------------------------------------------------------------- pair tables
// Passed by value in the kernel arguments (scalar loads; no device table).
struct PairTable {
  int npairs;
  int flags;  // per launch: bit0 scale_dst, bit1 scale_src, bit2 writeback_src
  int64_t tile_end[TDM_MAX_PAIRS];  // running tile count
  char* dst[TDM_MAX_PAIRS];
  char* src[TDM_MAX_PAIRS];
  int64_t count[TDM_MAX_PAIRS];
  int32_t head[TDM_MAX_PAIRS];    // elements before dst reaches a 16-byte boundary
  int32_t vec_ok[TDM_MAX_PAIRS];  // dst and src share the same phase within 16 bytes
};

template <typename T>
struct Divisor {
  typename Elem<T>::acc divisor, reciprocal;
};

// dst = (dst[/w]) + (src[/w]) on one element
template <typename T, int kDiv>
__device__ __forceinline__ void reduce_elem(T& d, T& s, bool scale_dst, bool scale_src, const Divisor<T>& dv) {
  using A = typename Elem<T>::acc;
  A x = Elem<T>::widen(d), y = Elem<T>::widen(s);
  if (scale_dst) x = scaled<T, kDiv>(x, dv.divisor, dv.reciprocal);
  if (scale_src) y = scaled<T, kDiv>(y, dv.divisor, dv.reciprocal);
  s = Elem<T>::narrow(y);
  d = Elem<T>::narrow(static_cast<A>(x + y));
}

template <typename T, int kDiv, int kMask>
__global__ __launch_bounds__(kThreads) void k1_reduce_kernel(PairTable tab, Divisor<T> dv) {
  constexpr int L = lanes<T>();
  constexpr int64_t kTileElems = static_cast<int64_t>(kK1TileVecs) * L;
  const bool scale_dst = tab.flags & 1, scale_src = tab.flags & 2, writeback = tab.flags & 4;
  const int64_t total = tab.tile_end[tab.npairs - 1];
  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    int p = 0;
    while (tile >= tab.tile_end[p]) ++p;
    const int64_t t = tile - (p ? tab.tile_end[p - 1] : 0);
    T* __restrict__ dst = reinterpret_cast<T*>(tab.dst[p]);
    T* __restrict__ src = reinterpret_cast<T*>(tab.src[p]);
    const int64_t n = tab.count[p];
    if (tab.vec_ok[p]) {
      const int64_t head = tab.head[p];
      const int64_t nv = (n - head) / L;
      char* dvp = reinterpret_cast<char*>(dst + head);
      char* svp = reinterpret_cast<char*>(src + head);
      const int64_t v0 = t * kK1TileVecs + threadIdx.x;
      if ((t + 1) * kK1TileVecs <= nv) {  // a full tile: all loads first, then the arithmetic, then the stores
        vec16 a[kK1Unroll], b[kK1Unroll];
#pragma unroll
        for (int k = 0; k < kK1Unroll; ++k) a[k] = load_rmw<kMask>(dvp + (v0 + k * kThreads) * 16);
#pragma unroll
        for (int k = 0; k < kK1Unroll; ++k) b[k] = load_stream<kMask>(svp + (v0 + k * kThreads) * 16);
#pragma unroll
        for (int k = 0; k < kK1Unroll; ++k) {
          Lanes<T> x = unpack<T>(a[k]), y = unpack<T>(b[k]);
#pragma unroll
          for (int l = 0; l < L; ++l) reduce_elem<T, kDiv>(x.v[l], y.v[l], scale_dst, scale_src, dv);
          store16<kMask>(dvp + (v0 + k * kThreads) * 16, pack<T>(x));
          if (writeback) store16<kMask>(svp + (v0 + k * kThreads) * 16, pack<T>(y));
        }
      } else {
#pragma unroll
        for (int k = 0; k < kK1Unroll; ++k) {
          const int64_t v = v0 + k * kThreads;
          if (v < nv) {
            Lanes<T> x = unpack<T>(load_rmw<kMask>(dvp + v * 16)), y = unpack<T>(load_stream<kMask>(svp + v * 16));
#pragma unroll
            for (int l = 0; l < L; ++l) reduce_elem<T, kDiv>(x.v[l], y.v[l], scale_dst, scale_src, dv);
            store16<kMask>(dvp + v * 16, pack<T>(x));
            if (writeback) store16<kMask>(svp + v * 16, pack<T>(y));
          }
        }
      }
      if (t == 0) {  // the few elements before and after the 16-byte body
        const int64_t tail0 = head + nv * L;
        int64_t i = -1;
        if (static_cast<int64_t>(threadIdx.x) < head) i = threadIdx.x;
        else if (threadIdx.x >= 32 && tail0 + (threadIdx.x - 32) < n && threadIdx.x - 32 < L) i = tail0 + (threadIdx.x - 32);
        if (i >= 0) {
          T x = dst[i], y = src[i];
          reduce_elem<T, kDiv>(x, y, scale_dst, scale_src, dv);
          dst[i] = x;
          if (writeback) src[i] = y;
        }
      }
    } else {  // the two pointers disagree within 16 bytes: element-wise, still coalesced
      const int64_t e0 = t * kTileElems + threadIdx.x;
#pragma unroll 4
      for (int k = 0; k < kK1Unroll * L; ++k) {
        const int64_t i = e0 + static_cast<int64_t>(k) * kThreads;
        if (i < n) {
          T x = dst[i], y = src[i];
          reduce_elem<T, kDiv>(x, y, scale_dst, scale_src, dv);
          dst[i] = x;
          if (writeback) src[i] = y;
        }
      }
    }
  }
}

template <typename T, int kDiv>
__device__ __forceinline__ T copy_elem(T s, const Divisor<T>& dv) {
  if constexpr (kDiv == 0) {
    return s;
  } else {
    return Elem<T>::narrow(scaled<T, kDiv>(Elem<T>::widen(s), dv.divisor, dv.reciprocal));
  }
}

template <typename T, int kDiv, int kMask>
__global__ __launch_bounds__(kThreads) void k1_copy_kernel(PairTable tab, Divisor<T> dv) {
  constexpr int L = lanes<T>();
  constexpr int64_t kTileElems = static_cast<int64_t>(kCopyTileVecs) * L;
  const int64_t total = tab.tile_end[tab.npairs - 1];
  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    int p = 0;
    while (tile >= tab.tile_end[p]) ++p;
    const int64_t t = tile - (p ? tab.tile_end[p - 1] : 0);
    T* __restrict__ dst = reinterpret_cast<T*>(tab.dst[p]);
    const T* __restrict__ src = reinterpret_cast<const T*>(tab.src[p]);
    const int64_t n = tab.count[p];
    if (tab.vec_ok[p]) {
      const int64_t head = tab.head[p];
      const int64_t nv = (n - head) / L;
      char* dvp = reinterpret_cast<char*>(dst + head);
      const char* svp = reinterpret_cast<const char*>(src + head);
      const int64_t v0 = t * kCopyTileVecs + threadIdx.x;
      if ((t + 1) * kCopyTileVecs <= nv) {
        vec16 b[kCopyUnroll];
#pragma unroll
        for (int k = 0; k < kCopyUnroll; ++k) b[k] = load_stream<kMask>(svp + (v0 + k * kThreads) * 16);
#pragma unroll
        for (int k = 0; k < kCopyUnroll; ++k) {
          if constexpr (kDiv != 0) {
            Lanes<T> y = unpack<T>(b[k]);
#pragma unroll
            for (int l = 0; l < L; ++l) y.v[l] = copy_elem<T, kDiv>(y.v[l], dv);
            b[k] = pack<T>(y);
          }
          store16<kMask>(dvp + (v0 + k * kThreads) * 16, b[k]);
        }
      } else {
#pragma unroll
        for (int k = 0; k < kCopyUnroll; ++k) {
          const int64_t v = v0 + k * kThreads;
          if (v < nv) {
            Lanes<T> y = unpack<T>(load_stream<kMask>(svp + v * 16));
#pragma unroll
            for (int l = 0; l < L; ++l) y.v[l] = copy_elem<T, kDiv>(y.v[l], dv);
            store16<kMask>(dvp + v * 16, pack<T>(y));
          }
        }
      }
      if (t == 0) {
        const int64_t tail0 = head + nv * L;
        int64_t i = -1;
        if (static_cast<int64_t>(threadIdx.x) < head) i = threadIdx.x;
        else if (threadIdx.x >= 32 && tail0 + (threadIdx.x - 32) < n && threadIdx.x - 32 < L) i = tail0 + (threadIdx.x - 32);
        if (i >= 0) dst[i] = copy_elem<T, kDiv>(src[i], dv);
      }
    } else {
      const int64_t e0 = t * kTileElems + threadIdx.x;
#pragma unroll 4
      for (int k = 0; k < kCopyUnroll * L; ++k) {
        const int64_t i = e0 + static_cast<int64_t>(k) * kThreads;
        if (i < n) dst[i] = copy_elem<T, kDiv>(src[i], dv);
      }
    }
  }
}

// ---------------------------------------------------------------- K2: bucket fold
// A segment as the kernels see it. The device table of K2 is an array of these, ONE
// PER TILE: the pointers already advanced to the tile's first element and `count`
// the tile's elements, so a workgroup needs a single lookup before its loads go out
// (a tile -> segment -> pointers chain cost 20% of the kernel's throughput).
struct FoldSegDev {
  const char* src[TDM_MAX_WORLD];
  char* dst[TDM_MAX_WORLD];
  int64_t count;
  int32_t chunk;
  int32_t vec_ok;  // every pointer of the segment is 16-byte aligned
};

// One tile of one segment: W loads per element, the fold in ring order, W stores.
// kAcc: the result is added into each destination (dst = dst + sum) instead of replacing it.
template <typename T, int kWorld, int kDiv, bool kAcc, int kMask>
__device__ __forceinline__ void fold_tile(const FoldSegDev& sg, int64_t t, const Divisor<T>& dv) {
  using A = typename Elem<T>::acc;
  constexpr int L = lanes<T>();
#ifndef TDM_K2_UNROLL_W2
#define TDM_K2_UNROLL_W2 4
#endif
#ifndef TDM_K2_UNROLL
#define TDM_K2_UNROLL 4
#endif
  // vectors per lane per tile step, per rank (worlds 3-4: 4 beats 2 by 2-3 %; beyond that the registers run out)
  constexpr int kU = kWorld <= 2 ? TDM_K2_UNROLL_W2 : kWorld <= 4 ? TDM_K2_UNROLL : 2;
  constexpr int64_t kTileElems = static_cast<int64_t>(kTileVecs) * L;
  const int64_t n = sg.count;
  const int c = sg.chunk;
  // ring order: the fold starts at rank chunk+1 and ends with the chunk's owner
  const char* sp[kWorld];
  char* dp[kWorld];
#pragma unroll
  for (int k = 0; k < kWorld; ++k) {
    sp[k] = sg.src[(c + 1 + k) % kWorld];
    dp[k] = sg.dst[k];
  }
  if (sg.vec_ok) {
    const int64_t nv = n / L;
#pragma unroll
    for (int u0 = 0; u0 < kUnroll; u0 += kU) {
      const int64_t vbase = t * kTileVecs + threadIdx.x + static_cast<int64_t>(u0) * kThreads;
      vec16 in[kWorld][kU];
#pragma unroll
      for (int k = 0; k < kWorld; ++k)
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int64_t v = vbase + u * kThreads;
          if (v < nv) in[k][u] = load_stream<kMask>(sp[k] + v * 16);
        }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t v = vbase + u * kThreads;
        if (v < nv) {
          Lanes<T> out;
#pragma unroll
          for (int l = 0; l < L; ++l) {
            A acc = scaled<T, kDiv>(Elem<T>::widen(unpack<T>(in[0][u]).v[l]), dv.divisor, dv.reciprocal);
#pragma unroll
            for (int k = 1; k < kWorld; ++k) {
              const A y = scaled<T, kDiv>(Elem<T>::widen(unpack<T>(in[k][u]).v[l]), dv.divisor, dv.reciprocal);
              acc = Elem<T>::widen(Elem<T>::narrow(static_cast<A>(y + acc)));
            }
            out.v[l] = Elem<T>::narrow(acc);
          }
          const vec16 packed = pack<T>(out);
#pragma unroll
          for (int k = 0; k < kWorld; ++k)
            if (dp[k]) {
              if constexpr (kAcc) {
                Lanes<T> cur = unpack<T>(load_rmw<kMask>(dp[k] + v * 16));
#pragma unroll
                for (int l = 0; l < L; ++l)
                  cur.v[l] = Elem<T>::narrow(static_cast<A>(Elem<T>::widen(cur.v[l]) + Elem<T>::widen(out.v[l])));
                store16<kMask>(dp[k] + v * 16, pack<T>(cur));
              } else {
                store16<kMask>(dp[k] + v * 16, packed);
              }
            }
        }
      }
    }
    if (t == 0 && threadIdx.x < n - nv * L) {  // tail elements
      const int64_t i = nv * L + threadIdx.x;
      A acc = scaled<T, kDiv>(Elem<T>::widen(reinterpret_cast<const T*>(sp[0])[i]), dv.divisor, dv.reciprocal);
#pragma unroll
      for (int k = 1; k < kWorld; ++k) {
        const A y = scaled<T, kDiv>(Elem<T>::widen(reinterpret_cast<const T*>(sp[k])[i]), dv.divisor, dv.reciprocal);
        acc = Elem<T>::widen(Elem<T>::narrow(static_cast<A>(y + acc)));
      }
#pragma unroll
      for (int k = 0; k < kWorld; ++k)
        if (dp[k]) {
          T* out1 = reinterpret_cast<T*>(dp[k]) + i;
          *out1 = kAcc ? Elem<T>::narrow(static_cast<A>(Elem<T>::widen(*out1) + Elem<T>::widen(Elem<T>::narrow(acc)))) : Elem<T>::narrow(acc);
        }
    }
  } else {
    const int64_t e0 = t * kTileElems + threadIdx.x;
    for (int k2 = 0; k2 < kUnroll * L; ++k2) {
      const int64_t i = e0 + static_cast<int64_t>(k2) * kThreads;
      if (i < n) {
        A acc = scaled<T, kDiv>(Elem<T>::widen(reinterpret_cast<const T*>(sp[0])[i]), dv.divisor, dv.reciprocal);
#pragma unroll
        for (int k = 1; k < kWorld; ++k) {
          const A y = scaled<T, kDiv>(Elem<T>::widen(reinterpret_cast<const T*>(sp[k])[i]), dv.divisor, dv.reciprocal);
          acc = Elem<T>::widen(Elem<T>::narrow(static_cast<A>(y + acc)));
        }
#pragma unroll
        for (int k = 0; k < kWorld; ++k)
          if (dp[k]) {
            T* out1 = reinterpret_cast<T*>(dp[k]) + i;
            *out1 = kAcc ? Elem<T>::narrow(static_cast<A>(Elem<T>::widen(*out1) + Elem<T>::widen(Elem<T>::narrow(acc)))) : Elem<T>::narrow(acc);
          }
      }
    }
  }
}

// Table in device memory, one record per tile (many segments: DDP's buckets).
template <typename T, int kWorld, int kDiv, bool kAcc>
__global__ __launch_bounds__(kThreads) void k2_fold_kernel(const FoldSegDev* __restrict__ tiles, int64_t total,
                                                           Divisor<T> dv) {
  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    fold_tile<T, kWorld, kDiv, kAcc, TDM_NT_MASK_K2>(tiles[tile], 0, dv);
  }
}

// Table by value (one segment per ring chunk: a whole all-reduce in one launch).
struct FoldSmall {
  int nseg;
  int64_t tile_end[TDM_MAX_WORLD];
  FoldSegDev seg[TDM_MAX_WORLD];
};

// kCold: the launch's footprint is far beyond the 256 MB Infinity Cache, so nothing it
// writes will be read from there: the cache policy of the once-per-step bucket fold.
template <typename T, int kWorld, int kDiv, bool kCold>
__global__ __launch_bounds__(kThreads) void k2_fold_small_kernel(FoldSmall tab, Divisor<T> dv) {
  const int64_t total = tab.tile_end[tab.nseg - 1];
  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    int lo = 0;
    while (tile >= tab.tile_end[lo]) ++lo;
    fold_tile<T, kWorld, kDiv, false, kCold ? TDM_NT_MASK_K2 : TDM_NT_MASK>(tab.seg[lo], tile - (lo ? tab.tile_end[lo - 1] : 0), dv);
  }
}

// ---------------------------------------------------------------- K3: AdamW
struct AdamwArgs {
  float* p;
  const float* g;
  float* m;
  float* v;
  int64_t n;
  tdm_adamw_scalars s;
  // Further copies of the updated parameters (the other ranks' flat buffers): the
  // update and the all-gather of the result in one pass.
  int ncopies;
  float* copy[TDM_MAX_WORLD - 1];
};

template <int kOrder>
__device__ __forceinline__ void adamw_elem(float& p, float g, float& m, float& v, const tdm_adamw_scalars& s,
                                           bool small_w) {
  if (s.use_decay) p = p * s.decay;
  const float diff = g - m;
  // lerp_: weight < 0.5 ? fma(w, end-start, start) : fma(w-1, end-start, end)
  m = small_w ? __builtin_fmaf(s.w1, diff, m) : __builtin_fmaf(s.w1 - 1.0f, diff, g);
  const float vs = v * s.beta2;
  if constexpr (kOrder == TDM_ADAMW_HOST_ORDER) {
    v = __builtin_fmaf(s.one_m_b2 * g, g, vs);  // CPU addcmul_: (value*g) rounded, then fused
  } else {
    v = __builtin_fmaf(s.one_m_b2, g * g, vs);  // GPU addcmul_: a + value * (g*g), contracted
  }
  if constexpr (kOrder == TDM_ADAMW_HOST_ORDER) {
    const float d = __builtin_sqrtf(v) / s.bc2_sqrt + s.eps;
    p = p + (s.neg_step * m) / d;  // CPU addcdiv_: (value*m)/d, then add; nothing fused
  } else {
    const float d = __builtin_sqrtf(v) * s.inv_bc2_sqrt + s.eps;  // GPU tensor / scalar: times the reciprocal
    p = __builtin_fmaf(s.neg_step, m / d, p);  // GPU addcdiv_: a + value * (m/d), contracted
  }
}

#ifndef TDM_K3_UNROLL
#define TDM_K3_UNROLL 1
#endif
constexpr int kAdamwUnroll = TDM_K3_UNROLL;  // vectors per lane and stream in flight

template <int kOrder, bool kVec, bool kCopies>
__global__ __launch_bounds__(kThreads) void k3_adamw_kernel(AdamwArgs a) {
  const bool small_w = __builtin_fabsf(a.s.w1) < 0.5f;
  if constexpr (kVec) {
    constexpr int kU = kAdamwUnroll;
    const int64_t nv = a.n / 4;
    const int64_t tiles = (nv + kThreads * kU - 1) / (kThreads * kU);
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
      const int64_t v0 = tile * (kThreads * kU) + threadIdx.x;
      vec16 rp[kU], rg[kU], rm[kU], rv[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t i = v0 + u * kThreads;
        if (i < nv) {
          rp[u] = load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.p) + i * 16);
          rg[u] = load_stream<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.g) + i * 16);
          rm[u] = load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.m) + i * 16);
          rv[u] = load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.v) + i * 16);
        }
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t i = v0 + u * kThreads;
        if (i < nv) {
          Lanes<float> P = unpack<float>(rp[u]), G = unpack<float>(rg[u]), M = unpack<float>(rm[u]),
                       V = unpack<float>(rv[u]);
#pragma unroll
          for (int l = 0; l < 4; ++l) adamw_elem<kOrder>(P.v[l], G.v[l], M.v[l], V.v[l], a.s, small_w);
          const vec16 packed = pack<float>(P);
          store16<TDM_NT_MASK_K3>(reinterpret_cast<char*>(a.p) + i * 16, packed);
          if constexpr (kCopies)
            for (int c = 0; c < a.ncopies; ++c) store16<TDM_NT_MASK_K3C>(reinterpret_cast<char*>(a.copy[c]) + i * 16, packed);
          store16<TDM_NT_MASK_K3>(reinterpret_cast<char*>(a.m) + i * 16, pack<float>(M));
          store16<TDM_NT_MASK_K3>(reinterpret_cast<char*>(a.v) + i * 16, pack<float>(V));
        }
      }
    }
    if (blockIdx.x == 0 && threadIdx.x < a.n - nv * 4) {
      const int64_t i = nv * 4 + threadIdx.x;
      adamw_elem<kOrder>(a.p[i], a.g[i], a.m[i], a.v[i], a.s, small_w);
      if constexpr (kCopies)
        for (int c = 0; c < a.ncopies; ++c) a.copy[c][i] = a.p[i];
    }
  } else {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < a.n; i += stride) {
      adamw_elem<kOrder>(a.p[i], a.g[i], a.m[i], a.v[i], a.s, small_w);
      if constexpr (kCopies)
        for (int c = 0; c < a.ncopies; ++c) a.copy[c][i] = a.p[i];
    }
  }
}

// ---------------------------------------------------------------- K2 + K3: ZeRO-2's whole step
// For every element of every bucket segment, in one launch: the gradients of all ranks
// are folded in the ring's order for the segment's chunk (K2), the sum is added to a zero
// gradient shard as ZeRO's grad_shard.add_(mine) would (0.0f + mine: a -0.0 becomes +0.0),
// the chunk's owner takes its AdamW step (K3), and the new parameter is written into every
// rank's flat buffer (the all-gather). 4W + 12 bytes read and 4W + 8 written per element,
// where reduce-scatter, add, AdamW and all-gather apart move 4(W+2) + 28 + 8(W-1).
struct StepSegDev {
  const char* g[TDM_MAX_WORLD];  // every rank's gradient for this tile
  char* p[TDM_MAX_WORLD];        // every rank's copy of the parameters for this tile
  char* m;                       // the owner's exp_avg
  char* v;                       // the owner's exp_avg_sq
  int64_t count;
  int32_t chunk;                 // the owner
  int32_t vec_ok;
};

#ifndef TDM_K23_UNROLL
#define TDM_K23_UNROLL 4
#endif
#ifndef TDM_NT_MASK_K23
#define TDM_NT_MASK_K23 TDM_NT_MASK_K3
#endif

// One tile (at most 16 KiB of every stream) of the step.
template <int kWorld, int kDiv, int kOrder>
__device__ __forceinline__ void step_tile(const StepSegDev& sg, int64_t at, int64_t n, const Divisor<float>& dv,
                                          const tdm_adamw_scalars& s, bool small_w) {
  constexpr int kU = kWorld <= 4 ? TDM_K23_UNROLL : 1;  // vectors per lane in flight, per stream
  constexpr int kM = TDM_NT_MASK_K23;
  {
    const int c = sg.chunk;  // `at`: the tile's offset in bytes from the record's pointers; n: its elements
    const char* gp[kWorld];
    char* pp[kWorld];
#pragma unroll
    for (int k = 0; k < kWorld; ++k) {
      gp[k] = sg.g[(c + 1 + k) % kWorld] + at;  // the fold ends with the owner's own term
      pp[k] = sg.p[k] + at;
    }
    char* own = sg.p[c] + at;
    char* const mm = sg.m + at;
    char* const vv = sg.v + at;
    auto one = [&](float grads_in_order[kWorld], float& P, float& M, float& V) {
      float acc = scaled<float, kDiv>(grads_in_order[0], dv.divisor, dv.reciprocal);
#pragma unroll
      for (int k = 1; k < kWorld; ++k) acc = scaled<float, kDiv>(grads_in_order[k], dv.divisor, dv.reciprocal) + acc;
      const float g = 0.0f + acc;  // grad_shard (zero) += mine
      adamw_elem<kOrder>(P, g, M, V, s, small_w);
    };
    if (sg.vec_ok) {
      const int64_t nv = n / 4;
#pragma unroll
      for (int u0 = 0; u0 < kUnroll; u0 += kU) {
        vec16 in[kWorld][kU], rp[kU], rm[kU], rv[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int64_t v = threadIdx.x + static_cast<int64_t>(u0 + u) * kThreads;
          if (v < nv) {
#pragma unroll
            for (int k = 0; k < kWorld; ++k) in[k][u] = load_stream<kM>(gp[k] + v * 16);
            rp[u] = load_rmw<kM>(own + v * 16);
            rm[u] = load_rmw<kM>(mm + v * 16);
            rv[u] = load_rmw<kM>(vv + v * 16);
          }
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int64_t v = threadIdx.x + static_cast<int64_t>(u0 + u) * kThreads;
          if (v < nv) {
            Lanes<float> P = unpack<float>(rp[u]), M = unpack<float>(rm[u]), V = unpack<float>(rv[u]);
#pragma unroll
            for (int l = 0; l < 4; ++l) {
              float gs[kWorld];
#pragma unroll
              for (int k = 0; k < kWorld; ++k) gs[k] = unpack<float>(in[k][u]).v[l];
              one(gs, P.v[l], M.v[l], V.v[l]);
            }
            const vec16 packed = pack<float>(P);
#pragma unroll
            for (int q = 0; q < kWorld; ++q) store16<kM>(pp[q] + v * 16, packed);
            store16<kM>(mm + v * 16, pack<float>(M));
            store16<kM>(vv + v * 16, pack<float>(V));
          }
        }
      }
      if (threadIdx.x < n - nv * 4) {  // the tile's last few elements
        const int64_t i = nv * 4 + threadIdx.x;
        float gs[kWorld];
#pragma unroll
        for (int k = 0; k < kWorld; ++k) gs[k] = reinterpret_cast<const float*>(gp[k])[i];
        float P = reinterpret_cast<float*>(own)[i], M = reinterpret_cast<float*>(mm)[i], V = reinterpret_cast<float*>(vv)[i];
        one(gs, P, M, V);
#pragma unroll
        for (int q = 0; q < kWorld; ++q) reinterpret_cast<float*>(pp[q])[i] = P;
        reinterpret_cast<float*>(mm)[i] = M;
        reinterpret_cast<float*>(vv)[i] = V;
      }
    } else {
      for (int64_t i = threadIdx.x; i < n; i += kThreads) {
        float gs[kWorld];
#pragma unroll
        for (int k = 0; k < kWorld; ++k) gs[k] = reinterpret_cast<const float*>(gp[k])[i];
        float P = reinterpret_cast<float*>(own)[i], M = reinterpret_cast<float*>(mm)[i], V = reinterpret_cast<float*>(vv)[i];
        one(gs, P, M, V);
#pragma unroll
        for (int q = 0; q < kWorld; ++q) reinterpret_cast<float*>(pp[q])[i] = P;
        reinterpret_cast<float*>(mm)[i] = M;
        reinterpret_cast<float*>(vv)[i] = V;
      }
    }
  }
}

template <int kWorld, int kDiv, int kOrder>
__global__ __launch_bounds__(kThreads) void k23_zero2_step_kernel(const StepSegDev* __restrict__ tiles, int64_t total,
                                                                  Divisor<float> dv, tdm_adamw_scalars s) {
  const bool small_w = __builtin_fabsf(s.w1) < 0.5f;
  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    step_tile<kWorld, kDiv, kOrder>(tiles[tile], 0, tiles[tile].count, dv, s, small_w);
  }
}

// The same for ONE segment, described in the kernel's arguments: no table to keep in
// device memory. A rank that is a process of its own steps exactly one segment, its
// shard, out of its peers' gradient buffers and into their parameter buffers.
template <int kWorld, int kDiv, int kOrder>
__global__ __launch_bounds__(kThreads) void k23_zero2_step_one_kernel(StepSegDev whole, int64_t total, Divisor<float> dv,
                                                                      tdm_adamw_scalars s) {
  const bool small_w = __builtin_fabsf(s.w1) < 0.5f;
  constexpr int64_t kTileBytes = static_cast<int64_t>(kTileVecs) * 16;
  for (int64_t tile = blockIdx.x; tile < total; tile += gridDim.x) {
    const int64_t n = min(static_cast<int64_t>(kTileVecs) * 4, whole.count - tile * kTileVecs * 4);
    step_tile<kWorld, kDiv, kOrder>(whole, tile * kTileBytes, n, dv, s, small_w);
  }
}

// ---------------------------------------------------------------- host side
int elem_size(int dtype) {
  switch (dtype) {
    case TDM_F32: case TDM_I32: return 4;
    case TDM_F64: case TDM_I64: return 8;
    case TDM_F16: case TDM_BF16: return 2;
    default: return 0;
  }
}

bool is_floating(int dtype) { return dtype == TDM_F32 || dtype == TDM_F64 || dtype == TDM_F16 || dtype == TDM_BF16; }

int compute_units() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev];
}

int grid_for(int64_t tiles) {
  const int64_t cap = static_cast<int64_t>(compute_units()) * g_blocks_per_cu;
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
  switch (div_kind(world, any_scale)) {
    case 0: hipLaunchKernelGGL((k1_reduce_kernel<T, 0, kMask>), grid, block, 0, stream, tab, dv); break;
    case 1: hipLaunchKernelGGL((k1_reduce_kernel<T, 1, kMask>), grid, block, 0, stream, tab, dv); break;
    default: hipLaunchKernelGGL((k1_reduce_kernel<T, 2, kMask>), grid, block, 0, stream, tab, dv); break;
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
  const dim3 grid(grid_for(tiles)), block(kThreads);
  switch (div_kind(world, true)) {
    case 0: hipLaunchKernelGGL((k1_copy_kernel<T, 0, kMask>), grid, block, 0, stream, tab, dv); break;
    case 1: hipLaunchKernelGGL((k1_copy_kernel<T, 1, kMask>), grid, block, 0, stream, tab, dv); break;
    default: hipLaunchKernelGGL((k1_copy_kernel<T, 2, kMask>), grid, block, 0, stream, tab, dv); break;
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
  const dim3 grid(grid_for(tiles)), block(kThreads);
  const FoldSegDev* img = static_cast<const FoldSegDev*>(image);
  switch (div_kind(kWorld, average != 0)) {
    case 0: hipLaunchKernelGGL((k2_fold_kernel<T, kWorld, 0, kAcc>), grid, block, 0, stream, img, tiles, dv); break;
    case 1: hipLaunchKernelGGL((k2_fold_kernel<T, kWorld, 1, kAcc>), grid, block, 0, stream, img, tiles, dv); break;
    default: hipLaunchKernelGGL((k2_fold_kernel<T, kWorld, 2, kAcc>), grid, block, 0, stream, img, tiles, dv); break;
  }
}

template <typename T, int kWorld>
void launch_fold_small_w(const FoldSmall& tab, int average, hipStream_t stream) {
  const Divisor<T> dv = make_divisor<T>(kWorld);
  const dim3 grid(grid_for(tab.tile_end[tab.nseg - 1])), block(kThreads);
  // bytes touched: every tile is read from kWorld ranks (and written back to most of them)
  const bool cold = tab.tile_end[tab.nseg - 1] * static_cast<int64_t>(kTileVecs) * 16 * kWorld > kColdFootprint;
  switch (div_kind(kWorld, average != 0) * 2 + (cold ? 1 : 0)) {
    case 0: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 0, false>), grid, block, 0, stream, tab, dv); break;
    case 1: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 0, true>), grid, block, 0, stream, tab, dv); break;
    case 2: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 1, false>), grid, block, 0, stream, tab, dv); break;
    case 3: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 1, true>), grid, block, 0, stream, tab, dv); break;
    case 4: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 2, false>), grid, block, 0, stream, tab, dv); break;
    default: hipLaunchKernelGGL((k2_fold_small_kernel<T, kWorld, 2, true>), grid, block, 0, stream, tab, dv); break;
  }
}

template <typename T>
void launch_fold_small(const FoldSmall& tab, int world, int average, hipStream_t stream) {
  switch (world) {
    case 2: launch_fold_small_w<T, 2>(tab, average, stream); break;
    case 3: launch_fold_small_w<T, 3>(tab, average, stream); break;
    case 4: launch_fold_small_w<T, 4>(tab, average, stream); break;
    case 5: launch_fold_small_w<T, 5>(tab, average, stream); break;
    case 6: launch_fold_small_w<T, 6>(tab, average, stream); break;
    case 7: launch_fold_small_w<T, 7>(tab, average, stream); break;
    case 8: launch_fold_small_w<T, 8>(tab, average, stream); break;
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
  const dim3 grid(grid_for(tiles)), block(kThreads);
  switch (div_kind(kWorld, average != 0)) {
    case 0: hipLaunchKernelGGL((k23_zero2_step_kernel<kWorld, 0, kOrder>), grid, block, 0, stream, t, tiles, dv, s); break;
    case 1: hipLaunchKernelGGL((k23_zero2_step_kernel<kWorld, 1, kOrder>), grid, block, 0, stream, t, tiles, dv, s); break;
    default: hipLaunchKernelGGL((k23_zero2_step_kernel<kWorld, 2, kOrder>), grid, block, 0, stream, t, tiles, dv, s); break;
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
  const dim3 grid(grid_for(tiles)), block(kThreads);
  switch (div_kind(kWorld, average != 0)) {
    case 0: hipLaunchKernelGGL((k23_zero2_step_one_kernel<kWorld, 0, kOrder>), grid, block, 0, stream, whole, tiles, dv, s); break;
    case 1: hipLaunchKernelGGL((k23_zero2_step_one_kernel<kWorld, 1, kOrder>), grid, block, 0, stream, whole, tiles, dv, s); break;
    default: hipLaunchKernelGGL((k23_zero2_step_one_kernel<kWorld, 2, kOrder>), grid, block, 0, stream, whole, tiles, dv, s); break;
  }
}

template <int kWorld>
void launch_step_one_w(const StepSegDev& whole, int64_t tiles, int average, const tdm_adamw_scalars& s, int order, hipStream_t stream) {
  if (order == TDM_ADAMW_HOST_ORDER) launch_step_one_o<kWorld, TDM_ADAMW_HOST_ORDER>(whole, tiles, average, s, stream);
  else launch_step_one_o<kWorld, TDM_ADAMW_DEVICE_ORDER>(whole, tiles, average, s, stream);
}

int64_t step_tiles(const tdm_step_seg* segs, int nseg) {
  const int64_t tile_elems = static_cast<int64_t>(kTileVecs) * 4;
  int64_t tiles = 0;
  for (int i = 0; i < nseg; ++i) tiles += segs[i].count > 0 ? (segs[i].count + tile_elems - 1) / tile_elems : 0;
  return tiles;
}

}  // namespace

// Used by the engine too: ZeRO-2's step over one segment (a rank's shard), see tdm_k23_zero2_step_segment.
void zero2_step_segment(const tdm_step_seg& sg, int world, bool average, const tdm_adamw_scalars& s, int order, hipStream_t stream) {
  if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
  if (order != TDM_ADAMW_HOST_ORDER && order != TDM_ADAMW_DEVICE_ORDER) throw Invalid("unknown update order");
  if (sg.count < 0) throw Invalid("negative count");
  if (sg.count == 0) return;
  if (sg.chunk < 0 || sg.chunk >= world) throw Invalid("chunk outside [0, world)");
  if (!sg.exp_avg || !sg.exp_avg_sq) throw Invalid("NULL optimizer state");
  StepSegDev whole;
  std::memset(&whole, 0, sizeof whole);
  bool vec = reinterpret_cast<uintptr_t>(sg.exp_avg) % 16 == 0 && reinterpret_cast<uintptr_t>(sg.exp_avg_sq) % 16 == 0;
  if (reinterpret_cast<uintptr_t>(sg.exp_avg) % 4 || reinterpret_cast<uintptr_t>(sg.exp_avg_sq) % 4) throw Invalid("pointer not aligned to 4 bytes");
  for (int r = 0; r < world; ++r) {
    if (!sg.grad[r] || !sg.param[r]) throw Invalid("NULL gradient or parameter");
    const uintptr_t a = reinterpret_cast<uintptr_t>(sg.grad[r]), b = reinterpret_cast<uintptr_t>(sg.param[r]);
    if (a % 4 || b % 4) throw Invalid("pointer not aligned to 4 bytes");
    vec = vec && a % 16 == 0 && b % 16 == 0;
    whole.g[r] = static_cast<const char*>(sg.grad[r]);
    whole.p[r] = static_cast<char*>(sg.param[r]);
  }
  whole.m = static_cast<char*>(sg.exp_avg);
  whole.v = static_cast<char*>(sg.exp_avg_sq);
  whole.count = sg.count;
  whole.chunk = sg.chunk;
  whole.vec_ok = vec;
  const int64_t tiles = step_tiles(&sg, 1);
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
  tab.flags = (any_scale && scale_dst ? 1 : 0) | (any_scale && scale_src ? 2 : 0) | (any_scale && scale_src && writeback_src ? 4 : 0);
  switch (dtype) {
    case TDM_F32: launch_reduce<float>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_F64: launch_reduce<double>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_F16: launch_reduce<f16_t>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_BF16: launch_reduce<bf16_t>(tab, tiles, world, any_scale, policy, stream); break;
    case TDM_I64: launch_reduce<int64_t>(tab, tiles, 1, false, policy, stream); break;
    default: launch_reduce<int32_t>(tab, tiles, 1, false, policy, stream); break;
  }
  check_hip(hipGetLastError(), "k1_reduce launch");
}

void copy_step(const tdm_pair* pairs, int npairs, int dtype, int world, hipStream_t stream, int policy) {
  const int es = elem_size(dtype);
  if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
  if (world > 1 && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
  PairTable tab;
  // dst == src is allowed when scaling in place (div_ of a chunk); partial overlap never is
  std::vector<tdm_pair> kept;
  for (int i = 0; i < npairs && pairs != nullptr; ++i) {
    if (pairs[i].dst == pairs[i].src && pairs[i].count > 0 && world <= 1) continue;  // copying onto itself
    kept.push_back(pairs[i]);
  }
  if (npairs > 0 && pairs == nullptr) throw Invalid("pairs is NULL");
  if (npairs < 0 || npairs > TDM_MAX_PAIRS) throw Invalid("npairs must be in [0, " + std::to_string(TDM_MAX_PAIRS) + "]");
  for (const tdm_pair& p : kept) {
    if (p.count > 0 && p.dst != p.src && p.dst != nullptr && p.src != nullptr) {
      const uintptr_t d = reinterpret_cast<uintptr_t>(p.dst), s = reinterpret_cast<uintptr_t>(p.src);
      const uintptr_t bytes = static_cast<uintptr_t>(p.count) * es;
      if (d < s + bytes && s < d + bytes) throw Invalid("copy: destination and source overlap");
    }
  }
  const int64_t tiles = build_pairs(kept.data(), static_cast<int>(kept.size()), es, false, kCopyTileVecs, &tab);
  if (tiles == 0) return;
  switch (dtype) {
    case TDM_F32: launch_copy<float>(tab, tiles, world, policy, stream); break;
    case TDM_F64: launch_copy<double>(tab, tiles, world, policy, stream); break;
    case TDM_F16: launch_copy<f16_t>(tab, tiles, world, policy, stream); break;
    case TDM_BF16: launch_copy<bf16_t>(tab, tiles, world, policy, stream); break;
    case TDM_I64: launch_copy<int64_t>(tab, tiles, 1, policy, stream); break;
    default: launch_copy<int32_t>(tab, tiles, 1, policy, stream); break;
  }
  check_hip(hipGetLastError(), "k1_copy launch");
}

// ---------------------------------------------------------------- a whole group in one process
// Rank r is bufs[r]; a ring step is ONE launch carrying every rank's pair.
namespace {

struct LocalRanks {
  std::vector<char*> base;
  std::vector<int64_t> lo, len;  // chunk bounds, in elements
  int world, es, dtype;
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
  for (int r = 0; r < world; ++r) {
    if (numel > 0 && bufs[r] == nullptr) throw Invalid("rank " + std::to_string(r) + ": NULL buffer");
    lr.base.push_back(static_cast<char*>(bufs[r]));
  }
  for (int a = 0; a < world && numel > 0; ++a)
    for (int b = a + 1; b < world; ++b) {
      const uintptr_t x = reinterpret_cast<uintptr_t>(bufs[a]), y = reinterpret_cast<uintptr_t>(bufs[b]);
      const uintptr_t bytes = static_cast<uintptr_t>(numel) * lr.es;
      if (x < y + bytes && y < x + bytes) throw Invalid("rank buffers overlap");
    }
  lr.lo.resize(world);
  lr.len.resize(world);
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
  if (const char* env = std::getenv("TDM_RING_POLICY")) {
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

int64_t footprint(const LocalRanks& lr) {  // bytes of all ranks' tensors together
  int64_t elems = 0;
  for (int64_t l : lr.len) elems += l;
  return elems * lr.es * lr.world;
}

void local_reduce_scatter(const LocalRanks& lr, bool average, bool keep_sent, hipStream_t stream) {
  const int n = lr.world;
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
void fold_step(const tdm_fold_seg* segs, int nseg, int world, int dtype, bool average, hipStream_t stream) {
  const int es = elem_size(dtype);
  if (es == 0) throw Invalid("unknown dtype " + std::to_string(dtype));
  if (world < 2 || world > TDM_MAX_WORLD) throw Invalid("the direct fold handles world sizes 2..8");
  if (nseg < 0 || nseg > TDM_MAX_WORLD || (nseg > 0 && segs == nullptr)) throw Invalid("the direct fold takes up to 8 segments");
  if (average && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
  FoldSmall tab;
  std::memset(&tab, 0, sizeof tab);
  const int64_t tile_elems = static_cast<int64_t>(kTileVecs) * (16 / es);
  int64_t tiles = 0;
  int k = 0;
  for (int i = 0; i < nseg; ++i) {
    const tdm_fold_seg& s = segs[i];
    if (s.count < 0) throw Invalid("fold: negative count");
    if (s.count == 0) continue;
    if (s.chunk < 0 || s.chunk >= world) throw Invalid("fold: chunk outside [0, world)");
    bool vec = true;
    for (int r = 0; r < world; ++r) {
      if (s.src[r] == nullptr) throw Invalid("fold: NULL source");
      const uintptr_t a = reinterpret_cast<uintptr_t>(s.src[r]), b = reinterpret_cast<uintptr_t>(s.dst[r]);
      if (a % es || b % es) throw Invalid("fold: pointer not aligned to the element size");
      vec = vec && a % 16 == 0 && b % 16 == 0;
      tab.seg[k].src[r] = static_cast<const char*>(s.src[r]);
      tab.seg[k].dst[r] = static_cast<char*>(s.dst[r]);
    }
    tab.seg[k].count = s.count;
    tab.seg[k].chunk = s.chunk;
    tab.seg[k].vec_ok = vec;
    tiles += (s.count + tile_elems - 1) / tile_elems;
    tab.tile_end[k] = tiles;
    ++k;
  }
  tab.nseg = k;
  if (k == 0) return;
  switch (dtype) {
    case TDM_F32: launch_fold_small<float>(tab, world, average, stream); break;
    case TDM_F64: launch_fold_small<double>(tab, world, average, stream); break;
    case TDM_F16: launch_fold_small<f16_t>(tab, world, average, stream); break;
    case TDM_BF16: launch_fold_small<bf16_t>(tab, world, average, stream); break;
    case TDM_I64: launch_fold_small<int64_t>(tab, world, 0, stream); break;
    default: launch_fold_small<int32_t>(tab, world, 0, stream); break;
  }
  check_hip(hipGetLastError(), "k2_fold_small launch");
}

}  // namespace tandem_hip

using namespace tandem_hip;

extern "C" {

int tdm_local_reduce_scatter(void* const* bufs, int world, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                             int average, int keep_sent, tdm_stream stream) {
  return guard([&] {
    if (average && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
    const LocalRanks lr = local_ranks(bufs, world, numel, dtype, sizes, nsizes);
    if (world > 1) local_reduce_scatter(lr, average != 0, keep_sent != 0, static_cast<hipStream_t>(stream));
  });
}

int tdm_local_all_gather(void* const* bufs, int world, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                         tdm_stream stream) {
  return guard([&] {
    const LocalRanks lr = local_ranks(bufs, world, numel, dtype, sizes, nsizes);
    if (world > 1) local_all_gather(lr, static_cast<hipStream_t>(stream));
  });
}

int tdm_local_all_reduce(void* const* bufs, int world, int64_t numel, int dtype, int average, int algorithm,
                         tdm_stream stream) {
  return guard([&] {
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

int tdm_set_blocks_per_cu(int blocks) {
  return guard([&] {
    if (blocks < 0 || blocks > 1024) throw Invalid("blocks per compute unit must be in [0, 1024]");
    g_blocks_per_cu = blocks == 0 ? kDefaultBlocksPerCu : blocks;
  });
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
  const int64_t tile_elems = static_cast<int64_t>(kTileVecs) * (16 / es);
  int64_t tiles = 0;
  for (int i = 0; i < nseg; ++i) tiles += segs[i].count > 0 ? (segs[i].count + tile_elems - 1) / tile_elems : 0;
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
      if (s.count < 0) throw Invalid("segment " + std::to_string(i) + ": negative count");
      if (s.chunk < 0 || s.chunk >= world) throw Invalid("segment " + std::to_string(i) + ": chunk outside [0, world)");
      bool vec = true;
      for (int r = 0; r < world; ++r) {
        if (s.count > 0 && s.src[r] == nullptr) throw Invalid("segment " + std::to_string(i) + ": NULL source");
        const uintptr_t a = reinterpret_cast<uintptr_t>(s.src[r]), b = reinterpret_cast<uintptr_t>(s.dst[r]);
        if (a % es || b % es) throw Invalid("segment " + std::to_string(i) + ": pointer not aligned to the element size");
        vec = vec && a % 16 == 0 && b % 16 == 0;
      }
      for (int64_t at = 0; at < s.count; at += tile_elems) {  // a tile's byte offset is a multiple of 16 KiB
        FoldSegDev& rec = out[tiles++];
        for (int r = 0; r < world; ++r) {
          rec.src[r] = static_cast<const char*>(s.src[r]) + at * es;
          rec.dst[r] = s.dst[r] ? static_cast<char*>(s.dst[r]) + at * es : nullptr;
        }
        rec.count = std::min<int64_t>(tile_elems, s.count - at);
        rec.chunk = s.chunk;
        rec.vec_ok = vec;
      }
    }
  });
}

int tdm_k2_bucket_fold(const void* table_dev, int64_t ntiles, int dtype, int world, int average, int accumulate,
                       tdm_stream stream) {
  return guard([&] {
    if (world < 1 || world > TDM_MAX_WORLD) throw Invalid("world must be in [1, 8]");
    if (ntiles < 0) throw Invalid("ntiles is negative");
    if (ntiles == 0) return;
    if (table_dev == nullptr) throw Invalid("table is NULL");
    if (average && world > 1 && !is_floating(dtype)) throw Invalid("integer tensors cannot be averaged in place");
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
      case TDM_F32: launch_fold<float>(table_dev, ntiles, world, average, accumulate != 0, st); break;
      case TDM_F64: launch_fold<double>(table_dev, ntiles, world, average, accumulate != 0, st); break;
      case TDM_F16: launch_fold<f16_t>(table_dev, ntiles, world, average, accumulate != 0, st); break;
      case TDM_BF16: launch_fold<bf16_t>(table_dev, ntiles, world, average, accumulate != 0, st); break;
      case TDM_I64: launch_fold<int64_t>(table_dev, ntiles, world, 0, accumulate != 0, st); break;
      case TDM_I32: launch_fold<int32_t>(table_dev, ntiles, world, 0, accumulate != 0, st); break;
      default: throw Invalid("unknown dtype " + std::to_string(dtype));
    }
    check_hip(hipGetLastError(), "k2_fold launch");
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
  AdamwArgs a{p, g, m, v, n, *s, ncopies, {}};
  for (int c = 0; c < ncopies; ++c) {
    if (!copies[c]) throw Invalid("NULL copy of the parameters");
    a.copy[c] = copies[c];
    ptrs[4 + c] = reinterpret_cast<uintptr_t>(copies[c]);
  }
  bool vec = true;
  for (int i = 0; i < 4 + ncopies; ++i) {
    if (ptrs[i] % 4) throw Invalid("pointer not aligned to 4 bytes");
    vec = vec && ptrs[i] % 16 == 0;
  }
  for (int i = 0; i < 4 + ncopies; ++i)
    for (int j = i + 1; j < 4 + ncopies; ++j) {
      const uintptr_t bytes = static_cast<uintptr_t>(n) * 4;
      if (ptrs[i] < ptrs[j] + bytes && ptrs[j] < ptrs[i] + bytes) throw Invalid("p, g, m, v and the copies must not overlap");
    }
  const dim3 block(kThreads);
  const int64_t tiles = vec ? (n / 4 + kThreads * kAdamwUnroll - 1) / (kThreads * kAdamwUnroll) : (n + kThreads - 1) / kThreads;
  const dim3 grid(grid_for(std::max<int64_t>(tiles, 1)));
  const int which = (order == TDM_ADAMW_HOST_ORDER ? 0 : 4) + (vec ? 2 : 0) + (ncopies > 0 ? 1 : 0);
  switch (which) {
    case 0: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, false, false>), grid, block, 0, st, a); break;
    case 1: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, false, true>), grid, block, 0, st, a); break;
    case 2: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, true, false>), grid, block, 0, st, a); break;
    case 3: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_HOST_ORDER, true, true>), grid, block, 0, st, a); break;
    case 4: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, false, false>), grid, block, 0, st, a); break;
    case 5: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, false, true>), grid, block, 0, st, a); break;
    case 6: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, true, false>), grid, block, 0, st, a); break;
    default: hipLaunchKernelGGL((k3_adamw_kernel<TDM_ADAMW_DEVICE_ORDER, true, true>), grid, block, 0, st, a); break;
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

int64_t tdm_k23_table_tiles(const tdm_step_seg* segs, int nseg) {
  if (nseg < 0 || (nseg > 0 && segs == nullptr)) return -1;
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
    std::memset(image, 0, static_cast<size_t>(tdm_k23_table_bytes(segs, nseg)));
    StepSegDev* out = static_cast<StepSegDev*>(image);
    const int64_t tile_elems = static_cast<int64_t>(kTileVecs) * 4;
    int64_t tiles = 0;
    for (int i = 0; i < nseg; ++i) {
      const tdm_step_seg& sg = segs[i];
      if (sg.count < 0) throw Invalid("segment " + std::to_string(i) + ": negative count");
      if (sg.count == 0) continue;
      if (sg.chunk < 0 || sg.chunk >= world) throw Invalid("segment " + std::to_string(i) + ": chunk outside [0, world)");
      if (!sg.exp_avg || !sg.exp_avg_sq) throw Invalid("segment " + std::to_string(i) + ": NULL optimizer state");
      bool vec = reinterpret_cast<uintptr_t>(sg.exp_avg) % 16 == 0 && reinterpret_cast<uintptr_t>(sg.exp_avg_sq) % 16 == 0;
      if (reinterpret_cast<uintptr_t>(sg.exp_avg) % 4 || reinterpret_cast<uintptr_t>(sg.exp_avg_sq) % 4) {
        throw Invalid("segment " + std::to_string(i) + ": pointer not aligned to 4 bytes");
      }
      for (int r = 0; r < world; ++r) {
        if (!sg.grad[r] || !sg.param[r]) throw Invalid("segment " + std::to_string(i) + ": NULL gradient or parameter");
        const uintptr_t a = reinterpret_cast<uintptr_t>(sg.grad[r]), b = reinterpret_cast<uintptr_t>(sg.param[r]);
        if (a % 4 || b % 4) throw Invalid("segment " + std::to_string(i) + ": pointer not aligned to 4 bytes");
        vec = vec && a % 16 == 0 && b % 16 == 0;
      }
      for (int64_t at = 0; at < sg.count; at += tile_elems) {
        StepSegDev& rec = out[tiles++];
        for (int r = 0; r < world; ++r) {
          rec.g[r] = static_cast<const char*>(sg.grad[r]) + at * 4;
          rec.p[r] = static_cast<char*>(sg.param[r]) + at * 4;
        }
        rec.m = static_cast<char*>(sg.exp_avg) + at * 4;
        rec.v = static_cast<char*>(sg.exp_avg_sq) + at * 4;
        rec.count = std::min<int64_t>(tile_elems, sg.count - at);
        rec.chunk = sg.chunk;
        rec.vec_ok = vec;
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

}  // extern "C"
