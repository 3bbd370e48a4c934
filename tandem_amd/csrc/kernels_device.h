// The device side of libtandem_hip: element types, load/store helpers with their cache
// policies, and the kernels K1 (ring-step reduce, copy), K2 (bucket fold), K3 (AdamW),
// K2+K3 (ZeRO-2's step) and K4's copies. Included by kernels.hip only: everything here
// has internal linkage.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "../../include/tandem_hip.h"
#include "common.h"

namespace tandem_hip {

namespace {


#ifndef TDM_THREADS
#define TDM_THREADS 128
#endif
#ifndef TDM_UNROLL
#define TDM_UNROLL 2
#endif
// Workgroups of two waves, two 16-byte vectors per lane and stream: 4 KiB of every stream per
// workgroup. How much one workgroup takes matters more than how many loads a lane keeps in flight,
// and it is the writes that are sensitive to it (a write-only probe over 2 GiB: 6.9 TB/s at 4 KiB
// per workgroup, 6.0 at 8-16 KiB, 5.7 at 32 KiB, 4.9 from a persistent grid, 5.5 at 2 KiB; read-only
// 7.0-7.1 at any of these). Against four waves and 8 KiB, in A/B runs inside one process on several
// machines: the ring's copy step 2.4-3.9 % faster, the two-rank bucket fold 3-7 %, the single-launch
// all-reduce at 256 MiB between 2.5 % faster and 1.8 % slower, K1's reduce step and AdamW equal, the
// one-launch ZeRO-2 step equal to 1.5 % slower. One wave per workgroup is slower throughout (too
// many workgroups to dispatch), and so is 16 KiB.
constexpr int kThreads = TDM_THREADS;
constexpr int kUnroll = TDM_UNROLL;             // 16-byte vectors per lane per tile and stream
#ifndef TDM_K1_UNROLL
#define TDM_K1_UNROLL 2
#endif
// K1 and the copy kernel cut their pairs into tiles of their own. Both must use the same tile: a ring
// whose reduce steps and gather steps differ in tile size or workgroup size is up to 5 % slower at
// 64 MiB per rank than with either size for both (what one kernel leaves in the caches, the other finds).
constexpr int kK1Unroll = TDM_K1_UNROLL;
constexpr int kK1TileVecs = kThreads * kK1Unroll;
#ifndef TDM_COPY_THREADS
#define TDM_COPY_THREADS TDM_THREADS
#endif
#ifndef TDM_COPY_UNROLL
#define TDM_COPY_UNROLL TDM_K1_UNROLL
#endif
constexpr int kCopyThreads = TDM_COPY_THREADS;
constexpr int kCopyUnroll = TDM_COPY_UNROLL;
constexpr int kCopyTileVecs = kCopyThreads * kCopyUnroll;
#ifndef TDM_WARM_VECS
#define TDM_WARM_VECS 2
#endif
// Vectors per lane and stream of the one-launch ring forms while the ranks' tensors stay in the caches. Measured, reduce-scatter +
// all-gather at world 4, 2 against 1: 16 MiB per rank 30.1 / 32.3 us, 32 MiB 56.8 / 58.1, 64 MiB 107.4 / 107.3 (world 3 alike).
constexpr int kWarmVecs = TDM_WARM_VECS;
constexpr int kTileVecs = kThreads * kUnroll;   // 256 vectors = 4 KiB of every stream
// Measured on MI355X: one tile per workgroup beats a persistent grid-stride
// loop by 5-8% (the hardware dispatcher balances 8 XCDs better than a fixed stride),
// so the grid covers the tiles one to one up to 4 Mi workgroups (16 GiB per launch and stream)
// and strides only beyond that. (With 256 Ki workgroups at most, four ranks of 4 GiB each lost
// 10 % on the ring's steps, 19 % on its one-launch forms and 23 % on the single-launch all-reduce.)
// 4 Mi workgroups of up to 256 lanes stay below HIP's limit of 2^32 lanes per launch.
constexpr int kDefaultBlocksPerCu = 16384;

int g_blocks_per_cu = kDefaultBlocksPerCu;
// From which footprint (all ranks' tensors together) a single-launch all-reduce takes the kernel built for data that
// is not found in the caches again (non-temporal stores, half tiles, an occupancy cap). Measured, cached against
// uncached kernel, footprints of 256 / 320 / 384 / 448 MiB: world 4 77 / 107 / 149 / 174 against 87 / 109 / 130 / 148 us
// (worlds 3 and 8 alike); world 2 82 / 102 / 138 / 165 against 92 / 120 / 147 / 163.
constexpr int64_t cold_footprint(int world) { return int64_t(world == 2 ? 448 : 352) << 20; }

// Which tile a workgroup takes. The dispatcher hands consecutive workgroups to the 8 XCDs in
// turn, so with tile = workgroup index every XCD touches every eighth 4 KiB of every stream.
// With shift > 0 the tiles are taken in groups of 8 << shift and each XCD gets (1 << shift)
// consecutive tiles of a group: the same tiles are in flight at any time, but each XCD's L2
// and its path to memory see runs of (4 KiB << shift) per stream. Measured on MI355X with
// streams of 336 MiB: nothing for one or two streams, +8-9 % for launches with four or more
// write streams. The tiles past the last whole group keep their own index; shift 0 is the identity.
__host__ __device__ __forceinline__ int64_t tile_of(int64_t idx, int64_t total, int shift) {
  const int64_t span = int64_t(8) << shift;
  if (idx >= (total & ~(span - 1))) return idx;
  const int64_t in = idx & (span - 1);
  return (idx - in) + ((in & 7) << shift) + (in >> 3);
}

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
// Narrow integers add in 32 bits and keep the low bits: the wrap-around sum of the element's own width,
// whatever the order of the terms. uint8 shares int8's kernels: the bits of the two sums are the same.
template <> struct Elem<int16_t> {
  using acc = int32_t;
  static constexpr bool floating = false;
  static __device__ __forceinline__ acc widen(int16_t x) { return x; }
  static __device__ __forceinline__ int16_t narrow(acc x) { return static_cast<int16_t>(static_cast<uint16_t>(x)); }
};
template <> struct Elem<int8_t> {
  using acc = int32_t;
  static constexpr bool floating = false;
  static __device__ __forceinline__ acc widen(int8_t x) { return x; }
  static __device__ __forceinline__ int8_t narrow(acc x) { return static_cast<int8_t>(static_cast<uint8_t>(x)); }
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
    if (x != x) out.bits = 0x7e00u;  // a NaN narrows to the canonical quiet NaN: sign and payload are not kept
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
      out.bits = 0x7fc0u;  // a NaN narrows to the canonical quiet NaN: sign and payload are not kept
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

// The lane-wise wrap-around sum of two vectors of the INTEGER type T, on the packed words: integers are never
// divided, so their kernels need no per-element code (unpacked, sixteen 8-bit lanes cost a kernel 100-250 registers).
// 8- and 16-bit lanes add inside their 32-bit word without carrying into the neighbour: the low bits of every lane are
// added with the top bit masked off, and the top bits are the exclusive or of the operands' and the carry's.
template <typename T>
__device__ __forceinline__ vec16 add_vec(const vec16& a, const vec16& b) {
  static_assert(!Elem<T>::floating, "integer element types only");
  vec16 r;
  if constexpr (sizeof(T) == 8) {
    unsigned long long x[2], y[2];
    __builtin_memcpy(x, &a, 16);
    __builtin_memcpy(y, &b, 16);
    x[0] += y[0];
    x[1] += y[1];
    __builtin_memcpy(&r, x, 16);
  } else if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = a[i] + b[i];
  } else {
    constexpr uint32_t top = sizeof(T) == 2 ? 0x80008000u : 0x80808080u;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = ((a[i] & ~top) + (b[i] & ~top)) ^ ((a[i] ^ b[i]) & top);
  }
  return r;
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
  int flags;  // per launch: bit0 scale_dst, bit1 scale_src, bit2 writeback_src; bits 8..: the shift of tile_of()
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
  const int shift = tab.flags >> 8;
  for (int64_t at = blockIdx.x; at < total; at += gridDim.x) {
    const int64_t tile = tile_of(at, total, shift);
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
          if constexpr (!Elem<T>::floating) {  // (never scaled: the source stays as it is)
            store16<kMask>(dvp + (v0 + k * kThreads) * 16, add_vec<T>(a[k], b[k]));
          } else {
            Lanes<T> x = unpack<T>(a[k]), y = unpack<T>(b[k]);
#pragma unroll
            for (int l = 0; l < L; ++l) reduce_elem<T, kDiv>(x.v[l], y.v[l], scale_dst, scale_src, dv);
            store16<kMask>(dvp + (v0 + k * kThreads) * 16, pack<T>(x));
            if (writeback) store16<kMask>(svp + (v0 + k * kThreads) * 16, pack<T>(y));
          }
        }
      } else {
#pragma unroll
        for (int k = 0; k < kK1Unroll; ++k) {
          const int64_t v = v0 + k * kThreads;
          if (v < nv) {
            if constexpr (!Elem<T>::floating) {
              store16<kMask>(dvp + v * 16, add_vec<T>(load_rmw<kMask>(dvp + v * 16), load_stream<kMask>(svp + v * 16)));
            } else {
              Lanes<T> x = unpack<T>(load_rmw<kMask>(dvp + v * 16)), y = unpack<T>(load_stream<kMask>(svp + v * 16));
#pragma unroll
              for (int l = 0; l < L; ++l) reduce_elem<T, kDiv>(x.v[l], y.v[l], scale_dst, scale_src, dv);
              store16<kMask>(dvp + v * 16, pack<T>(x));
              if (writeback) store16<kMask>(svp + v * 16, pack<T>(y));
            }
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
__global__ __launch_bounds__(kCopyThreads) void k1_copy_kernel(PairTable tab, Divisor<T> dv) {
  constexpr int L = lanes<T>();
  constexpr int64_t kTileElems = static_cast<int64_t>(kCopyTileVecs) * L;
  const int64_t total = tab.tile_end[tab.npairs - 1];
  const int shift = tab.flags >> 8;
  for (int64_t at = blockIdx.x; at < total; at += gridDim.x) {
    const int64_t tile = tile_of(at, total, shift);
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
        for (int k = 0; k < kCopyUnroll; ++k) b[k] = load_stream<kMask>(svp + (v0 + k * kCopyThreads) * 16);
#pragma unroll
        for (int k = 0; k < kCopyUnroll; ++k) {
          if constexpr (kDiv != 0) {
            Lanes<T> y = unpack<T>(b[k]);
#pragma unroll
            for (int l = 0; l < L; ++l) y.v[l] = copy_elem<T, kDiv>(y.v[l], dv);
            b[k] = pack<T>(y);
          }
          store16<kMask>(dvp + (v0 + k * kCopyThreads) * 16, b[k]);
        }
      } else {
#pragma unroll
        for (int k = 0; k < kCopyUnroll; ++k) {
          const int64_t v = v0 + k * kCopyThreads;
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
        const int64_t i = e0 + static_cast<int64_t>(k) * kCopyThreads;
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
  // 0: the pointers disagree within 16 bytes, element by element. Otherwise 1 + h: every pointer is
  // 16-byte aligned and h (< 16 / element size) further elements lie directly BEFORE the pointers:
  // the head of a segment whose pointers all started at the same distance from a 16-byte boundary.
  int32_t vec_ok;
};

// One tile of one segment: W loads per element, the fold in ring order, W stores.
// kAcc: the result is added into each destination (dst = dst + sum) instead of replacing it.
// kRounds: the part of the segment one call covers, in rounds of one vector per lane
// (kT vectors, kT = the workgroup's lanes); `t` counts such parts from the segment's start.
template <typename T, int kWorld, int kDiv, bool kAcc, int kMask, int kRounds = kUnroll, int kT = kThreads>
__device__ __forceinline__ void fold_tile(const FoldSegDev& sg, int64_t t, const Divisor<T>& dv) {
  using A = typename Elem<T>::acc;
  constexpr int L = lanes<T>();
#ifndef TDM_K2_UNROLL_W2
#define TDM_K2_UNROLL_W2 2
#endif
#ifndef TDM_K2_UNROLL
#define TDM_K2_UNROLL 2
#endif
  // vectors per lane in flight, per rank
  constexpr int kWant = kWorld <= 2 ? TDM_K2_UNROLL_W2 : kWorld <= 4 ? TDM_K2_UNROLL : 2;
  constexpr int kU = kWant < kRounds ? kWant : kRounds;
  constexpr int kPartVecs = kT * kRounds;
  constexpr int64_t kTileElems = static_cast<int64_t>(kPartVecs) * L;
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
    for (int u0 = 0; u0 < kRounds; u0 += kU) {
      const int64_t vbase = t * kPartVecs + threadIdx.x + static_cast<int64_t>(u0) * kT;
      vec16 in[kWorld][kU];
#pragma unroll
      for (int k = 0; k < kWorld; ++k)
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int64_t v = vbase + u * kT;
          if (v < nv) in[k][u] = load_stream<kMask>(sp[k] + v * 16);
        }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t v = vbase + u * kT;
        if (v < nv) {
          vec16 packed;
          [[maybe_unused]] Lanes<T> out;
          if constexpr (!Elem<T>::floating) {
            packed = in[0][u];
#pragma unroll
            for (int k = 1; k < kWorld; ++k) packed = add_vec<T>(in[k][u], packed);
          } else {
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
            packed = pack<T>(out);
          }
#pragma unroll
          for (int k = 0; k < kWorld; ++k)
            if (dp[k]) {
              if constexpr (kAcc && !Elem<T>::floating) {
                store16<kMask>(dp[k] + v * 16, add_vec<T>(load_rmw<kMask>(dp[k] + v * 16), packed));
              } else if constexpr (kAcc) {
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
    const int head = sg.vec_ok - 1;
    // the few elements after the last whole vector (lanes 0..) and before the first (lanes 32..)
    if (t == 0 && (threadIdx.x < n - nv * L || (threadIdx.x >= 32 && static_cast<int>(threadIdx.x) - 32 < head))) {
      const int64_t i = threadIdx.x < 32 ? nv * L + threadIdx.x : -1 - (static_cast<int64_t>(threadIdx.x) - 32);
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
    for (int k2 = 0; k2 < kRounds * L; ++k2) {
      const int64_t i = e0 + static_cast<int64_t>(k2) * kT;
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

// Table in device memory, one record per tile (many segments: DDP's buckets). A record
// describes 4 KiB of every stream and is taken in two parts of 2 KiB, by one workgroup each:
// launches that stream from HBM through many streams at once do better with the smaller part
// (two-rank bucket fold 3-7 %, ZeRO-2's fold into the shards 2 %, against a build with one
// workgroup per 4 KiB; one workgroup that takes the record's two parts one after the other, so that every
// record is fetched once, is slower still: two-rank bucket fold 0.228 against 0.2125 ms, the fold into
// the shards 0.372 against 0.357).
#ifndef TDM_K2_SPLIT
#define TDM_K2_SPLIT 1  // 0 (measurement builds): one workgroup per record
#endif
template <int kWorld>
struct FoldShape {
  static constexpr bool kSmall = TDM_K2_SPLIT && kThreads >= 128 && kTileVecs % 128 == 0;
  static constexpr int kT = kSmall ? 128 : kThreads;
  static constexpr int kRounds = kSmall ? 1 : kUnroll;
  static constexpr int kParts = kTileVecs / (kT * kRounds);
};

template <typename T, int kWorld, int kDiv, bool kAcc>
__global__ __launch_bounds__(kThreads) void k2_fold_kernel(const FoldSegDev* __restrict__ tiles, int64_t total,
                                                           Divisor<T> dv, int shift) {
  using S = FoldShape<kWorld>;
  for (int64_t at = blockIdx.x; at < total * S::kParts; at += gridDim.x) {
    const int64_t part = tile_of(at, total * S::kParts, shift);
    fold_tile<T, kWorld, kDiv, kAcc, TDM_NT_MASK_K2, S::kRounds, S::kT>(tiles[part / S::kParts], part % S::kParts, dv);
  }
}

// Writes K2's table on the device: one thread per tile of up to kFillSegs segments that
// arrive in the launch itself. For callers that may not allocate or copy from the host
// (tdm_k2_bucket_fold_static): the records land in a fixed array inside the library.
constexpr int kFillSegs = 16;
struct FillBatch {
  int nseg;
  int world;
  int es;               // element size in bytes
  int64_t tile_elems;   // elements per record
  int64_t first[kFillSegs + 1];  // first[k]: index of segment k's first record; first[nseg]: one past the batch's last
  int32_t vec_ok[kFillSegs];
  tdm_fold_seg seg[kFillSegs];
};

__global__ __launch_bounds__(256) __attribute__((unused)) void k2_table_fill_kernel(FillBatch b, FoldSegDev* __restrict__ out) {
  const int64_t tile = b.first[0] + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tile >= b.first[b.nseg]) return;
  int k = 0;
  while (tile >= b.first[k + 1]) ++k;
  const tdm_fold_seg& s = b.seg[k];
  const int64_t at = (tile - b.first[k]) * b.tile_elems;
  FoldSegDev rec;
#pragma unroll
  for (int r = 0; r < TDM_MAX_WORLD; ++r) {
    rec.src[r] = r < b.world && s.src[r] ? static_cast<const char*>(s.src[r]) + at * b.es : nullptr;
    rec.dst[r] = r < b.world && s.dst[r] ? static_cast<char*>(s.dst[r]) + at * b.es : nullptr;
  }
  rec.count = min(b.tile_elems, s.count - at);
  rec.chunk = s.chunk;
  rec.vec_ok = b.vec_ok[k] == 0 ? 0 : (tile == b.first[k] ? b.vec_ok[k] : 1);  // the head belongs to the first record
  out[tile] = rec;
}

// Parts per tile of a launch with its table by value whose footprint is beyond the caches.
template <int kWorld>
constexpr int fold_small_parts() {
  return FoldShape<kWorld>::kSmall && FoldShape<kWorld>::kT == kThreads ? FoldShape<kWorld>::kParts : 1;
}

// Table by value (one segment per ring chunk: a whole all-reduce in one launch).
struct FoldSmall {
  int nseg;
  int shift;  // of tile_of()
  int64_t tile_end[TDM_MAX_WORLD];
  FoldSegDev seg[TDM_MAX_WORLD];
};

// kCold: the launch's footprint is far beyond the 256 MB Infinity Cache, so nothing it
// writes will be read from there: the cache policy of the once-per-step bucket fold.
// Such a launch also takes its tiles in two parts of 2 KiB, one workgroup each (256 MiB per rank at
// world 4: 3 % faster; within the cache, 64 MiB per rank, the whole tile per workgroup is 6 % faster).
template <typename T, int kWorld, int kDiv, bool kCold>
__global__ __launch_bounds__(kThreads) void k2_fold_small_kernel(FoldSmall tab, Divisor<T> dv) {
  constexpr int kParts = kCold ? fold_small_parts<kWorld>() : 1;
  const int64_t total = tab.tile_end[tab.nseg - 1] * kParts;
  for (int64_t at = blockIdx.x; at < total; at += gridDim.x) {
    const int64_t part = tile_of(at, total, tab.shift);
    const int64_t tile = part / kParts;
    int lo = 0;
    while (tile >= tab.tile_end[lo]) ++lo;
    const int64_t t = (tile - (lo ? tab.tile_end[lo - 1] : 0)) * kParts + part % kParts;
    fold_tile<T, kWorld, kDiv, false, kCold ? TDM_NT_MASK_K2 : TDM_NT_MASK, kUnroll / kParts>(tab.seg[lo], t, dv);
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
  int shift;  // of tile_of()
  int head;   // vector path: elements (at most 31: up to a cache line) that lie before the pointers, peeled off an unaligned shard
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
#ifndef TDM_K3_THREADS
#define TDM_K3_THREADS TDM_THREADS
#endif
constexpr int kAdamwThreads = TDM_K3_THREADS;  // lanes per workgroup of K3

template <int kOrder, bool kVec, bool kCopies>
__global__ __launch_bounds__(kAdamwThreads) void k3_adamw_kernel(AdamwArgs a) {
  const bool small_w = __builtin_fabsf(a.s.w1) < 0.5f;
  if constexpr (kVec) {
    constexpr int kU = kAdamwUnroll;
    const int64_t nv = a.n / 4;
    const int64_t tiles = (nv + kAdamwThreads * kU - 1) / (kAdamwThreads * kU);
    for (int64_t at = blockIdx.x; at < tiles; at += gridDim.x) {
      const int64_t v0 = tile_of(at, tiles, a.shift) * (kAdamwThreads * kU) + threadIdx.x;
      vec16 rp[kU], rg[kU], rm[kU], rv[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t i = v0 + u * kAdamwThreads;
        if (i < nv) {
          rp[u] = load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.p) + i * 16);
          rg[u] = load_stream<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.g) + i * 16);
          rm[u] = load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.m) + i * 16);
          rv[u] = load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.v) + i * 16);
        }
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int64_t i = v0 + u * kAdamwThreads;
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
    // the last few elements (lanes 0..3), and the head before the first vector (lanes 32..62)
    if (blockIdx.x == 0 && (threadIdx.x < a.n - nv * 4 || (threadIdx.x >= 32 && static_cast<int>(threadIdx.x) - 32 < a.head))) {
      const int64_t i = threadIdx.x < 32 ? nv * 4 + threadIdx.x : -1 - (static_cast<int64_t>(threadIdx.x) - 32);
      adamw_elem<kOrder>(a.p[i], a.g[i], a.m[i], a.v[i], a.s, small_w);
      if constexpr (kCopies)
        for (int c = 0; c < a.ncopies; ++c) a.copy[c][i] = a.p[i];
    }
  } else {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kAdamwThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kAdamwThreads + threadIdx.x; i < a.n; i += stride) {
      adamw_elem<kOrder>(a.p[i], a.g[i], a.m[i], a.v[i], a.s, small_w);
      if constexpr (kCopies)
        for (int c = 0; c < a.ncopies; ++c) a.copy[c][i] = a.p[i];
    }
  }
}

// ---------------------------------------------------------------- K3 on other element types
// The reference's update is seven torch operations that take any floating dtype (tandem/optim.py:28-37).
// float64: the same arithmetic on doubles, the step's scalars unrounded. bfloat16 and float16: every operation
// reads the 16-bit type, computes in fp32 and writes the 16-bit type, so the value is rounded to nearest even
// after EACH operation; add_(eps) adds eps rounded to the type (ATen wraps that scalar in the tensor's dtype),
// the other scalars act as fp32. Host order only: these follow torch's CPU kernels, which is what the reference's engine runs.
template <typename S>
struct AdamwHyper {
  int use_decay;
  S decay, w1, beta2, one_m_b2, bc2_sqrt, eps, neg_step;
  // bfloat16 only (see AdamwMath16::root_over): 1 / bc2_sqrt rounded to fp32, and the window around a rounding tie inside
  // which the quotient is recomputed by a true division: low 16 bits + tie_bias (mod 2^16) <= tie_span.
  // tie_span = 0xffff sends every element the exact way.
  S inv_bc2;
  uint32_t tie_bias, tie_span;
};

template <typename T> struct AdamwMath;

template <> struct AdamwMath<double> {
  using S = double;
  static constexpr int kGroup = 1;
  template <int N>
  static __device__ __forceinline__ void step_n(double* p, const double* g, double* m, double* v, const AdamwHyper<double>& s, bool small_w) {
    static_assert(N == 1, "doubles are stepped one at a time");
    step(*p, *g, *m, *v, s, small_w);
  }
  static __device__ __forceinline__ void step(double& p, double g, double& m, double& v, const AdamwHyper<double>& s, bool small_w) {
    if (s.use_decay) p = p * s.decay;
    const double diff = g - m;
    m = small_w ? __builtin_fma(s.w1, diff, m) : __builtin_fma(s.w1 - 1.0, diff, g);
    const double vs = v * s.beta2;
    v = __builtin_fma(s.one_m_b2 * g, g, vs);
    const double d = __builtin_sqrt(v) / s.bc2_sqrt + s.eps;
    p = p + (s.neg_step * m) / d;
  }
};

// The two 16-bit types share the step; they differ in how a float is rounded to the type and back (a conversion
// instruction either way: v_cvt_pk_bf16_f32, v_cvt_f16_f32) and in the canonical NaN that is stored.
template <typename T> struct Round16;
template <> struct Round16<bf16_t> {
  static __device__ __forceinline__ float rb(float x) {
    const __bf16 h = static_cast<__bf16>(x);
    return static_cast<float>(h);
  }
  // two floats through one conversion instruction (v_cvt_pk_bf16_f32 takes a pair)
  static __device__ __forceinline__ void rb2(float& x, float& y) {
    typedef float float_pair __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16_pair __attribute__((ext_vector_type(2)));
    const float_pair in = {x, y};
    const bf16_pair h = __builtin_convertvector(in, bf16_pair);
    uint32_t u;
    __builtin_memcpy(&u, &h, 4);
    x = __uint_as_float(u << 16);
    y = __uint_as_float(u & 0xffff0000u);
  }
  // the bits of a float that rb() has already rounded: its upper half
  static __device__ __forceinline__ uint16_t bits(float x) { return static_cast<uint16_t>(__float_as_uint(x) >> 16); }
  static constexpr uint16_t kNan = 0x7fc0u;
};
template <> struct Round16<f16_t> {
  // The float must exist as a float before it is narrowed: left to itself the compiler folds the multiplication or
  // fused multiply-add that produced it into a mixed-precision instruction that rounds the exact result to f16 ONCE,
  // where torch rounds to fp32 and then to f16. With operands that are not all f16 values (beta2, the step's other
  // constants) the two differ on ties: 10 ulps x f32(0.95) is 9.49999988 exactly, 9.5 as a float, and rounds to 9 the
  // one way and to 10 the other. The empty asm is the barrier; it emits nothing.
  static __device__ __forceinline__ float rb(float x) {
    asm volatile("" : "+v"(x));
    const _Float16 h = static_cast<_Float16>(x);
    return static_cast<float>(h);
  }
  static __device__ __forceinline__ uint16_t bits(float x) {  // exact: x is representable
    const _Float16 h = static_cast<_Float16>(x);
    uint16_t b;
    __builtin_memcpy(&b, &h, 2);
    return b;
  }
  static constexpr uint16_t kNan = 0x7e00u;
};

// x is rounded to the 16-bit type and back by the conversion instruction instead of the integer operations of
// Elem<T>::narrow: this kernel rounds eight times per element, and on bfloat16 its arithmetic showed in the time
// until the root and the division by bc2_sqrt were shortened (root_over below; TDM_BF16_SHORT_ROOT=0 builds the
// version that does them to the letter, for comparison). A NaN stays a NaN through the roundings; what is stored is
// the canonical one, as narrow() makes it.
#ifndef TDM_BF16_SHORT_ROOT
#define TDM_BF16_SHORT_ROOT 1
#endif
template <typename T>
struct AdamwMath16 {
  using S = float;
  using R = Round16<T>;
  static constexpr bool kBf16 = std::is_same<T, bf16_t>::value;
  // Elements are stepped in groups: bfloat16 rounds two floats with one conversion instruction.
  static constexpr int kGroup = kBf16 ? 2 : 1;

  template <int N>
  static __device__ __forceinline__ void round_all(float (&x)[N]) {
    if constexpr (N == 2 && kBf16) {
      R::rb2(x[0], x[1]);
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) x[i] = R::rb(x[i]);
    }
  }

  // d = rb(rb(sqrt(v)) / bc2_sqrt), the two operations that cost the most arithmetic when done to the letter (a
  // correctly rounded fp32 square root and a true division are a dozen instructions each).
  //
  // bfloat16 takes a shorter way to the same bits. (1) The hardware's square root (within 1 ulp of fp32) instead of the
  // correctly rounded one: v has 8 significant bits, so sqrt(v) cannot come close to a value half way between two
  // bfloat16 neighbours (such a T has an odd 9-bit significand, T*T an odd significand of 17 or 18 bits, v's has at
  // most 8, so |v - T*T| is at least one unit of T*T's last place and sqrt(v) stays more than 30 fp32 ulps away from
  // T): every float within a few ulps of sqrt(v) rounds to the same bfloat16. The instruction does not take denormal
  // floats: a nonzero v below 2^-96 goes the exact way. (2) A multiplication by 1 / bc2_sqrt instead of the division:
  // the product lies within 2.5 fp32 ulps of the correctly rounded quotient, so both round to the same bfloat16 unless
  // a tie (low 16 bits 0x8000) lies within a few ulps; then the pair goes the exact way (about 3 % of a wave's pairs).
  // The host sets the window, and sets it to everything when bc2_sqrt is outside [2^-30, 2^30].
  template <int N>
  static __device__ __forceinline__ void root_over(const float (&v)[N], float (&d)[N], const AdamwHyper<float>& s) {
    if constexpr (kBf16 && TDM_BF16_SHORT_ROOT) {
      float q[N];
      bool exact_way = false;
#pragma unroll
      for (int i = 0; i < N; ++i) d[i] = __builtin_amdgcn_sqrtf(v[i]);
      round_all(d);
#pragma unroll
      for (int i = 0; i < N; ++i) {
        q[i] = d[i] * s.inv_bc2;
        exact_way |= ((__float_as_uint(q[i]) + s.tie_bias) & 0xffffu) <= s.tie_span;
        exact_way |= !(v[i] >= 0x1p-96f) && v[i] != 0.0f;  // denormal floats, negative numbers, NaN
      }
      if (__builtin_expect(exact_way, 0)) {
#pragma unroll
        for (int i = 0; i < N; ++i) q[i] = R::rb(__builtin_sqrtf(v[i])) / s.bc2_sqrt;
      }
#pragma unroll
      for (int i = 0; i < N; ++i) d[i] = q[i];
      round_all(d);
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) d[i] = R::rb(__builtin_sqrtf(v[i]));
#pragma unroll
      for (int i = 0; i < N; ++i) d[i] = R::rb(d[i] / s.bc2_sqrt);
    }
  }

  template <int N>
  static __device__ __forceinline__ void step_n(T* p, const T* g, T* m, T* v, const AdamwHyper<float>& s, bool small_w) {
    float P[N], G[N], M[N], V[N], D[N];
#pragma unroll
    for (int i = 0; i < N; ++i) P[i] = Elem<T>::widen(p[i]), G[i] = Elem<T>::widen(g[i]), M[i] = Elem<T>::widen(m[i]), V[i] = Elem<T>::widen(v[i]);
    if (s.use_decay) {
#pragma unroll
      for (int i = 0; i < N; ++i) P[i] = P[i] * s.decay;
      round_all(P);
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const float diff = G[i] - M[i];  // inside lerp_: not rounded
      M[i] = small_w ? __builtin_fmaf(s.w1, diff, M[i]) : __builtin_fmaf(s.w1 - 1.0f, diff, G[i]);
    }
    round_all(M);
#pragma unroll
    for (int i = 0; i < N; ++i) V[i] = V[i] * s.beta2;
    round_all(V);
#pragma unroll
    for (int i = 0; i < N; ++i) V[i] = __builtin_fmaf(s.one_m_b2 * G[i], G[i], V[i]);
    round_all(V);
    root_over(V, D, s);
#pragma unroll
    for (int i = 0; i < N; ++i) D[i] = D[i] + s.eps;  // s.eps arrives rounded to the 16-bit type
    round_all(D);
#pragma unroll
    for (int i = 0; i < N; ++i) P[i] = P[i] + (s.neg_step * M[i]) / D[i];
    round_all(P);
#pragma unroll
    for (int i = 0; i < N; ++i) p[i] = exact(P[i]), m[i] = exact(M[i]), v[i] = exact(V[i]);
  }
  static __device__ __forceinline__ void step(T& p, T g, T& m, T& v, const AdamwHyper<float>& s, bool small_w) {
    step_n<1>(&p, &g, &m, &v, s, small_w);
  }
  static __device__ __forceinline__ T exact(float x) {
    T out;
    out.bits = x != x ? R::kNan : R::bits(x);
    return out;
  }
};
template <> struct AdamwMath<bf16_t> : AdamwMath16<bf16_t> {};
template <> struct AdamwMath<f16_t> : AdamwMath16<f16_t> {};

template <typename T>
struct AdamwArgsT {
  T* p;
  const T* g;
  T* m;
  T* v;
  int64_t n;
  AdamwHyper<typename AdamwMath<T>::S> s;
  int ncopies;
  int shift;  // of tile_of()
  int head;   // vector path: elements before the pointers (up to a cache line), peeled off an unaligned shard
  T* copy[TDM_MAX_WORLD - 1];
};

template <typename T, bool kVec, bool kCopies>
__global__ __launch_bounds__(kAdamwThreads) void k3_adamw_typed_kernel(AdamwArgsT<T> a) {
  using S = typename AdamwMath<T>::S;
  const bool small_w = (a.s.w1 < S(0) ? -a.s.w1 : a.s.w1) < S(0.5);
  constexpr int kL = lanes<T>(), kG = AdamwMath<T>::kGroup;
  static_assert(kL % kG == 0, "a vector holds whole groups");
  static_assert(kL <= 32 && 32 + 128 / static_cast<int>(sizeof(T)) <= kAdamwThreads, "lanes 0.. take the tail, lanes 32.. a head of up to a cache line");
  if constexpr (kVec) {
    const int64_t nv = a.n / kL;
    const int64_t tiles = (nv + kAdamwThreads - 1) / kAdamwThreads;
    for (int64_t at = blockIdx.x; at < tiles; at += gridDim.x) {
      const int64_t i = tile_of(at, tiles, a.shift) * kAdamwThreads + threadIdx.x;
      if (i < nv) {
        Lanes<T> P = unpack<T>(load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.p) + i * 16));
        const Lanes<T> G = unpack<T>(load_stream<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.g) + i * 16));
        Lanes<T> M = unpack<T>(load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.m) + i * 16));
        Lanes<T> V = unpack<T>(load_rmw<TDM_NT_MASK_K3>(reinterpret_cast<const char*>(a.v) + i * 16));
#pragma unroll
        for (int l = 0; l < kL; l += kG) AdamwMath<T>::template step_n<kG>(&P.v[l], &G.v[l], &M.v[l], &V.v[l], a.s, small_w);
        const vec16 packed = pack<T>(P);
        store16<TDM_NT_MASK_K3>(reinterpret_cast<char*>(a.p) + i * 16, packed);
        if constexpr (kCopies)
          for (int c = 0; c < a.ncopies; ++c) store16<TDM_NT_MASK_K3C>(reinterpret_cast<char*>(a.copy[c]) + i * 16, packed);
        store16<TDM_NT_MASK_K3>(reinterpret_cast<char*>(a.m) + i * 16, pack<T>(M));
        store16<TDM_NT_MASK_K3>(reinterpret_cast<char*>(a.v) + i * 16, pack<T>(V));
      }
    }
    // the last few elements (lanes 0..7), and the head before the first vector (lanes 32..): up to a cache line
    if (blockIdx.x == 0 && (threadIdx.x < a.n - nv * kL || (threadIdx.x >= 32 && static_cast<int>(threadIdx.x) - 32 < a.head))) {
      const int64_t i = threadIdx.x < 32 ? nv * kL + threadIdx.x : -1 - (static_cast<int64_t>(threadIdx.x) - 32);
      AdamwMath<T>::step(a.p[i], a.g[i], a.m[i], a.v[i], a.s, small_w);
      if constexpr (kCopies)
        for (int c = 0; c < a.ncopies; ++c) a.copy[c][i] = a.p[i];
    }
  } else {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kAdamwThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kAdamwThreads + threadIdx.x; i < a.n; i += stride) {
      AdamwMath<T>::step(a.p[i], a.g[i], a.m[i], a.v[i], a.s, small_w);
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
  int32_t vec_ok;                // as FoldSegDev's
};

#ifndef TDM_K23_UNROLL
#define TDM_K23_UNROLL 2
#endif
// A record of the step's table (4 KiB of every stream) is taken in two parts of 2 KiB, by one
// workgroup each: 3 % faster at the 85.8M-parameter step than one workgroup per record.
#ifndef TDM_K23_PARTS
#define TDM_K23_PARTS 2
#endif
constexpr int kStepParts = (TDM_K23_PARTS <= kUnroll && kUnroll % TDM_K23_PARTS == 0) ? TDM_K23_PARTS : 1;
#ifndef TDM_NT_MASK_K23
#define TDM_NT_MASK_K23 TDM_NT_MASK_K3
#endif

// One part (at most kRounds vectors per lane and stream) of the step.
template <int kWorld, int kDiv, int kOrder, int kRounds>
__device__ __forceinline__ void step_tile(const StepSegDev& sg, int64_t at, int64_t n, int head, const Divisor<float>& dv,
                                          const tdm_adamw_scalars& s, bool small_w) {
  constexpr int kWant = kWorld <= 4 ? TDM_K23_UNROLL : 1;
  constexpr int kU = kWant < kRounds ? kWant : kRounds;  // vectors per lane in flight, per stream
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
      for (int u0 = 0; u0 < kRounds; u0 += kU) {
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
      // the tile's last few elements (lanes 0..), and the segment's head before its first vector (lanes 32..)
      if (threadIdx.x < n - nv * 4 || (threadIdx.x >= 32 && static_cast<int>(threadIdx.x) - 32 < head)) {
        const int64_t i = threadIdx.x < 32 ? nv * 4 + threadIdx.x : -1 - (static_cast<int64_t>(threadIdx.x) - 32);
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
                                                                  Divisor<float> dv, tdm_adamw_scalars s, int shift) {
  const bool small_w = __builtin_fabsf(s.w1) < 0.5f;
  constexpr int64_t kPartElems = static_cast<int64_t>(kTileVecs / kStepParts) * 4;
  for (int64_t at = blockIdx.x; at < total * kStepParts; at += gridDim.x) {
    const int64_t part = tile_of(at, total * kStepParts, shift);
    const StepSegDev& rec = tiles[part / kStepParts];
    const int64_t first = (part % kStepParts) * kPartElems;  // the part's first element within the record
    const int64_t n = min(kPartElems, rec.count - first);
    const int head = first == 0 ? rec.vec_ok - 1 : 0;
    if (n > 0) step_tile<kWorld, kDiv, kOrder, kUnroll / kStepParts>(rec, first * 4, n, head, dv, s, small_w);
  }
}

// The same for ONE segment, described in the kernel's arguments: no table to keep in
// device memory. A rank that is a process of its own steps exactly one segment, its
// shard, out of its peers' gradient buffers and into their parameter buffers.
template <int kWorld, int kDiv, int kOrder>
__global__ __launch_bounds__(kThreads) void k23_zero2_step_one_kernel(StepSegDev whole, int64_t total, Divisor<float> dv,
                                                                      tdm_adamw_scalars s, int shift) {
  const bool small_w = __builtin_fabsf(s.w1) < 0.5f;
  constexpr int64_t kPartElems = static_cast<int64_t>(kTileVecs / kStepParts) * 4;
  for (int64_t at = blockIdx.x; at < total * kStepParts; at += gridDim.x) {
    const int64_t part = tile_of(at, total * kStepParts, shift);
    const int64_t n = min(kPartElems, whole.count - part * kPartElems);
    const int head = part == 0 ? whole.vec_ok - 1 : 0;
    if (n > 0) step_tile<kWorld, kDiv, kOrder, kUnroll / kStepParts>(whole, part * kPartElems * 4, n, head, dv, s, small_w);
  }
}

// ---------------------------------------------------------------- K2 + K3 on float64 and bfloat16
// The one-launch step on the other shard types of K3: the gradients folded in the ring's order with the
// element type's own rounding (as K2 folds them: every addition rounded to the type), 0 + mine as
// grad_shard.add_(mine) leaves it, the typed AdamW step of AdamwMath<T>, the new parameter stored into every
// rank's buffer. Host order. One vector per lane and stream in flight (a vector is 2 doubles or 8 bf16).
template <typename T, int kWorld, int kDiv, int kRounds>
__device__ __forceinline__ void step_tile_typed(const StepSegDev& sg, int64_t at, int64_t n, int head, const Divisor<T>& dv,
                                                const AdamwHyper<typename AdamwMath<T>::S>& s, bool small_w) {
  using A = typename Elem<T>::acc;
  constexpr int L = lanes<T>(), kG = AdamwMath<T>::kGroup;
  constexpr int kM = TDM_NT_MASK_K23;
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
  auto folded = [&](const T (&gs)[kWorld]) {
    A acc = scaled<T, kDiv>(Elem<T>::widen(gs[0]), dv.divisor, dv.reciprocal);
#pragma unroll
    for (int k = 1; k < kWorld; ++k) {
      const A y = scaled<T, kDiv>(Elem<T>::widen(gs[k]), dv.divisor, dv.reciprocal);
      acc = Elem<T>::widen(Elem<T>::narrow(static_cast<A>(y + acc)));
    }
    return Elem<T>::narrow(static_cast<A>(A(0) + acc));  // grad_shard (zero) += mine
  };
  auto one = [&](const T (&gs)[kWorld], T& P, T& M, T& V) { AdamwMath<T>::step(P, folded(gs), M, V, s, small_w); };
  auto scalar_at = [&](int64_t i) {
    T gs[kWorld];
#pragma unroll
    for (int k = 0; k < kWorld; ++k) gs[k] = reinterpret_cast<const T*>(gp[k])[i];
    T P = reinterpret_cast<T*>(own)[i], M = reinterpret_cast<T*>(mm)[i], V = reinterpret_cast<T*>(vv)[i];
    one(gs, P, M, V);
#pragma unroll
    for (int q = 0; q < kWorld; ++q) reinterpret_cast<T*>(pp[q])[i] = P;
    reinterpret_cast<T*>(mm)[i] = M;
    reinterpret_cast<T*>(vv)[i] = V;
  };
  if (sg.vec_ok) {
    const int64_t nv = n / L;
#pragma unroll
    for (int u = 0; u < kRounds; ++u) {
      const int64_t v = threadIdx.x + static_cast<int64_t>(u) * kThreads;
      if (v < nv) {
        vec16 in[kWorld];
#pragma unroll
        for (int k = 0; k < kWorld; ++k) in[k] = load_stream<kM>(gp[k] + v * 16);
        Lanes<T> P = unpack<T>(load_rmw<kM>(own + v * 16)), M = unpack<T>(load_rmw<kM>(mm + v * 16)),
                 V = unpack<T>(load_rmw<kM>(vv + v * 16));
#pragma unroll
        for (int l = 0; l < L; l += kG) {
          T g[kG];
#pragma unroll
          for (int j = 0; j < kG; ++j) {
            T gs[kWorld];
#pragma unroll
            for (int k = 0; k < kWorld; ++k) gs[k] = unpack<T>(in[k]).v[l + j];
            g[j] = folded(gs);
          }
          AdamwMath<T>::template step_n<kG>(&P.v[l], g, &M.v[l], &V.v[l], s, small_w);
        }
        const vec16 packed = pack<T>(P);
#pragma unroll
        for (int q = 0; q < kWorld; ++q) store16<kM>(pp[q] + v * 16, packed);
        store16<kM>(mm + v * 16, pack<T>(M));
        store16<kM>(vv + v * 16, pack<T>(V));
      }
    }
    // the tile's last few elements (lanes 0..), and the segment's head before its first vector (lanes 32..)
    if (threadIdx.x < n - nv * L || (threadIdx.x >= 32 && static_cast<int>(threadIdx.x) - 32 < head)) {
      scalar_at(threadIdx.x < 32 ? nv * L + threadIdx.x : -1 - (static_cast<int64_t>(threadIdx.x) - 32));
    }
  } else {
    for (int64_t i = threadIdx.x; i < n; i += kThreads) scalar_at(i);
  }
}

template <typename T, int kWorld, int kDiv>
__global__ __launch_bounds__(kThreads) void k23_zero2_step_typed_kernel(const StepSegDev* __restrict__ tiles, int64_t total, Divisor<T> dv,
                                                                        AdamwHyper<typename AdamwMath<T>::S> s, int shift) {
  using S = typename AdamwMath<T>::S;
  const bool small_w = (s.w1 < S(0) ? -s.w1 : s.w1) < S(0.5);
  constexpr int64_t kPartElems = static_cast<int64_t>(kTileVecs / kStepParts) * lanes<T>();
  for (int64_t at = blockIdx.x; at < total * kStepParts; at += gridDim.x) {
    const int64_t part = tile_of(at, total * kStepParts, shift);
    const StepSegDev& rec = tiles[part / kStepParts];
    const int64_t first = (part % kStepParts) * kPartElems;  // the part's first element within the record
    const int64_t n = min(kPartElems, rec.count - first);
    const int head = first == 0 ? rec.vec_ok - 1 : 0;
    if (n > 0) step_tile_typed<T, kWorld, kDiv, kUnroll / kStepParts>(rec, first * static_cast<int64_t>(sizeof(T)), n, head, dv, s, small_w);
  }
}

// The typed step for ONE segment described in the kernel's arguments (as k23_zero2_step_one_kernel is for fp32).
template <typename T, int kWorld, int kDiv>
__global__ __launch_bounds__(kThreads) void k23_zero2_step_one_typed_kernel(StepSegDev whole, int64_t total, Divisor<T> dv,
                                                                            AdamwHyper<typename AdamwMath<T>::S> s, int shift) {
  using S = typename AdamwMath<T>::S;
  const bool small_w = (s.w1 < S(0) ? -s.w1 : s.w1) < S(0.5);
  constexpr int64_t kPartElems = static_cast<int64_t>(kTileVecs / kStepParts) * lanes<T>();
  for (int64_t at = blockIdx.x; at < total * kStepParts; at += gridDim.x) {
    const int64_t part = tile_of(at, total * kStepParts, shift);
    const int64_t n = min(kPartElems, whole.count - part * kPartElems);
    const int head = part == 0 ? whole.vec_ok - 1 : 0;
    if (n > 0) step_tile_typed<T, kWorld, kDiv, kUnroll / kStepParts>(whole, part * kPartElems * static_cast<int64_t>(sizeof(T)), n, head, dv, s, small_w);
  }
}

}  // namespace

}  // namespace tandem_hip
