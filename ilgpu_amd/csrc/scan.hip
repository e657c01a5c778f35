// Inclusive / exclusive scan, single pass with decoupled look-back.
//
// Stands in for the Scan delegates of ScanExtensions.cs:930-959.  The
// reference's single-pass kernel (ScanExtensions.cs:530-597) chains the groups
// strictly through one global word (SequentialGroupExecutor.cs:58-77) and reads
// the input twice; here each tile publishes its aggregate as soon as it has
// it, and a tile's first wave resolves the prefix of up to 64 predecessor
// tiles per step, so tiles only wait for data, never for their turn.
//
// Tile layout (kBlock = 512 threads, 8 waves, kVecs = 16 16-byte vectors per
// lane, i.e. 128 KiB per tile: time per launch falls with the number of tiles
// until about this size, then register pressure takes over):
//   wave w owns a contiguous chunk of kVecs*64 vectors; vector j of lane l is
//   chunk[j*64 + l], so every load/store instruction of a wave covers 1 KiB of
//   consecutive addresses (dwordx4 per lane).  Scan order inside a wave is
//   (j, lane, element): each lane scans its vector, the wave scans the vector
//   totals once per j, and the running totals of earlier j are folded in.
//
// Tile ids come from a global ticket, so a tile's predecessors have always
// started.  Status words are read and written with agent-scope atomics: the
// eight XCDs of the device have separate L2s.
//   4-byte T: one 64-bit word {flag, value} per tile;
//   8-byte T: two such words per tile, one per half of the value.
// Each tile's words sit in a 128-byte line of their own.
//
// Algorithmic HBM traffic: 2 * n * sizeof(T) bytes (status: 128 B/tile).
#include <atomic>
#include <mutex>

#include "kernels.hpp"

namespace ilgpu_hip {

namespace {

#ifndef ILGPU_HIP_SCAN_BLOCK
#define ILGPU_HIP_SCAN_BLOCK 512
#endif
#ifndef ILGPU_HIP_SCAN_VECS
#define ILGPU_HIP_SCAN_VECS 16
#endif
#ifndef ILGPU_HIP_SCAN_WAVES_PER_EU
#define ILGPU_HIP_SCAN_WAVES_PER_EU 4
#endif
#ifndef ILGPU_HIP_SCAN_NT_LOAD
#define ILGPU_HIP_SCAN_NT_LOAD 1
#endif
#ifndef ILGPU_HIP_SCAN_NT_STORE
#define ILGPU_HIP_SCAN_NT_STORE 1
#endif
// Measurement only: 1 takes every tile's prefix as the identity (wrong results
// beyond the first tile) to time the kernel without its look-back.
#ifndef ILGPU_HIP_SCAN_PROBE_NO_LOOKBACK
#define ILGPU_HIP_SCAN_PROBE_NO_LOOKBACK 0
#endif
// 1 issues the loads of a tile's second half only after the first half has
// been scanned (half as many bytes in flight per wave).
#ifndef ILGPU_HIP_SCAN_LOAD_HALVES
#define ILGPU_HIP_SCAN_LOAD_HALVES 0
#endif
// 8-byte status words per tile: one 128-byte line each.  Every resident block
// polls the words of the few dozen tiles before it with loads that go past the
// L2; packed eight bytes apart those words share a handful of lines, and the
// memory channels that hold them fall behind on the data streams (measured at
// 2^28 int32: 0.384 ms packed, 0.363 at 64 bytes per tile, 0.360 at 128 to 512).
constexpr int kStatusStride = 16;
constexpr int64_t kStatusBytes = 8 * kStatusStride;
constexpr int kBlock = ILGPU_HIP_SCAN_BLOCK;
constexpr int kWaves = kBlock / kWaveSize;
constexpr int kVecs = ILGPU_HIP_SCAN_VECS;
#ifndef ILGPU_HIP_SCAN_VECS8
#define ILGPU_HIP_SCAN_VECS8 16
#endif
// 16-byte vectors per thread and tile, by element size (the same 128 KiB tile
// for both: measured at 2^27 int64 in the register-lean form, 10 vectors
// 0.456 ms, 12: 0.401, 14: 0.394, 16: 0.382, 18 and 20 the same as 16 for Add
// but 0.48 and 0.54 for the floating-point Max, which then spills).
template <typename T> constexpr int scan_vecs() {
  return sizeof(T) == 8 ? ILGPU_HIP_SCAN_VECS8 : kVecs;
}
constexpr uint32_t kFlagInvalid = 0, kFlagAggregate = 1, kFlagPrefix = 2;
constexpr int64_t kHeaderBytes = 256;  // ticket counter, padded

template <typename T> constexpr int tile_elems() {
  return kBlock * scan_vecs<T>() * Vec16<T>::N;
}

template <typename T> struct Bits;
template <> struct Bits<int32_t> { using type = uint32_t; };
template <> struct Bits<uint32_t> { using type = uint32_t; };
template <> struct Bits<float> { using type = uint32_t; };
template <> struct Bits<int64_t> { using type = uint64_t; };
template <> struct Bits<uint64_t> { using type = uint64_t; };
template <> struct Bits<double> { using type = uint64_t; };

template <typename T>
__device__ __forceinline__ typename Bits<T>::type to_bits(T v) {
  typename Bits<T>::type b;
  __builtin_memcpy(&b, &v, sizeof(T));
  return b;
}
template <typename T>
__device__ __forceinline__ T from_bits(typename Bits<T>::type b) {
  T v;
  __builtin_memcpy(&v, &b, sizeof(T));
  return v;
}

// Look-back state in temp memory.
template <typename T, int SIZE = sizeof(T)> struct TileState;

template <typename T> struct TileState<T, 4> {
  uint64_t* words;
  __device__ __forceinline__ void publish(int tile, uint32_t flag, T v) const {
    const uint64_t w = ((uint64_t)flag << 32) | to_bits(v);
    __hip_atomic_store(&words[(int64_t)tile * kStatusStride], w, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
  // Spins until the tile has published something; returns its flag.
  __device__ __forceinline__ uint32_t wait(int tile, T* v) const {
    uint64_t w;
    while (true) {
      w = __hip_atomic_load(&words[(int64_t)tile * kStatusStride], __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
      if ((uint32_t)(w >> 32) != kFlagInvalid) break;
      __builtin_amdgcn_s_sleep(1);
    }
    *v = from_bits<T>((uint32_t)w);
    return (uint32_t)(w >> 32);
  }
};

// 8-byte values: two 64-bit words in the tile's line, {flag, low half} and
// {flag, high half}, each written and read with one relaxed atomic.  A tile writes each
// state (aggregate, then prefix) once, so two words with the same flag hold
// the halves of the same value; a reader that catches the words in different
// states reads again.  No fences: an agent-scope release would write back the
// whole L2 of the XCD for every tile.
template <typename T> struct TileState<T, 8> {
  uint64_t* words;
  __device__ __forceinline__ void publish(int tile, uint32_t flag, T v) const {
    const uint64_t bits = to_bits(v);
    uint64_t* w = &words[(int64_t)tile * kStatusStride];
    __hip_atomic_store(&w[0], ((uint64_t)flag << 32) | (uint32_t)bits,
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&w[1], ((uint64_t)flag << 32) | (bits >> 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __device__ __forceinline__ uint32_t wait(int tile, T* v) const {
    uint64_t lo, hi;
    const uint64_t* w = &words[(int64_t)tile * kStatusStride];
    while (true) {
      lo = __hip_atomic_load(&w[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      hi = __hip_atomic_load(&w[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((uint32_t)(lo >> 32) != kFlagInvalid && (lo >> 32) == (hi >> 32)) break;
      __builtin_amdgcn_s_sleep(1);
    }
    *v = from_bits<T>((uint64_t)(uint32_t)lo | (hi << 32));
    return (uint32_t)(lo >> 32);
  }
};

// Data-parallel-primitive move: lane i receives `v` of the lane that the
// control word CTRL names (row_shr:n = 0x110 + n within rows of 16 lanes,
// row_bcast:15 = 0x142, row_bcast:31 = 0x143, wave_shr:1 = 0x138); lanes
// without a source, and rows outside ROW_MASK, receive `fill`.
template <typename T, int CTRL, int ROW_MASK>
__device__ __forceinline__ T dpp_move(T fill, T v) {
  if constexpr (sizeof(T) == 8) {
    union { T t; int32_t w[2]; } f, a, b;
    f.t = fill;
    a.t = v;
    b.w[0] = __builtin_amdgcn_update_dpp(f.w[0], a.w[0], CTRL, ROW_MASK, 0xf, false);
    b.w[1] = __builtin_amdgcn_update_dpp(f.w[1], a.w[1], CTRL, ROW_MASK, 0xf, false);
    return b.t;
  } else {
    union { T t; int32_t w; } f, a, b;
    f.t = fill;
    a.t = v;
    b.w = __builtin_amdgcn_update_dpp(f.w, a.w, CTRL, ROW_MASK, 0xf, false);
    return b.t;
  }
}

// Inclusive scan over the 64 lanes of a wave: four shifted steps inside each
// row of 16 lanes, then the last lane of row 0 (2) is folded into row 1 (3),
// then lane 31 into rows 2 and 3.
template <typename T, int OP>
__device__ __forceinline__ T wave_inclusive_scan(T v, int) {
  using F = Functor<T, OP>;
  const T id = F::identity();
  v = F::apply(dpp_move<T, 0x111, 0xf>(id, v), v);
  v = F::apply(dpp_move<T, 0x112, 0xf>(id, v), v);
  v = F::apply(dpp_move<T, 0x114, 0xf>(id, v), v);
  v = F::apply(dpp_move<T, 0x118, 0xf>(id, v), v);
  v = F::apply(dpp_move<T, 0x142, 0xa>(id, v), v);
  v = F::apply(dpp_move<T, 0x143, 0xc>(id, v), v);
  return v;
}

// Value of `v` in lane `src` as a wave-uniform (scalar register) value.
template <typename T>
__device__ __forceinline__ T read_lane(T v, int src) {
  if constexpr (sizeof(T) == 8) {
    union { T t; int32_t w[2]; } a, b;
    a.t = v;
    b.w[0] = __builtin_amdgcn_readlane(a.w[0], src);
    b.w[1] = __builtin_amdgcn_readlane(a.w[1], src);
    return b.t;
  } else {
    union { T t; int32_t w; } a, b;
    a.t = v;
    b.w = __builtin_amdgcn_readlane(a.w, src);
    return b.t;
  }
}

// Keeps a value where it is in program order: the scheduler otherwise
// interleaves the row scans of a tile and keeps a copy of every row alive.
template <typename T> __device__ __forceinline__ void pin(T& v) {
  if constexpr (sizeof(T) == 8) {
    union { T t; int32_t w[2]; } a;
    a.t = v;
    asm volatile("" : "+v"(a.w[0]), "+v"(a.w[1]));
    v = a.t;
  } else {
    union { T t; int32_t w; } a;
    a.t = v;
    asm volatile("" : "+v"(a.w));
    v = a.t;
  }
}

// Value of the previous lane; lane 0 receives `fill`.
template <typename T>
__device__ __forceinline__ T lane_shift_up(T fill, T v) {
  return dpp_move<T, 0x138, 0xf>(fill, v);
}

template <typename T, int OP>
__device__ __forceinline__ T wave_reduce(T v) {
  using F = Functor<T, OP>;
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1)
    v = F::apply(v, shfl_down(v, off));
  return shfl(v, 0);
}

// Executed by the first wave of the block.  Publishes the tile's aggregate,
// resolves the exclusive prefix of the tile and publishes the inclusive one.
template <typename T, int OP>
__device__ __forceinline__ T resolve_prefix(const TileState<T>& st, int tile,
                                            T aggregate, int lane) {
  using F = Functor<T, OP>;
  if (tile == 0) {
    if (lane == 0) st.publish(0, kFlagPrefix, aggregate);
    return F::identity();
  }
  if (lane == 0) st.publish(tile, kFlagAggregate, aggregate);
  T exclusive = F::identity();
  int base = tile - 1;
  while (true) {
    const int idx = base - lane;
    T val = F::identity();
    uint32_t flag = kFlagPrefix;  // virtual prefix in front of tile 0
    if (idx >= 0) flag = st.wait(idx, &val);
    const uint64_t has_prefix = __ballot(flag == kFlagPrefix);
    // Lanes run from the nearest predecessor (lane 0) to the farthest; the
    // first lane holding an inclusive prefix ends the walk.
    const int first = has_prefix != 0
                          ? __ffsll((unsigned long long)has_prefix) - 1
                          : kWaveSize - 1;
    const T contrib = lane <= first ? val : F::identity();
    exclusive = F::apply(wave_reduce<T, OP>(contrib), exclusive);
    if (has_prefix != 0) break;  // wave-uniform
    base -= kWaveSize;
  }
  if (lane == 0) st.publish(tile, kFlagPrefix, F::apply(exclusive, aggregate));
  return exclusive;
}

// Four waves per SIMD, i.e. 128 registers and two blocks per CU: left to itself
// the compiler takes 180 to 256 registers for the floating-point Max and Min
// kernels, which halves their residency (measured 0.56 -> 0.44 ms at 2^28 float).
template <typename T, int OP, bool VECTOR>
__global__ __launch_bounds__(kBlock, ILGPU_HIP_SCAN_WAVES_PER_EU) void scan_kernel(
    const T* __restrict__ in, T* __restrict__ out, int64_t n,
    int64_t in_stride, int64_t out_stride, int inclusive,
    uint32_t* __restrict__ ticket, TileState<T> st) {
  using F = Functor<T, OP>;
  using V = typename Vec16<T>::type;
  constexpr int VN = Vec16<T>::N;
  constexpr int kTileVecs = scan_vecs<T>();
  constexpr int kTile = tile_elems<T>();
  constexpr int kWaveElems = kTile / kWaves;

  __shared__ int s_tile;
  __shared__ T s_wave_total[kWaves];
  __shared__ T s_prefix;

  // An input of one tile comes without ticket and status words (and without
  // the launch that clears them): there is nobody to wait for or to tell.
  const bool alone = ticket == nullptr;
  if (!alone) {
    if (threadIdx.x == 0) s_tile = (int)atomicAdd(ticket, 1u);
    __syncthreads();
  }
  const int tile = alone ? 0 : s_tile;
  const int lane = threadIdx.x & (kWaveSize - 1);
  // The wave index and everything derived from it are wave-uniform: kept in
  // scalar registers, so a lane addresses its vectors by one 32-bit offset.
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize);
  const int64_t tile_base = (int64_t)tile * kTile;
  const int64_t wave_base = tile_base + (int64_t)wave * kWaveElems;
  const bool full = tile_base + kTile <= n;
  // Elements of this wave's chunk that lie inside the view (tail path only).
  const int wave_valid =
      (int)(n - wave_base < kWaveElems ? (n - wave_base < 0 ? 0 : n - wave_base)
                                       : kWaveElems);

  T x[kTileVecs][VN];
  constexpr bool kHalves = ILGPU_HIP_SCAN_LOAD_HALVES && sizeof(T) == 4 && kTileVecs % 2 == 0;
  auto load_rows = [&](int j0, int j1) {
    const V* src = reinterpret_cast<const V*>(in + wave_base);
#pragma unroll
    for (int j = j0; j < j1; ++j) {
      V v = ILGPU_HIP_SCAN_NT_LOAD ? __builtin_nontemporal_load(&src[j * kWaveSize + lane])
                                   : src[j * kWaveSize + lane];
#pragma unroll
      for (int k = 0; k < VN; ++k) x[j][k] = v[k];
    }
  };
  if (VECTOR && full) {
    load_rows(0, kHalves ? kTileVecs / 2 : kTileVecs);
  } else {
#pragma unroll
    for (int j = 0; j < kTileVecs; ++j)
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        const int e = (j * kWaveSize + lane) * VN + k;
        x[j][k] = e < wave_valid ? in[(wave_base + e) * in_stride] : F::identity();
      }
  }

  if constexpr (sizeof(T) == 8) {
    // Register-lean form for 8-byte elements, whose per-row prefixes would
    // take two registers each: the prefix of the lower lanes is folded into
    // the row at once, so no per-row prefix outlives this loop, and the row
    // totals are wave-uniform values in scalar registers (104 registers at 16
    // vectors; 2^27 int64 Add 0.419 -> 0.382 ms against the form below at 10
    // vectors).  For 4-byte elements the two forms measure the same.
    T seg_total[kTileVecs];
#pragma unroll
    for (int j = 0; j < kTileVecs; ++j) {
#pragma unroll
      for (int k = 1; k < VN; ++k) x[j][k] = F::apply(x[j][k - 1], x[j][k]);
      const T inc = wave_inclusive_scan<T, OP>(x[j][VN - 1], lane);
      seg_total[j] = read_lane<T>(inc, kWaveSize - 1);
      const T up = lane_shift_up<T>(F::identity(), inc);
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        x[j][k] = F::apply(up, x[j][k]);
        pin(x[j][k]);
      }
    }
    T wave_total = seg_total[0];
#pragma unroll
    for (int j = 1; j < kTileVecs; ++j) wave_total = F::apply(wave_total, seg_total[j]);
    if (lane == 0) s_wave_total[wave] = wave_total;
    __syncthreads();
    T wave_prefix = F::identity();
    T block_total = s_wave_total[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      if (w == wave) wave_prefix = block_total;
      block_total = F::apply(block_total, s_wave_total[w]);
    }
    if (wave == 0) {
      const T exclusive = ILGPU_HIP_SCAN_PROBE_NO_LOOKBACK || alone
                              ? F::identity()
                              : resolve_prefix<T, OP>(st, tile, block_total, lane);
      if (lane == 0) s_prefix = exclusive;
    }
    __syncthreads();
    T running = F::apply(s_prefix, wave_prefix);
    V* dst = reinterpret_cast<V*>(out + wave_base);
#pragma unroll
    for (int j = 0; j < kTileVecs; ++j) {
      T r[VN];
      if (inclusive) {
#pragma unroll
        for (int k = 0; k < VN; ++k) r[k] = F::apply(running, x[j][k]);
      } else {
        r[0] = F::apply(running, lane_shift_up<T>(F::identity(), x[j][VN - 1]));
#pragma unroll
        for (int k = 1; k < VN; ++k) r[k] = F::apply(running, x[j][k - 1]);
      }
      if (VECTOR && full) {
        V v;
#pragma unroll
        for (int k = 0; k < VN; ++k) v[k] = r[k];
        if (ILGPU_HIP_SCAN_NT_STORE) __builtin_nontemporal_store(v, &dst[j * kWaveSize + lane]);
        else dst[j * kWaveSize + lane] = v;
      } else {
#pragma unroll
        for (int k = 0; k < VN; ++k) {
          const int e = (j * kWaveSize + lane) * VN + k;
          if (e < wave_valid) out[(wave_base + e) * out_stride] = r[k];
        }
      }
      running = F::apply(running, seg_total[j]);
    }
    return;
  }
  // Lane-local inclusive scan of each vector, then one wave scan per j.
  T lane_excl[kTileVecs];   // fold of the vectors of lower lanes, same j
  T seg_total[kTileVecs];   // fold of the whole 64-lane row j
  auto scan_rows = [&](int j0, int j1) {
#pragma unroll
    for (int j = j0; j < j1; ++j) {
#pragma unroll
      for (int k = 1; k < VN; ++k) x[j][k] = F::apply(x[j][k - 1], x[j][k]);
      const T inc = wave_inclusive_scan<T, OP>(x[j][VN - 1], lane);
      seg_total[j] = shfl(inc, kWaveSize - 1);
      lane_excl[j] = lane_shift_up<T>(F::identity(), inc);
    }
  };
  if (kHalves && VECTOR && full) {
    scan_rows(0, kTileVecs / 2);
    __builtin_amdgcn_sched_barrier(0);
    load_rows(kTileVecs / 2, kTileVecs);
    scan_rows(kTileVecs / 2, kTileVecs);
  } else {
    scan_rows(0, kTileVecs);
  }
  T wave_total = seg_total[0];
#pragma unroll
  for (int j = 1; j < kTileVecs; ++j) wave_total = F::apply(wave_total, seg_total[j]);
  if (lane == 0) s_wave_total[wave] = wave_total;
  __syncthreads();

  T wave_prefix = F::identity();
  T block_total = s_wave_total[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) {
    if (w == wave) wave_prefix = block_total;
    block_total = F::apply(block_total, s_wave_total[w]);
  }

  if (wave == 0) {
    const T exclusive = ILGPU_HIP_SCAN_PROBE_NO_LOOKBACK || alone
                            ? F::identity()
                            : resolve_prefix<T, OP>(st, tile, block_total, lane);
    if (lane == 0) s_prefix = exclusive;
  }
  __syncthreads();

  T running = F::apply(s_prefix, wave_prefix);  // prefix of row 0 of this wave
  V* dst = reinterpret_cast<V*>(out + wave_base);
#pragma unroll
  for (int j = 0; j < kTileVecs; ++j) {
    const T before = F::apply(running, lane_excl[j]);  // prefix of x[j][0]
    T r[VN];
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      if (inclusive) r[k] = F::apply(before, x[j][k]);
      else r[k] = k == 0 ? before : F::apply(before, x[j][k - 1]);
    }
    if (VECTOR && full) {
      V v;
#pragma unroll
      for (int k = 0; k < VN; ++k) v[k] = r[k];
      if (ILGPU_HIP_SCAN_NT_STORE) __builtin_nontemporal_store(v, &dst[j * kWaveSize + lane]);
      else dst[j * kWaveSize + lane] = v;
    } else {
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        const int e = (j * kWaveSize + lane) * VN + k;
        if (e < wave_valid) out[(wave_base + e) * out_stride] = r[k];
      }
    }
    running = F::apply(running, seg_total[j]);
  }
}

// ---- unique ------------------------------------------------------------------
// Removes consecutive duplicates in place and reports the new length; stands
// in for the Unique delegate of UniqueExtensions.cs:59-209, whose kernel runs
// the groups strictly one after the other (SequentialGroupExecutor) with a
// serial compaction loop per group.  Here it is the same single-pass chain as
// the scan: an element is kept if it differs from its predecessor, a tile
// publishes its number of kept elements, resolves how many were kept in front
// of it, and writes its kept elements to data[kept_before + local rank].
//
// In place is safe without a second buffer: a tile loads all of its elements
// (and the element in front of each vector) before it publishes anything, a
// tile learns its offset only after every earlier tile has published, and it
// writes only at or below the positions it read, so no element is overwritten
// before its owner (or its successor's comparison) has read it.
//
// "Differs" is Comparison<T>.Compare(a, b) != 0 (ComparisonOperations.tt:30-45),
// i.e. CompareTo: all NaNs are equal to each other and -0.0 equals +0.0.
#ifndef ILGPU_HIP_UNIQUE_VECS
#define ILGPU_HIP_UNIQUE_VECS 12
#endif
#ifndef ILGPU_HIP_UNIQUE_NT_STORE
#define ILGPU_HIP_UNIQUE_NT_STORE 1
#endif
#ifndef ILGPU_HIP_UNIQUE_VECS1
#define ILGPU_HIP_UNIQUE_VECS1 4
#endif
#ifndef ILGPU_HIP_UNIQUE_VECS2
#define ILGPU_HIP_UNIQUE_VECS2 8
#endif
// 16-byte vectors per thread and tile, by element size: every element of a
// vector is unpacked into a register of its own, so a vector of bytes costs
// sixteen registers and one of 2-byte elements eight.
constexpr int unique_vecs(int elem_bytes) {
  return elem_bytes == 1 ? ILGPU_HIP_UNIQUE_VECS1
                         : elem_bytes == 2 ? ILGPU_HIP_UNIQUE_VECS2 : ILGPU_HIP_UNIQUE_VECS;
}

template <typename T> struct is_float_like { static constexpr bool value = is_fp<T>::value; };
template <> struct is_float_like<_Float16> { static constexpr bool value = true; };

template <typename T> __device__ __forceinline__ bool differs(T a, T b) {
  if constexpr (is_float_like<T>::value) return !(a == b) && !(a != a && b != b);
  else return a != b;
}

template <typename T> constexpr int unique_tile_elems() {
  return kBlock * unique_vecs(sizeof(T)) * Vec16<T>::N;
}

template <typename T, bool VECTOR>
__global__ __launch_bounds__(kBlock) void unique_kernel(
    T* data, int64_t n, int64_t* __restrict__ out_length,
    uint32_t* __restrict__ ticket, TileState<uint32_t> st, int num_tiles) {
  using V = typename Vec16<T>::type;
  constexpr int VN = Vec16<T>::N;
  constexpr int kUniqueVecs = unique_vecs(sizeof(T));
  constexpr int kTile = unique_tile_elems<T>();
  constexpr int kWaveElems = kTile / kWaves;

  __shared__ int s_tile;
  __shared__ uint32_t s_wave_total[kWaves];
  __shared__ uint32_t s_prefix;

  const bool alone = ticket == nullptr;  // one tile: no ticket, no status words
  if (!alone) {
    if (threadIdx.x == 0) s_tile = (int)atomicAdd(ticket, 1u);
    __syncthreads();
  }
  const int tile = alone ? 0 : s_tile;
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave = threadIdx.x / kWaveSize;
  const int64_t tile_base = (int64_t)tile * kTile;
  const int64_t wave_base = tile_base + (int64_t)wave * kWaveElems;
  const bool full = tile_base + kTile <= n;

  T x[kUniqueVecs][VN];
  // The element in front of the wave's chunk; every other predecessor is in a
  // register of this wave.
  const T chunk_before = wave_base > 0 && wave_base < n ? data[wave_base - 1] : T();
#pragma unroll
  for (int j = 0; j < kUniqueVecs; ++j) {
    const int64_t first = wave_base + (int64_t)(j * kWaveSize + lane) * VN;
    if (VECTOR && full) {
      const V v = __builtin_nontemporal_load(reinterpret_cast<const V*>(data + first));
#pragma unroll
      for (int k = 0; k < VN; ++k) x[j][k] = v[k];
    } else {
#pragma unroll
      for (int k = 0; k < VN; ++k) x[j][k] = first + k < n ? data[first + k] : T();
    }
  }
  T before[kUniqueVecs];  // the element in front of each vector
#pragma unroll
  for (int j = 0; j < kUniqueVecs; ++j) {
    const T from_left = shfl_up(x[j][VN - 1], 1);
    const T row_before = j == 0 ? chunk_before : shfl(x[j > 0 ? j - 1 : 0][VN - 1], kWaveSize - 1);
    before[j] = lane == 0 ? row_before : from_left;
  }

  // keep bit k of vector j; kept elements per vector; wave scan per row.
  uint32_t keep[kUniqueVecs], lane_excl[kUniqueVecs], seg_total[kUniqueVecs];
#pragma unroll
  for (int j = 0; j < kUniqueVecs; ++j) {
    const int64_t first = wave_base + (int64_t)(j * kWaveSize + lane) * VN;
    uint32_t bits = 0;
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      const bool valid = first + k < n;
      const bool is_first = first + k == 0;
      const bool d = differs<T>(x[j][k], k == 0 ? before[j] : x[j][k - 1]);
      if (valid && (is_first || d)) bits |= 1u << k;
    }
    keep[j] = bits;
    const uint32_t cnt = (uint32_t)__popc(bits);
    const uint32_t inc = wave_inclusive_scan<uint32_t, ILGPU_HIP_OP_ADD>(cnt, lane);
    seg_total[j] = shfl(inc, kWaveSize - 1);
    lane_excl[j] = inc - cnt;
  }
  uint32_t wave_total = 0;
#pragma unroll
  for (int j = 0; j < kUniqueVecs; ++j) wave_total += seg_total[j];
  if (lane == 0) s_wave_total[wave] = wave_total;
  __syncthreads();

  uint32_t wave_prefix = 0, block_total = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    if (w == wave) wave_prefix = block_total;
    block_total += s_wave_total[w];
  }
  if (wave == 0) {
    const uint32_t exclusive =
        alone ? 0u : resolve_prefix<uint32_t, ILGPU_HIP_OP_ADD>(st, tile, block_total, lane);
    if (lane == 0) s_prefix = exclusive;
  }
  __syncthreads();

  uint32_t running = s_prefix + wave_prefix;
#pragma unroll
  for (int j = 0; j < kUniqueVecs; ++j) {
    uint32_t pos = running + lane_excl[j];
    if (keep[j] == (1u << VN) - 1u) {
      // the whole vector survives: one 16-byte store, aligned like an element
      typedef V UnalignedV __attribute__((aligned(sizeof(T))));
      V v;
#pragma unroll
      for (int k = 0; k < VN; ++k) v[k] = x[j][k];
      if (ILGPU_HIP_UNIQUE_NT_STORE) __builtin_nontemporal_store(v, reinterpret_cast<UnalignedV*>(data + pos));
      else *reinterpret_cast<UnalignedV*>(data + pos) = v;
    } else {
#pragma unroll
      for (int k = 0; k < VN; ++k)
        if (keep[j] >> k & 1u) data[pos++] = x[j][k];
    }
    running += seg_total[j];
  }
  if (tile == num_tiles - 1 && threadIdx.x == 0)
    out_length[0] = (int64_t)s_prefix + (int64_t)block_total;
}

__global__ void zero_words_kernel(uint32_t* words, int64_t count) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count;
       i += stride)
    words[i] = 0u;
}

template <typename T> int64_t num_tiles(int64_t n) {
  return div_up(n, tile_elems<T>());
}

template <typename T, int OP>
int32_t launch_typed(hipStream_t stream, const void* in, int64_t in_stride,
                     void* out, int64_t out_stride, int64_t n, int32_t kind,
                     void* temp) {
  const int64_t tiles = num_tiles<T>(n);
  char* base = reinterpret_cast<char*>(align_up((int64_t)(uintptr_t)temp, 256));
  uint32_t* ticket = reinterpret_cast<uint32_t*>(base);
  TileState<T> st;
  st.words = reinterpret_cast<uint64_t*>(base + kHeaderBytes);
  if (tiles > 1) {
    const int64_t zero_words = (kHeaderBytes + tiles * kStatusBytes) / 4;
    const int32_t rc = launch_zero_words(stream, reinterpret_cast<uint32_t*>(base), zero_words);
    if (rc != ILGPU_HIP_SUCCESS) return rc;
  } else {
    ticket = nullptr;  // one tile: one launch
  }
  // Element strides above one (Stride1D.General) take the scalar path.
  const bool vector = in_stride == 1 && out_stride == 1 &&
                      (reinterpret_cast<uintptr_t>(in) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  const int inclusive = kind == ILGPU_HIP_SCAN_INCLUSIVE ? 1 : 0;
  ProfileScope scope(stream, "scan");
  if (vector) {
    hipLaunchKernelGGL((scan_kernel<T, OP, true>), dim3((unsigned)tiles),
                       dim3(kBlock), 0, stream, static_cast<const T*>(in),
                       static_cast<T*>(out), n, in_stride, out_stride,
                       inclusive, ticket, st);
  } else {
    hipLaunchKernelGGL((scan_kernel<T, OP, false>), dim3((unsigned)tiles),
                       dim3(kBlock), 0, stream, static_cast<const T*>(in),
                       static_cast<T*>(out), n, in_stride, out_stride,
                       inclusive, ticket, st);
  }
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

template <typename T>
int32_t launch_op(hipStream_t stream, const void* in, int64_t in_stride,
                  void* out, int64_t out_stride, int64_t n, int32_t op,
                  int32_t kind, void* temp) {
  switch (op) {
    case ILGPU_HIP_OP_ADD:
      return launch_typed<T, ILGPU_HIP_OP_ADD>(stream, in, in_stride, out, out_stride, n,
                                               kind, temp);
    case ILGPU_HIP_OP_MAX:
      return launch_typed<T, ILGPU_HIP_OP_MAX>(stream, in, in_stride, out, out_stride, n,
                                               kind, temp);
    case ILGPU_HIP_OP_MIN:
      return launch_typed<T, ILGPU_HIP_OP_MIN>(stream, in, in_stride, out, out_stride, n,
                                               kind, temp);
    default:
      return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace

int32_t launch_zero_words(hipStream_t stream, uint32_t* words, int64_t count) {
  if (count <= 0) return ILGPU_HIP_SUCCESS;
  int64_t blocks = div_up(count, 256 * 4);
  if (blocks > 2048) blocks = 2048;
  ProfileScope scope(stream, "zero_words");
  hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     stream, words, count);
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

int64_t scan_temp_bytes(int64_t n, int elem_bytes) {
  // 256 bytes of alignment slack + header + per-tile state.
  const int64_t tiles =
      elem_bytes == 4 ? num_tiles<uint32_t>(n) : num_tiles<uint64_t>(n);
  return 256 + kHeaderBytes + tiles * kStatusBytes;
}

int32_t launch_scan(hipStream_t stream, const void* in, int64_t in_stride,
                    void* out, int64_t out_stride, int64_t n, int32_t type,
                    int32_t op, int32_t kind, void* temp) {
  switch (type) {
    case ILGPU_HIP_I32: return launch_op<int32_t>(stream, in, in_stride, out, out_stride, n, op, kind, temp);
    case ILGPU_HIP_U32: return launch_op<uint32_t>(stream, in, in_stride, out, out_stride, n, op, kind, temp);
    case ILGPU_HIP_I64: return launch_op<int64_t>(stream, in, in_stride, out, out_stride, n, op, kind, temp);
    case ILGPU_HIP_U64: return launch_op<uint64_t>(stream, in, in_stride, out, out_stride, n, op, kind, temp);
    case ILGPU_HIP_F32: return launch_op<float>(stream, in, in_stride, out, out_stride, n, op, kind, temp);
    case ILGPU_HIP_F64: return launch_op<double>(stream, in, in_stride, out, out_stride, n, op, kind, temp);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

// ---- scan on the library's own scratch ---------------------------------------
// For callers that cannot allocate or carry a temp view: the tile states of one
// scan live in a device array that is part of the library's code object.  It is
// sized for kStaticScanTiles tiles (1 GiB of input); every call on a GPU shares
// that GPU's copy, so calls that overlap in time on one GPU race.
constexpr int64_t kSmallestTileBytes =
    (int64_t)kBlock * 16 * (scan_vecs<uint32_t>() < scan_vecs<uint64_t>() ? scan_vecs<uint32_t>()
                                                                           : scan_vecs<uint64_t>());
constexpr int64_t kStaticScanTiles = ILGPU_HIP_SCAN_STATIC_MAX_BYTES / kSmallestTileBytes;
constexpr int64_t kStaticScratchBytes = kHeaderBytes + kStaticScanTiles * kStatusBytes;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
}  // namespace

int32_t launch_scan_static(hipStream_t stream, const void* in, int64_t in_stride,
                           void* out, int64_t out_stride, int64_t n, int32_t type,
                           int32_t op, int32_t kind) {
  // The tiles of this call must fit the array: scan_temp_bytes() minus the
  // alignment slack a caller's temp needs (the array is aligned itself).
  if (scan_temp_bytes(n, elem_size(type)) - 256 > kStaticScratchBytes)
    return ILGPU_HIP_ERROR_STATIC_LIMIT;
  int device = -1;
  ILGPU_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  // Every GPU holds its own copy of the array at its own address; the array's
  // name is no device address on the host.  Looked up once per device.
  void* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ptr = g_scratch_ptr[device].load(std::memory_order_relaxed);
    if (ptr == nullptr) {
      ILGPU_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
      if (ptr == nullptr) return ILGPU_HIP_ERROR_RUNTIME;
      g_scratch_ptr[device].store(ptr, std::memory_order_release);
    }
  }
  // launch_scan clears the ticket and the status lines it will use with a fill
  // kernel (the array keeps the previous call's contents) and hands `ptr` to
  // the scan kernel as it does with a caller's temp.
  return launch_scan(stream, in, in_stride, out, out_stride, n, type, op, kind, ptr);
}

int64_t unique_temp_bytes(int64_t n, int elem_bytes) {
  const int64_t tile = (int64_t)kBlock * unique_vecs(elem_bytes) * (16 / elem_bytes);
  return 256 + kHeaderBytes + div_up(n, tile) * kStatusBytes;
}

namespace {
template <typename T>
int32_t launch_unique_typed(hipStream_t stream, void* data, int64_t n,
                            int64_t* out_length, void* temp) {
  const int64_t tiles = div_up(n, (int64_t)unique_tile_elems<T>());
  char* base = reinterpret_cast<char*>(align_up((int64_t)(uintptr_t)temp, 256));
  uint32_t* ticket = reinterpret_cast<uint32_t*>(base);
  TileState<uint32_t> st;
  st.words = reinterpret_cast<uint64_t*>(base + kHeaderBytes);
  if (tiles > 1) {
    const int32_t rc = launch_zero_words(stream, reinterpret_cast<uint32_t*>(base),
                                         (kHeaderBytes + tiles * kStatusBytes) / 4);
    if (rc != ILGPU_HIP_SUCCESS) return rc;
  } else {
    ticket = nullptr;  // one tile: one launch
  }
  const bool vector = (reinterpret_cast<uintptr_t>(data) & 15) == 0;
  ProfileScope scope(stream, "unique");
  if (vector)
    hipLaunchKernelGGL((unique_kernel<T, true>), dim3((unsigned)tiles), dim3(kBlock), 0,
                       stream, static_cast<T*>(data), n, out_length, ticket, st,
                       (int)tiles);
  else
    hipLaunchKernelGGL((unique_kernel<T, false>), dim3((unsigned)tiles), dim3(kBlock), 0,
                       stream, static_cast<T*>(data), n, out_length, ticket, st,
                       (int)tiles);
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}
}  // namespace

int32_t launch_unique(hipStream_t stream, void* data, int64_t n, int32_t type,
                      int64_t* out_length, void* temp) {
  switch (type) {
    case ILGPU_HIP_I8: return launch_unique_typed<int8_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_U8: return launch_unique_typed<uint8_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_I16: return launch_unique_typed<int16_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_U16: return launch_unique_typed<uint16_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_I32: return launch_unique_typed<int32_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_U32: return launch_unique_typed<uint32_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_I64: return launch_unique_typed<int64_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_U64: return launch_unique_typed<uint64_t>(stream, data, n, out_length, temp);
    case ILGPU_HIP_F16: return launch_unique_typed<_Float16>(stream, data, n, out_length, temp);
    case ILGPU_HIP_F32: return launch_unique_typed<float>(stream, data, n, out_length, temp);
    case ILGPU_HIP_F64: return launch_unique_typed<double>(stream, data, n, out_length, temp);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace ilgpu_hip
