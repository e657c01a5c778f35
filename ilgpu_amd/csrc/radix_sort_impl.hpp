// Radix sort of keys and key/value pairs: onesweep LSD sort, 8-bit digits.
//
// Stands in for the RadixSort / RadixSortPairs delegates of
// RadixSortExtensions.cs:1017-1337.  The reference runs NumBits/2 passes of
// {memset, local 4-way split, counter scan, scatter} (:1276-1334) and packs
// pairs into an array of structs first (:1057-1072).  Here a sort of k-byte
// keys is
//
//   zero      clears the global digit histograms, tile tickets and look-back
//             status words (one launch);
//   histogram one read of the keys builds the 256-bin histogram of every digit
//             position in LDS (replicated counters) and adds it to global;
//   plan      one block turns the histograms into exclusive digit offsets,
//             marks passes whose digit is the same for every key (they are
//             skipped) and records which buffer each pass reads;
//   pass x k  onesweep: a block takes a tile by ticket, ranks its keys (one
//             returning LDS add per key on per-wave digit counters; the LDS
//             serves the lanes of an instruction in lane order, so equal digits
//             keep memory order: every pass is stable), publishes
//             its 256 digit counts, resolves the counts of all earlier tiles by
//             decoupled look-back, stages the tile in digit order through LDS
//             and writes each digit's run to its final place;
//   finish    copies the result back if an odd number of passes ran.
//
// Keys and values stay in separate arrays (structure of arrays); a value
// travels with its key through the same tile-local permutation.
//
// Key order: digit(k) = ((k ^ xor_mask ^ f(k)) >> shift) & 0xFF, where
// xor_mask folds the sign-bit flip of signed/float types and the complement
// of Descending* (RadixSortOperations.tt:77-93, 122-123) and f(k) is the
// per-key term of the float transforms.  Float keys are converted once, by the
// first pass that runs, and converted back by the last one.
//
// Algorithmic HBM traffic for n keys of k bytes, values of v bytes and P
// executed passes: n * (k * (2P + 1) + v * 2P) bytes.
//
// This header holds the kernels and their launch code as templates; one
// translation unit per key size (radix_sort_k1/2/4/8.hip) instantiates them, so
// that the key sizes compile side by side, and radix_sort.hip holds what does
// not depend on the key size.  (A kernel has to be defined in the translation
// unit that launches it, hence a header and not a library of kernels.)
#pragma once

#include <hip/hip_fp16.h>

#include <atomic>
#include <type_traits>

#include "kernels.hpp"

namespace ilgpu_hip {

// Process-wide sort parameters (ilgpu_hip_sort_set_parameter), defined in
// radix_sort.hip.
extern std::atomic<uint32_t> g_sort_spin_limit;
extern std::atomic<int32_t> g_sort_large_min_tiles_per_cu;  // negative: the defaults
extern std::atomic<int32_t> g_sort_small_kernel;            // 0: one-tile inputs take the passes too
extern std::atomic<int32_t> g_sort_short_tile_max_tiles;    // negative: the default

namespace {

constexpr int kRadix = 256;
constexpr int kMaxPasses = 8;
// Launch shape of the onesweep pass.  The block size fixes the number of
// per-wave sub-tiles (and with it the LDS footprint of the ranking counters);
// items per thread fix the tile size.
#ifndef ILGPU_HIP_SORT_BLOCK
#define ILGPU_HIP_SORT_BLOCK 512
#endif
#ifndef ILGPU_HIP_SORT_ITEMS
#define ILGPU_HIP_SORT_ITEMS 36
#endif
#ifndef ILGPU_HIP_SORT_ITEMS8
#define ILGPU_HIP_SORT_ITEMS8 18
#endif
#ifndef ILGPU_HIP_SORT_PAIR_ITEMS2
#define ILGPU_HIP_SORT_PAIR_ITEMS2 16
#endif
#ifndef ILGPU_HIP_SORT_PAIR_ITEMS4
#define ILGPU_HIP_SORT_PAIR_ITEMS4 10
#endif
#ifndef ILGPU_HIP_SORT_PAIR_ITEMS3
#define ILGPU_HIP_SORT_PAIR_ITEMS3 14
#endif
#ifndef ILGPU_HIP_SORT_LOOKBACK
#define ILGPU_HIP_SORT_LOOKBACK 4
#endif
// Rows whose LDS operations are in flight together while ranking, and staged
// keys a thread reads per batch of the write-out.
#ifndef ILGPU_HIP_SORT_RANK_GROUP
#define ILGPU_HIP_SORT_RANK_GROUP 6
#endif
#ifndef ILGPU_HIP_SORT_PAIR_RANK_GROUP
#define ILGPU_HIP_SORT_PAIR_RANK_GROUP 2
#endif
#ifndef ILGPU_HIP_SORT_PAIR_WRITE_GROUP
#define ILGPU_HIP_SORT_PAIR_WRITE_GROUP 4
#endif
// Tiles are handed out in chunks of consecutive tiles, one chunk at a time to
// each of kTicketGroups groups of blocks (block b is in group b % 8: blocks are
// dispatched round-robin over the eight XCDs, so a group is the blocks of one
// XCD).  Neighbouring tiles write neighbouring runs; when they run on one XCD
// the partially written lines between their runs merge in that XCD's L2.
#ifndef ILGPU_HIP_SORT_MAX_CHUNK_SHIFT
#define ILGPU_HIP_SORT_MAX_CHUNK_SHIFT 3
#endif
constexpr int kTicketGroups = 8;
constexpr int kTicketStride = 32;          // words: one 128-byte line per group
constexpr int kMaxChunkShift = ILGPU_HIP_SORT_MAX_CHUNK_SHIFT;
// Polls of an empty status word before a look-back stops waiting for the tile
// and counts its digit itself.
constexpr uint32_t kDefaultSpinLimit = 4096;
#ifndef ILGPU_HIP_SORT_WRITE_GROUP
#define ILGPU_HIP_SORT_WRITE_GROUP 12
#endif
// Two block sizes.  Large inputs take 1024-thread blocks, one per compute unit:
// twice the tile, so every digit's run is twice as long (it is run length that
// the scattered writes pay for, pairs above all, whose tiles are short), and
// half as many tiles to chain.  Smaller inputs take 512-thread blocks, two per
// compute unit, which fill the GPU with fewer keys.
constexpr int kSortBlock = ILGPU_HIP_SORT_BLOCK;      // small inputs, and the self-test
constexpr int kSortBlockLarge = 1024;
// The large block is used from this many of its tiles per compute unit on.
// Keys without values take the pipelined pass there, measured against the
// 512-thread classic pass on u32 keys (ms per sort): 2^24.6 keys (2.7 tiles
// per CU) 0.291 / 0.277, 2^25 (3.6) 0.328 / 0.347, 2^25.6 (5.3) 0.461 / 0.480,
// 2^26 (7.1) 0.572 / 0.617, 2^27 1.040 / 1.136.  The classic 1024-thread pass
// (ILGPU_HIP_SORT_PIPELINED=0) pays from ten tiles per CU on; pairs of u64 keys
// and u32 values gain 4 to 8 % from 2^23 pairs on.
#ifndef ILGPU_HIP_SORT_PIPELINED
#define ILGPU_HIP_SORT_PIPELINED 1
#endif
constexpr int kLargeMinTilesPerCuKeys = ILGPU_HIP_SORT_PIPELINED ? 3 : 10;
constexpr int kLargeMinTilesPerCuPairs = 2;
// Lanes that rank together (a sub-tile row): one wave.
constexpr int kSubLanes = kWaveSize;
constexpr int kLookback = ILGPU_HIP_SORT_LOOKBACK;
#ifndef ILGPU_HIP_SORT_HIST_BLOCK
#define ILGPU_HIP_SORT_HIST_BLOCK 512
#endif
#ifndef ILGPU_HIP_SORT_HIST_BLOCKS_PER_CU
#define ILGPU_HIP_SORT_HIST_BLOCKS_PER_CU 2
#endif
#ifndef ILGPU_HIP_SORT_HIST_RUNS
#define ILGPU_HIP_SORT_HIST_RUNS 1
#endif
#ifndef ILGPU_HIP_SORT_HIST_NT
#define ILGPU_HIP_SORT_HIST_NT 1
#endif
#ifndef ILGPU_HIP_SORT_HIST_UNROLL
#define ILGPU_HIP_SORT_HIST_UNROLL 2
#endif
constexpr int kHistUnroll = ILGPU_HIP_SORT_HIST_UNROLL;
constexpr int kHistBlock = ILGPU_HIP_SORT_HIST_BLOCK;
#ifndef ILGPU_HIP_SORT_HIST_LDS_WORDS
#define ILGPU_HIP_SORT_HIST_LDS_WORDS 16384
#endif
constexpr int kHistLdsWords = ILGPU_HIP_SORT_HIST_LDS_WORDS;
// Look-back status word of a (tile, digit): 0 = nothing published yet;
// top bits 11 = the tile's own count in the low 30 bits (a count is at most a
// tile); anything else = inclusive count over all tiles up to this one, plus
// one.  An inclusive count is at most n <= 2^31 - 1, so count + 1 <= 2^31
// never has both top bits set and is never 0.
constexpr uint32_t kStatusAggregate = 3u << 30;
constexpr uint32_t kStatusCountMask = (1u << 30) - 1u;
__device__ __forceinline__ uint32_t status_aggregate(uint32_t count) {
  return kStatusAggregate | count;
}
__device__ __forceinline__ uint32_t status_prefix(uint32_t inclusive) { return inclusive + 1u; }
__device__ __forceinline__ bool status_is_aggregate(uint32_t w) {
  return (w & kStatusAggregate) == kStatusAggregate;
}
// Value of a non-empty word and whether it ends the look-back.
__device__ __forceinline__ uint32_t status_value(uint32_t w) {
  return status_is_aggregate(w) ? w & kStatusCountMask : w - 1u;
}
constexpr int64_t kMaxSortLength = 0x7fffffffll;  // like the reference: int.MaxValue

template <int KEY_BYTES> struct KeyOf;
template <> struct KeyOf<1> { using type = uint8_t; };
template <> struct KeyOf<2> { using type = uint16_t; };
template <> struct KeyOf<4> { using type = uint32_t; };
template <> struct KeyOf<8> { using type = uint64_t; };

struct alignas(16) Bytes16 { uint32_t x, y, z, w; };
template <int VALUE_BYTES> struct ValueOf { using type = uint8_t; };
template <> struct ValueOf<2> { using type = uint16_t; };
template <> struct ValueOf<4> { using type = uint32_t; };
template <> struct ValueOf<8> { using type = uint64_t; };
template <> struct ValueOf<16> { using type = Bytes16; };

// The value a sequencer gives element i (Sequencers.tt:25-37, Sequencer.cs:36-75):
// mode 1 = the integer sequencers and IndexSequencer, (T)i with T as wide as the
// value; mode 2 = HalfSequencer, FloatSequencer and DoubleSequencer, (T)i in
// floating point (long to float rounds to nearest even, Half goes through
// float as the C# conversion does).
template <int VALUE_BYTES>
__device__ __forceinline__ typename ValueOf<VALUE_BYTES>::type index_value(int64_t i, int mode) {
  using Val = typename ValueOf<VALUE_BYTES>::type;
  if constexpr (VALUE_BYTES == 1) {
    return (Val)(uint8_t)i;
  } else if constexpr (VALUE_BYTES == 2) {
    if (mode == 2) return (Val)__half_as_ushort(__float2half((float)i));
    return (Val)(uint16_t)i;
  } else if constexpr (VALUE_BYTES == 4) {
    if (mode == 2) return (Val)__float_as_uint((float)i);
    return (Val)(uint32_t)i;
  } else if constexpr (VALUE_BYTES == 8) {
    if (mode == 2) return (Val)(uint64_t)__double_as_longlong((double)i);
    return (Val)(uint64_t)i;
  } else {
    return Val{};  // 16-byte values are never generated (refused by the entry point)
  }
}

// Keys per thread and tile.  Long tiles pay: the runs they scatter are longer
// (fewer partial cache lines) and there are fewer tiles to chain.  Keys-only
// sorts take 36 keys of up to 4 bytes or 18 of 8 bytes per thread: the most
// that the 160 KiB of LDS of a compute unit stage for sixteen waves.  Values
// live in registers next to the keys, which caps pairs lower, by the registers
// one pair takes: at two (key and value of up to 4 bytes each) 16 items with
// 4-byte values and 20 with shorter ones, 14 at three, 10 at four, 8 with
// 16-byte values.  (Measured per pass on 2^27 pairs with 1024-thread blocks:
// u32 + u32 at 16 / 18 / 20 / 24 items 0.470 / 0.486 / 0.486 / 0.972 ms; u64 +
// u32 at 10 / 12 / 14 / 16 / 18 items 0.714 / 0.681 / 0.667 / 0.702 / 0.691;
// u64 + u64 at 10 / 12 / 14 items 0.902 / 0.919 / 0.947; u32 + u8 at 16 / 18 /
// 20 items 0.597 / 0.594 / 0.579.)
constexpr int items_per_thread(int key_bytes, int value_bytes) {
  if (value_bytes == 0) return key_bytes == 8 ? ILGPU_HIP_SORT_ITEMS8 : ILGPU_HIP_SORT_ITEMS;
  if (value_bytes == 16) return 8;
  const int registers = (key_bytes == 8 ? 2 : 1) + (value_bytes == 8 ? 2 : 1);
  if (registers == 2) return value_bytes <= 2 ? 20 : ILGPU_HIP_SORT_PAIR_ITEMS2;
  return registers == 3 ? ILGPU_HIP_SORT_PAIR_ITEMS3 : ILGPU_HIP_SORT_PAIR_ITEMS4;
}
constexpr int tile_keys(int key_bytes, int value_bytes, int block) {
  return block * items_per_thread(key_bytes, value_bytes);
}
// Short tiles.  A sort of a few hundred tiles leaves compute units idle, and
// each of its passes lasts as long as one tile takes from its first load to its
// last store.  Keys without values that fit kShortTileMaxTiles tiles of a
// shorter class (a third, a half or two thirds of the usual keys per thread)
// take the shortest class that does: every tile resident at once, in one
// round, more compute units at work and fewer rows to rank and to write per
// block.
#ifndef ILGPU_HIP_SORT_SHORT_TILE_MAX_TILES
#define ILGPU_HIP_SORT_SHORT_TILE_MAX_TILES 512
#endif
constexpr int kShortTileMaxTiles = ILGPU_HIP_SORT_SHORT_TILE_MAX_TILES;
constexpr int kShortTileClasses = 3;
constexpr int short_items_per_thread(int key_bytes, int short_class) {
  const int full = items_per_thread(key_bytes, 0);
  const int items = short_class == 0 ? full / 3 : (short_class == 1 ? full / 2 : full * 2 / 3);
  return items < 2 ? 2 : items & ~1;
}

// How raw key bits map to unsigned bits that sort in the requested order.
// ordered(k) = k ^ xor_mask ^ (lsr(~k, bits-1) & reference_term) ^ (asr(k, bits-1) & total_term):
// branch-free for every mode.  reference_term is 1 for the float order of the
// reference (RadixSortOperations.tt:81-89 as written: the complement mask is a
// LOGICAL shift of ~bits, i.e. 1 for non-negative values and 0 otherwise);
// total_term is all bits below the sign for IEEE totalOrder (negative values
// have them flipped); both are 0 for integer keys.
struct KeyXform {
  uint64_t xor_mask;
  uint64_t reference_term;
  uint64_t total_term;
};

template <typename K>
__device__ __forceinline__ K key_term(K k, const KeyXform& xf) {
  constexpr int kBits = sizeof(K) * 8;
  using S = typename std::make_signed<K>::type;
  return (K)(((K)((K)(~k) >> (kBits - 1)) & (K)xf.reference_term) ^
             ((K)((S)k >> (kBits - 1)) & (K)xf.total_term));
}

template <typename K>
__device__ __forceinline__ K ordered_bits(K k, const KeyXform& xf) {
  return (K)(k ^ (K)xf.xor_mask ^ key_term(k, xf));
}

template <typename K>
__device__ __forceinline__ uint32_t digit_of(K k, const KeyXform& xf, int shift) {
  return (uint32_t)(ordered_bits(k, xf) >> shift) & (kRadix - 1);
}

// Inverse of ordered_bits.  The per-key term depends on the key's sign bit
// only and never changes it, so u = o ^ xor_mask has the sign bit of the key
// and the same term taken from u gives the key back.
template <typename K>
__device__ __forceinline__ K raw_bits(K o, const KeyXform& xf) {
  const K u = (K)(o ^ (K)xf.xor_mask);
  return (K)(u ^ key_term(u, xf));
}

constexpr uint32_t kNoHotDigit = 0xFFFFFFFFu;
constexpr int kMaxHot = 4;
// Device-resident description of the passes, written by plan_kernel.
struct SortPlan {
  uint32_t skip[kMaxPasses];        // digit identical for all keys
  uint32_t src_is_alt[kMaxPasses];  // pass reads the alternate buffer
  // Up to kMaxHot digits that each hold an eighth of the keys or more, most
  // frequent first; unused entries are kNoHotDigit.
  uint32_t hot[kMaxPasses][kMaxHot];
  uint32_t first_executed;          // index of the first pass that runs
  uint32_t last_executed;           // index of the last pass that runs
  uint32_t executed;                // number of passes that run
  uint32_t final_in_alt;            // result sits in the alternate buffer
};

// The first active lane's key, as a wave-uniform value.
__device__ __forceinline__ uint64_t readfirstlane_key(uint64_t k) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)k);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(k >> 32));
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint32_t readfirstlane_key(uint32_t k) {
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)k);
}
__device__ __forceinline__ uint32_t readfirstlane_key(uint16_t k) {
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)k);
}
__device__ __forceinline__ uint32_t readfirstlane_key(uint8_t k) {
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)k);
}

// ---- histogram of all digit positions ------------------------------------
template <typename K, bool FLOAT_KEYS>
__global__ __launch_bounds__(kHistBlock) void sort_histogram_kernel(
    const K* __restrict__ keys, int64_t n, KeyXform xf, int passes,
    int replica_shift, uint32_t* __restrict__ global_hist) {
  using V = typename Vec16<K>::type;
  constexpr int VN = Vec16<K>::N;
  extern __shared__ uint32_t s_hist[];  // [passes][256][replicas]
  const int words = (passes * kRadix) << replica_shift;
  for (int i = threadIdx.x; i < words; i += kHistBlock) s_hist[i] = 0u;
  __syncthreads();

  const uint32_t replica = threadIdx.x & ((1u << replica_shift) - 1u);
  auto count = [&](K k) {
    K o = (K)(k ^ (K)xf.xor_mask);
    if constexpr (FLOAT_KEYS) o ^= key_term(k, xf);
#pragma unroll
    for (int p = 0; p < (int)sizeof(K); ++p) {
      const uint32_t d = (uint32_t)(o >> (8 * p)) & (kRadix - 1);
      atomicAdd(&s_hist[((p * kRadix + d) << replica_shift) + replica], 1u);
    }
    // Key by key: with the digits of all keys of a vector extracted first and
    // their atomics issued in one burst the kernel measured 4 % slower.
    __builtin_amdgcn_sched_barrier(0);
  };

  // Non-temporal loads: 0.180 against 0.217 ms for 2^28 u32 keys.  The kernel
  // is bound by the rate of LDS instructions (a wave's atomic takes the LDS of
  // a compute unit about five cycles whatever its addresses) next to the key
  // stream, and the two overlap better when the keys do not allocate in L2.
  // Two vectors per round: one is 0.235 ms, four 0.208.
  auto load_keys = [](const V* p) -> V {
    return ILGPU_HIP_SORT_HIST_NT ? __builtin_nontemporal_load(p) : *p;
  };
  // Vectors whose keys are the same in every lane of a wave, wholly or in their
  // upper half (constant input; small values under large types), would meet
  // in one counter 256 keys deep.  They are counted as runs in registers, one
  // check per vector, and reach the counters when the value changes; only
  // with all 64 lanes at work, so that the run is the same in every lane.
  // (Sorts of 2^28 u32 keys: all equal 0.269 -> 0.197 ms, Zipf values below
  // 2^16 1.174 -> 1.120, uniform 2.056 -> 2.059.)
  constexpr int kHalfBits = 4 * (int)sizeof(K);
  K run_key = 0, run_half = 0;
  uint32_t run_key_count = 0, run_half_count = 0;
  auto flush_key_run = [&]() {
    if ((threadIdx.x & (kWaveSize - 1)) == 0 && run_key_count != 0u) {
      K o = (K)(run_key ^ (K)xf.xor_mask);
      if constexpr (FLOAT_KEYS) o ^= key_term(run_key, xf);
#pragma unroll
      for (int p = 0; p < (int)sizeof(K); ++p)
        atomicAdd(&s_hist[((p * kRadix + ((uint32_t)(o >> (8 * p)) & (kRadix - 1))) << replica_shift) + replica],
                  run_key_count);
    }
    run_key_count = 0u;
  };
  auto flush_half_run = [&]() {  // run_half: ordered bits above the lower half
    if constexpr (sizeof(K) >= 2) {  // a 1-byte key has no upper half of whole digits
      if ((threadIdx.x & (kWaveSize - 1)) == 0 && run_half_count != 0u) {
#pragma unroll
        for (int p = (int)sizeof(K) / 2; p < (int)sizeof(K); ++p)
          atomicAdd(&s_hist[((p * kRadix + ((uint32_t)(run_half >> (8 * p - kHalfBits)) & (kRadix - 1))) << replica_shift) + replica],
                    run_half_count);
      }
    }
    run_half_count = 0u;
  };
  // Whether a vector's keys agree in every lane of the (full) wave: wholly
  // (returns 2), in their upper half (1), or not (0).
  auto uniformity = [&](const V& v, K& first) -> int {
    K diff = 0;
#pragma unroll
    for (int k = 1; k < VN; ++k) diff |= (K)(v[k] ^ v[0]);
    first = (K)readfirstlane_key(v[0]);
    diff |= (K)(v[0] ^ first);
    if (__ballot(true) != ~0ull) return 0;
    if (__ballot(diff != 0) == 0ull) return 2;
    if (FLOAT_KEYS) return 0;  // the upper half of their ordered bits depends on the sign
    return __ballot((K)(diff >> kHalfBits) != 0) == 0ull ? 1 : 0;
  };
  auto count_vector = [&](auto checked, const V& v) {
    if constexpr (decltype(checked)::value) {
      K first;
      const int same = uniformity(v, first);
      if (same == 2) {
        if (first != run_key) { flush_key_run(); run_key = first; }
        run_key_count += (uint32_t)(kWaveSize * VN);
        return;
      }
      if (same == 1) {
        const K half = (K)((K)(first ^ (K)xf.xor_mask) >> kHalfBits);
        if (half != run_half) { flush_half_run(); run_half = half; }
        run_half_count += (uint32_t)(kWaveSize * VN);
#pragma unroll
        for (int k = 0; k < VN; ++k) {
          const K o = (K)(v[k] ^ (K)xf.xor_mask);
#pragma unroll
          for (int p = 0; p < (int)sizeof(K) / 2; ++p)
            atomicAdd(&s_hist[((p * kRadix + ((uint32_t)(o >> (8 * p)) & (kRadix - 1))) << replica_shift) + replica], 1u);
          __builtin_amdgcn_sched_barrier(0);
        }
        return;
      }
    }
#pragma unroll
    for (int k = 0; k < VN; ++k) count(v[k]);
  };
  const uintptr_t addr = reinterpret_cast<uintptr_t>(keys);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(K));
  if (head > n) head = n;
  const V* body = reinterpret_cast<const V*>(keys + head);
  const int64_t nvec = (n - head) / VN;
  const int64_t tail_start = head + nvec * VN;
  const int64_t stride = (int64_t)gridDim.x * kHistBlock;
  // The first round's vectors are requested, and by the first of them a wave
  // decides whether it looks for runs at all: the check costs keys that vary
  // 1 to 2 % of a sort when every vector pays it.
  int64_t i = (int64_t)blockIdx.x * kHistBlock + threadIdx.x;
  V v0[kHistUnroll];
  const bool have_first = i + (kHistUnroll - 1) * stride < nvec;
  if (have_first) {
#pragma unroll
    for (int u = 0; u < kHistUnroll; ++u) v0[u] = load_keys(&body[i + u * stride]);
  }
  bool look_for_runs = false;
  if (ILGPU_HIP_SORT_HIST_RUNS && sizeof(K) >= 2 && have_first) {
    K first;
    look_for_runs = uniformity(v0[0], first) != 0;
  }
  auto count_body = [&](auto checked) {
    if (have_first) {
#pragma unroll
      for (int u = 0; u < kHistUnroll; ++u) count_vector(checked, v0[u]);
      i += kHistUnroll * stride;
    }
    for (; i + (kHistUnroll - 1) * stride < nvec; i += kHistUnroll * stride) {
      V v[kHistUnroll];
#pragma unroll
      for (int u = 0; u < kHistUnroll; ++u) v[u] = load_keys(&body[i + u * stride]);
#pragma unroll
      for (int u = 0; u < kHistUnroll; ++u) count_vector(checked, v[u]);
    }
    for (; i < nvec; i += stride) {
      V a = load_keys(&body[i]);
      count_vector(checked, a);
    }
  };
  if (look_for_runs) count_body(std::true_type{});
  else count_body(std::false_type{});
  if (blockIdx.x == 0) {
    const int64_t extra = head + (n - tail_start);
    if ((int64_t)threadIdx.x < extra) {
      const int64_t idx = (int64_t)threadIdx.x < head
                              ? (int64_t)threadIdx.x
                              : tail_start + ((int64_t)threadIdx.x - head);
      count(keys[idx]);
    }
  }
  flush_key_run();
  flush_half_run();
  __syncthreads();

  const int replicas = 1 << replica_shift;
  for (int b = threadIdx.x; b < passes * kRadix; b += kHistBlock) {
    uint32_t c = 0;
    for (int r = 0; r < replicas; ++r)
      c += s_hist[(b << replica_shift) + ((r + b) & (replicas - 1))];
    if (c != 0) atomicAdd(&global_hist[b], c);
  }
}

// ---- plan: exclusive digit offsets, skipped passes, buffer parity ---------
__global__ __launch_bounds__(kRadix) void plan_kernel(
    const uint32_t* __restrict__ global_hist, uint32_t* __restrict__ excl,
    SortPlan* __restrict__ plan, int passes, uint32_t n) {
  __shared__ uint32_t s_wave[kRadix / kWaveSize];
  __shared__ int s_trivial;
  __shared__ unsigned long long s_hot[kMaxHot];  // count << 8 | digit, most frequent first
  const int d = threadIdx.x;
  const int lane = d & (kWaveSize - 1);
  const int wave = d / kWaveSize;
  uint32_t parity = 0, executed = 0, first = passes, last = passes;
  // The counts of every pass in one round trip (the loop below is a chain of
  // barriers that a load inside it would wait behind, pass after pass).
  uint32_t counts[kMaxPasses];
#pragma unroll
  for (int p = 0; p < kMaxPasses; ++p) counts[p] = p < passes ? global_hist[p * kRadix + d] : 0u;
#pragma unroll
  for (int p = 0; p < kMaxPasses; ++p) {
    if (p >= passes) break;
    if (d < kMaxHot) s_hot[d] = 0ull;
    if (d == 0) s_trivial = 0;
    __syncthreads();
    const uint32_t c = counts[p];
    if (c == n) s_trivial = 1;
    // A digit qualifies with an eighth of the keys (two lanes of a
    // sub-tile row on average); kMaxHot rounds of "largest below the previous
    // one" order the most frequent ones.
    const unsigned long long mine = ((unsigned long long)c << 8) | (unsigned long long)d;
    const bool frequent = (uint64_t)c * 8 >= (uint64_t)n;
    for (int h = 0; h < kMaxHot; ++h) {
      if (frequent && (h == 0 || mine < s_hot[h - 1])) atomicMax(&s_hot[h], mine);
      __syncthreads();
    }
    uint32_t inc = c;
#pragma unroll
    for (int s = 1; s < kWaveSize; s <<= 1) {
      const uint32_t o = shfl_up(inc, s);
      if (lane >= s) inc += o;
    }
    if (lane == kWaveSize - 1) s_wave[wave] = inc;
    __syncthreads();
    uint32_t off = 0;
    for (int w = 0; w < wave; ++w) off += s_wave[w];
    excl[p * kRadix + d] = off + inc - c;
    const bool trivial = s_trivial != 0;
    if (d == 0) {
      plan->skip[p] = trivial ? 1u : 0u;
      plan->src_is_alt[p] = parity;
      for (int h = 0; h < kMaxHot; ++h)
        plan->hot[p][h] = s_hot[h] != 0ull ? (uint32_t)(s_hot[h] & 0xFFull) : kNoHotDigit;
    }
    if (!trivial) {
      if (executed == 0) first = p;
      last = p;
      parity ^= 1u;
      ++executed;
    }
    __syncthreads();
  }
  if (d == 0) {
    plan->first_executed = first;
    plan->last_executed = last;
    plan->executed = executed;
    plan->final_in_alt = parity;
  }
}

// ---- onesweep pass ---------------------------------------------------------
// Ranking.  A block's tile is cut into sub-tiles, one per wave; lane l of wave
// w holds items w*64*kItems + j*64 + l, j = 0 .. kItems-1, so memory order
// inside a sub-tile is (row j, lane) and a row is one 256-byte load.  Every
// (wave, digit) pair owns one 32-bit LDS counter.  For row j every lane adds
// one to the counter of its digit with a returning LDS atomic; the value that
// comes back is the key's rank among the keys of that digit in the sub-tile.
//
// That the rank follows memory order rests on two properties of the LDS:
// instructions of one wave execute in issue order (rows chain through the
// counters without barriers), and the lanes of ONE atomic instruction that
// meet in one address are served in ascending lane order.  The second is a
// property of this hardware (gfx950), not of the programming model; it is
// checked on the device by ilgpu_hip_selftest_lds_atomic_order and, end to
// end, by every stability test of the pair sorts.  With it the pass is stable
// at one LDS operation per key and no cross-lane arithmetic.
template <int KEY_BYTES, int VALUE_BYTES, int BLOCK,
          int ITEMS = items_per_thread(KEY_BYTES, VALUE_BYTES)>
struct SortTile {
  static constexpr int kSubTiles = BLOCK / kSubLanes;
  static constexpr int kCounterWords = kSubTiles * kRadix;
  static constexpr int kCounterBytes = kCounterWords * 4;
  static constexpr int kItems = ITEMS;
  static constexpr int kTile = BLOCK * ITEMS;
  static constexpr int kSubTileKeys = kSubLanes * kItems;
  static constexpr int kKeyStageBytes = kTile * KEY_BYTES;
  // The values of a tile go through the same LDS bytes after the keys, all at
  // once when they fit (72 KiB per 512 threads: two such blocks or one of 1024
  // threads share a compute unit's LDS), else in rounds.
#ifndef ILGPU_HIP_SORT_VALUE_STAGE
#define ILGPU_HIP_SORT_VALUE_STAGE 1
#endif
  static constexpr int kValueStageLimit = ILGPU_HIP_SORT_VALUE_STAGE ? (BLOCK / 512) * 72 * 1024 : 0;
  static constexpr int kValueStageBytes =
      kTile * VALUE_BYTES <= kValueStageLimit ? kTile * VALUE_BYTES : 0;
  static constexpr int kKeyOrCounterBytes =
      kCounterBytes > kKeyStageBytes ? kCounterBytes : kKeyStageBytes;
  static constexpr int kStageBytes =
      kValueStageBytes > kKeyOrCounterBytes ? kValueStageBytes : kKeyOrCounterBytes;
};

// Cache policy of a pass's key loads and scattered stores.  Measured on 2^28
// u32 keys, ms per pass: plain / plain 0.477, non-temporal loads 0.486,
// non-temporal stores 0.658 (the scattered stores rely on L2 to merge the
// pieces of a line that different waves write).
#ifndef ILGPU_HIP_SORT_NT_LOAD
#define ILGPU_HIP_SORT_NT_LOAD 0
#endif
// Rows of a tile whose loads the pipelined pass issues before it starts to
// rank; the loads of the other rows follow one rank group at a time, so that
// a wave never has more than this many loads in flight (more than about 24
// stall a wave on an idle device).  Under load the effect is small: 2.045 ms
// per sort of 2^28 u32 keys with 24 against 2.053 with all 36 up front.
#ifndef ILGPU_HIP_SORT_LOAD_AHEAD
#define ILGPU_HIP_SORT_LOAD_AHEAD 24
#endif
#ifndef ILGPU_HIP_SORT_NT_STORE
#define ILGPU_HIP_SORT_NT_STORE 0
#endif
template <int KEY_BYTES, int ITEMS, bool FULL>
__device__ __forceinline__ void load_tile_keys(
    const typename KeyOf<KEY_BYTES>::type* __restrict__ src, int64_t tile_base,
    int valid, int first_local,
    typename KeyOf<KEY_BYTES>::type (&key)[ITEMS]) {
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int local = first_local + j * kSubLanes;
    if (FULL || local < valid)
      key[j] = ILGPU_HIP_SORT_NT_LOAD ? __builtin_nontemporal_load(&src[tile_base + local])
                                      : src[tile_base + local];
    else key[j] = 0;
  }
}

// Waves per SIMD the pass kernel is compiled for: sixteen waves per CU, as two
// 512-thread blocks or one 1024-thread block.  That bounds a thread at 128
// registers (36 keys and 18 registers of packed ranks in a keys-only sort;
// fewer items when values ride along) and the blocks of a CU at 160 KiB of
// LDS together (a 36-key tile stages 72 KiB per 512 threads).
#ifndef ILGPU_HIP_SORT_WAVES_PER_EU
#define ILGPU_HIP_SORT_WAVES_PER_EU 4
#endif

// Tile of a group's k-th draw: its chunks are g, g + 8, g + 16, ... of
// 2^chunk_shift consecutive tiles.
__device__ __forceinline__ int ticket_tile(uint32_t k, uint32_t g, uint32_t groups, int chunk_shift) {
  const uint32_t chunk = (k >> chunk_shift) * groups + g;
  return (int)((chunk << chunk_shift) + (k & ((1u << chunk_shift) - 1u)));
}

// Sorts one tile by the digit of `pass` and scatters it.
template <int KEY_BYTES, int VALUE_BYTES, bool FLOAT_KEYS, bool FULL, bool HOT, int BLOCK, int ITEMS>
__device__ __forceinline__ void sort_tile(
    typename KeyOf<KEY_BYTES>::type (&key)[ITEMS],
    const typename KeyOf<KEY_BYTES>::type* __restrict__ src_keys,
    typename KeyOf<KEY_BYTES>::type* __restrict__ dst_keys,
    const typename ValueOf<VALUE_BYTES>::type* __restrict__ src_vals,
    typename ValueOf<VALUE_BYTES>::type* __restrict__ dst_vals,
    int64_t tile_base, int valid, int tile, int pass, const KeyXform& xf,
    const uint32_t* __restrict__ excl, uint32_t* status, int make_index,
    unsigned char* s_stage, uint32_t* s_global_off, uint32_t* s_scan,
    const uint32_t (&hot)[kMaxHot], uint32_t spin_limit, bool in_raw, bool out_raw) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Val = typename ValueOf<VALUE_BYTES>::type;
  using TileCfg = SortTile<KEY_BYTES, VALUE_BYTES, BLOCK, ITEMS>;
  constexpr int kItems = TileCfg::kItems;
  constexpr int kSubTiles = TileCfg::kSubTiles;
  constexpr bool kPairs = VALUE_BYTES > 0;
  constexpr int kValuesPerRound =
      kPairs ? TileCfg::kStageBytes / (VALUE_BYTES > 0 ? VALUE_BYTES : 1) : 1;
  constexpr int kRounds =
      kPairs ? (TileCfg::kTile + kValuesPerRound - 1) / kValuesPerRound : 0;
  static_assert(kItems % 2 == 0 && TileCfg::kTile <= 65536,
                "ranks and tile positions are packed two to a register");
  static_assert(kItems * kSubLanes < 65536, "a sub-tile's digit count fits 16 bits");

  // Counter of (sub-tile, digit): keys of that digit in the rows ranked so far.
  uint32_t* s_counter = reinterpret_cast<uint32_t*>(s_stage);
  K* s_keys = reinterpret_cast<K*>(s_stage);
  Val* s_vals = reinterpret_cast<Val*>(s_stage);

  // The thread index is made opaque per tile (and again for the write-out):
  // otherwise every per-item index derived from it is hoisted out of the
  // tile loop and held in a register of its own, dozens of them.
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & (kWaveSize - 1);
  const int wave = tid / kWaveSize;
  const int sub = wave;                     // sub-tile index in the block
  const int first_local = sub * TileCfg::kSubTileKeys + lane;
  const int shift = pass * 8;


  // Float keys travel between the passes in their ordered form: the first
  // pass that runs converts them as it ranks them (in_raw), the last one
  // converts them back as it writes them (out_raw), and in between a digit is
  // a shift and a mask.  Other keys keep their bits; their order is one xor.
  // (A pass that finds them converted applies the identity: no mask, no term.)
  KeyXform xf_in = xf;
  if (!in_raw) xf_in = KeyXform{0, 0, 0};
  auto digit = [&](K k) -> uint32_t {
    if constexpr (FLOAT_KEYS) return (uint32_t)(k >> shift) & (kRadix - 1);
    else return (uint32_t)((K)(k ^ (K)xf.xor_mask) >> shift) & (kRadix - 1);
  };
  // Keys past the end of the input take digit 255; they come last in memory
  // order, so they rank behind every real key and are dropped on write-out.
  auto item_digit = [&](int j) -> uint32_t {
    return (FULL || first_local + j * kSubLanes < valid) ? digit(key[j])
                                                          : (uint32_t)(kRadix - 1);
  };

  Val val[kPairs ? kItems : 1];
  if constexpr (kPairs) {
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const int local = first_local + j * kSubLanes;
      if (FULL || local < valid) {
        if (make_index) {
          val[j] = index_value<VALUE_BYTES>(tile_base + local, make_index);
        } else {
          val[j] = src_vals[tile_base + local];
        }
      }
    }
  }

  // Rank inside the sub-tile, later position inside the tile: 16 bits each.
  uint32_t* my_counters = s_counter + sub * kRadix;
  uint32_t packed[kItems / 2];
  // HOT: some digits hold a large share of the keys each (known from the
  // global histogram).  Their keys would all meet in one counter, and LDS
  // serialises the atomics of a wave to one address; they are ranked by one
  // ballot per such digit instead and only the other keys go through the
  // counters.
  uint32_t hot_count[kMaxHot] = {};  // keys of each hot digit in this sub-tile so far
  // Rows are ranked in groups: the LDS operations of a group are issued back
  // to back and their results consumed together, so a wave waits for one LDS
  // round trip per group, not per row.
  // (Pairs hold their values in registers too and take smaller groups.)
  constexpr int kGroup = kPairs ? ILGPU_HIP_SORT_PAIR_RANK_GROUP : ILGPU_HIP_SORT_RANK_GROUP;
  static_assert(kGroup % 2 == 0, "ranks are packed in pairs");
#pragma unroll
  for (int j0 = 0; j0 < kItems; j0 += kGroup) {
    uint32_t fetched[kGroup];   // what the LDS returned for the row
    uint32_t offset[kGroup];    // added to it: lane index of a one-digit row
    bool broadcast[kGroup];     // wave-uniform: take lane 0's result
#pragma unroll
    for (int g = 0; g < kGroup; ++g) {
      const int j = j0 + g;
      if (j >= kItems) break;
      const uint32_t d = item_digit(j);
      fetched[g] = 0;
      offset[g] = 0;
      broadcast[g] = false;
      bool through_counter = true;
      if constexpr (HOT) {
#pragma unroll
        for (int h = 0; h < kMaxHot; ++h) {
          if (hot[h] == kNoHotDigit) continue;  // wave-uniform
          const bool is_hot = d == hot[h];
          const uint64_t hot_lanes = __ballot(is_hot);
          if (is_hot) {
            offset[g] = hot_count[h] + (uint32_t)mbcnt(hot_lanes);
            through_counter = false;
          }
          hot_count[h] += (uint32_t)__popcll(hot_lanes);
        }
      } else {
        // Keys that arrive in runs put one digit into whole rows of a
        // sub-tile; the 64 atomics of such a row would meet in one word and
        // serialise.  In a row that is all one digit only lane 0 adds (the
        // whole row at once) and the others take its result plus their lane
        // index.  Passes with dominant digits leave the check out: the
        // ballots above already took their frequent digits.
        const uint32_t row_digit = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
        broadcast[g] = __ballot(d == row_digit) == ~0ull;
        if (broadcast[g]) {
          offset[g] = (uint32_t)lane;
          through_counter = lane == 0;
        }
      }
      if (through_counter)
        fetched[g] = __hip_atomic_fetch_add(my_counters + d,
                                            broadcast[g] ? (uint32_t)kSubLanes : 1u,
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
#pragma unroll
    for (int g = 0; g < kGroup; ++g) {
      const int j = j0 + g;
      if (j >= kItems) break;
      uint32_t rank = fetched[g];
      if constexpr (!HOT) {
        if (broadcast[g]) rank = (uint32_t)__builtin_amdgcn_readfirstlane((int)rank);
      }
      rank += offset[g];
      if (j % 2 == 0) packed[j / 2] = rank;
      else packed[j / 2] |= rank << 16;
    }
    // Pin the packed ranks here: left alone, the compiler sinks the rank
    // arithmetic of all rows to where the ranks are used and keeps two live
    // registers per key until then.
#pragma unroll
    for (int g = 0; g < kGroup; g += 2)
      if (j0 + g < kItems) asm volatile("" : "+v"(packed[(j0 + g) / 2]));
  }
  if constexpr (HOT) {
#pragma unroll
    for (int h = 0; h < kMaxHot; ++h)  // these counters are untouched so far: still zero
      if (hot[h] != kNoHotDigit && lane == 0) my_counters[hot[h]] = hot_count[h];
  }
  __syncthreads();

  // One thread per digit: totals over the sub-tiles, look-back over the tiles.
  uint32_t count = 0, inc = 0;
  uint32_t* tile_status = status + (int64_t)tile * kRadix;
  if (tid < kRadix) {
#pragma unroll
    for (int s = 0; s < kSubTiles; ++s) count += s_counter[s * kRadix + tid];
    __hip_atomic_store(&tile_status[tid],
                       tile == 0 ? status_prefix(count) : status_aggregate(count),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    inc = count;
#pragma unroll
    for (int s = 1; s < kWaveSize; s <<= 1) {
      const uint32_t o = shfl_up(inc, s);
      if (lane >= s) inc += o;
    }
    if (lane == kWaveSize - 1) s_scan[wave] = inc;
  }
  __syncthreads();
  // Digit threads: run starts, and the first step of the look-back is put in
  // flight; it is consumed after the keys are staged, so its round trip
  // overlaps the position and staging work of the whole block.
  uint32_t digit_start = 0;
  uint32_t first_step[kLookback];
  if (tid < kRadix) {
    digit_start = inc - count;
    for (int w = 0; w < wave; ++w) digit_start += s_scan[w];
    // Tile-local position of the first key of every (sub-tile, digit) run.
    {
      uint32_t run = digit_start;
#pragma unroll
      for (int s = 0; s < kSubTiles; ++s) {
        const uint32_t t = s_counter[s * kRadix + tid];
        s_counter[s * kRadix + tid] = run;
        run += t;
      }
    }
#pragma unroll
    for (int u = 0; u < kLookback; ++u) {
      const int idx = tile - 1 - u < 0 ? 0 : tile - 1 - u;
      first_step[u] = __hip_atomic_load(&status[(int64_t)idx * kRadix + tid],
                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __syncthreads();

  // Tile-local position of every key; afterwards the counters are dead and
  // the same LDS bytes stage the keys in digit order.
#pragma unroll
  for (int j = 0; j < kItems; j += 2) {
    const uint32_t p0 = my_counters[item_digit(j)] + (packed[j / 2] & 0xFFFFu);
    const uint32_t p1 = my_counters[item_digit(j + 1)] + (packed[j / 2] >> 16);
    packed[j / 2] = p0 | (p1 << 16);
    if (j % 8 == 6) __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kItems; ++j)
    s_keys[j % 2 == 0 ? packed[j / 2] & 0xFFFFu : packed[j / 2] >> 16] = key[j];

  if (tid < kRadix) {
    // Keys with this digit in earlier tiles: walk back over the status words,
    // kLookback tiles per step.  The loads of a step are unconditional (index
    // clamped) so that they are in flight together; positions in front of
    // tile 0 read as an empty inclusive prefix.
    uint32_t before = 0;
    bool done = tile == 0;
    bool preloaded = true;
    for (int t = tile - 1; !done; t -= kLookback) {
      uint32_t s[kLookback];
#pragma unroll
      for (int u = 0; u < kLookback; ++u) {
        if (preloaded) {
          s[u] = first_step[u];
        } else {
          const int idx = t - u < 0 ? 0 : t - u;
          s[u] = __hip_atomic_load(&status[(int64_t)idx * kRadix + tid],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      preloaded = false;
#pragma unroll
      for (int u = 0; u < kLookback; ++u)
        if (t - u < 0) s[u] = status_prefix(0u);
#pragma unroll
      for (int u = 0; u < kLookback; ++u) {
        if (done) continue;
        uint32_t polls = 0;
        while (s[u] == 0u) {
          if (polls++ >= spin_limit) {
            // Nobody has published tile t - u: its owner may not be running.
            // Count this thread's digit in that tile from the source keys (a
            // full tile: it precedes this one) and go on as if the tile had
            // published its own count.  Slow, and never needed while every
            // group of blocks is resident.
            const K* other = src_keys + (int64_t)(t - u) * TileCfg::kTile;
            uint32_t c = 0;
#pragma unroll 4
            for (int i = 0; i < TileCfg::kTile; ++i) {
              K k = other[i];
              if constexpr (FLOAT_KEYS) k = ordered_bits(k, xf_in);
              c += digit(k) == (uint32_t)tid;
            }
            s[u] = status_aggregate(c);
            break;
          }
          __builtin_amdgcn_s_sleep(1);
          s[u] = __hip_atomic_load(&status[(int64_t)(t - u) * kRadix + tid],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        before += status_value(s[u]);
        done = !status_is_aggregate(s[u]);
      }
    }
    if (tile > 0)
      __hip_atomic_store(&tile_status[tid], status_prefix(before + count),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_global_off[tid] = excl[pass * kRadix + tid] + before - digit_start;
  }
  __syncthreads();

  uint32_t gpos[kPairs ? kItems : 1];
  asm volatile("" : "+v"(tid));
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const int i = j * BLOCK + tid;
    if (FULL || i < valid) {
      const K k = s_keys[i];
      const uint32_t g = s_global_off[digit(k)] + (uint32_t)i;
      if constexpr (FLOAT_KEYS) dst_keys[g] = out_raw ? raw_bits(k, xf) : k;
      else dst_keys[g] = k;
      if constexpr (kPairs) gpos[j] = g;
    }
    constexpr int kWriteGroup = kPairs ? ILGPU_HIP_SORT_PAIR_WRITE_GROUP : ILGPU_HIP_SORT_WRITE_GROUP;
    if (j % kWriteGroup == kWriteGroup - 1) __builtin_amdgcn_sched_barrier(0);
  }

  if constexpr (kPairs) {
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
      const uint32_t lo = (uint32_t)r * kValuesPerRound;
      __syncthreads();  // the stage buffer is free again
#pragma unroll
      for (int j = 0; j < kItems; ++j) {
        const uint32_t pos = j % 2 == 0 ? packed[j / 2] & 0xFFFFu : packed[j / 2] >> 16;
        if (pos - lo < (uint32_t)kValuesPerRound) s_vals[pos - lo] = val[j];
      }
      __syncthreads();
#pragma unroll
      for (int j = 0; j < kItems; ++j) {
        const uint32_t i = (uint32_t)(j * BLOCK + tid);
        if ((FULL || i < (uint32_t)valid) && i - lo < (uint32_t)kValuesPerRound)
          dst_vals[gpos[j]] = s_vals[i - lo];
      }
    }
  }
}

template <int KEY_BYTES, int VALUE_BYTES, bool FLOAT_KEYS, int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK, ILGPU_HIP_SORT_WAVES_PER_EU)
void onesweep_kernel(
    typename KeyOf<KEY_BYTES>::type* keys_a,
    typename KeyOf<KEY_BYTES>::type* keys_b,
    typename ValueOf<VALUE_BYTES>::type* vals_a,
    typename ValueOf<VALUE_BYTES>::type* vals_b, int64_t n, int pass,
    KeyXform xf, const uint32_t* __restrict__ excl, uint32_t* status,
    uint32_t* ticket, const SortPlan* __restrict__ plan, int num_tiles,
    int values_from_index, int groups, int chunk_shift, uint32_t spin_limit) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Val = typename ValueOf<VALUE_BYTES>::type;
  using TileCfg = SortTile<KEY_BYTES, VALUE_BYTES, BLOCK, ITEMS>;
  constexpr int kTile = TileCfg::kTile;
  constexpr int kItems = TileCfg::kItems;

  __shared__ __attribute__((aligned(16))) unsigned char s_stage[TileCfg::kStageBytes];
  __shared__ uint32_t s_global_off[kRadix];
  __shared__ uint32_t s_scan[kRadix / kWaveSize];
  __shared__ int s_tile;

  if (plan->skip[pass]) return;
  const bool src_alt = plan->src_is_alt[pass] != 0;
  uint32_t hot[kMaxHot];
#pragma unroll
  for (int h = 0; h < kMaxHot; ++h) hot[h] = plan->hot[pass][h];
  const K* src_keys = src_alt ? keys_b : keys_a;
  K* dst_keys = src_alt ? keys_a : keys_b;
  const Val* src_vals = src_alt ? vals_b : vals_a;
  Val* dst_vals = src_alt ? vals_a : vals_b;
  // 0, or the kind of index values the first pass that runs generates
  const int make_index =
      VALUE_BYTES > 0 && plan->first_executed == (uint32_t)pass ? values_from_index : 0;
  const bool in_raw = plan->first_executed == (uint32_t)pass;
  const bool out_raw = plan->last_executed == (uint32_t)pass;
  const int tid = threadIdx.x;
  const int first_local = (tid / kSubLanes) * TileCfg::kSubTileKeys + tid % kSubLanes;

  auto valid_keys = [&](int t) -> int {
    const int64_t remaining = n - (int64_t)t * kTile;
    return remaining >= kTile ? kTile : (remaining > 0 ? (int)remaining : 0);
  };

  // Tickets: group g (= blockIdx % 8) owns the chunks g, g + 8, g + 16, ... of
  // 2^chunk_shift consecutive tiles and draws their tiles in order from its
  // own counter.  Unlike a single counter this does not start tiles in index
  // order across groups: a tile can find that a predecessor owned by another
  // group has not been started, and if that group had no resident block it
  // would wait for ever.  The look-back therefore never waits without bound:
  // after spin_limit polls of an empty word it counts the tile's digit itself
  // (sort_tile), so every block finishes whatever the other blocks do.
  // A block draws its next tile only when it is about to start it: the time
  // between a tile's ticket and the publication of its digit counts is what
  // every later tile's look-back waits for.  (Drawing it earlier, to load the
  // next keys during the look-back and the write-out, measured 3 to 12 % slower,
  // with the global ticket and again with the per-group ones.)  The key loads
  // fly while the ranking counters are cleared.
  // A grid of as many blocks as there are tiles (a short input) needs no
  // tickets (ticket == nullptr): block b takes tile b and is done, which saves
  // a pass two round trips to the ticket, one of them only to learn that
  // there is nothing left.  Blocks start in index order in practice, so a
  // tile's predecessors are running; where they are not, the bounded look-back
  // covers that as it does with tickets.
  for (int round = 0;; ++round) {
    int tile;
    if (ticket == nullptr) {
      if (round > 0) break;
      tile = (int)blockIdx.x;
    } else {
      if (tid == 0) {
        const uint32_t g = blockIdx.x % (uint32_t)groups;
        s_tile = ticket_tile(atomicAdd(ticket + g * kTicketStride, 1u), g, (uint32_t)groups, chunk_shift);
      }
      __syncthreads();  // also: the previous tile's staged keys have been read
      tile = s_tile;
    }
    if (tile >= num_tiles) break;
    const int64_t tile_base = (int64_t)tile * kTile;
    const int valid = valid_keys(tile);
    // Three instantiations of the tile code: full tiles with and without
    // dominant digits, and the tail tile (bounds-checked; the dominant-digit
    // form serves it either way: without such digits every key goes through
    // the counters).  Each loads its keys itself, so that the loads, the
    // clearing of the counters and the ranking are one straight line and the
    // rows are ranked as their keys arrive.
    auto run = [&](auto full, auto with_hot) {
      constexpr bool kFull = decltype(full)::value;
      constexpr bool kHot = decltype(with_hot)::value;
      K key[kItems];
      load_tile_keys<KEY_BYTES, kItems, kFull>(src_keys, tile_base, valid, first_local, key);
      if constexpr (FLOAT_KEYS) {
        if (in_raw) {
#pragma unroll
          for (int j = 0; j < kItems; ++j) key[j] = ordered_bits(key[j], xf);
        }
      }
      {  // clear the ranking counters
        uint4* z = reinterpret_cast<uint4*>(s_stage);
        for (int i = tid; i < TileCfg::kCounterBytes / 16; i += BLOCK)
          z[i] = make_uint4(0u, 0u, 0u, 0u);
      }
      __syncthreads();
      sort_tile<KEY_BYTES, VALUE_BYTES, FLOAT_KEYS, kFull, kHot, BLOCK, ITEMS>(
          key, src_keys, dst_keys, src_vals, dst_vals, tile_base, valid, tile, pass, xf, excl,
          status, make_index, s_stage, s_global_off, s_scan, hot, spin_limit, in_raw, out_raw);
    };
    if (valid != kTile) run(std::false_type{}, std::true_type{});
    else if (hot[0] == kNoHotDigit) run(std::true_type{}, std::false_type{});
    else run(std::true_type{}, std::true_type{});
  }
}

// ---- onesweep pass, pipelined form (keys without values, large inputs) --------
// The pass above runs a tile's phases one after the other: while a block waits
// for its keys nothing else happens on its compute unit, and while it ranks,
// walks and stages, no load is in flight.  This form overlaps them.
//
//   * The write-out of a tile is deferred until the next tile is ranked.  Per
//     tile: positions and staging of tile T (its keys leave the registers),
//     load and ranking of the block's next tile T', digit totals of T'
//     published, T written out from LDS, and so on.  The stores of T drain
//     while T' is staged and T'' is loaded; T is resolved (the digit counts of
//     all earlier tiles) while T' is loaded and ranked.
//   * A 1024-thread block is fifteen waves that sort and one that resolves.
//     The sorting waves hold the keys (15 x 64 x kItems per tile).  The other
//     wave holds none and hands the 256 global offsets of a tile over through
//     LDS.  A wave that sorts could not do this beside its loads: vector memory
//     results return to a wave, and to a compute unit, in request order, so a
//     status word asked for behind a tile of keys arrives behind the keys.  For
//     the same reason a look-back step on a compute unit that streams keys
//     takes three times what it takes on an idle one, and a walk of the usual
//     depth (thirty tiles) would outlast the tile.
//   * So the walking is done elsewhere.  Four blocks of the grid sort nothing:
//     their compute units issue no key traffic and their memory round trips are
//     short.  Each takes 64 of the 256 digits and turns the published counts of
//     the tiles into inclusive prefixes, in tile order, a window of 64 tiles per
//     round trip.  A sorting block's sixteenth wave only polls the row of its
//     own tile until the prefixes are there.  Every status row is read by the
//     scanning blocks and by its owner, not by the thirty tiles behind it.
//     Nothing waits without bound: a wave that has polled its row often enough
//     walks back itself (pipelined_walk), and a scanning block that waits for a
//     tile nobody publishes counts that tile's digits itself.
//   * A tile's digit counts are published a fixed time after its ticket is
//     drawn (staging of the previous tile, load, ranking), whatever any other
//     block does and however long the tile before takes to be resolved: a
//     ticket commits the block to the tile, and every later tile waits for
//     those counts.  That is why the sorting waves never meet the sixteenth
//     wave inside their own steps: among themselves they synchronise through
//     counters in LDS (arrive: one add by a wave's first lane; wait: poll), and
//     the block-wide barrier is used once per tile, where the offsets of the
//     tile before are handed over.
//   * The ranking counters have LDS of their own (the tile is 1/16 shorter,
//     which frees it): a wave clears its counters itself as soon as it has read
//     its run starts, and no barrier separates positions from staging.
//
// Floating-point keys are converted by the first pass that runs and back by
// the last one (in_xf, out_xf in the kernel); pairs take the pass above.
template <int KEY_BYTES> struct PipelinedTile {
  static constexpr int kBlock = 1024;
  static constexpr int kSorterWaves = kBlock / kWaveSize - 1;
  static constexpr int kSorters = kSorterWaves * kWaveSize;
  static constexpr int kItems = items_per_thread(KEY_BYTES, 0);
  static constexpr int kSubTileKeys = kWaveSize * kItems;
  static constexpr int kTile = kSorterWaves * kSubTileKeys;
};
constexpr int pipelined_tile_keys(int key_bytes) {
  return (1024 / kWaveSize - 1) * kWaveSize * items_per_thread(key_bytes, 0);
}
#ifndef ILGPU_HIP_SORT_WALK_STEP
#define ILGPU_HIP_SORT_WALK_STEP 4
#endif
constexpr int kWalkStep = ILGPU_HIP_SORT_WALK_STEP;   // tiles per look-back step of a resolving wave that walks back itself
constexpr int kWalkDigits = kRadix / kWaveSize;       // digits per lane of a resolving wave

// Loads the calling wave's keys of one tile into `key` and ranks them on the
// wave's counters, which are zero on entry: as in sort_tile.
template <int KEY_BYTES, bool FULL, bool HOT, bool FLOAT_KEYS>
__device__ __forceinline__ void pipelined_rank(
    typename KeyOf<KEY_BYTES>::type (&key)[(items_per_thread(KEY_BYTES, 0))],
    uint32_t (&packed)[(items_per_thread(KEY_BYTES, 0)) / 2],
    const typename KeyOf<KEY_BYTES>::type* __restrict__ src_keys, int64_t tile_base, int valid,
    int shift, const KeyXform& in_xf, uint32_t* my_counters, int lane, int first_local,
    const uint32_t (&hot)[kMaxHot]) {
  using K = typename KeyOf<KEY_BYTES>::type;
  constexpr int kItems = items_per_thread(KEY_BYTES, 0);
  // Rows whose loads are issued before the ranking starts; the others follow
  // one rank group at a time.
  constexpr int kAhead = ILGPU_HIP_SORT_LOAD_AHEAD < kItems ? ILGPU_HIP_SORT_LOAD_AHEAD : kItems;
  auto load_rows = [&](int j0, int j1) {
#pragma unroll
    for (int j = j0; j < j1 && j < kItems; ++j) {
      const int local = first_local + j * kWaveSize;
      if (FULL || local < valid)
        key[j] = ILGPU_HIP_SORT_NT_LOAD ? __builtin_nontemporal_load(&src_keys[tile_base + local])
                                        : src_keys[tile_base + local];
      else key[j] = 0;
    }
  };
  load_rows(0, kAhead);
  if (kAhead < kItems) __builtin_amdgcn_sched_barrier(0);
  // Float keys leave this function in their ordered form (in_xf is the
  // identity when they arrive in it); integer keys keep their bits.
  auto item_digit = [&](int j) -> uint32_t {
    if constexpr (FLOAT_KEYS) key[j] = ordered_bits(key[j], in_xf);
    const K o = FLOAT_KEYS ? key[j] : (K)(key[j] ^ (K)in_xf.xor_mask);
    const uint32_t d = (uint32_t)(o >> shift) & (kRadix - 1);
    return (FULL || first_local + j * kWaveSize < valid) ? d : (uint32_t)(kRadix - 1);
  };
  uint32_t hot_count[kMaxHot] = {};
  constexpr int kGroup = ILGPU_HIP_SORT_RANK_GROUP;
  static_assert(kGroup % 2 == 0, "ranks are packed in pairs");
#pragma unroll
  for (int j0 = 0; j0 < kItems; j0 += kGroup) {
    uint32_t fetched[kGroup];
    uint32_t offset[kGroup];
    bool broadcast[kGroup];
    if (kAhead < kItems) {
      load_rows(kAhead + j0, kAhead + j0 + kGroup);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int g = 0; g < kGroup; ++g) {
      const int j = j0 + g;
      if (j >= kItems) break;
      const uint32_t d = item_digit(j);
      fetched[g] = 0;
      offset[g] = 0;
      broadcast[g] = false;
      bool through_counter = true;
      if constexpr (HOT) {
#pragma unroll
        for (int h = 0; h < kMaxHot; ++h) {
          if (hot[h] == kNoHotDigit) continue;  // wave-uniform
          const bool is_hot = d == hot[h];
          const uint64_t hot_lanes = __ballot(is_hot);
          if (is_hot) {
            offset[g] = hot_count[h] + (uint32_t)mbcnt(hot_lanes);
            through_counter = false;
          }
          hot_count[h] += (uint32_t)__popcll(hot_lanes);
        }
      } else {
        const uint32_t row_digit = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
        broadcast[g] = __ballot(d == row_digit) == ~0ull;
        if (broadcast[g]) {
          offset[g] = (uint32_t)lane;
          through_counter = lane == 0;
        }
      }
      if (through_counter)
        fetched[g] = __hip_atomic_fetch_add(my_counters + d,
                                            broadcast[g] ? (uint32_t)kWaveSize : 1u,
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
#pragma unroll
    for (int g = 0; g < kGroup; ++g) {
      const int j = j0 + g;
      if (j >= kItems) break;
      uint32_t rank = fetched[g];
      if constexpr (!HOT) {
        if (broadcast[g]) rank = (uint32_t)__builtin_amdgcn_readfirstlane((int)rank);
      }
      rank += offset[g];
      if (j % 2 == 0) packed[j / 2] = rank;
      else packed[j / 2] |= rank << 16;
    }
#pragma unroll
    for (int g = 0; g < kGroup; g += 2)
      if (j0 + g < kItems) asm volatile("" : "+v"(packed[(j0 + g) / 2]));
  }
  if constexpr (HOT) {
#pragma unroll
    for (int h = 0; h < kMaxHot; ++h)  // these counters are untouched so far: still zero
      if (hot[h] != kNoHotDigit && lane == 0) my_counters[hot[h]] = hot_count[h];
  }
}

// A resolving wave that walks back itself: the digit counts of all earlier tiles by
// look-back, the tile's inclusive counts published, the global offsets of its
// 256 runs into s_global_off.  Lane l owns digits 4l .. 4l+3, so a tile's
// status row is one 16-byte load per lane: the time of a look-back step grows
// with the number of load instructions in it, not with their width.
typedef uint32_t StatusVec __attribute__((ext_vector_type(4)));
constexpr int kStatusCoherent = 16;  // cache policy of the buffer operations: sc1, agent scope
__device__ __forceinline__ StatusVec load_status_row(__amdgpu_buffer_rsrc_t rsrc, int tile,
                                                      int lane) {
  return __builtin_amdgcn_raw_buffer_load_b128(rsrc, (tile * kRadix + lane * kWalkDigits) * 4, 0,
                                               kStatusCoherent);
}

template <int KEY_BYTES, bool FLOAT_KEYS>
__device__ __forceinline__ void pipelined_walk(
    const typename KeyOf<KEY_BYTES>::type* __restrict__ src_keys, int tile, int shift,
    const KeyXform& in_xf, __amdgpu_buffer_rsrc_t status,
    const uint32_t* __restrict__ excl_row, const uint32_t* s_total, const uint32_t* s_start,
    uint32_t* s_global_off, int lane, uint32_t spin_limit) {
  using K = typename KeyOf<KEY_BYTES>::type;
  constexpr int kTile = PipelinedTile<KEY_BYTES>::kTile;
  static_assert(kWalkDigits == 4, "a lane's digits are one 16-byte vector");
  auto digit = [&](K k) -> uint32_t {  // of a key as the source holds it
    const K o = FLOAT_KEYS ? ordered_bits(k, in_xf) : (K)(k ^ (K)in_xf.xor_mask);
    return (uint32_t)(o >> shift) & (kRadix - 1);
  };
  const StatusVec my_count = reinterpret_cast<const StatusVec*>(s_total)[lane];
  const StatusVec my_excl = reinterpret_cast<const StatusVec*>(excl_row)[lane];
  uint32_t before[kWalkDigits];
  bool done[kWalkDigits];
#pragma unroll
  for (int c = 0; c < kWalkDigits; ++c) {
    before[c] = 0;
    done[c] = tile == 0;
  }
  for (int t = tile - 1; t >= 0; t -= kWalkStep) {
    bool all_done = true;
#pragma unroll
    for (int c = 0; c < kWalkDigits; ++c) all_done = all_done && done[c];
    if (__all(all_done)) break;
    // The loads of a step are unconditional (index clamped) so that they are in
    // flight together; positions in front of tile 0 read as an empty prefix.
    StatusVec s[kWalkStep];
#pragma unroll
    for (int u = 0; u < kWalkStep; ++u)
      s[u] = load_status_row(status, t - u < 0 ? 0 : t - u, lane);
#pragma unroll
    for (int u = 0; u < kWalkStep; ++u) {
      if (t - u < 0) s[u] = StatusVec{status_prefix(0u), status_prefix(0u), status_prefix(0u),
                                      status_prefix(0u)};
      // Words of tile t - u that this lane still needs and that are empty:
      // the tile's row is polled until they are there, never without bound.
      uint32_t polls = 0;
      while (true) {
        bool missing = false;
#pragma unroll
        for (int c = 0; c < kWalkDigits; ++c) missing = missing || (!done[c] && s[u][c] == 0u);
        if (!__any(missing)) break;
        if (polls++ >= spin_limit) {
          // Nobody has published tile t - u: its owner may not be running.
          // Count the digits of that (full) tile from the source keys and go
          // on as if the tile had published its own counts.  Slow, and never
          // needed while every group of blocks is resident.
          const K* other = src_keys + (int64_t)(t - u) * kTile;
          uint32_t cnt[kWalkDigits] = {};
#pragma unroll 4
          for (int i = 0; i < kTile; ++i) {
            K k = other[i];
            const uint32_t d = digit(k);
#pragma unroll
            for (int c = 0; c < kWalkDigits; ++c) cnt[c] += d == (uint32_t)(lane * kWalkDigits + c);
          }
#pragma unroll
          for (int c = 0; c < kWalkDigits; ++c)
            if (s[u][c] == 0u) s[u][c] = status_aggregate(cnt[c]);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
        s[u] = load_status_row(status, t - u, lane);
      }
#pragma unroll
      for (int c = 0; c < kWalkDigits; ++c) {
        if (!done[c]) {
          before[c] += status_value(s[u][c]);
          done[c] = !status_is_aggregate(s[u][c]);
        }
      }
    }
  }
  StatusVec prefix, offset;
  const StatusVec start = reinterpret_cast<const StatusVec*>(s_start)[lane];
#pragma unroll
  for (int c = 0; c < kWalkDigits; ++c) {
    prefix[c] = status_prefix(before[c] + my_count[c]);
    offset[c] = my_excl[c] + before[c] - start[c];
  }
  if (tile > 0)
    __builtin_amdgcn_raw_buffer_store_b128(prefix, status, (tile * kRadix + lane * kWalkDigits) * 4,
                                           0, kStatusCoherent);
  reinterpret_cast<StatusVec*>(s_global_off)[lane] = offset;
}

#ifndef ILGPU_HIP_SORT_OWN_ROW_SLEEP
#define ILGPU_HIP_SORT_OWN_ROW_SLEEP 20
#endif
// Rows (tiles) a scanning block takes per round trip: four per wave, and as
// many again requested ahead.  (A wave with more than about 24 dwords per lane
// in flight stalls: measured.)
#ifndef ILGPU_HIP_SORT_SCAN_SEG_ROWS
#define ILGPU_HIP_SORT_SCAN_SEG_ROWS 4
#endif
constexpr int kScanSegRows = ILGPU_HIP_SORT_SCAN_SEG_ROWS;
constexpr int kScanSegs = 16;
constexpr int kScanWindow = kScanSegs * kScanSegRows;
constexpr int kScanBlocks = kRadix / kWaveSize;  // one scanning block per 64 digits
// Polls of its own row before a resolving wave stops waiting for the scanning
// block and walks back itself.
constexpr uint32_t kScannerPolls = 64;

// A scanning block's loop: status words of the tiles in order, counts into
// inclusive prefixes, for the 64 digits of the block (lane = digit).  Wave w
// takes the rows 4w .. 4w+3 of a window of 64 tiles: one round trip reads the
// window, the rows that are complete at its front are scanned (four rows per
// thread in registers, the sixteen waves combined through LDS) and their
// prefixes written back.  A row's word either adds its count or (tile 0, or a
// tile whose owner walked back itself) sets the running value.
// s_lds: 16 + 17 x 64 words.
template <int KEY_BYTES, bool FLOAT_KEYS>
__device__ __forceinline__ void pipelined_scan(
    const typename KeyOf<KEY_BYTES>::type* __restrict__ src_keys, int shift,
    const KeyXform& in_xf, uint32_t* status, int num_tiles, uint32_t spin_limit,
    uint32_t* s_lds) {
  using K = typename KeyOf<KEY_BYTES>::type;
  constexpr int kTile = PipelinedTile<KEY_BYTES>::kTile;
  uint32_t* s_avail = s_lds;                          // [segments]: leading complete rows of every wave's segment
  uint32_t* s_part = s_lds + kScanSegs;               // [segments][64]: what a segment's rows do to the running value
  uint32_t* s_prefix = s_part + kScanSegs * kWaveSize;  // [64]: the running inclusive counts
  static_assert(kScanSegs * kWaveSize >= kRadix, "the fallback counts 256 digit values in s_part");
  constexpr uint32_t kAbsolute = 0x80000000u; // a segment that sets the running value
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = tid / kWaveSize;
  const int quarter = blockIdx.x;  // this block's 64 digits
  const int seg = wave;            // this wave's rows of the window
  const int dgt = quarter * kWaveSize + lane;
  auto combine = [&](uint32_t running, uint32_t part) -> uint32_t {
    return (part & kAbsolute) ? (part & ~kAbsolute) : running + part;
  };
  if (seg == 0) s_prefix[lane] = 0u;
  __syncthreads();
  uint32_t polls = 0;
  int t = 0;
  uint32_t w[kScanSegRows], w_next[kScanSegRows];
  bool ahead = false;  // w already holds the window at t
  auto load_window = [&](int first_tile, uint32_t (&words)[kScanSegRows]) {
#pragma unroll
    for (int u = 0; u < kScanSegRows; ++u) {
      int row = first_tile + seg * kScanSegRows + u;
      row = row < num_tiles ? row : num_tiles - 1;
      words[u] = __hip_atomic_load(&status[(int64_t)row * kRadix + dgt], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  while (t < num_tiles) {
    const int first_row = t + seg * kScanSegRows;
    // The window was requested by the previous turn if that consumed a whole
    // window (the scan is behind and the rows are there); the next one is
    // requested before this one is worked on, so that its round trip runs
    // beside the scan and ahead of this window's stores.
    if (!ahead) load_window(t, w);
    load_window(t + kScanWindow, w_next);
    int there = 0;  // complete rows at the front of this wave's segment (wave-uniform)
    bool open = true;
#pragma unroll
    for (int u = 0; u < kScanSegRows; ++u) {
      open = open && first_row + u < num_tiles && __all(w[u] != 0u);
      there += open ? 1 : 0;
    }
    if (lane == 0) s_avail[seg] = (uint32_t)there;
    __syncthreads();
    // Complete rows at the front of the window.
    int avail = 0;
    {
      bool full = true;
#pragma unroll
      for (int g = 0; g < kScanSegs; ++g) {
        const int a = (int)s_avail[g];
        avail += full ? a : 0;
        full = full && a == kScanSegRows;
      }
    }
    int mine = avail - seg * kScanSegRows;  // rows of this segment that are consumed
    mine = mine < 0 ? 0 : (mine > kScanSegRows ? kScanSegRows : mine);
    uint32_t value = 0;
    bool absolute = false;
    uint32_t was_aggregate = 0;  // bit u: row u held a count
#pragma unroll
    for (int u = 0; u < kScanSegRows; ++u) {
      if (u < mine) {
        if (status_is_aggregate(w[u])) {
          value += w[u] & kStatusCountMask;
          was_aggregate |= 1u << u;
        } else {
          value = w[u] - 1u;
          absolute = true;
        }
      }
      // From here w[u] is the running value within the segment, and whether it
      // is already absolute rides in the top bit.
      w[u] = value | (absolute ? kAbsolute : 0u);
    }
    s_part[seg * kWaveSize + lane] = value | (absolute ? kAbsolute : 0u);
    __syncthreads();
    uint32_t running = s_prefix[lane];
    uint32_t base = running;
#pragma unroll
    for (int g = 0; g < kScanSegs; ++g) {
      const uint32_t part = s_part[g * kWaveSize + lane];
      if (g < seg) base = combine(base, part);
      running = combine(running, part);
    }
#pragma unroll
    for (int u = 0; u < kScanSegRows; ++u) {
      if (u < mine && ((was_aggregate >> u) & 1u))
        __hip_atomic_store(&status[(int64_t)(first_row + u) * kRadix + dgt],
                           status_prefix(combine(base, w[u])), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();  // the segment results and the running counts have been read
    if (seg == 0) s_prefix[lane] = running;
    t += avail;
    ahead = avail == kScanWindow;
    if (ahead) {
#pragma unroll
      for (int u = 0; u < kScanSegRows; ++u) w[u] = w_next[u];
    }
    if (avail != 0) {
      polls = 0;
    } else if (polls++ >= spin_limit) {
      // Nobody has published tile t: its owner may not be running.  Count its
      // digits from the source keys (a full tile: the last one is left to its
      // owner) and go on; the owner, if it ever runs, resolves itself.  Slow,
      // and never needed while every block is resident.
      if (t == num_tiles - 1) return;
      if (tid < kRadix) s_part[tid] = 0u;
      __syncthreads();
      const K* other = src_keys + (int64_t)t * kTile;
      for (int i = tid; i < kTile; i += kScanSegs * kWaveSize) {
        const K k = other[i];
        const K o = FLOAT_KEYS ? ordered_bits(k, in_xf) : (K)(k ^ (K)in_xf.xor_mask);
        atomicAdd(&s_part[(uint32_t)(o >> shift) & (kRadix - 1)], 1u);
      }
      __syncthreads();
      if (seg == 0) s_prefix[lane] += s_part[dgt];
      __syncthreads();
      ++t;
      polls = 0;
    } else {
      __builtin_amdgcn_s_sleep(2);
    }
  }
}

template <int KEY_BYTES, bool FLOAT_KEYS>
__global__ __launch_bounds__(1024, ILGPU_HIP_SORT_WAVES_PER_EU)
void onesweep_pipelined_kernel(
    typename KeyOf<KEY_BYTES>::type* keys_a, typename KeyOf<KEY_BYTES>::type* keys_b, int64_t n,
    int pass, KeyXform xf, const uint32_t* __restrict__ excl, uint32_t* status, uint32_t* ticket,
    const SortPlan* __restrict__ plan, int num_tiles, int groups, int chunk_shift,
    uint32_t spin_limit, int with_scanner) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Cfg = PipelinedTile<KEY_BYTES>;
  constexpr int kTile = Cfg::kTile;
  constexpr int kItems = Cfg::kItems;
  constexpr int kSorterWaves = Cfg::kSorterWaves;
  constexpr int kDigitWaves = kRadix / kWaveSize;
  constexpr int kDrawThread = kRadix;  // first lane of the first wave without digits
  static_assert(kItems % 2 == 0 && kTile <= 65536,
                "ranks and tile positions are packed two to a register");

  __shared__ __attribute__((aligned(16))) K s_keys[kTile];
  __shared__ __attribute__((aligned(16))) uint32_t s_counter[kSorterWaves * kRadix];
  // Handed between the sorting waves and the resolving wave, which runs up to a
  // tile behind: two copies each, by the parity of the block's tile count.
  __shared__ __attribute__((aligned(16))) uint32_t s_total[2][kRadix];
  __shared__ __attribute__((aligned(16))) uint32_t s_start[2][kRadix];
  __shared__ __attribute__((aligned(16))) uint32_t s_global_off[2][kRadix];
  __shared__ int s_next[2];
  __shared__ uint32_t s_scan[kDigitWaves];
  __shared__ uint32_t s_bar[4];

  if (plan->skip[pass]) return;
  const bool src_alt = plan->src_is_alt[pass] != 0;
  const K* src_keys = src_alt ? keys_b : keys_a;
  K* dst_keys = src_alt ? keys_a : keys_b;
  const int shift = pass * 8;
  const uint32_t group = blockIdx.x % (uint32_t)groups;
  uint32_t* my_ticket = ticket + group * kTicketStride;
  // Float keys travel between the passes in their ordered form: the first pass
  // that runs converts them as it ranks them, the last one converts them back
  // as it writes them, and in between a digit is a shift and a mask (in_xf and
  // out_xf are the identity then).  Integer keys keep their bits throughout;
  // their order is one xor wherever a digit is taken.
  KeyXform in_xf = xf, out_xf = xf;
  if constexpr (FLOAT_KEYS) {
    if (plan->first_executed != (uint32_t)pass) in_xf = KeyXform{0, 0, 0};
    if (plan->last_executed != (uint32_t)pass) out_xf = KeyXform{0, 0, 0};
  }

  if (with_scanner && blockIdx.x < kScanBlocks) {
    // ---- a scanning block: the prefixes of 64 digits ----
    pipelined_scan<KEY_BYTES, FLOAT_KEYS>(src_keys, shift, in_xf, status, num_tiles,
                                          spin_limit, s_counter);
    return;
  }
  if (threadIdx.x == 0)
    s_next[0] = ticket_tile(atomicAdd(my_ticket, 1u), group, (uint32_t)groups, chunk_shift);
  if (threadIdx.x < 4) s_bar[threadIdx.x] = 0u;
  for (int i = threadIdx.x; i < kSorterWaves * kRadix / 4; i += Cfg::kBlock)
    reinterpret_cast<uint4*>(s_counter)[i] = make_uint4(0u, 0u, 0u, 0u);
  __syncthreads();
  int tile = s_next[0];
  __syncthreads();  // s_next[0] is written again by the first tile
  auto is_full = [&](int t) -> bool { return n - (int64_t)t * kTile >= kTile; };

  // Synchronisation.  The block-wide barrier (all sixteen waves) is used once
  // per tile, where the sixteenth wave hands over: it must never be waited for
  // inside the sorting waves' steps, or the publication of a tile's counts
  // would wait for the resolution of the tile before.  Among themselves the
  // sorting waves meet at counters in LDS: a wave arrives with one add by its
  // first lane (after its own LDS operations have completed) and, where it
  // needs the others, polls the counter.  it = tiles this block has finished.

  if (__builtin_amdgcn_readfirstlane(threadIdx.x / kWaveSize) == kSorterWaves) {
    // ---- the resolving wave ----
    const int lane = threadIdx.x & (kWaveSize - 1);
    // The status words of this pass as a buffer: 16-byte loads and stores with
    // the cache policy of an agent-scope atomic.
    const __amdgpu_buffer_rsrc_t status_rows = __builtin_amdgcn_make_buffer_rsrc(
        status, 0, num_tiles * kRadix * 4, 0x00027000);
    uint32_t it = 0;
    __syncthreads();  // the first tile's totals and run starts are there, or there is no tile
    while (tile < num_tiles) {
      const uint32_t par = it & 1u;
      bool resolved = false;
      if (!resolved && with_scanner && tile > 0) {
        // The scanning block turns this tile's counts into prefixes; its row is
        // polled until it has, but never without bound.
        const StatusVec my_count = reinterpret_cast<const StatusVec*>(s_total[par])[lane];
        for (uint32_t polls = 0; polls <= spin_limit && polls < kScannerPolls; ++polls) {
          __builtin_amdgcn_s_sleep(ILGPU_HIP_SORT_OWN_ROW_SLEEP);
          const StatusVec row = load_status_row(status_rows, tile, lane);
          bool all = true;
#pragma unroll
          for (int c = 0; c < kWalkDigits; ++c)
            all = all && row[c] != 0u && !status_is_aggregate(row[c]);
          if (__all(all)) {
            const StatusVec my_excl =
                reinterpret_cast<const StatusVec*>(excl + pass * kRadix)[lane];
            const StatusVec start = reinterpret_cast<const StatusVec*>(s_start[par])[lane];
            StatusVec offset;
#pragma unroll
            for (int c = 0; c < kWalkDigits; ++c)
              offset[c] = my_excl[c] + (status_value(row[c]) - my_count[c]) - start[c];
            reinterpret_cast<StatusVec*>(s_global_off[par])[lane] = offset;
            resolved = true;
            break;
          }
        }
      }
      if (!resolved)
        pipelined_walk<KEY_BYTES, FLOAT_KEYS>(src_keys, tile, shift, in_xf, status_rows,
                                              excl + pass * kRadix, s_total[par], s_start[par],
                                              s_global_off[par], lane, spin_limit);
      __syncthreads();  // this tile is resolved; the next one's totals are there, if there is one
      tile = s_next[par];
      ++it;
    }
    return;
  }

  // ---- the sorting waves ----
  uint32_t hot[kMaxHot];
#pragma unroll
  for (int h = 0; h < kMaxHot; ++h) hot[h] = plan->hot[pass][h];
  auto digit = [&](K k) -> uint32_t {  // of a ranked or staged key
    const K o = FLOAT_KEYS ? k : (K)(k ^ (K)xf.xor_mask);
    return (uint32_t)(o >> shift) & (kRadix - 1);
  };
  auto arrive = [&](int which, int lane) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (lane == 0)
      __hip_atomic_fetch_add(&s_bar[which], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  auto wait_for = [&](int which, uint32_t target, int lane) {
    if (lane == 0) {
      while (__hip_atomic_load(&s_bar[which], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) <
             target)
        __builtin_amdgcn_s_sleep(1);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  };
  // Tile-local positions from the run starts, the wave's counters cleared for
  // the next tile, the keys staged in digit order.
  auto stage = [&](auto full, K (&key)[kItems], uint32_t (&packed)[kItems / 2], int valid,
                   uint32_t* my_counters, int lane, int first_local) {
    constexpr bool kFull = decltype(full)::value;
    auto item_digit = [&](int j) -> uint32_t {
      return (kFull || first_local + j * kWaveSize < valid) ? digit(key[j])
                                                             : (uint32_t)(kRadix - 1);
    };
#pragma unroll
    for (int j = 0; j < kItems; j += 2) {
      const uint32_t p0 = my_counters[item_digit(j)] + (packed[j / 2] & 0xFFFFu);
      const uint32_t p1 = my_counters[item_digit(j + 1)] + (packed[j / 2] >> 16);
      packed[j / 2] = p0 | (p1 << 16);
      if (j % 8 == 6) __builtin_amdgcn_sched_barrier(0);
    }
    reinterpret_cast<uint4*>(my_counters)[lane] = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int j = 0; j < kItems; ++j)
      s_keys[j % 2 == 0 ? packed[j / 2] & 0xFFFFu : packed[j / 2] >> 16] = key[j];
  };
  auto write_out = [&](auto full, int valid, const uint32_t* global_off) {
    constexpr bool kFull = decltype(full)::value;
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const int i = j * Cfg::kSorters + tid;
      if (kFull || i < valid) {
        const K k = s_keys[i];
        const uint32_t g = global_off[digit(k)] + (uint32_t)i;
        const K out = FLOAT_KEYS ? raw_bits(k, out_xf) : k;
        if (ILGPU_HIP_SORT_NT_STORE) __builtin_nontemporal_store(out, &dst_keys[g]);
        else dst_keys[g] = out;
      }
      if (j % ILGPU_HIP_SORT_WRITE_GROUP == ILGPU_HIP_SORT_WRITE_GROUP - 1)
        __builtin_amdgcn_sched_barrier(0);
    }
  };
  // What follows the ranking of a tile, up to the point where its keys are
  // staged in LDS: digit totals published, run starts, the hand-over with the
  // resolving wave, the write-out of the tile before, staging.
  uint32_t it = 0;       // tiles this block has finished
  bool pending = false;  // a staged tile waits to be written out
  auto after_ranking = [&](auto full, K (&key)[kItems], uint32_t (&packed)[kItems / 2],
                           int valid) {
    // The thread index is made opaque per tile: see sort_tile.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid / kWaveSize;
    const int first_local = wave * Cfg::kSubTileKeys + lane;
    uint32_t* my_counters = s_counter + wave * kRadix;
    const uint32_t par = it & 1u;
    arrive(0, lane);  // ranked
    uint32_t drawn = 0;
    if (tid < kRadix) {
      // One thread per digit (waves 0..3): totals over the sub-tiles, published
      // at once; then the tile-local start of every (sub-tile, digit) run.
      wait_for(0, (it + 1u) * kSorterWaves, lane);
      uint32_t count = 0;
#pragma unroll
      for (int s = 0; s < kSorterWaves; ++s) count += s_counter[s * kRadix + tid];
      __hip_atomic_store(&status[(int64_t)tile * kRadix + tid],
                         tile == 0 ? status_prefix(count) : status_aggregate(count),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_total[par][tid] = count;
      uint32_t inc = count;
#pragma unroll
      for (int s = 1; s < kWaveSize; s <<= 1) {
        const uint32_t o = shfl_up(inc, s);
        if (lane >= s) inc += o;
      }
      if (lane == kWaveSize - 1) s_scan[wave] = inc;
      arrive(1, lane);
      wait_for(1, (it + 1u) * kDigitWaves, lane);
      uint32_t run = inc - count;
      for (int w = 0; w < wave; ++w) run += s_scan[w];
      s_start[par][tid] = run;
#pragma unroll
      for (int s = 0; s < kSorterWaves; ++s) {
        const uint32_t c = s_counter[s * kRadix + tid];
        s_counter[s * kRadix + tid] = run;
        run += c;
      }
    } else if (tid == kDrawThread) {
      // The block's next tile is drawn now: its keys are loaded as soon as this
      // tile is staged, and its counts are published right after their ranking,
      // whatever the look-back of this tile does.
      drawn = atomicAdd(my_ticket, 1u);
    }
    __syncthreads();  // run starts and totals are there; the tile before is resolved
    if (pending) write_out(std::true_type{}, kTile, s_global_off[par ^ 1u]);
    if (tid == kDrawThread) s_next[par] = ticket_tile(drawn, group, (uint32_t)groups, chunk_shift);
    arrive(2, lane);  // the staged tile has been read
    wait_for(2, (it + 1u) * kSorterWaves, lane);
    stage(full, key, packed, valid, my_counters, lane, first_local);
    pending = true;
    const int next_tile = s_next[par];
    ++it;
    return next_tile;
  };

  auto full_tiles = [&](auto with_hot) {
    constexpr bool kHot = decltype(with_hot)::value;
    if (!(tile < num_tiles && is_full(tile))) return;
    K key[kItems];
    uint32_t packed[kItems / 2];
    {
      int tid = threadIdx.x;
      asm volatile("" : "+v"(tid));
      const int lane = tid & (kWaveSize - 1), wave = tid / kWaveSize;
      pipelined_rank<KEY_BYTES, true, kHot, FLOAT_KEYS>(
          key, packed, src_keys, (int64_t)tile * kTile, kTile, shift, in_xf, s_counter + wave * kRadix,
          lane, wave * Cfg::kSubTileKeys + lane, hot);
    }
    bool ranked = true;
    while (ranked) {
      const int next_tile = after_ranking(std::true_type{}, key, packed, kTile);
      ranked = next_tile < num_tiles && is_full(next_tile);
      if (ranked) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const int lane = tid & (kWaveSize - 1), wave = tid / kWaveSize;
        pipelined_rank<KEY_BYTES, true, kHot, FLOAT_KEYS>(
            key, packed, src_keys, (int64_t)next_tile * kTile, kTile, shift, in_xf,
            s_counter + wave * kRadix, lane, wave * Cfg::kSubTileKeys + lane, hot);
      }
      tile = next_tile;
    }
  };
  if (hot[0] == kNoHotDigit) full_tiles(std::false_type{});
  else full_tiles(std::true_type{});
  // Here the block's next tile, if any, is the one at the end of the input; it
  // is the last of its group and so of this block.
  int last_valid = kTile;
  if (tile < num_tiles) {
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid / kWaveSize;
    last_valid = (int)(n - (int64_t)tile * kTile);
    K key[kItems];
    uint32_t packed[kItems / 2];
    pipelined_rank<KEY_BYTES, false, true, FLOAT_KEYS>(
        key, packed, src_keys, (int64_t)tile * kTile, last_valid, shift, in_xf,
        s_counter + wave * kRadix, lane, wave * Cfg::kSubTileKeys + lane, hot);
    after_ranking(std::false_type{}, key, packed, last_valid);
  }
  __syncthreads();  // the last tile is resolved
  if (pending) {
    if (last_valid == kTile) write_out(std::true_type{}, kTile, s_global_off[(it & 1u) ^ 1u]);
    else write_out(std::false_type{}, last_valid, s_global_off[(it & 1u) ^ 1u]);
  }
}

// ---- inputs of one tile ---------------------------------------------------------
// A sort of at most one 512-thread tile runs as one block and one launch: the
// keys (and values) stay in registers, every pass ranks them like a pass above,
// moves them through LDS into digit order and takes them back in memory order
// (lane l of wave w holds positions w*64*I + j*64 + l again), and the last pass
// is followed by one coalesced write.  No histogram, plan, tickets, look-back
// or temp memory; a pass whose digit is the same for every key simply leaves
// the order as it is.  ITEMS keys per thread: every row costs its rank, its
// staging and its share of five barriers per pass whether it holds keys or
// not, so short inputs take an instantiation with few rows (4, 12 or 24:
// 32 to 2048 u32 keys 8 to 9 us instead of 24 to 27, up to 6144 keys 13
// instead of 31).
constexpr int kSmallSortItemsA = 4, kSmallSortItemsB = 12, kSmallSortItemsC = 24;
template <int KEY_BYTES, int VALUE_BYTES, bool FLOAT_KEYS, int ITEMS>
__global__ __launch_bounds__(kSortBlock, ILGPU_HIP_SORT_WAVES_PER_EU)
void small_sort_kernel(typename KeyOf<KEY_BYTES>::type* keys,
                       typename ValueOf<VALUE_BYTES>::type* vals, int n, KeyXform xf,
                       int values_from_index) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Val = typename ValueOf<VALUE_BYTES>::type;
  using TileCfg = SortTile<KEY_BYTES, VALUE_BYTES, kSortBlock>;
  constexpr int kItems = ITEMS;
  constexpr int kSubTiles = TileCfg::kSubTiles;
  constexpr int kSubTileKeys = kSubLanes * kItems;
  constexpr bool kPairs = VALUE_BYTES > 0;
  static_assert(kItems % 2 == 0 && kItems <= TileCfg::kItems, "ranks are packed in pairs");
  // Counters, then the keys, then the values of the tile share these bytes.
  constexpr int kEntryBytes = KEY_BYTES > VALUE_BYTES ? KEY_BYTES : VALUE_BYTES;
  constexpr int kStageBytes = kSortBlock * kItems * kEntryBytes > TileCfg::kCounterBytes
                                  ? kSortBlock * kItems * kEntryBytes
                                  : TileCfg::kCounterBytes;

  __shared__ __attribute__((aligned(16))) unsigned char s_stage[kStageBytes];
  __shared__ uint32_t s_scan[kRadix / kWaveSize];
  uint32_t* s_counter = reinterpret_cast<uint32_t*>(s_stage);
  K* s_keys = reinterpret_cast<K*>(s_stage);
  Val* s_vals = reinterpret_cast<Val*>(s_stage);

  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = tid / kWaveSize;
  const int first_local = wave * kSubTileKeys + lane;
  uint32_t* my_counters = s_counter + wave * kRadix;

  K key[kItems];
  Val val[kPairs ? kItems : 1];
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const int local = first_local + j * kSubLanes;
    key[j] = 0;
    if (local < n) {
      key[j] = keys[local];
      if constexpr (FLOAT_KEYS) key[j] = ordered_bits(key[j], xf);
      if constexpr (kPairs) {
        if (values_from_index) {
          val[j] = index_value<VALUE_BYTES>(local, values_from_index);
        } else {
          val[j] = vals[local];
        }
      }
    }
  }

#pragma unroll 1
  for (int pass = 0; pass < KEY_BYTES; ++pass) {
    const int shift = pass * 8;
    // Positions past the end take digit 255 and come last in memory order, so
    // they stay behind every key through every pass.
    auto item_digit = [&](int j) -> uint32_t {
      if (first_local + j * kSubLanes >= n) return (uint32_t)(kRadix - 1);
      if constexpr (FLOAT_KEYS) return (uint32_t)(key[j] >> shift) & (kRadix - 1);
      else return (uint32_t)((K)(key[j] ^ (K)xf.xor_mask) >> shift) & (kRadix - 1);
    };
    __syncthreads();  // the stage of the previous pass has been read
    for (int i = tid; i < TileCfg::kCounterWords; i += kSortBlock) s_counter[i] = 0u;
    __syncthreads();

    uint32_t packed[kItems / 2];  // rank in the sub-tile, then position in the tile
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const uint32_t d = item_digit(j);
      // a row that is all one digit: lane 0 adds for the row (see sort_tile)
      const uint32_t row_digit = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
      const bool whole_row = __ballot(d == row_digit) == ~0ull;
      uint32_t rank = 0;
      if (!whole_row || lane == 0)
        rank = __hip_atomic_fetch_add(my_counters + d, whole_row ? (uint32_t)kSubLanes : 1u,
                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (whole_row) rank = (uint32_t)__builtin_amdgcn_readfirstlane((int)rank) + (uint32_t)lane;
      if (j % 2 == 0) packed[j / 2] = rank;
      else packed[j / 2] |= rank << 16;
    }
    __syncthreads();

    // One thread per digit: totals over the sub-tiles, exclusive scan over the
    // digits, then the tile position of the first key of every (sub-tile, digit).
    uint32_t count = 0, inc = 0;
    if (tid < kRadix) {
#pragma unroll
      for (int s = 0; s < kSubTiles; ++s) count += s_counter[s * kRadix + tid];
      inc = count;
#pragma unroll
      for (int s = 1; s < kWaveSize; s <<= 1) {
        const uint32_t o = shfl_up(inc, s);
        if (lane >= s) inc += o;
      }
      if (lane == kWaveSize - 1) s_scan[wave] = inc;
    }
    __syncthreads();
    if (tid < kRadix) {
      uint32_t run = inc - count;
      for (int w = 0; w < wave; ++w) run += s_scan[w];
#pragma unroll
      for (int s = 0; s < kSubTiles; ++s) {
        const uint32_t t = s_counter[s * kRadix + tid];
        s_counter[s * kRadix + tid] = run;
        run += t;
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kItems; j += 2) {
      const uint32_t p0 = my_counters[item_digit(j)] + (packed[j / 2] & 0xFFFFu);
      const uint32_t p1 = my_counters[item_digit(j + 1)] + (packed[j / 2] >> 16);
      packed[j / 2] = p0 | (p1 << 16);
    }
    __syncthreads();  // the run starts have been read; the same bytes stage the keys
#pragma unroll
    for (int j = 0; j < kItems; ++j)
      s_keys[j % 2 == 0 ? packed[j / 2] & 0xFFFFu : packed[j / 2] >> 16] = key[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kItems; ++j) key[j] = s_keys[first_local + j * kSubLanes];
    if constexpr (kPairs) {
      __syncthreads();
#pragma unroll
      for (int j = 0; j < kItems; ++j)
        s_vals[j % 2 == 0 ? packed[j / 2] & 0xFFFFu : packed[j / 2] >> 16] = val[j];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < kItems; ++j) val[j] = s_vals[first_local + j * kSubLanes];
    }
  }

#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const int local = first_local + j * kSubLanes;
    if (local < n) {
      if constexpr (FLOAT_KEYS) keys[local] = raw_bits(key[j], xf);
      else keys[local] = key[j];
      if constexpr (kPairs) vals[local] = val[j];
    }
  }
}

// ---- finish ----------------------------------------------------------------
template <int KEY_BYTES, int VALUE_BYTES>
__global__ __launch_bounds__(256) void finish_kernel(
    typename KeyOf<KEY_BYTES>::type* keys_a,
    const typename KeyOf<KEY_BYTES>::type* keys_b,
    typename ValueOf<VALUE_BYTES>::type* vals_a,
    const typename ValueOf<VALUE_BYTES>::type* vals_b, int64_t n,
    const SortPlan* __restrict__ plan, int values_from_index) {
  const bool copy_back = plan->final_in_alt != 0;
  const bool fill_index =
      VALUE_BYTES > 0 && values_from_index && plan->executed == 0;
  if (!copy_back && !fill_index) return;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    if (copy_back) {
      keys_a[i] = keys_b[i];
      if constexpr (VALUE_BYTES > 0) vals_a[i] = vals_b[i];
    } else {
      if constexpr (VALUE_BYTES > 0) vals_a[i] = index_value<VALUE_BYTES>(i, values_from_index);
    }
  }
}

// ---- host side -------------------------------------------------------------

struct TempLayout {
  int64_t alt_keys, alt_vals, excl, plan, zero_begin, hist, tickets, status,
      status_stride, total;
  int64_t tiles;
};

// Layout for tiles of `block` threads.  Temp views are sized for the small
// block (more tiles, more status words); the large block's layout fits inside.
// Keys per thread of the class of short tiles an input takes (the shortest
// that makes at most `max_tiles` tiles), or 0: full tiles.
inline int pick_short_items(int64_t n, int key_bytes, int value_bytes, int64_t max_tiles) {
  if (value_bytes != 0) return 0;
  // 8-byte keys: their full tiles are half as long to begin with, and beyond
  // 128 short ones the longer look-back costs what the shorter tiles save.
  if (key_bytes == 8 && max_tiles > kShortTileMaxTiles / 4) max_tiles = kShortTileMaxTiles / 4;
  for (int c = 0; c < kShortTileClasses; ++c) {
    const int items = short_items_per_thread(key_bytes, c);
    if (div_up(n, (int64_t)kSortBlock * items) <= max_tiles) return items;
  }
  return 0;
}
// With the defaults (what temp views are sized by) the layout is that of the
// shortest tiles the input can be given: the 512-thread block's, or short
// tiles where they apply.
TempLayout make_layout(int64_t n, int key_bytes, int value_bytes, int block = kSortBlock,
                       int64_t tile_override = 0) {
  TempLayout L;
  int64_t tile = tile_override > 0 ? tile_override : tile_keys(key_bytes, value_bytes, block);
  if (tile_override <= 0 && block == kSortBlock) {
    const int short_items = pick_short_items(n, key_bytes, value_bytes, kShortTileMaxTiles);
    if (short_items > 0) tile = (int64_t)kSortBlock * short_items;
  }
  L.tiles = div_up(n, tile);
  int64_t off = 0;
  L.alt_keys = off; off += align_up(n * key_bytes, 256);
  L.alt_vals = off; off += align_up(n * value_bytes, 256);
  L.excl = off; off += kMaxPasses * kRadix * 4;
  L.plan = off; off += 256;
  L.zero_begin = off;
  L.hist = off; off += kMaxPasses * kRadix * 4;
  L.tickets = off; off += kMaxPasses * kTicketGroups * kTicketStride * 4;
  L.status = off;
  L.status_stride = L.tiles * kRadix * 4;
  off += L.status_stride * key_bytes;  // one status array per pass
  L.total = off;
  return L;
}

KeyXform make_xform(int32_t key_type, int32_t flags) {
  const int bits = elem_size(key_type) * 8;
  const uint64_t all = bits == 64 ? ~0ull : ((1ull << bits) - 1ull);
  const uint64_t sign = 1ull << (bits - 1);
  KeyXform xf{0, 0, 0};
  switch (key_type) {
    case ILGPU_HIP_I8: case ILGPU_HIP_I16: case ILGPU_HIP_I32: case ILGPU_HIP_I64:
      xf.xor_mask = sign;
      break;
    case ILGPU_HIP_F16: case ILGPU_HIP_F32: case ILGPU_HIP_F64:
      if (flags & ILGPU_HIP_SORT_FLOAT_TOTAL_ORDER) {
        xf.xor_mask = sign;
        xf.total_term = sign - 1ull;
      } else {
        // Half: (uint)~bits >> 15 keeps the sign-extended upper ones, so bits
        // 1..15 are always flipped (RadixSortOperations.tt:77-80).
        xf.xor_mask = key_type == ILGPU_HIP_F16 ? 0xFFFEull : sign;
        xf.reference_term = 1ull;
      }
      break;
    default:
      break;
  }
  if (flags & ILGPU_HIP_SORT_DESCENDING) xf.xor_mask ^= all;
  return xf;
}

// The passes of one sort with tiles of BLOCK threads and ITEMS keys per thread.
template <int KEY_BYTES, int VALUE_BYTES, int BLOCK,
          int ITEMS = items_per_thread(KEY_BYTES, VALUE_BYTES)>
int32_t launch_passes(hipStream_t stream, const SortArgs& a, const TempLayout& L, char* base,
                      const KeyXform& xf, int cus) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Val = typename ValueOf<VALUE_BYTES>::type;
  K* keys_a = static_cast<K*>(a.keys);
  K* keys_b = reinterpret_cast<K*>(base + L.alt_keys);
  Val* vals_a = static_cast<Val*>(a.values);
  Val* vals_b = reinterpret_cast<Val*>(base + L.alt_vals);
  uint32_t* excl = reinterpret_cast<uint32_t*>(base + L.excl);
  SortPlan* plan = reinterpret_cast<SortPlan*>(base + L.plan);
  uint32_t* tickets = reinterpret_cast<uint32_t*>(base + L.tickets);
  const int passes = KEY_BYTES;
  const int from_index = a.value_source == ILGPU_HIP_VALUES_FROM_INDEX
                             ? 1
                             : (a.value_source == ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT ? 2 : 0);
  const bool float_keys = (xf.reference_term | xf.total_term) != 0;
  auto* pass_kernel = onesweep_kernel<KEY_BYTES, VALUE_BYTES, false, BLOCK, ITEMS>;
  if constexpr (KEY_BYTES >= 2) {  // there is no 1-byte floating-point key
    if (float_keys) pass_kernel = onesweep_kernel<KEY_BYTES, VALUE_BYTES, true, BLOCK, ITEMS>;
  }
  // Resident blocks per CU of this instantiation: asked once per device and
  // kernel (the query costs microseconds, which small sorts would feel).
  static std::atomic<int> cached_per_cu[kMaxCachedDevices][2];  // per instantiation
  const int device = current_device();
  std::atomic<int>* cached =
      device >= 0 && device < kMaxCachedDevices ? &cached_per_cu[device][float_keys ? 1 : 0]
                                                : nullptr;
  int per_cu = cached ? cached->load(std::memory_order_relaxed) : 0;
  if (per_cu == 0) {
    ILGPU_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(
        &per_cu, pass_kernel, BLOCK, 0));
    if (per_cu < 1) per_cu = 1;
    if (cached) cached->store(per_cu, std::memory_order_relaxed);
  }
  int64_t grid = (int64_t)cus * per_cu;
  if (grid > L.tiles) grid = L.tiles;
  // Every group of blocks needs a block: a grid below eight blocks (few tiles, or
  // a device with very few compute units) forms as many groups as it has blocks.
  const int groups = grid < kTicketGroups ? (int)grid : kTicketGroups;
  // Chunks as long as leave every block of the grid a tile of its own in the
  // first round (short inputs: single tiles, handed out round-robin).
  int chunk_shift = 0;
  while (chunk_shift < kMaxChunkShift && (grid << (chunk_shift + 1)) <= L.tiles) ++chunk_shift;
  const uint32_t spin_limit = g_sort_spin_limit.load(std::memory_order_relaxed);
  for (int p = 0; p < passes; ++p) {
    uint32_t* status =
        reinterpret_cast<uint32_t*>(base + L.status + (int64_t)p * L.status_stride);
    {
      ProfileScope scope(stream, "sort_onesweep");
      hipLaunchKernelGGL(pass_kernel,
                         dim3((unsigned)grid), dim3(BLOCK), 0, stream,
                         keys_a, keys_b, vals_a, vals_b, a.n, p, xf, excl,
                         status,
                         grid == L.tiles ? nullptr : tickets + p * kTicketGroups * kTicketStride,
                         plan, (int)L.tiles, from_index, groups, chunk_shift, spin_limit);
    }
    ILGPU_HIP_CHECK(hipGetLastError());
  }
  return ILGPU_HIP_SUCCESS;
}

// The passes of a keys-only sort in the pipelined form (one block per compute unit).
template <int KEY_BYTES>
int32_t launch_passes_pipelined(hipStream_t stream, const SortArgs& a, const TempLayout& L,
                                char* base, const KeyXform& xf, int cus) {
  using K = typename KeyOf<KEY_BYTES>::type;
  K* keys_a = static_cast<K*>(a.keys);
  K* keys_b = reinterpret_cast<K*>(base + L.alt_keys);
  uint32_t* excl = reinterpret_cast<uint32_t*>(base + L.excl);
  SortPlan* plan = reinterpret_cast<SortPlan*>(base + L.plan);
  uint32_t* tickets = reinterpret_cast<uint32_t*>(base + L.tickets);
  auto* pass_kernel = onesweep_pipelined_kernel<KEY_BYTES, false>;
  if constexpr (KEY_BYTES >= 2) {  // there is no 1-byte floating-point key
    if ((xf.reference_term | xf.total_term) != 0)
      pass_kernel = onesweep_pipelined_kernel<KEY_BYTES, true>;
  }
  int64_t grid = cus;  // 1024 threads and 150 KiB of LDS: one block per compute unit
  if (grid > L.tiles) grid = L.tiles;
  const int groups = grid < kTicketGroups ? (int)grid : kTicketGroups;
  // Chunks of 16 and 32 tiles, which the write pattern by itself prefers
  // (bench_bounds scatter), lose here: 0.492 and 0.572 ms per pass against 0.484.
  int chunk_shift = 0;
  while (chunk_shift < kMaxChunkShift && (grid << (chunk_shift + 1)) <= L.tiles) ++chunk_shift;
  const uint32_t spin_limit = g_sort_spin_limit.load(std::memory_order_relaxed);
#ifndef ILGPU_HIP_SORT_SCANNER
#define ILGPU_HIP_SORT_SCANNER 1
#endif
  // One block scans instead of sorting when the grid can spare it.
  const int with_scanner = ILGPU_HIP_SORT_SCANNER && grid >= 64 ? 1 : 0;
  for (int p = 0; p < KEY_BYTES; ++p) {
    uint32_t* status =
        reinterpret_cast<uint32_t*>(base + L.status + (int64_t)p * L.status_stride);
    {
      ProfileScope scope(stream, "sort_onesweep");
      hipLaunchKernelGGL(pass_kernel, dim3((unsigned)grid), dim3(1024), 0, stream, keys_a, keys_b,
                         a.n, p, xf, excl, status, tickets + p * kTicketGroups * kTicketStride,
                         plan, (int)L.tiles, groups, chunk_shift, spin_limit, with_scanner);
    }
    ILGPU_HIP_CHECK(hipGetLastError());
  }
  return ILGPU_HIP_SUCCESS;
}

template <int KEY_BYTES, int VALUE_BYTES>
int32_t launch_sized(hipStream_t stream, const SortArgs& a) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Val = typename ValueOf<VALUE_BYTES>::type;
  if (a.n <= (int64_t)tile_keys(KEY_BYTES, VALUE_BYTES, kSortBlock) &&
      g_sort_small_kernel.load(std::memory_order_relaxed) != 0) {
    // one tile: one block, one launch, no temp
    const KeyXform xf = make_xform(a.key_type, a.flags);
    constexpr int kFullItems = items_per_thread(KEY_BYTES, VALUE_BYTES);
    auto launch_small = [&](auto items) -> int32_t {
      constexpr int kItems = decltype(items)::value;
      auto* kernel = small_sort_kernel<KEY_BYTES, VALUE_BYTES, false, kItems>;
      if constexpr (KEY_BYTES >= 2) {  // there is no 1-byte floating-point key
        if ((xf.reference_term | xf.total_term) != 0)
          kernel = small_sort_kernel<KEY_BYTES, VALUE_BYTES, true, kItems>;
      }
      ProfileScope scope(stream, "sort_small");
      hipLaunchKernelGGL(kernel, dim3(1), dim3(kSortBlock), 0, stream, static_cast<K*>(a.keys),
                         static_cast<Val*>(a.values), (int)a.n, xf,
                         a.value_source == ILGPU_HIP_VALUES_FROM_INDEX
                               ? 1
                               : (a.value_source == ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT ? 2 : 0));
      ILGPU_HIP_CHECK(hipGetLastError());
      return ILGPU_HIP_SUCCESS;
    };
    if constexpr (kSmallSortItemsA < kFullItems) {
      if (a.n <= (int64_t)kSortBlock * kSmallSortItemsA)
        return launch_small(std::integral_constant<int, kSmallSortItemsA>{});
    }
    if constexpr (kSmallSortItemsB < kFullItems) {
      if (a.n <= (int64_t)kSortBlock * kSmallSortItemsB)
        return launch_small(std::integral_constant<int, kSmallSortItemsB>{});
    }
    if constexpr (kSmallSortItemsC < kFullItems) {
      if (a.n <= (int64_t)kSortBlock * kSmallSortItemsC)
        return launch_small(std::integral_constant<int, kSmallSortItemsC>{});
    }
    return launch_small(std::integral_constant<int, kFullItems>{});
  }
  const int cus = device_cu_count();
  int64_t min_tiles_per_cu = g_sort_large_min_tiles_per_cu.load(std::memory_order_relaxed);
  if (min_tiles_per_cu < 0)
    min_tiles_per_cu = VALUE_BYTES > 0 ? kLargeMinTilesPerCuPairs : kLargeMinTilesPerCuKeys;
  const bool use_large =
      div_up(a.n, (int64_t)tile_keys(KEY_BYTES, VALUE_BYTES, kSortBlockLarge)) >=
      min_tiles_per_cu * cus;
  const KeyXform xf = make_xform(a.key_type, a.flags);
#ifndef ILGPU_HIP_SORT_PIPELINED
#define ILGPU_HIP_SORT_PIPELINED 1
#endif
#ifndef ILGPU_HIP_SORT_PIPELINED_FLOAT
#define ILGPU_HIP_SORT_PIPELINED_FLOAT 1
#endif
  // Large keys-only sorts take the pipelined form of the pass.
  const bool use_pipelined =
      ILGPU_HIP_SORT_PIPELINED && VALUE_BYTES == 0 && use_large &&
      (ILGPU_HIP_SORT_PIPELINED_FLOAT || (xf.reference_term | xf.total_term) == 0);
  // Short inputs of keys take short tiles (the parameter can only lower the
  // limit: temp views are sized by the default).
  int64_t short_max_tiles = g_sort_short_tile_max_tiles.load(std::memory_order_relaxed);
  if (short_max_tiles < 0 || short_max_tiles > kShortTileMaxTiles)
    short_max_tiles = kShortTileMaxTiles;
  // Two 512-thread blocks are resident per compute unit; a second round of
  // short tiles would cost more than full tiles do.
  if (short_max_tiles > 2 * (int64_t)cus) short_max_tiles = 2 * (int64_t)cus;
  const int short_items =
      use_large ? 0 : pick_short_items(a.n, KEY_BYTES, VALUE_BYTES, short_max_tiles);
  const TempLayout L =
      make_layout(a.n, KEY_BYTES, VALUE_BYTES, use_large ? kSortBlockLarge : kSortBlock,
                  use_pipelined ? pipelined_tile_keys(KEY_BYTES)
                                : (short_items > 0 ? kSortBlock * short_items
                                             : tile_keys(KEY_BYTES, VALUE_BYTES,
                                                         use_large ? kSortBlockLarge : kSortBlock)));
  char* base = reinterpret_cast<char*>(align_up((int64_t)(uintptr_t)a.temp, 256));
  K* keys_a = static_cast<K*>(a.keys);
  K* keys_b = reinterpret_cast<K*>(base + L.alt_keys);
  Val* vals_a = static_cast<Val*>(a.values);
  Val* vals_b = reinterpret_cast<Val*>(base + L.alt_vals);
  uint32_t* excl = reinterpret_cast<uint32_t*>(base + L.excl);
  SortPlan* plan = reinterpret_cast<SortPlan*>(base + L.plan);
  uint32_t* hist = reinterpret_cast<uint32_t*>(base + L.hist);
  const int passes = KEY_BYTES;
  const int from_index = a.value_source == ILGPU_HIP_VALUES_FROM_INDEX
                             ? 1
                             : (a.value_source == ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT ? 2 : 0);

  int32_t rc = launch_zero_words(stream, hist, (L.total - L.zero_begin) / 4);
  if (rc != ILGPU_HIP_SUCCESS) return rc;

  {
    int shift = 0;  // replicas: as many as kHistLdsWords of LDS counters hold
    while ((1 << (shift + 1)) <= 32 &&
           ((passes * kRadix) << (shift + 1)) <= kHistLdsWords)
      ++shift;
    const size_t lds = (size_t)((passes * kRadix) << shift) * 4;
    // A block's fixed cost is its flush, one global atomic per digit value and
    // position, which all blocks issue at about the same time.  Up to half a
    // block per CU as soon as every thread has four vectors to count, more
    // only when every thread has sixteen (2^20 u32 keys: 7.5 us instead of
    // 15.5 with one vector per thread; 2^22: 12.3 instead of 17.1).
    const int64_t vectors = div_up(a.n, Vec16<K>::N);
    const int64_t few = std::min<int64_t>(div_up(vectors, kHistBlock * 4), std::max(cus / 2, 1));
    int64_t blocks = std::max(few, div_up(vectors, kHistBlock * 16));
    // Two blocks of 64 KiB of counters are resident per CU: no second round.
    if (blocks > (int64_t)cus * ILGPU_HIP_SORT_HIST_BLOCKS_PER_CU)
      blocks = (int64_t)cus * ILGPU_HIP_SORT_HIST_BLOCKS_PER_CU;
    if (blocks < 1) blocks = 1;
    ProfileScope scope(stream, "sort_histogram");
    auto* histogram_kernel = sort_histogram_kernel<K, false>;
    if constexpr (KEY_BYTES >= 2) {  // there is no 1-byte floating-point key
      if ((xf.reference_term | xf.total_term) != 0) histogram_kernel = sort_histogram_kernel<K, true>;
    }
    hipLaunchKernelGGL(histogram_kernel, dim3((unsigned)blocks),
                       dim3(kHistBlock), lds, stream, keys_a, a.n, xf, passes,
                       shift, hist);
    ILGPU_HIP_CHECK(hipGetLastError());
  }
  {
    ProfileScope scope(stream, "sort_plan");
    hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(kRadix), 0, stream, hist, excl,
                       plan, passes, (uint32_t)a.n);
  }
  ILGPU_HIP_CHECK(hipGetLastError());

  if (use_pipelined) {
    if constexpr (VALUE_BYTES == 0)
      rc = launch_passes_pipelined<KEY_BYTES>(stream, a, L, base, xf, cus);
  } else if (use_large) {
    rc = launch_passes<KEY_BYTES, VALUE_BYTES, kSortBlockLarge>(stream, a, L, base, xf, cus);
  } else if (short_items > 0) {
    if constexpr (VALUE_BYTES == 0) {
      constexpr int kA = short_items_per_thread(KEY_BYTES, 0);
      constexpr int kB = short_items_per_thread(KEY_BYTES, 1);
      constexpr int kC = short_items_per_thread(KEY_BYTES, 2);
      if (short_items == kA)
        rc = launch_passes<KEY_BYTES, 0, kSortBlock, kA>(stream, a, L, base, xf, cus);
      else if (short_items == kB)
        rc = launch_passes<KEY_BYTES, 0, kSortBlock, kB>(stream, a, L, base, xf, cus);
      else
        rc = launch_passes<KEY_BYTES, 0, kSortBlock, kC>(stream, a, L, base, xf, cus);
    }
  } else
    rc = launch_passes<KEY_BYTES, VALUE_BYTES, kSortBlock>(stream, a, L, base, xf, cus);
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  {
    // Mostly there is nothing to copy and every block returns at once; 16
    // keys per thread are few enough blocks for that and enough for the copy.
    int64_t blocks = div_up(a.n, 256 * 16);
    if (blocks > (int64_t)cus * 8) blocks = (int64_t)cus * 8;
    ProfileScope scope(stream, "sort_finish");
    hipLaunchKernelGGL((finish_kernel<KEY_BYTES, VALUE_BYTES>),
                       dim3((unsigned)blocks), dim3(256), 0, stream, keys_a,
                       keys_b, vals_a, vals_b, a.n, plan, from_index);
    ILGPU_HIP_CHECK(hipGetLastError());
  }
  return ILGPU_HIP_SUCCESS;
}

template <int KEY_BYTES>
int32_t launch_value(hipStream_t stream, const SortArgs& a) {
  switch (a.value_bytes) {
    case 0: return launch_sized<KEY_BYTES, 0>(stream, a);
    case 1: return launch_sized<KEY_BYTES, 1>(stream, a);
    case 2: return launch_sized<KEY_BYTES, 2>(stream, a);
    case 4: return launch_sized<KEY_BYTES, 4>(stream, a);
    case 8: return launch_sized<KEY_BYTES, 8>(stream, a);
    case 16: return launch_sized<KEY_BYTES, 16>(stream, a);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}


}  // namespace

}  // namespace ilgpu_hip
