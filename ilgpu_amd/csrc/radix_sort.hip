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
//   pass x k  onesweep: a block takes a tile by ticket, ranks its keys
//             (per-wave digit counters in LDS, wave64 ballot matching, so
//             equal digits keep memory order: every pass is stable), publishes
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
// per-key term of the float transforms.
//
// Algorithmic HBM traffic for n keys of k bytes, values of v bytes and P
// executed passes: n * (k * (2P + 1) + v * 2P) bytes.
#include "kernels.hpp"

namespace ilgpu_hip {

namespace {

constexpr int kRadix = 256;
constexpr int kMaxPasses = 8;
constexpr int kSortBlock = 512;
constexpr int kSortWaves = kSortBlock / kWaveSize;
constexpr int kHistBlock = 512;
constexpr uint32_t kStatusAggregate = 1u << 30;
constexpr uint32_t kStatusPrefix = 2u << 30;
constexpr uint32_t kStatusValueMask = (1u << 30) - 1u;
constexpr int64_t kMaxSortLength = (1ll << 30) - 1;  // counts must fit 30 bits

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

template <int KEY_BYTES> constexpr int items_per_thread() {
  return KEY_BYTES == 8 ? 8 : 16;
}
template <int KEY_BYTES> constexpr int tile_keys() {
  return kSortBlock * items_per_thread<KEY_BYTES>();
}

// How raw key bits map to unsigned bits that sort in the requested order.
enum { kModePlain = 0, kModeFloatReference = 1, kModeFloatTotalOrder = 2 };
struct KeyXform {
  uint64_t xor_mask;
  int32_t mode;
};

template <typename K>
__device__ __forceinline__ K ordered_bits(K k, const KeyXform& xf) {
  constexpr int kBits = sizeof(K) * 8;
  K o = k ^ (K)xf.xor_mask;
  if (xf.mode == kModeFloatReference) {
    // RadixSortOperations.tt:81-89 as written: the complement mask is a
    // LOGICAL shift of ~bits, i.e. 1 for non-negative values and 0 otherwise.
    o ^= (K)((K)(~k) >> (kBits - 1));
  } else if (xf.mode == kModeFloatTotalOrder) {
    const K sign = (K)((K)1 << (kBits - 1));
    if (k & sign) o ^= (K)(sign - 1);
  }
  return o;
}

template <typename K>
__device__ __forceinline__ uint32_t digit_of(K k, const KeyXform& xf, int shift) {
  return (uint32_t)(ordered_bits(k, xf) >> shift) & (kRadix - 1);
}

// Device-resident description of the passes, written by plan_kernel.
struct SortPlan {
  uint32_t skip[kMaxPasses];        // digit identical for all keys
  uint32_t src_is_alt[kMaxPasses];  // pass reads the alternate buffer
  uint32_t first_executed;          // index of the first pass that runs
  uint32_t executed;                // number of passes that run
  uint32_t final_in_alt;            // result sits in the alternate buffer
};

// ---- histogram of all digit positions ------------------------------------
template <typename K>
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
    const K o = ordered_bits(k, xf);
#pragma unroll
    for (int p = 0; p < (int)sizeof(K); ++p) {
      const uint32_t d = (uint32_t)(o >> (8 * p)) & (kRadix - 1);
      atomicAdd(&s_hist[((p * kRadix + d) << replica_shift) + replica], 1u);
    }
  };

  const uintptr_t addr = reinterpret_cast<uintptr_t>(keys);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(K));
  if (head > n) head = n;
  const V* body = reinterpret_cast<const V*>(keys + head);
  const int64_t nvec = (n - head) / VN;
  const int64_t tail_start = head + nvec * VN;
  const int64_t stride = (int64_t)gridDim.x * kHistBlock;
  int64_t i = (int64_t)blockIdx.x * kHistBlock + threadIdx.x;
  for (; i + stride < nvec; i += 2 * stride) {
    V a = body[i];
    V b = body[i + stride];
#pragma unroll
    for (int k = 0; k < VN; ++k) count(a[k]);
#pragma unroll
    for (int k = 0; k < VN; ++k) count(b[k]);
  }
  for (; i < nvec; i += stride) {
    V a = body[i];
#pragma unroll
    for (int k = 0; k < VN; ++k) count(a[k]);
  }
  if (blockIdx.x == 0) {
    const int64_t extra = head + (n - tail_start);
    if ((int64_t)threadIdx.x < extra) {
      const int64_t idx = (int64_t)threadIdx.x < head
                              ? (int64_t)threadIdx.x
                              : tail_start + ((int64_t)threadIdx.x - head);
      count(keys[idx]);
    }
  }
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
  const int d = threadIdx.x;
  const int lane = d & (kWaveSize - 1);
  const int wave = d / kWaveSize;
  uint32_t parity = 0, executed = 0, first = passes;
  for (int p = 0; p < passes; ++p) {
    if (d == 0) s_trivial = 0;
    __syncthreads();
    const uint32_t c = global_hist[p * kRadix + d];
    if (c == n) s_trivial = 1;
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
    }
    if (!trivial) {
      if (executed == 0) first = p;
      parity ^= 1u;
      ++executed;
    }
    __syncthreads();
  }
  if (d == 0) {
    plan->first_executed = first;
    plan->executed = executed;
    plan->final_in_alt = parity;
  }
}

// ---- onesweep pass ---------------------------------------------------------
// Lanes holding the same digit, as a 64-bit mask: eight ballots, one per bit.
__device__ __forceinline__ uint64_t match_digit(uint32_t d) {
  uint64_t peers = ~0ull;
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const bool bit = (d >> b) & 1u;
    const uint64_t m = __ballot(bit);
    peers &= bit ? m : ~m;
  }
  return peers;
}

template <int KEY_BYTES, int VALUE_BYTES>
__global__ __launch_bounds__(kSortBlock) void onesweep_kernel(
    typename KeyOf<KEY_BYTES>::type* keys_a,
    typename KeyOf<KEY_BYTES>::type* keys_b,
    typename ValueOf<VALUE_BYTES>::type* vals_a,
    typename ValueOf<VALUE_BYTES>::type* vals_b, int64_t n, int pass,
    KeyXform xf, const uint32_t* __restrict__ excl, uint32_t* status,
    uint32_t* ticket, const SortPlan* __restrict__ plan, int num_tiles,
    int values_from_index) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Val = typename ValueOf<VALUE_BYTES>::type;
  constexpr int kItems = items_per_thread<KEY_BYTES>();
  constexpr int kTile = tile_keys<KEY_BYTES>();
  constexpr bool kPairs = VALUE_BYTES > 0;
  // Values are staged through the key buffer, kTile * KEY_BYTES bytes at a time.
  constexpr int kStageBytes = kTile * (KEY_BYTES < 4 ? 4 : KEY_BYTES);
  constexpr int kValuesPerRound = kPairs ? kStageBytes / (VALUE_BYTES > 0 ? VALUE_BYTES : 1) : 1;
  constexpr int kRounds = kPairs ? (kTile + kValuesPerRound - 1) / kValuesPerRound : 0;

  __shared__ uint32_t s_wave_hist[kSortWaves][kRadix];
  __shared__ uint32_t s_global_off[kRadix];
  __shared__ uint32_t s_scan[kRadix / kWaveSize];
  __shared__ int s_tile;
  __shared__ __attribute__((aligned(16))) unsigned char s_stage[kStageBytes];
  K* s_keys = reinterpret_cast<K*>(s_stage);
  Val* s_vals = reinterpret_cast<Val*>(s_stage);

  if (plan->skip[pass]) return;
  const bool src_alt = plan->src_is_alt[pass] != 0;
  const K* src_keys = src_alt ? keys_b : keys_a;
  K* dst_keys = src_alt ? keys_a : keys_b;
  const Val* src_vals = src_alt ? vals_b : vals_a;
  Val* dst_vals = src_alt ? vals_a : vals_b;
  const bool make_index = kPairs && values_from_index &&
                          plan->first_executed == (uint32_t)pass;
  const int shift = pass * 8;
  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int wave = tid / kWaveSize;

  while (true) {
    if (tid == 0) s_tile = (int)atomicAdd(ticket, 1u);
    for (int i = tid; i < kSortWaves * kRadix; i += kSortBlock)
      (&s_wave_hist[0][0])[i] = 0u;
    __syncthreads();
    const int tile = s_tile;
    if (tile >= num_tiles) break;

    const int64_t tile_base = (int64_t)tile * kTile;
    const int64_t remaining = n - tile_base;
    const int valid = remaining < kTile ? (int)remaining : kTile;
    const int wave_first = wave * (kWaveSize * kItems) + lane;

    K key[kItems];
    Val val[kPairs ? kItems : 1];
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const int local = wave_first + j * kWaveSize;
      if (local < valid) {
        key[j] = src_keys[tile_base + local];
        if constexpr (kPairs) {
          if (make_index) {
            if constexpr (VALUE_BYTES == 4) val[j] = (Val)(uint32_t)(tile_base + local);
            else if constexpr (VALUE_BYTES == 8) val[j] = (Val)(uint64_t)(tile_base + local);
          } else {
            val[j] = src_vals[tile_base + local];
          }
        }
      } else {
        key[j] = 0;
      }
    }

    // Rank every key among the keys of its wave that share its digit; keys
    // past the end of the input take digit 255 and, coming last in memory
    // order, rank behind every real key.
    uint32_t rank[kItems];
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const int local = wave_first + j * kWaveSize;
      const uint32_t d = local < valid ? digit_of(key[j], xf, shift) : (kRadix - 1);
      const uint64_t peers = match_digit(d);
      const uint32_t below = (uint32_t)mbcnt(peers);
      const uint32_t prev = s_wave_hist[wave][d];
      if (below == 0) s_wave_hist[wave][d] = prev + (uint32_t)__popcll(peers);
      rank[j] = prev + below;
    }
    __syncthreads();

    // One thread per digit: totals over the waves, look-back over the tiles.
    uint32_t count = 0, inc = 0;
    uint32_t* tile_status = status + (int64_t)tile * kRadix;
    if (tid < kRadix) {
#pragma unroll
      for (int w = 0; w < kSortWaves; ++w) {
        const uint32_t t = s_wave_hist[w][tid];
        s_wave_hist[w][tid] = count;
        count += t;
      }
      __hip_atomic_store(&tile_status[tid],
                         (tile == 0 ? kStatusPrefix : kStatusAggregate) | count,
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
    if (tid < kRadix) {
      uint32_t digit_start = inc - count;
      for (int w = 0; w < wave; ++w) digit_start += s_scan[w];
#pragma unroll
      for (int w = 0; w < kSortWaves; ++w) s_wave_hist[w][tid] += digit_start;

      uint32_t before = 0;  // keys with this digit in earlier tiles
      for (int t = tile - 1; t >= 0; --t) {
        uint32_t s;
        while (true) {
          s = __hip_atomic_load(&status[(int64_t)t * kRadix + tid],
                                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if ((s & ~kStatusValueMask) != 0) break;
          __builtin_amdgcn_s_sleep(1);
        }
        before += s & kStatusValueMask;
        if ((s & ~kStatusValueMask) == kStatusPrefix) break;
      }
      if (tile > 0)
        __hip_atomic_store(&tile_status[tid], kStatusPrefix | (before + count),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_global_off[tid] = excl[pass * kRadix + tid] + before - digit_start;
    }
    __syncthreads();

    // Tile-local position of every key, then the keys in digit order in LDS.
    uint32_t pos[kItems];
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const int local = wave_first + j * kWaveSize;
      const uint32_t d = local < valid ? digit_of(key[j], xf, shift) : (kRadix - 1);
      pos[j] = s_wave_hist[wave][d] + rank[j];
      s_keys[pos[j]] = key[j];
    }
    __syncthreads();

    uint32_t gpos[kPairs ? kItems : 1];
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const int i = j * kSortBlock + tid;
      if (i < valid) {
        const K k = s_keys[i];
        const uint32_t g = s_global_off[digit_of(k, xf, shift)] + (uint32_t)i;
        dst_keys[g] = k;
        if constexpr (kPairs) gpos[j] = g;
      }
    }

    if constexpr (kPairs) {
#pragma unroll
      for (int r = 0; r < kRounds; ++r) {
        const uint32_t lo = (uint32_t)r * kValuesPerRound;
        __syncthreads();  // the stage buffer is free again
#pragma unroll
        for (int j = 0; j < kItems; ++j)
          if (pos[j] - lo < (uint32_t)kValuesPerRound) s_vals[pos[j] - lo] = val[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
          const uint32_t i = (uint32_t)(j * kSortBlock + tid);
          if (i < (uint32_t)valid && i - lo < (uint32_t)kValuesPerRound)
            dst_vals[gpos[j]] = s_vals[i - lo];
        }
      }
    }
    __syncthreads();  // LDS is reused by the next tile
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
  using Val = typename ValueOf<VALUE_BYTES>::type;
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
      if constexpr (VALUE_BYTES == 4) vals_a[i] = (Val)(uint32_t)i;
      else if constexpr (VALUE_BYTES == 8) vals_a[i] = (Val)(uint64_t)i;
    }
  }
}

// ---- host side -------------------------------------------------------------
struct TempLayout {
  int64_t alt_keys, alt_vals, excl, plan, zero_begin, hist, tickets, status,
      status_stride, total;
  int64_t tiles;
};

TempLayout make_layout(int64_t n, int key_bytes, int value_bytes) {
  TempLayout L;
  const int64_t tile = key_bytes == 8 ? tile_keys<8>() : tile_keys<4>();
  L.tiles = div_up(n, tile);
  int64_t off = 0;
  L.alt_keys = off; off += align_up(n * key_bytes, 256);
  L.alt_vals = off; off += align_up(n * value_bytes, 256);
  L.excl = off; off += kMaxPasses * kRadix * 4;
  L.plan = off; off += 256;
  L.zero_begin = off;
  L.hist = off; off += kMaxPasses * kRadix * 4;
  L.tickets = off; off += 256;
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
  KeyXform xf{0, kModePlain};
  switch (key_type) {
    case ILGPU_HIP_I8: case ILGPU_HIP_I16: case ILGPU_HIP_I32: case ILGPU_HIP_I64:
      xf.xor_mask = sign;
      break;
    case ILGPU_HIP_F16: case ILGPU_HIP_F32: case ILGPU_HIP_F64:
      if (flags & ILGPU_HIP_SORT_FLOAT_TOTAL_ORDER) {
        xf.xor_mask = sign;
        xf.mode = kModeFloatTotalOrder;
      } else {
        // Half: (uint)~bits >> 15 keeps the sign-extended upper ones, so bits
        // 1..15 are always flipped (RadixSortOperations.tt:77-80).
        xf.xor_mask = key_type == ILGPU_HIP_F16 ? 0xFFFEull : sign;
        xf.mode = kModeFloatReference;
      }
      break;
    default:
      break;
  }
  if (flags & ILGPU_HIP_SORT_DESCENDING) xf.xor_mask ^= all;
  return xf;
}

template <int KEY_BYTES, int VALUE_BYTES>
int32_t launch_sized(hipStream_t stream, const SortArgs& a) {
  using K = typename KeyOf<KEY_BYTES>::type;
  using Val = typename ValueOf<VALUE_BYTES>::type;
  const TempLayout L = make_layout(a.n, KEY_BYTES, VALUE_BYTES);
  char* base = reinterpret_cast<char*>(align_up((int64_t)(uintptr_t)a.temp, 256));
  K* keys_a = static_cast<K*>(a.keys);
  K* keys_b = reinterpret_cast<K*>(base + L.alt_keys);
  Val* vals_a = static_cast<Val*>(a.values);
  Val* vals_b = reinterpret_cast<Val*>(base + L.alt_vals);
  uint32_t* excl = reinterpret_cast<uint32_t*>(base + L.excl);
  SortPlan* plan = reinterpret_cast<SortPlan*>(base + L.plan);
  uint32_t* hist = reinterpret_cast<uint32_t*>(base + L.hist);
  uint32_t* tickets = reinterpret_cast<uint32_t*>(base + L.tickets);
  const KeyXform xf = make_xform(a.key_type, a.flags);
  const int passes = KEY_BYTES;
  const int cus = device_cu_count();
  const int from_index = a.value_source == ILGPU_HIP_VALUES_FROM_INDEX ? 1 : 0;

  int32_t rc = launch_zero_words(stream, hist, (L.total - L.zero_begin) / 4);
  if (rc != ILGPU_HIP_SUCCESS) return rc;

  {
    int shift = 0;  // replicas: 32 KiB of LDS counters
    while ((1 << (shift + 1)) <= 32 &&
           ((passes * kRadix) << (shift + 1)) <= 8192)
      ++shift;
    const size_t lds = (size_t)((passes * kRadix) << shift) * 4;
    int64_t blocks = div_up(div_up(a.n, Vec16<K>::N), kHistBlock);
    if (blocks > (int64_t)cus * 4) blocks = (int64_t)cus * 4;
    if (blocks < 1) blocks = 1;
    ProfileScope scope(stream, "sort_histogram");
    hipLaunchKernelGGL((sort_histogram_kernel<K>), dim3((unsigned)blocks),
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

  int per_cu = 0;
  ILGPU_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(
      &per_cu, onesweep_kernel<KEY_BYTES, VALUE_BYTES>, kSortBlock, 0));
  if (per_cu < 1) per_cu = 1;
  int64_t grid = (int64_t)cus * per_cu;
  if (grid > L.tiles) grid = L.tiles;
  for (int p = 0; p < passes; ++p) {
    uint32_t* status =
        reinterpret_cast<uint32_t*>(base + L.status + (int64_t)p * L.status_stride);
    {
      ProfileScope scope(stream, "sort_onesweep");
      hipLaunchKernelGGL((onesweep_kernel<KEY_BYTES, VALUE_BYTES>),
                         dim3((unsigned)grid), dim3(kSortBlock), 0, stream,
                         keys_a, keys_b, vals_a, vals_b, a.n, p, xf, excl,
                         status, tickets + p, plan, (int)L.tiles, from_index);
    }
    ILGPU_HIP_CHECK(hipGetLastError());
  }
  {
    int64_t blocks = div_up(a.n, 256);
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

int64_t radix_sort_max_length() { return kMaxSortLength; }

int64_t radix_sort_temp_bytes(int64_t n, int key_bytes, int value_bytes) {
  return 256 + make_layout(n, key_bytes, value_bytes).total;
}

int32_t launch_radix_sort(hipStream_t stream, const SortArgs& a) {
  switch (elem_size(a.key_type)) {
    case 1: return launch_value<1>(stream, a);
    case 2: return launch_value<2>(stream, a);
    case 4: return launch_value<4>(stream, a);
    case 8: return launch_value<8>(stream, a);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace ilgpu_hip
