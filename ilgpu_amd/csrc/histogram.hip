// Histogram: bins[locator(v)] += 1 for every input element.
//
// Stands in for HistogramKernel / HistogramUncheckedKernel and the launchers
// (HistogramExtensions.cs:176-354, HistogramLaunchers.tt:52-101).  The
// reference issues one global atomic per element (HistogramOperations.tt:
// 36-40); here each block counts into a private LDS histogram and adds each
// non-zero bin to the global bins once.
//
// LDS layout: R replicas of every bin, word index = bin * R + (lane % R).
// With R = 32 a wave's 64 LDS atomics land in 32 different banks whatever the
// data (uniform, skewed or constant), so neither bank conflicts nor
// same-address serialisation depend on the input.  R is the largest power of
// two <= 32 for which num_bins * R counters fit in 48 KiB; histograms with
// more than 12288 bins fall through to global atomics per element.
//
// Overflow (checked variant): the reference flags an increment that saw
// old == MaxValue.  A bulk add of c > 0 to a bin holding `old` passes through
// MaxValue exactly when old + c, in wider arithmetic, exceeds it.
//
// Algorithmic HBM traffic: n * sizeof(T) bytes read; bins are negligible.
#include "kernels.hpp"

namespace ilgpu_hip {

namespace {

constexpr int kBlock = 512;
constexpr int kUnroll = 2;
constexpr int kLdsBudgetWords = 12288;  // 48 KiB of counters per block
constexpr int kMaxReplicas = 32;

// ---- bin locators ---------------------------------------------------------
// IDENTITY: bin = (int)value.  MODULO: |value % num_bins| with the sign of the
// dividend (C# remainder; HistogramTests.tt:83-94), i.e. |value| mod num_bins;
// floating point uses fmod.
template <typename T, int LOC>
__device__ __forceinline__ int64_t locate(T v, int num_bins) {
  if constexpr (LOC == ILGPU_HIP_LOCATOR_IDENTITY) {
    if constexpr (is_fp<T>::value) {
      // Saturating conversion keeps NaN/inf/huge values out of range.
      if (!(v > (T)-1 && v < (T)2147483648.0)) return -1;
      return (int64_t)(int32_t)v;
    } else if constexpr (sizeof(T) == 8) {
      if constexpr (T(-1) < T(0)) return (int64_t)v;
      else return v > (T)INT64_MAX ? -1 : (int64_t)v;
    } else {
      return (int64_t)v;
    }
  } else {
    if constexpr (is_fp<T>::value) {
      T r = sizeof(T) == 4 ? (T)fmodf((float)v, (float)num_bins)
                           : (T)fmod((double)v, (double)num_bins);
      r = r < 0 ? -r : r;
      if (!(r >= 0)) return -1;  // NaN
      return (int64_t)(int32_t)r;
    } else if constexpr (sizeof(T) == 8) {
      uint64_t mag;
      if constexpr (T(-1) < T(0)) mag = v < 0 ? (uint64_t)0 - (uint64_t)v : (uint64_t)v;
      else mag = (uint64_t)v;
      return (int64_t)(mag % (uint64_t)num_bins);
    } else {
      const int64_t w = (int64_t)v;
      const uint32_t mag = (uint32_t)(w < 0 ? -w : w);
      return (int64_t)(mag % (uint32_t)num_bins);
    }
  }
}

template <typename B> struct BinTraits;
template <> struct BinTraits<int32_t> {
  static __device__ __forceinline__ bool passes_max(int32_t old, uint32_t c) {
    return (int64_t)old + (int64_t)c > (int64_t)INT32_MAX;
  }
};
template <> struct BinTraits<uint32_t> {
  static __device__ __forceinline__ bool passes_max(uint32_t old, uint32_t c) {
    return (uint64_t)old + (uint64_t)c > (uint64_t)UINT32_MAX;
  }
};
template <> struct BinTraits<int64_t> {
  static __device__ __forceinline__ bool passes_max(int64_t old, uint32_t c) {
    return old > INT64_MAX - (int64_t)c;
  }
};
template <> struct BinTraits<uint64_t> {
  static __device__ __forceinline__ bool passes_max(uint64_t old, uint32_t c) {
    return old > UINT64_MAX - (uint64_t)c;
  }
};

// Adds c to bins[b] as bin type B; returns whether the add passed MaxValue.
template <typename B>
__device__ __forceinline__ bool add_to_bin(void* bins, int64_t b, uint32_t c,
                                           bool checked) {
  if constexpr (sizeof(B) == 4) {
    uint32_t* p = static_cast<uint32_t*>(bins) + b;
    if (!checked) {
      __hip_atomic_fetch_add(p, c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
    const uint32_t old = __hip_atomic_fetch_add(p, c, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
    return BinTraits<B>::passes_max((B)old, c);
  } else {
    uint64_t* p = static_cast<uint64_t*>(bins) + b;
    if (!checked) {
      __hip_atomic_fetch_add(p, (uint64_t)c, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
    const uint64_t old = __hip_atomic_fetch_add(p, (uint64_t)c, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
    return BinTraits<B>::passes_max((B)old, c);
  }
}

// ---- floating-point bins ------------------------------------------------------
// The reference adds 1.0 to a float or double bin once per element, each
// addition rounded in the bin's precision (Atomic.Add(ref target, 1),
// HistogramOperations.tt:36-40), so a float bin stops growing at 2^24.  Every
// increment is the same function x -> fl(x + 1), so the value of a bin after c
// of them does not depend on their order, and add_ones gives exactly that
// value without c additions: inside a binade whose spacing is at most one,
// steps of one are exact (x, 1 and x + 1 are multiples of the spacing), so
// whole runs of steps up to the top of the binade (or, for negative values,
// down to magnitude below one) are taken at once; the steps that can round —
// into a coarser binade, across zero, beyond 2^24 or 2^53 — are single
// additions in hardware.
template <typename F>
__device__ __forceinline__ F add_ones(F x, uint32_t c) {
  constexpr int kDigits = sizeof(F) == 4 ? 24 : 53;
  const F limit = (F)(1ull << kDigits);
  if (x != x) return x;  // NaN stays NaN
  while (c > 0) {
    const F y = x + (F)1;
    if (y == x) return x;  // stuck: the spacing has outgrown one (or x is infinite)
    uint32_t k = 1;
    F next = y;
    const F ax = x < (F)0 ? -x : x;
    if (ax >= (F)1 && ax < limit) {
      uint64_t whole;
      if (x > (F)0) {
        int e;
        if constexpr (sizeof(F) == 4) (void)frexpf(x, &e);
        else (void)frexp(x, &e);
        F top;  // 2^e: the first value of the next binade, above x
        if constexpr (sizeof(F) == 4) top = ldexpf(1.0f, e);
        else top = ldexp(1.0, e);
        whole = (uint64_t)(top - x);  // steps that end at or below it
      } else {
        whole = (uint64_t)ax;         // steps that end at or below zero
      }
      if (whole >= 1) {
        k = whole < (uint64_t)c ? (uint32_t)whole : c;
        next = x + (F)k;  // exact
      }
    }
    x = next;
    c -= k;
  }
  return x;
}

// Adds c ones to the floating-point bin b; returns whether an increment found
// the bin at MaxValue (only a bin that holds MaxValue already: it is not
// reachable by steps of one).
template <typename F, typename U>
__device__ __forceinline__ bool add_to_fp_bin(void* bins, int64_t b, uint32_t c,
                                              bool checked) {
  const F max_value = sizeof(F) == 4 ? (F)3.402823466e+38f : (F)1.7976931348623157e+308;
  if (c == 1u) {
    // One element: the hardware's floating-point add in L2 is the reference's
    // operation itself (one addition of 1.0, rounded in the bin's precision),
    // and it does not retry: many elements for one bin do not starve each
    // other as compare-and-swap loops would.
    const F before = unsafeAtomicAdd(static_cast<F*>(bins) + b, (F)1);
    return checked && before == max_value;
  }
  U* p = static_cast<U*>(bins) + b;
  U old = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
    F x;
    __builtin_memcpy(&x, &old, sizeof(F));
    const F y = add_ones<F>(x, c);
    U desired;
    __builtin_memcpy(&desired, &y, sizeof(F));
    if (desired == old) break;  // nothing to store
    if (__hip_atomic_compare_exchange_strong(p, &old, desired, __ATOMIC_RELAXED,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      break;
  }
  F before;
  __builtin_memcpy(&before, &old, sizeof(F));
  return checked && before == max_value;
}

__device__ __forceinline__ bool add_to_bin_dyn(int bin_type, void* bins,
                                               int64_t b, uint32_t c,
                                               bool checked) {
  switch (bin_type) {
    case ILGPU_HIP_I32: return add_to_bin<int32_t>(bins, b, c, checked);
    case ILGPU_HIP_U32: return add_to_bin<uint32_t>(bins, b, c, checked);
    case ILGPU_HIP_I64: return add_to_bin<int64_t>(bins, b, c, checked);
    case ILGPU_HIP_F32: return add_to_fp_bin<float, uint32_t>(bins, b, c, checked);
    case ILGPU_HIP_F64: return add_to_fp_bin<double, uint64_t>(bins, b, c, checked);
    default: return add_to_bin<uint64_t>(bins, b, c, checked);
  }
}

// RANGE_CHECK = false when every value of T is a valid bin (e.g. u8 into
// >= 256 bins with the identity locator).
template <typename T, int LOC, bool RANGE_CHECK>
__global__ __launch_bounds__(kBlock) void histogram_lds_kernel(
    const T* __restrict__ in, int64_t n, int64_t in_stride, void* bins,
    int num_bins, int bin_type, int32_t* overflow, int replica_shift) {
  using V = typename Vec16<T>::type;
  constexpr int VN = Vec16<T>::N;
  extern __shared__ uint32_t s_counts[];
  __shared__ int s_overflow;

  const int words = num_bins << replica_shift;
  for (int i = threadIdx.x; i < words; i += kBlock) s_counts[i] = 0u;
  if (threadIdx.x == 0) s_overflow = 0;
  __syncthreads();

  const uint32_t replica = threadIdx.x & ((1u << replica_shift) - 1u);
  auto count = [&](T v) {
    const int64_t b = locate<T, LOC>(v, num_bins);
    if (!RANGE_CHECK || (uint64_t)b < (uint64_t)num_bins)
      atomicAdd(&s_counts[((uint32_t)b << replica_shift) + replica], 1u);
  };

  const uintptr_t addr = reinterpret_cast<uintptr_t>(in);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(T));
  if (head > n) head = n;
  const V* body = reinterpret_cast<const V*>(in + head);
  int64_t nvec = (n - head) / VN;
  int64_t tail_start = head + nvec * VN;

  const int64_t stride = (int64_t)gridDim.x * kBlock;
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (in_stride != 1) {
    // Stride1D.General with an element stride above one: sample i lives at
    // in[i * in_stride]; one scalar load per sample, no vector body.
    for (int64_t e = i; e < n; e += stride) count(in[e * in_stride]);
    nvec = 0;
    head = 0;
    tail_start = n;
  }
  for (; i + (kUnroll - 1) * stride < nvec; i += kUnroll * stride) {
    V v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      v[u] = __builtin_nontemporal_load(&body[i + u * stride]);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int k = 0; k < VN; ++k) count(v[u][k]);
  }
  for (; i < nvec; i += stride) {
    V v = __builtin_nontemporal_load(&body[i]);
#pragma unroll
    for (int k = 0; k < VN; ++k) count(v[k]);
  }
  if (blockIdx.x == 0) {
    const int64_t extra = head + (n - tail_start);
    if ((int64_t)threadIdx.x < extra) {
      const int64_t idx = (int64_t)threadIdx.x < head
                              ? (int64_t)threadIdx.x
                              : tail_start + ((int64_t)threadIdx.x - head);
      count(in[idx]);
    }
  }
  __syncthreads();

  const bool checked = overflow != nullptr;
  bool passed = false;
  const int replicas = 1 << replica_shift;
  for (int b = threadIdx.x; b < num_bins; b += kBlock) {
    uint32_t c = 0;
    // Rotate the start so that neighbouring bins read different banks.
    for (int r = 0; r < replicas; ++r)
      c += s_counts[(b << replica_shift) + ((r + b) & (replicas - 1))];
    if (c != 0) passed |= add_to_bin_dyn(bin_type, bins, b, c, checked);
  }
  if (checked) {
    if (passed) s_overflow = 1;
    __syncthreads();
    if (threadIdx.x == 0 && s_overflow)
      __hip_atomic_fetch_or(overflow, 1, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
  }
}

// More bins than LDS holds: one global atomic per element, as the reference.
template <typename T, int LOC>
__global__ __launch_bounds__(kBlock) void histogram_global_kernel(
    const T* __restrict__ in, int64_t n, int64_t in_stride, void* bins,
    int64_t num_bins, int bin_type, int32_t* overflow) {
  const bool checked = overflow != nullptr;
  bool passed = false;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n;
       i += stride) {
    const int64_t b = locate<T, LOC>(in[i * in_stride], (int)num_bins);
    if ((uint64_t)b < (uint64_t)num_bins)
      passed |= add_to_bin_dyn(bin_type, bins, b, 1u, checked);
  }
  if (checked && __ballot(passed) != 0 && (threadIdx.x & (kWaveSize - 1)) == 0)
    __hip_atomic_fetch_or(overflow, 1, __ATOMIC_RELAXED,
                          __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T> constexpr double type_max_as_double();
template <> constexpr double type_max_as_double<int8_t>() { return 127.0; }
template <> constexpr double type_max_as_double<uint8_t>() { return 255.0; }
template <> constexpr double type_max_as_double<int16_t>() { return 32767.0; }
template <> constexpr double type_max_as_double<uint16_t>() { return 65535.0; }
template <> constexpr double type_max_as_double<int32_t>() { return 2147483647.0; }
template <> constexpr double type_max_as_double<uint32_t>() { return 4294967295.0; }
template <> constexpr double type_max_as_double<int64_t>() { return 9.3e18; }
template <> constexpr double type_max_as_double<uint64_t>() { return 1.9e19; }
template <> constexpr double type_max_as_double<float>() { return 3.5e38; }
template <> constexpr double type_max_as_double<double>() { return 1.7e308; }

template <typename T, int LOC>
int32_t launch_typed(hipStream_t stream, const void* in, int64_t n,
                     int64_t in_stride, void* bins, int64_t num_bins,
                     int32_t bin_type, int32_t* overflow) {
  const T* src = static_cast<const T*>(in);
  const int cus = device_cu_count();
  ProfileScope scope(stream, "histogram");
  if (num_bins > kLdsBudgetWords) {
    int64_t blocks = div_up(n, kBlock);
    if (blocks > (int64_t)cus * 4) blocks = (int64_t)cus * 4;
    hipLaunchKernelGGL((histogram_global_kernel<T, LOC>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, stream, src, n, in_stride, bins,
                       num_bins, bin_type, overflow);
    ILGPU_HIP_CHECK(hipGetLastError());
    return ILGPU_HIP_SUCCESS;
  }
  int shift = 0;
  while ((1 << (shift + 1)) <= kMaxReplicas &&
         (num_bins << (shift + 1)) <= kLdsBudgetWords)
    ++shift;
  const size_t lds_bytes = (size_t)(num_bins << shift) * sizeof(uint32_t);
  const int64_t nvec = n / Vec16<T>::N;
  int64_t blocks = div_up(nvec > 0 ? nvec : 1, kBlock);
  // 160 KiB of LDS per CU: as many resident blocks as fit, at most 3 (every
  // block flushes all of its bins with global atomics at the end: measured
  // 0.165 ms at 2 or 3 blocks per CU against 0.186 at 4 for 2^28 keys into
  // 4096 bins, and 0.182 against 0.188 for 2^30 bytes into 256 bins).
  int64_t per_cu = (int64_t)(160 * 1024) / (int64_t)(lds_bytes + 1024);
  if (per_cu > 3) per_cu = 3;
  if (per_cu < 1) per_cu = 1;
  if (blocks > cus * per_cu) blocks = cus * per_cu;
  // Values of T that cannot leave [0, num_bins) need no range check.
  const bool unsigned_small =
      LOC == ILGPU_HIP_LOCATOR_IDENTITY && !(T(-1) < T(0)) &&
      !is_fp<T>::value && type_max_as_double<T>() < (double)num_bins;
  const bool no_check = LOC == ILGPU_HIP_LOCATOR_MODULO ? !is_fp<T>::value
                                                        : unsigned_small;
  if (no_check) {
    hipLaunchKernelGGL((histogram_lds_kernel<T, LOC, false>),
                       dim3((unsigned)blocks), dim3(kBlock), lds_bytes, stream,
                       src, n, in_stride, bins, (int)num_bins, bin_type, overflow,
                       shift);
  } else {
    hipLaunchKernelGGL((histogram_lds_kernel<T, LOC, true>),
                       dim3((unsigned)blocks), dim3(kBlock), lds_bytes, stream,
                       src, n, in_stride, bins, (int)num_bins, bin_type, overflow,
                       shift);
  }
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

template <typename T>
int32_t launch_locator(hipStream_t stream, const void* in, int64_t n,
                       int64_t in_stride, void* bins, int64_t num_bins,
                       int32_t bin_type, int32_t locator, int32_t* overflow) {
  switch (locator) {
    case ILGPU_HIP_LOCATOR_IDENTITY:
      return launch_typed<T, ILGPU_HIP_LOCATOR_IDENTITY>(
          stream, in, n, in_stride, bins, num_bins, bin_type, overflow);
    case ILGPU_HIP_LOCATOR_MODULO:
      return launch_typed<T, ILGPU_HIP_LOCATOR_MODULO>(
          stream, in, n, in_stride, bins, num_bins, bin_type, overflow);
    default:
      return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace

int32_t launch_histogram(hipStream_t stream, const void* in, int64_t n,
                         int64_t in_stride, int32_t in_type, void* bins,
                         int64_t num_bins, int32_t bin_type, int32_t locator,
                         int32_t* overflow) {
#define ILGPU_HIP_HIST_CASE(CODE, T)                                      \
  case CODE:                                                              \
    return launch_locator<T>(stream, in, n, in_stride, bins, num_bins,    \
                             bin_type, locator, overflow)
  switch (in_type) {
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_I8, int8_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_I16, int16_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_I32, int32_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_I64, int64_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_U8, uint8_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_U16, uint16_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_U32, uint32_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_U64, uint64_t);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_F32, float);
    ILGPU_HIP_HIST_CASE(ILGPU_HIP_F64, double);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
#undef ILGPU_HIP_HIST_CASE
}

}  // namespace ilgpu_hip
