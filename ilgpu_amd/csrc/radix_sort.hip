// Radix sort: what does not depend on the key size — process-wide parameters,
// the device self-test of the LDS property the ranking rests on, strided
// views, temp sizing and the dispatch to the translation units of the key
// sizes (radix_sort_k1/2/4/8.hip, which instantiate radix_sort_impl.hpp).
#include "radix_sort_impl.hpp"

namespace ilgpu_hip {

std::atomic<uint32_t> g_sort_spin_limit{kDefaultSpinLimit};
std::atomic<int32_t> g_sort_large_min_tiles_per_cu{-1};
std::atomic<int32_t> g_sort_short_tile_max_tiles{-1};
std::atomic<int32_t> g_sort_small_kernel{1};
// Test hook: -1 = ask the device (the default), 0 / 1 = every device is taken
// to have failed / passed the check of its LDS atomics.
std::atomic<int32_t> g_sort_assume_lds_order{-1};

// radix_sort_k<bytes>.hip
int32_t launch_sort_key_bytes_1(hipStream_t stream, const SortArgs& a);
int32_t launch_sort_key_bytes_2(hipStream_t stream, const SortArgs& a);
int32_t launch_sort_key_bytes_4(hipStream_t stream, const SortArgs& a);
int32_t launch_sort_key_bytes_8(hipStream_t stream, const SortArgs& a);

namespace {

// ---- device check of the LDS property the ranking rests on -------------------
// Every wave keeps 256 counters and plays `rows` ranking rows on pseudo-random
// digits drawn from `distinct` values: one returning LDS add per lane, then the
// rank a lane got is compared with the rank memory order demands (count before
// the row + lanes below it with the same digit, from eight ballots).  Lanes
// served out of order are counted into *mismatches.
__global__ __launch_bounds__(kSortBlock) void lds_atomic_order_kernel(
    int rows, uint32_t distinct, uint64_t seed, unsigned long long* mismatches) {
  __shared__ uint32_t s_counter[(kSortBlock / kWaveSize) * kRadix];
  const int tid = threadIdx.x;
  for (int i = tid; i < (kSortBlock / kWaveSize) * kRadix; i += kSortBlock) s_counter[i] = 0u;
  __syncthreads();
  uint32_t* mine = s_counter + (tid / kWaveSize) * kRadix;
  unsigned long long wrong = 0;
  for (int r = 0; r < rows; ++r) {
    uint64_t z = seed + ((uint64_t)blockIdx.x << 40) + ((uint64_t)r << 12) + (uint64_t)tid;
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const uint32_t d = (uint32_t)(z % distinct) * ((uint32_t)kRadix / distinct);
    uint64_t peers = ~0ull;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const bool bit = ((d >> b) & 1u) != 0;
      const uint64_t m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    const uint32_t before =
        __hip_atomic_load(mine + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const uint32_t rank =
        __hip_atomic_fetch_add(mine + d, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (rank != before + (uint32_t)mbcnt(peers)) ++wrong;
  }
  if (wrong != 0) atomicAdd(mismatches, wrong);
}


// What the check found, per device: 0 = not asked yet, 1 = lanes served in
// order, 2 = not.  The counter the check kernels add to is a device array of
// the library, so the check allocates nothing.
std::atomic<int> g_lds_order_state[kMaxCachedDevices];
__device__ __align__(8) unsigned long long g_lds_order_mismatches[2];

// ---- strided views ------------------------------------------------------------
// Stride1D.General with an element stride above one: the view is gathered
// into a dense staging copy behind the dense sort's temp area, sorted there
// and scattered back; elements between the strided ones are never touched.
template <typename E>
__global__ __launch_bounds__(256) void gather_strided_kernel(
    const E* __restrict__ src, int64_t stride, E* __restrict__ dst, int64_t n) {
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step)
    dst[i] = src[i * stride];
}

template <typename E>
__global__ __launch_bounds__(256) void scatter_strided_kernel(
    const E* __restrict__ src, E* __restrict__ dst, int64_t stride, int64_t n) {
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step)
    dst[i * stride] = src[i];
}

template <typename E>
int32_t copy_strided(hipStream_t stream, bool gather, void* strided, int64_t stride,
                     void* dense, int64_t n) {
  int64_t blocks = div_up(n, 256);
  const int64_t cap = (int64_t)device_cu_count() * 8;
  if (blocks > cap) blocks = cap;
  ProfileScope scope(stream, gather ? "sort_gather" : "sort_scatter");
  if (gather)
    hipLaunchKernelGGL((gather_strided_kernel<E>), dim3((unsigned)blocks), dim3(256), 0,
                       stream, static_cast<const E*>(strided), stride,
                       static_cast<E*>(dense), n);
  else
    hipLaunchKernelGGL((scatter_strided_kernel<E>), dim3((unsigned)blocks), dim3(256), 0,
                       stream, static_cast<const E*>(dense), static_cast<E*>(strided),
                       stride, n);
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

int32_t copy_strided_bytes(hipStream_t stream, bool gather, int elem_bytes, void* strided,
                           int64_t stride, void* dense, int64_t n) {
  switch (elem_bytes) {
    case 1: return copy_strided<uint8_t>(stream, gather, strided, stride, dense, n);
    case 2: return copy_strided<uint16_t>(stream, gather, strided, stride, dense, n);
    case 4: return copy_strided<uint32_t>(stream, gather, strided, stride, dense, n);
    case 8: return copy_strided<uint64_t>(stream, gather, strided, stride, dense, n);
    case 16: return copy_strided<Bytes16>(stream, gather, strided, stride, dense, n);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

int32_t launch_dense(hipStream_t stream, const SortArgs& a) {
  switch (elem_size(a.key_type)) {
    case 1: return launch_sort_key_bytes_1(stream, a);
    case 2: return launch_sort_key_bytes_2(stream, a);
    case 4: return launch_sort_key_bytes_4(stream, a);
    case 8: return launch_sort_key_bytes_8(stream, a);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace

void set_sort_parameter(int32_t parameter, int32_t value) {
  if (parameter == ILGPU_HIP_SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER) {
    g_sort_assume_lds_order.store(value < 0 ? -1 : (value == 0 ? 0 : 1), std::memory_order_relaxed);
    if (value < 0)  // and ask the devices again
      for (auto& state : g_lds_order_state) state.store(0, std::memory_order_relaxed);
  } else if (parameter == ILGPU_HIP_SORT_PARAM_LOOKBACK_SPIN_LIMIT)
    g_sort_spin_limit.store(value < 0 ? kDefaultSpinLimit : (uint32_t)value, std::memory_order_relaxed);
  else if (parameter == ILGPU_HIP_SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU)
    g_sort_large_min_tiles_per_cu.store(value < 0 ? -1 : value, std::memory_order_relaxed);
  else if (parameter == ILGPU_HIP_SORT_PARAM_SHORT_TILE_MAX_TILES)
    g_sort_short_tile_max_tiles.store(value < 0 ? -1 : value, std::memory_order_relaxed);
  else
    g_sort_small_kernel.store(value == 0 ? 0 : 1, std::memory_order_relaxed);
}

int32_t launch_lds_atomic_order_selftest(hipStream_t stream, int rows, int64_t* mismatches) {
  int32_t rc = launch_zero_words(stream, reinterpret_cast<uint32_t*>(mismatches), 2);
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  const int blocks = device_cu_count() * 4;  // every CU busy with several blocks
  const uint32_t distinct[] = {1u, 2u, 4u, 16u, 64u, 256u};
  for (int i = 0; i < 6; ++i) {
    hipLaunchKernelGGL(lds_atomic_order_kernel, dim3((unsigned)blocks), dim3(kSortBlock), 0,
                       stream, rows, distinct[i], 0x1234ull + (uint64_t)i,
                       reinterpret_cast<unsigned long long*>(mismatches));
    ILGPU_HIP_CHECK(hipGetLastError());
  }
  return ILGPU_HIP_SUCCESS;
}

// Every sort goes through here first.  The ranking of a pass is stable only if
// the lanes of one returning LDS atomic that meet in one address are served in
// lane order, which the hardware does and no document promises: the first sort
// on a device plays the check kernels once (some tens of microseconds and one
// wait for the stream) and the answer is kept per device; a device that fails
// is refused rather than sorted wrongly.
int32_t check_sort_device(hipStream_t stream) {
  const int32_t assumed = g_sort_assume_lds_order.load(std::memory_order_relaxed);
  if (assumed >= 0) return assumed ? ILGPU_HIP_SUCCESS : ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int device = current_device();
  std::atomic<int>* state =
      device >= 0 && device < kMaxCachedDevices ? &g_lds_order_state[device] : nullptr;
  const int known = state ? state->load(std::memory_order_acquire) : 0;
  if (known == 1) return ILGPU_HIP_SUCCESS;
  if (known == 2) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  // The answer has to come back to the host, which a stream that is being
  // captured cannot give: such callers check the device before they capture.
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) == hipSuccess &&
      capturing != hipStreamCaptureStatusNone)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  void* counter = nullptr;
  ILGPU_HIP_CHECK(hipGetSymbolAddress(&counter, HIP_SYMBOL(g_lds_order_mismatches)));
  const int32_t rc =
      launch_lds_atomic_order_selftest(stream, 64, static_cast<int64_t*>(counter));
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  unsigned long long mismatches = ~0ull;
  ILGPU_HIP_CHECK(hipMemcpyAsync(&mismatches, counter, sizeof(mismatches), hipMemcpyDeviceToHost,
                                 stream));
  ILGPU_HIP_CHECK(hipStreamSynchronize(stream));
  if (state) state->store(mismatches == 0 ? 1 : 2, std::memory_order_release);
  return mismatches == 0 ? ILGPU_HIP_SUCCESS : ILGPU_HIP_ERROR_NOT_SUPPORTED;
}

int32_t read_sort_plan(hipStream_t stream, const void* temp, int64_t n, int key_bytes,
                       int value_bytes, int32_t* executed, int32_t* skipped) {
  // Inputs of one tile are sorted by one block without a plan: every pass runs.
  if (n <= (int64_t)tile_keys(key_bytes, value_bytes, kSortBlock) &&
      g_sort_small_kernel.load(std::memory_order_relaxed) != 0) {
    *executed = key_bytes;
    *skipped = 0;
    return ILGPU_HIP_SUCCESS;
  }
  const TempLayout L = make_layout(n, key_bytes, value_bytes);
  const char* base = reinterpret_cast<const char*>(align_up((int64_t)(uintptr_t)temp, 256));
  SortPlan plan;
  ILGPU_HIP_CHECK(hipMemcpyAsync(&plan, base + L.plan, sizeof(plan), hipMemcpyDeviceToHost,
                                 stream));
  ILGPU_HIP_CHECK(hipStreamSynchronize(stream));
  *executed = (int32_t)plan.executed;
  *skipped = key_bytes - (int32_t)plan.executed;
  return ILGPU_HIP_SUCCESS;
}

int64_t radix_sort_max_length() { return kMaxSortLength; }

int64_t radix_sort_temp_bytes(int64_t n, int key_bytes, int value_bytes,
                              int64_t key_stride, int64_t value_stride) {
  int64_t total = 256 + make_layout(n, key_bytes, value_bytes).total;
  if (key_stride != 1 || (value_bytes > 0 && value_stride != 1)) {
    total = align_up(total, 256);
    if (key_stride != 1) total += align_up(n * key_bytes, 256);
    if (value_bytes > 0 && value_stride != 1) total += align_up(n * value_bytes, 256);
  }
  return total;
}

int32_t launch_radix_sort(hipStream_t stream, const SortArgs& a) {
  const int32_t checked = check_sort_device(stream);
  if (checked != ILGPU_HIP_SUCCESS) return checked;
  const bool has_values = a.values != nullptr && a.value_bytes > 0;
  const bool keys_strided = a.key_stride != 1;
  const bool values_strided = has_values && a.value_stride != 1;
  if (!keys_strided && !values_strided) return launch_dense(stream, a);

  const int kb = elem_size(a.key_type);
  char* base = reinterpret_cast<char*>(align_up((int64_t)(uintptr_t)a.temp, 256));
  char* staging = base + align_up(make_layout(a.n, kb, a.value_bytes).total, 256);
  SortArgs dense = a;
  dense.key_stride = 1;
  dense.value_stride = 1;
  int32_t rc;
  if (keys_strided) {
    dense.keys = staging;
    staging += align_up(a.n * kb, 256);
    rc = copy_strided_bytes(stream, true, kb, a.keys, a.key_stride, dense.keys, a.n);
    if (rc != ILGPU_HIP_SUCCESS) return rc;
  }
  if (values_strided) {
    dense.values = staging;
    if (a.value_source == ILGPU_HIP_VALUES_FROM_VIEW) {
      rc = copy_strided_bytes(stream, true, a.value_bytes, a.values, a.value_stride,
                              dense.values, a.n);
      if (rc != ILGPU_HIP_SUCCESS) return rc;
    }
  }
  rc = launch_dense(stream, dense);
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  if (keys_strided) {
    rc = copy_strided_bytes(stream, false, kb, a.keys, a.key_stride, dense.keys, a.n);
    if (rc != ILGPU_HIP_SUCCESS) return rc;
  }
  if (values_strided)
    rc = copy_strided_bytes(stream, false, a.value_bytes, a.values, a.value_stride,
                            dense.values, a.n);
  return rc;
}

}  // namespace ilgpu_hip
