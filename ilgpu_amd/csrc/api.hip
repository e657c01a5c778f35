// C ABI of libilgpu_hip_algorithms.so: argument validation (mirroring the
// checks and exception kinds of the reference's host-side delegates) and
// dispatch to the kernel launchers.  No GPU work is enqueued when validation
// fails, and nothing here allocates device memory.
#include <atomic>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "kernels.hpp"

namespace ilgpu_hip {

namespace {
thread_local int32_t g_last_runtime_error = 0;
std::atomic<int> g_cu_count[kMaxCachedDevices];
}  // namespace

void set_last_runtime_error(hipError_t e) { g_last_runtime_error = (int32_t)e; }

int current_device() {
  int dev = -1;
  return hipGetDevice(&dev) == hipSuccess ? dev : -1;
}

int device_cu_count() {
  const int dev = current_device();
  const bool cacheable = dev >= 0 && dev < kMaxCachedDevices;
  if (cacheable) {
    const int cached = g_cu_count[dev].load(std::memory_order_relaxed);
    if (cached > 0) return cached;
  }
  int cus = 0;
  if (dev < 0 ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) !=
          hipSuccess ||
      cus <= 0)
    cus = 256;
  if (cacheable) g_cu_count[dev].store(cus, std::memory_order_relaxed);
  return cus;
}

// ---- per-kernel timing ------------------------------------------------------
namespace {
struct ProfileRecord {
  const char* name;
  hipEvent_t start, stop;
};
struct ProfileTotal {
  std::string name;
  int64_t launches;
  double total_ms;
};
std::atomic<bool> g_profiling{false};
std::mutex g_profile_mutex;
std::vector<ProfileRecord> g_profile_pending;
std::vector<ProfileTotal> g_profile_totals;

// Waits for every pending event pair and folds it into the totals.
void drain_profile_records() {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  for (const ProfileRecord& r : g_profile_pending) {
    float ms = 0.0f;
    if (hipEventSynchronize(r.stop) == hipSuccess &&
        hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
      ProfileTotal* t = nullptr;
      for (ProfileTotal& c : g_profile_totals)
        if (c.name == r.name) t = &c;
      if (t == nullptr) {
        g_profile_totals.push_back({r.name, 0, 0.0});
        t = &g_profile_totals.back();
      }
      t->launches += 1;
      t->total_ms += ms;
    }
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_profile_pending.clear();
}
}  // namespace

ProfileScope::ProfileScope(hipStream_t stream, const char* name)
    : stream_(stream), name_(name), start_(nullptr), active_(false) {
  if (!g_profiling.load(std::memory_order_relaxed)) return;
  if (hipEventCreate(&start_) != hipSuccess) return;
  if (hipEventRecord(start_, stream_) != hipSuccess) {
    (void)hipEventDestroy(start_);
    return;
  }
  active_ = true;
}

ProfileScope::~ProfileScope() {
  if (!active_) return;
  hipEvent_t stop = nullptr;
  if (hipEventCreate(&stop) != hipSuccess ||
      hipEventRecord(stop, stream_) != hipSuccess) {
    (void)hipEventDestroy(start_);
    if (stop) (void)hipEventDestroy(stop);
    return;
  }
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  g_profile_pending.push_back({name_, start_, stop});
}

namespace {

inline bool aligned_to(const void* p, int bytes) {
  return (reinterpret_cast<uintptr_t>(p) % (uintptr_t)bytes) == 0;
}

// A view is valid when it has a buffer and a positive length
// (ArrayView.IsValid, ArrayView.cs:261-265).
inline bool valid_view(const void* p, int64_t length) {
  return p != nullptr && length > 0;
}

// The checks TempViewManager makes on the caller's ArrayView<int> temp
// (TempViewManager.cs:33-41, 84-89).
inline int32_t check_temp(const void* temp, int64_t temp_bytes,
                          int64_t required) {
  if (temp == nullptr || temp_bytes <= 0) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!aligned_to(temp, 4)) return ILGPU_HIP_ERROR_UNALIGNED_TEMP;
  if (temp_bytes < required) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  return ILGPU_HIP_SUCCESS;
}

inline bool scan_reduce_type(int32_t t) {
  return t == ILGPU_HIP_I32 || t == ILGPU_HIP_I64 || t == ILGPU_HIP_U32 ||
         t == ILGPU_HIP_U64 || t == ILGPU_HIP_F32 || t == ILGPU_HIP_F64;
}

inline bool valid_op(int32_t op) {
  return op == ILGPU_HIP_OP_ADD || op == ILGPU_HIP_OP_MAX ||
         op == ILGPU_HIP_OP_MIN;
}

}  // namespace
}  // namespace ilgpu_hip

using namespace ilgpu_hip;

extern "C" {

int32_t ilgpu_hip_version(void) { return ILGPU_HIP_ALGORITHMS_VERSION; }

const char* ilgpu_hip_status_string(int32_t status) {
  switch (status) {
    case ILGPU_HIP_SUCCESS: return "success";
    case ILGPU_HIP_ERROR_NULL_VIEW: return "invalid (null or empty) view";
    case ILGPU_HIP_ERROR_OUT_OF_RANGE: return "argument out of range";
    case ILGPU_HIP_ERROR_NOT_SUPPORTED: return "not supported";
    case ILGPU_HIP_ERROR_UNALIGNED_TEMP: return "unaligned temp allocation";
    case ILGPU_HIP_ERROR_RUNTIME: return "HIP runtime error";
    case ILGPU_HIP_ERROR_STATIC_LIMIT:
      return "input exceeds what the library's static scratch serves "
             "(ilgpu_hip_scan_static: 1 GiB of input)";
    default: return "unknown status";
  }
}

int32_t ilgpu_hip_last_runtime_error(void) { return g_last_runtime_error; }

int32_t ilgpu_hip_profile_enable(int32_t enabled) {
  drain_profile_records();
  if (enabled) {
    std::lock_guard<std::mutex> lock(g_profile_mutex);
    g_profile_totals.clear();
  }
  g_profiling.store(enabled != 0, std::memory_order_relaxed);
  return ILGPU_HIP_SUCCESS;
}

int32_t ilgpu_hip_profile_query(const char* kernel_name, int64_t* launches,
                                double* total_ms) {
  if (kernel_name == nullptr || launches == nullptr || total_ms == nullptr)
    return ILGPU_HIP_ERROR_NULL_VIEW;
  drain_profile_records();
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  *launches = 0;
  *total_ms = 0.0;
  for (const ProfileTotal& t : g_profile_totals)
    if (t.name == kernel_name) {
      *launches = t.launches;
      *total_ms = t.total_ms;
    }
  return ILGPU_HIP_SUCCESS;
}

/* ---- radix sort -------------------------------------------------------- */

int32_t ilgpu_hip_radix_sort_temp_bytes(int64_t n, int32_t key_type,
                                        int32_t value_bytes,
                                        int64_t* temp_bytes) {
  if (temp_bytes == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  const int kb = elem_size(key_type);
  if (kb < 0) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (value_bytes != 0 && value_bytes != 1 && value_bytes != 2 &&
      value_bytes != 4 && value_bytes != 8 && value_bytes != 16)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (n < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (n > radix_sort_max_length()) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  *temp_bytes = radix_sort_temp_bytes(n, kb, value_bytes);
  return ILGPU_HIP_SUCCESS;
}

int32_t ilgpu_hip_radix_sort_temp_bytes_strided(int64_t n, int32_t key_type,
                                                int32_t value_bytes,
                                                int64_t key_stride,
                                                int64_t value_stride,
                                                int64_t* temp_bytes) {
  if (temp_bytes == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (key_stride < 1 || value_stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  const int32_t rc =
      ilgpu_hip_radix_sort_temp_bytes(n, key_type, value_bytes, temp_bytes);
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  *temp_bytes = radix_sort_temp_bytes(n, elem_size(key_type), value_bytes,
                                      key_stride, value_stride);
  return ILGPU_HIP_SUCCESS;
}

int32_t ilgpu_hip_radix_sort_keys(ilgpu_hip_stream_t stream, void* keys,
                                  int64_t n, int64_t stride, int32_t key_type,
                                  int32_t flags, void* temp,
                                  int64_t temp_bytes) {
  const int kb = elem_size(key_type);
  if (kb < 0) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(keys, n)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (n > radix_sort_max_length()) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(keys, kb)) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (flags & ~(ILGPU_HIP_SORT_DESCENDING | ILGPU_HIP_SORT_FLOAT_TOTAL_ORDER))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int32_t rc = check_temp(temp, temp_bytes,
                                radix_sort_temp_bytes(n, kb, 0, stride, 1));
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  SortArgs a{keys, nullptr, stride, 1, n, key_type, 0, flags,
             ILGPU_HIP_VALUES_FROM_VIEW, temp};
  return launch_radix_sort(static_cast<hipStream_t>(stream), a);
}

int32_t ilgpu_hip_radix_sort_pairs(ilgpu_hip_stream_t stream, void* keys,
                                   int64_t key_stride, void* values,
                                   int64_t value_stride, int64_t n,
                                   int32_t key_type, int32_t value_bytes,
                                   int32_t flags, int32_t value_source,
                                   void* temp, int64_t temp_bytes) {
  const int kb = elem_size(key_type);
  if (kb < 0) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (value_bytes != 1 && value_bytes != 2 && value_bytes != 4 &&
      value_bytes != 8 && value_bytes != 16)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(keys, n) || values == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (n > radix_sort_max_length()) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (key_stride < 1 || value_stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(keys, kb) || !aligned_to(values, value_bytes))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (flags & ~(ILGPU_HIP_SORT_DESCENDING | ILGPU_HIP_SORT_FLOAT_TOTAL_ORDER))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (value_source != ILGPU_HIP_VALUES_FROM_VIEW &&
      value_source != ILGPU_HIP_VALUES_FROM_INDEX &&
      value_source != ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (value_source == ILGPU_HIP_VALUES_FROM_INDEX && value_bytes == 16)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (value_source == ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT && value_bytes != 2 &&
      value_bytes != 4 && value_bytes != 8)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int32_t rc = check_temp(
      temp, temp_bytes,
      radix_sort_temp_bytes(n, kb, value_bytes, key_stride, value_stride));
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  SortArgs a{keys, values, key_stride, value_stride, n, key_type, value_bytes,
             flags, value_source, temp};
  return launch_radix_sort(static_cast<hipStream_t>(stream), a);
}

int32_t ilgpu_hip_selftest_lds_atomic_order(ilgpu_hip_stream_t stream,
                                            int32_t rows, int64_t* mismatches) {
  if (mismatches == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (rows < 1 || rows > (1 << 20)) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(mismatches, 8)) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  return launch_lds_atomic_order_selftest(static_cast<hipStream_t>(stream), rows,
                                          mismatches);
}

int32_t ilgpu_hip_radix_sort_passes(ilgpu_hip_stream_t stream, const void* temp,
                                    int64_t temp_bytes, int64_t n, int32_t key_type,
                                    int32_t value_bytes, int32_t* executed,
                                    int32_t* skipped) {
  if (executed == nullptr || skipped == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  const int kb = elem_size(key_type);
  if (kb < 0) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (value_bytes != 0 && value_bytes != 1 && value_bytes != 2 && value_bytes != 4 &&
      value_bytes != 8 && value_bytes != 16)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (n < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (n > radix_sort_max_length()) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int32_t rc = check_temp(temp, temp_bytes, radix_sort_temp_bytes(n, kb, value_bytes));
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  return read_sort_plan(static_cast<hipStream_t>(stream), temp, n, kb, value_bytes, executed,
                        skipped);
}

int32_t ilgpu_hip_sort_check_device(ilgpu_hip_stream_t stream) {
  return check_sort_device(static_cast<hipStream_t>(stream));
}

int32_t ilgpu_hip_sort_set_parameter(int32_t parameter, int32_t value) {
  if (parameter != ILGPU_HIP_SORT_PARAM_LOOKBACK_SPIN_LIMIT &&
      parameter != ILGPU_HIP_SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU &&
      parameter != ILGPU_HIP_SORT_PARAM_ONE_TILE_KERNEL &&
      parameter != ILGPU_HIP_SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER &&
      parameter != ILGPU_HIP_SORT_PARAM_SHORT_TILE_MAX_TILES)
    return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  set_sort_parameter(parameter, value);
  return ILGPU_HIP_SUCCESS;
}

/* ---- scan -------------------------------------------------------------- */

int32_t ilgpu_hip_scan_temp_bytes(int64_t n, int32_t elem_type,
                                  int64_t* temp_bytes) {
  if (temp_bytes == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!scan_reduce_type(elem_type)) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (n < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (n > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  *temp_bytes = scan_temp_bytes(n, elem_size(elem_type));
  return ILGPU_HIP_SUCCESS;
}

int32_t ilgpu_hip_scan(ilgpu_hip_stream_t stream, const void* in,
                       int64_t in_length, int64_t in_stride, void* out,
                       int64_t out_length, int64_t out_stride,
                       int32_t elem_type, int32_t op, int32_t kind, void* temp,
                       int64_t temp_bytes) {
  /* Order of checks as in ScanExtensions.cs:675-685. */
  if (!scan_reduce_type(elem_type) || !valid_op(op) ||
      (kind != ILGPU_HIP_SCAN_INCLUSIVE && kind != ILGPU_HIP_SCAN_EXCLUSIVE))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(in, in_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!valid_view(out, out_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (out_length < in_length) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (in_length > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int eb = elem_size(elem_type);
  if (in_stride < 1 || out_stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(in, eb) || !aligned_to(out, eb))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int32_t rc = check_temp(temp, temp_bytes, scan_temp_bytes(in_length, eb));
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  return launch_scan(static_cast<hipStream_t>(stream), in, in_stride, out,
                     out_stride, in_length, elem_type, op, kind, temp);
}

int32_t ilgpu_hip_scan_static(ilgpu_hip_stream_t stream, const void* in,
                              int64_t in_length, int64_t in_stride, void* out,
                              int64_t out_length, int64_t out_stride,
                              int32_t elem_type, int32_t op, int32_t kind) {
  /* The checks of ilgpu_hip_scan, in its order; no temp to check. */
  if (!scan_reduce_type(elem_type) || !valid_op(op) ||
      (kind != ILGPU_HIP_SCAN_INCLUSIVE && kind != ILGPU_HIP_SCAN_EXCLUSIVE))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(in, in_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!valid_view(out, out_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (out_length < in_length) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (in_length > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int eb = elem_size(elem_type);
  if (in_stride < 1 || out_stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(in, eb) || !aligned_to(out, eb))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (in_length * eb > ILGPU_HIP_SCAN_STATIC_MAX_BYTES)
    return ILGPU_HIP_ERROR_STATIC_LIMIT;
  return launch_scan_static(static_cast<hipStream_t>(stream), in, in_stride, out,
                            out_stride, in_length, elem_type, op, kind);
}

/* ---- reduce ------------------------------------------------------------ */

int32_t ilgpu_hip_reduce_temp_bytes(int64_t n, int32_t elem_type,
                                    int64_t* temp_bytes) {
  if (temp_bytes == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!scan_reduce_type(elem_type)) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (n < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  *temp_bytes = reduce_temp_bytes();
  return ILGPU_HIP_SUCCESS;
}

int32_t ilgpu_hip_reduce(ilgpu_hip_stream_t stream, const void* in, int64_t n,
                         int64_t stride, int32_t elem_type, int32_t op,
                         void* out, int64_t out_length, void* temp,
                         int64_t temp_bytes) {
  /* Order of checks as in ReductionExtensions.cs:146-153. */
  if (!scan_reduce_type(elem_type) || !valid_op(op))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(in, n)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!valid_view(out, out_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (n > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int eb = elem_size(elem_type);
  if (stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(in, eb) || !aligned_to(out, eb))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int32_t rc = check_temp(temp, temp_bytes, reduce_temp_bytes());
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  return launch_reduce(static_cast<hipStream_t>(stream), in, n, stride,
                       elem_type, op, out, temp);
}

/* ---- histogram --------------------------------------------------------- */

int32_t ilgpu_hip_histogram(ilgpu_hip_stream_t stream, const void* in,
                            int64_t n, int64_t stride, int32_t in_type,
                            void* bins, int64_t num_bins, int32_t bin_type,
                            int32_t locator, int32_t* overflow) {
  /* Order of checks as in HistogramExtensions.cs:322-338. */
  const int eb = elem_size(in_type);
  if (eb < 0 || in_type == ILGPU_HIP_F16) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (bin_type != ILGPU_HIP_I32 && bin_type != ILGPU_HIP_U32 &&
      bin_type != ILGPU_HIP_I64 && bin_type != ILGPU_HIP_U64 &&
      bin_type != ILGPU_HIP_F32 && bin_type != ILGPU_HIP_F64)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (locator != ILGPU_HIP_LOCATOR_IDENTITY &&
      locator != ILGPU_HIP_LOCATOR_MODULO)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(in, n)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!valid_view(bins, num_bins)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (n > INT32_MAX || num_bins > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(in, eb) || !aligned_to(bins, elem_size(bin_type)) ||
      (overflow != nullptr && !aligned_to(overflow, 4)))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  return launch_histogram(static_cast<hipStream_t>(stream), in, n, stride,
                          in_type, bins, num_bins, bin_type, locator, overflow);
}

/* ---- unique ------------------------------------------------------------ */

int32_t ilgpu_hip_unique_temp_bytes(int64_t n, int32_t elem_type,
                                    int64_t* temp_bytes) {
  if (temp_bytes == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  const int eb = elem_size(elem_type);
  if (eb < 0) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (n < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (n > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  *temp_bytes = unique_temp_bytes(n, eb);
  return ILGPU_HIP_SUCCESS;
}

int32_t ilgpu_hip_unique(ilgpu_hip_stream_t stream, void* input, int64_t n,
                         int32_t elem_type, int64_t* new_length,
                         int64_t new_length_extent, void* temp,
                         int64_t temp_bytes) {
  /* Order of checks as in UniqueExtensions.cs:160-178. */
  const int eb = elem_size(elem_type);
  if (eb < 0) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(input, n)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!valid_view(new_length, new_length_extent)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (temp == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (n > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!aligned_to(input, eb) || !aligned_to(new_length, 8))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const int32_t rc = check_temp(temp, temp_bytes, unique_temp_bytes(n, eb));
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  return launch_unique(static_cast<hipStream_t>(stream), input, n, elem_type,
                       new_length, temp);
}

/* ---- initialize, sequence, reorder -------------------------------------- */

int32_t ilgpu_hip_initialize(ilgpu_hip_stream_t stream, void* view, int64_t n,
                             int64_t stride, int32_t elem_bytes,
                             const void* value) {
  /* InitializeExtensions.cs:124-127. */
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 &&
      elem_bytes != 8 && elem_bytes != 16)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(view, n) || value == nullptr) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(view, elem_bytes)) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  return launch_initialize(static_cast<hipStream_t>(stream), view, n, stride,
                           elem_bytes, value);
}

int32_t ilgpu_hip_sequence(ilgpu_hip_stream_t stream, void* view, int64_t n,
                           int64_t stride, int32_t elem_type,
                           int64_t sequence_length, int64_t batch_length) {
  /* SequenceExtensions.cs:362-371. */
  const int eb = elem_size(elem_type);
  if (eb < 0) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(view, n)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (sequence_length < 1 || batch_length < 1 || stride < 1)
    return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(view, eb)) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  return launch_sequence(static_cast<hipStream_t>(stream), view, n, stride,
                         elem_type, sequence_length, batch_length);
}

int32_t ilgpu_hip_reorder(ilgpu_hip_stream_t stream, const void* source,
                          int64_t source_length, void* target,
                          int64_t target_length, const int32_t* order,
                          int64_t order_length, int32_t elem_bytes) {
  /* ReorderExtensions.cs:158-171, then TransformExtensions.cs:318-332 with the
   * order view as the transformer's source. */
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 &&
      elem_bytes != 8 && elem_bytes != 16)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(source, source_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!valid_view(order, order_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (order_length < source_length) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (source_length > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(target, target_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (target_length < order_length) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(source, elem_bytes) || !aligned_to(target, elem_bytes) ||
      !aligned_to(order, 4))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  return launch_reorder(static_cast<hipStream_t>(stream), source, target, order,
                        order_length, elem_bytes);
}

/* ---- transform, reorder-transform --------------------------------------- */

static int32_t check_transformer(int32_t source_type, int32_t target_type,
                                 int32_t transformer) {
  if (elem_size(source_type) < 0 || elem_size(target_type) < 0)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (transformer < ILGPU_HIP_TRANSFORM_CONVERT ||
      transformer > ILGPU_HIP_TRANSFORM_MULTIPLY)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  const bool float_source = source_type >= ILGPU_HIP_F16;
  const bool float_target = target_type >= ILGPU_HIP_F16;
  if (float_source && !float_target) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (float_source && transformer == ILGPU_HIP_TRANSFORM_BIT_COMPLEMENT)
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  return ILGPU_HIP_SUCCESS;
}

int32_t ilgpu_hip_transform(ilgpu_hip_stream_t stream, const void* source,
                            int64_t source_length, int64_t source_stride,
                            int32_t source_type, void* target,
                            int64_t target_length, int64_t target_stride,
                            int32_t target_type, int32_t transformer,
                            int64_t factor) {
  /* TransformExtensions.cs:304-317. */
  const int32_t rc = check_transformer(source_type, target_type, transformer);
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  if (!valid_view(source, source_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (target == nullptr || target_length < 0) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (target_length < source_length) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (source_stride < 1 || target_stride < 1) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(source, elem_size(source_type)) ||
      !aligned_to(target, elem_size(target_type)))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  TransformArgs a{source, source_stride, source_type, target, target_stride,
                  target_type, nullptr, source_length, transformer, factor};
  return launch_transform(static_cast<hipStream_t>(stream), a);
}

int32_t ilgpu_hip_reorder_transform(ilgpu_hip_stream_t stream,
                                    const void* source, int64_t source_length,
                                    int32_t source_type, void* target,
                                    int64_t target_length, int32_t target_type,
                                    const int32_t* order, int64_t order_length,
                                    int32_t transformer, int64_t factor) {
  /* ReorderExtensions.cs:158-171, then TransformExtensions.cs:304-317 with
   * the order view as the transformer's source. */
  const int32_t rc = check_transformer(source_type, target_type, transformer);
  if (rc != ILGPU_HIP_SUCCESS) return rc;
  if (!valid_view(source, source_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (!valid_view(order, order_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (order_length < source_length) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (source_length > INT32_MAX) return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  if (!valid_view(target, target_length)) return ILGPU_HIP_ERROR_NULL_VIEW;
  if (target_length < order_length) return ILGPU_HIP_ERROR_OUT_OF_RANGE;
  if (!aligned_to(source, elem_size(source_type)) ||
      !aligned_to(target, elem_size(target_type)) || !aligned_to(order, 4))
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  TransformArgs a{source, 1, source_type, target, 1, target_type, order,
                  order_length, transformer, factor};
  return launch_transform(static_cast<hipStream_t>(stream), a);
}

}  // extern "C"
