// Internal launch interface between the C ABI (api.hip) and the kernel files.
// All launchers assume validated arguments: non-null, naturally aligned
// device pointers, 1 <= n <= INT32_MAX, element strides >= 1, temp large
// enough.
#pragma once

#include "common.hpp"

namespace ilgpu_hip {

// reduce.hip
int64_t reduce_temp_bytes();
int32_t launch_reduce(hipStream_t stream, const void* in, int64_t n,
                      int64_t in_stride, int32_t type, int32_t op, void* out,
                      void* temp);

// scan.hip
int64_t scan_temp_bytes(int64_t n, int elem_bytes);
int32_t launch_scan(hipStream_t stream, const void* in, int64_t in_stride,
                    void* out, int64_t out_stride, int64_t n, int32_t type,
                    int32_t op, int32_t kind, void* temp);

// Same on the library's static scratch (no temp view, no allocation); inputs of
// more than ILGPU_HIP_SCAN_STATIC_MAX_BYTES return ILGPU_HIP_ERROR_STATIC_LIMIT.
int32_t launch_scan_static(hipStream_t stream, const void* in, int64_t in_stride,
                           void* out, int64_t out_stride, int64_t n, int32_t type,
                           int32_t op, int32_t kind);

// histogram.hip
int32_t launch_histogram(hipStream_t stream, const void* in, int64_t n,
                         int64_t in_stride, int32_t in_type, void* bins,
                         int64_t num_bins, int32_t bin_type, int32_t locator,
                         int32_t* overflow);

// radix_sort.hip (kernels: radix_sort_impl.hpp, radix_sort_k*.hip)
struct SortArgs {
  void* keys;
  void* values;      // nullptr for a keys-only sort
  int64_t key_stride;    // element strides of the two views
  int64_t value_stride;
  int64_t n;
  int32_t key_type;
  int32_t value_bytes;   // 0 for keys only
  int32_t flags;
  int32_t value_source;
  void* temp;
};
// Strides above one add a dense staging copy of that view to the temp.
int64_t radix_sort_temp_bytes(int64_t n, int key_bytes, int value_bytes,
                              int64_t key_stride = 1, int64_t value_stride = 1);
int64_t radix_sort_max_length();
int32_t launch_radix_sort(hipStream_t stream, const SortArgs& args);
// ILGPU_HIP_SORT_PARAM_* (validated by the caller); negative = default.
void set_sort_parameter(int32_t parameter, int32_t value);
// Device check of the LDS behaviour the sort's ranking relies on: lanes of one
// returning LDS atomic that share an address are served in lane order.
// mismatches[0] (device) receives the number of lanes found out of order.
int32_t launch_lds_atomic_order_selftest(hipStream_t stream, int rows, int64_t* mismatches);
// The same check once per device, with the answer kept: SUCCESS, or
// NOT_SUPPORTED for a device that serves the lanes in another order (or while
// `stream` is being captured and the device has not been asked yet).  Every
// sort calls it first.
int32_t check_sort_device(hipStream_t stream);
// How many passes the last sort that used `temp` (same n, key size, value size,
// dense views) ran, and how many it found unnecessary; waits for the stream.
int32_t read_sort_plan(hipStream_t stream, const void* temp, int64_t n, int key_bytes,
                       int value_bytes, int32_t* executed, int32_t* skipped);

// scan.hip: Unique (consecutive duplicates removed in place, new length to
// out_length[0] on the device).
int64_t unique_temp_bytes(int64_t n, int elem_bytes);
int32_t launch_unique(hipStream_t stream, void* data, int64_t n, int32_t type,
                      int64_t* out_length, void* temp);

// sequence.hip
int32_t launch_initialize(hipStream_t stream, void* view, int64_t n, int64_t stride,
                          int elem_bytes, const void* value);
int32_t launch_sequence(hipStream_t stream, void* view, int64_t n, int64_t stride,
                        int32_t type, int64_t sequence_length, int64_t batch_length);
int32_t launch_reorder(hipStream_t stream, const void* source, void* target,
                       const int32_t* order, int64_t n, int elem_bytes);

// transform.hip: target[i] = (T)op((S)source[order ? order[i] : i]).
struct TransformArgs {
  const void* source;
  int64_t source_stride;  // ignored when order is given (dense source)
  int32_t source_type;
  void* target;
  int64_t target_stride;
  int32_t target_type;
  const int32_t* order;   // nullptr for a plain transform
  int64_t n;
  int32_t transformer;
  int64_t factor;
};
int32_t launch_transform(hipStream_t stream, const TransformArgs& args);

// fill kernel shared by scan and sort: words[0..count) = 0, as a kernel so
// that callers may capture the stream into a graph.
int32_t launch_zero_words(hipStream_t stream, uint32_t* words, int64_t count);

}  // namespace ilgpu_hip
