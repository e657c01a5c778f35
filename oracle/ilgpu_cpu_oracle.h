/*
 * TEST INFRASTRUCTURE ONLY — CPU oracle for the ILGPU.Algorithms hot path.
 *
 * A plain-C restatement of what ILGPU's CPUAccelerator computes for radix sort
 * (keys and pairs), scan, reduce and histogram.  It exists so that the HIP
 * library can be checked against it; nothing in the shipped library may call,
 * link or import it.  Every function cites the reference lines it follows
 * (paths are relative to the ILGPU source tree).
 *
 * Pinning status of each function (what independent evidence holds it in place):
 *   oracle_extract_radix_bits   integers: pinned (numeric order; the reference's own
 *                               sequences RadixSortExtensionTests.tt:37-131).
 *                               float/double >= 0 at integer values and constant -1:
 *                               pinned by the same sequences.  Negative floats,
 *                               adjacent positive floats and Half: no reference test
 *                               covers them; pinned by golden vectors worked out by
 *                               hand from RadixSortOperations.tt:81-89, 122-123 with
 *                               C#'s integer promotion rules, in Python integers only
 *                               (tests/golden/make_known_answers.py, ops
 *                               sort_float_bits and sort_pairs_float_bits: Half,
 *                               float and double, both orders, keys and pairs).
 *   oracle_radix_sort[_pairs]   pinned against stable sort by extracted key.
 *   oracle_scan                 integers pinned against serial fold
 *                               (ScanExtensionTests.tt:286-305); floating point
 *                               pinned only where every partial sum is exact.
 *   oracle_reduce               integers pinned against serial fold; float Add is
 *                               one admissible order of a non-deterministic
 *                               reference (tolerance contract, see oracle_sum_f64).
 *   oracle_histogram            pinned against HistogramTests.tt:50-76 vectors.
 *   oracle_unique               pinned against RemoveConsecutiveDuplicates on the
 *                               reference's inputs (UniqueExtensionTests.tt:36-67,
 *                               integers) and against a first-of-run filter for
 *                               every tile size; NaN and signed-zero equality follow
 *                               .NET CompareTo and are pinned by that definition
 *                               only (no reference test has such inputs).
 *   sequence / initialize / reorder (numpy restatements in cpu_oracle.py) pinned by
 *                               SequencerTests.tt:56-70 and ReorderExtensionTests.tt.
 *   transform / reorder_transform (numpy restatements in cpu_oracle.py) pinned by the
 *                               expectations of TransformerExtensionTests.tt:66-162
 *                               and ReorderExtensionTests.tt:160-290, and by Python
 *                               big-integer arithmetic for every integer type pair;
 *                               float16/32/64 rounding by hand-picked ties.
 *   temp-size helpers           pinned by the closed formulas they restate.
 */
#ifndef ILGPU_CPU_ORACLE_H
#define ILGPU_CPU_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types: the eleven NumericTypes of TypeInformation.ttinclude:94-121. */
enum {
  ORACLE_I8 = 0, ORACLE_I16 = 1, ORACLE_I32 = 2, ORACLE_I64 = 3,
  ORACLE_U8 = 4, ORACLE_U16 = 5, ORACLE_U32 = 6, ORACLE_U64 = 7,
  ORACLE_F16 = 8, ORACLE_F32 = 9, ORACLE_F64 = 10
};
enum { ORACLE_OP_ADD = 0, ORACLE_OP_MAX = 1, ORACLE_OP_MIN = 2 };
enum { ORACLE_LOCATOR_IDENTITY = 0, ORACLE_LOCATOR_MODULO = 1 };

/* Default CPUDevice: 4 lanes x 4 warps x 1 multiprocessor (CPUDevice.cs:67-77). */
#define ORACLE_CPU_WARP_SIZE 4
#define ORACLE_CPU_GROUP_SIZE 16
#define ORACLE_CPU_MAX_NUM_THREADS 16

int oracle_elem_size(int type);

/* RadixSortOperations.tt:52-93 (ascending), :122-123 (descending). */
int oracle_extract_radix_bits(int type, int descending, const void *value,
                              int shift, int bit_mask);

/* RadixSortExtensions.cs:1168-1227 with CPURadixSortKernel1/2 (:755-826,:929-979).
 * Sorts `data` in place.  num_groups = accelerator.MaxNumThreads (16 by default).
 * Returns 0, or -1 on bad arguments / allocation failure. */
int oracle_radix_sort(int type, int descending, void *data, int64_t n,
                      int num_groups);

/* RadixSortExtensions.cs:1017-1074: gather (key,value) records, sort the
 * records by key with the same passes, scatter back.  value_bytes in 1..16. */
int oracle_radix_sort_pairs(int key_type, int descending, void *keys,
                            void *values, int value_bytes, int64_t n,
                            int num_groups);

/* ScanExtensions.cs:407-439 (single group) with ComputeTileScan (:340-388) and
 * the serial group scan of IL/ILGroupExtensions.cs:76-192.  Types: I32 I64 U32
 * U64 F32 F64 (ScanReduceOperations.tt:20).  `out` may alias nothing. */
int oracle_scan(int type, int op, int inclusive, const void *in, void *out,
                int64_t n, int group_size);

/* ReductionExtensions.cs:104-124 on the default CPU launch shape: one group of
 * 16 threads striding by 16 (GridExtensions.cs:182-196), warp tree reduce
 * (PTX/PTXWarpExtensions.cs:26-37 used by IL/ILWarpExtensions.cs:28-33), warps
 * folded in index order.  Writes one element to out. */
int oracle_reduce(int type, int op, const void *in, int64_t n, void *out,
                  int group_size, int warp_size);

/* The float32 Add contract: float64 sum of the inputs, serial order. */
double oracle_sum_f64(int type, const void *in, int64_t n);

/* HistogramExtensions.cs:237-277 + HistogramLaunchers.tt:89-100 +
 * HistogramOperations.tt:36-40, run serially like HistogramTests.tt:50-76.
 * Bins accumulate; *overflow is OR-ed with 1 when an increment saw MaxValue.
 * bin types: I32 I64 U32 U64.  Locators: identity (bin = value, caller keeps
 * values in range) and the test suite's modulo (HistogramTests.tt:83-94). */
int oracle_histogram(int in_type, int bin_type, int locator, const void *in,
                     int64_t n, void *bins, int64_t num_bins,
                     int32_t *overflow);

/* UniqueKernel (UniqueExtensions.cs:59-118): consecutive duplicates under
 * Comparison<T> (CompareTo) removed in place, groups of `tile` elements run in
 * sequence; returns the new length (-1 on bad arguments). */
int64_t oracle_unique(int type, void *data, int64_t n, int64_t tile);

/* Temp sizing on the CPU accelerator, in 32-bit ints
 * (RadixSortExtensions.cs:419-447, :384-404; ScanExtensions.cs:158-170). */
int64_t oracle_scan_temp_ints_cpu(void);
int64_t oracle_radix_sort_temp_ints_cpu(int elem_bytes, int64_t n,
                                        int max_num_threads);

/* TempViewManager.Allocate (TempViewManager.cs:84-112): returns the new
 * NumInts, -1 for "temp too small", -2 for the unaligned-allocation error. */
int64_t oracle_temp_view_allocate(int64_t num_ints, int64_t temp_len_ints,
                                  int elem_bytes, int is_primitive,
                                  int64_t length);

#ifdef __cplusplus
}
#endif
#endif
