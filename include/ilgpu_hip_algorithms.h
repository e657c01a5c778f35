/*
 * ilgpu_hip_algorithms.h — C ABI of libilgpu_hip_algorithms.so
 *
 * Hand-written gfx950 (MI355X, CDNA4) implementation of the data-parallel
 * primitives of ILGPU.Algorithms: radix sort (keys, key/value pairs), inclusive
 * and exclusive scan, reduction and histogram.  The entry points below are
 * what a P/Invoke layer behind ILGPU's existing C# surface binds; each one
 * names the reference interface it stands in for (paths relative to the ILGPU
 * source tree).
 *
 * Conventions
 *  - Every pointer named keys/values/in/out/bins/overflow/temp is a DEVICE
 *    pointer to memory the caller owns (the address an ArrayView yields from
 *    LoadEffectiveAddressAsPtr, ArrayViewExtensions.cs:48-50).
 *  - `stream` is a hipStream_t (NULL = the default stream).  All work is
 *    enqueued asynchronously on it, like the reference's delegates; the
 *    caller synchronises before reading results.
 *  - Lengths and strides count ELEMENTS: element i of a view is at
 *    base[i * stride] (ArrayView1D<T, Stride1D.General>, ArrayViews.tt:114-119;
 *    Stride1D.Dense is stride 1).  Stride 1 takes the vectorised kernels;
 *    larger strides are served by scalar loads and stores (scan, reduce,
 *    histogram) or by a dense staging copy in temp (sort), and elements
 *    between the strided ones are never read or written.  Strides below 1
 *    return ILGPU_HIP_ERROR_OUT_OF_RANGE.
 *  - Lengths above INT32_MAX return ILGPU_HIP_ERROR_NOT_SUPPORTED, like
 *    ErrorMessages.NotSupportedArrayView64 in the reference.
 *  - The library allocates no device memory and keeps no pointer after a call
 *    returns.  Scratch space comes from `temp` (the reference's
 *    ArrayView<int> temp), sized by the *_temp_bytes queries; its contents on
 *    entry are irrelevant and on exit undefined.  One in-flight call per temp
 *    buffer; calls on different streams with different temps may overlap.
 *  - Return value: ilgpu_hip_status (0 = success).  Argument errors are
 *    detected before any GPU work is enqueued.
 */
#ifndef ILGPU_HIP_ALGORITHMS_H
#define ILGPU_HIP_ALGORITHMS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ILGPU_HIP_ALGORITHMS_VERSION 100 /* major*10000 + minor*100 + patch */

typedef void *ilgpu_hip_stream_t; /* hipStream_t */

/* Status codes and the .NET exception each maps to in the C# layer. */
typedef enum ilgpu_hip_status {
  ILGPU_HIP_SUCCESS = 0,
  ILGPU_HIP_ERROR_NULL_VIEW = 1,      /* ArgumentNullException: invalid view */
  ILGPU_HIP_ERROR_OUT_OF_RANGE = 2,   /* ArgumentOutOfRangeException */
  ILGPU_HIP_ERROR_NOT_SUPPORTED = 3,  /* NotSupportedException */
  ILGPU_HIP_ERROR_UNALIGNED_TEMP = 4, /* InvalidOperationException
                                         (TempViewManager.cs:98-106) */
  ILGPU_HIP_ERROR_RUNTIME = 5,        /* a HIP call failed; see
                                         ilgpu_hip_last_runtime_error() */
  ILGPU_HIP_ERROR_STATIC_LIMIT = 6    /* NotSupportedException: the input is
                                         larger than the library's static
                                         scratch serves (ilgpu_hip_scan_static) */
} ilgpu_hip_status;

/* Element types: NumericTypes of TypeInformation.ttinclude:94-121. */
typedef enum ilgpu_hip_type {
  ILGPU_HIP_I8 = 0, ILGPU_HIP_I16 = 1, ILGPU_HIP_I32 = 2, ILGPU_HIP_I64 = 3,
  ILGPU_HIP_U8 = 4, ILGPU_HIP_U16 = 5, ILGPU_HIP_U32 = 6, ILGPU_HIP_U64 = 7,
  ILGPU_HIP_F16 = 8, ILGPU_HIP_F32 = 9, ILGPU_HIP_F64 = 10
} ilgpu_hip_type;

/* Scan/reduce functors: Add/Max/Min of ScanReduceOperations.tt:20-27. */
typedef enum ilgpu_hip_op {
  ILGPU_HIP_OP_ADD = 0, ILGPU_HIP_OP_MAX = 1, ILGPU_HIP_OP_MIN = 2
} ilgpu_hip_op;

/* ScanKind (ScanExtensions.cs:27-38). */
typedef enum ilgpu_hip_scan_kind {
  ILGPU_HIP_SCAN_INCLUSIVE = 0, ILGPU_HIP_SCAN_EXCLUSIVE = 1
} ilgpu_hip_scan_kind;

/* Sort flags.  DESCENDING selects the Descending* functor
 * (RadixSortOperations.tt:98-125).  By default floating-point keys are
 * ordered exactly as the reference's ExtractRadixBits orders them
 * (RadixSortOperations.tt:81-89), and that order is NOT numerically monotone:
 * the mask meant to complement negative values comes from a logical shift of
 * an unsigned pattern, so an "ascending" sort of float or double keys leaves
 * the negative ones in ascending magnitude ([-0.5, -1, -2, 0.5, 1, 2]) and
 * positive keys that differ only in the last mantissa bit swapped; for Half
 * (whose bits are promoted to a 32-bit int before the shift) the negative
 * keys are in numeric order and the positive ones in descending order
 * ([-2, -1, -0.5, 2, 1, 0.5]).  FLOAT_TOTAL_ORDER instead sorts in IEEE-754
 * totalOrder (-NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN), the
 * numerically sorted result; it has no counterpart in the reference. */
enum {
  ILGPU_HIP_SORT_DESCENDING = 1,
  ILGPU_HIP_SORT_FLOAT_TOTAL_ORDER = 2
};

/* Where the values of a key/value sort come from: the values view itself
 * (ViewSourceSequencer, Sequencer.cs:79-102) or value[i] = (TValue)i computed
 * on the fly.  FROM_INDEX: TValue is the integer type as wide as the value
 * (IndexSequencer, Sequencer.cs:36-45, and Int8Sequencer .. UInt64Sequencer,
 * Sequencers.tt:25-37: the index truncated to 1, 2, 4 or 8 bytes).
 * FROM_INDEX_AS_FLOAT: TValue is the floating-point type as wide as the value
 * (HalfSequencer, FloatSequencer, DoubleSequencer, Sequencer.cs:47-75: 2, 4 or
 * 8 bytes; long to float rounds to nearest even, Half goes through float as
 * the C# conversion does, so indices from 65520 on give +infinity). */
typedef enum ilgpu_hip_value_source {
  ILGPU_HIP_VALUES_FROM_VIEW = 0,
  ILGPU_HIP_VALUES_FROM_INDEX = 1,
  ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT = 2
} ilgpu_hip_value_source;

/* Histogram bin locators (IComputeSingleBinOperation, IHistogramOperations.cs:
 * 19-30, is arbitrary user code in the reference; a native library offers a
 * closed set).  IDENTITY: bin = (int)value, elements outside [0, num_bins)
 * are ignored.  MODULO: bin = |value % num_bins|, the locator of the
 * reference's own tests (HistogramTests.tt:83-94). */
typedef enum ilgpu_hip_locator {
  ILGPU_HIP_LOCATOR_IDENTITY = 0,
  ILGPU_HIP_LOCATOR_MODULO = 1
} ilgpu_hip_locator;

/* ---- library ----------------------------------------------------------- */

int32_t ilgpu_hip_version(void);
const char *ilgpu_hip_status_string(int32_t status);
/* hipError_t of the most recent failing HIP call on the calling thread. */
int32_t ilgpu_hip_last_runtime_error(void);

/* Per-kernel timing, the library's counterpart of ILGPU's profiling markers
 * (ProfilingMarker.cs:19-61, enabled by Context.Builder.Profiling(),
 * Context.Builder.cs:315-319).  While enabled, each kernel launch is bracketed
 * by a pair of HIP events on its stream.  Enabling clears earlier totals.
 * ilgpu_hip_profile_query waits for the recorded events and returns how often
 * the named kernel ran and its summed duration.  Kernel names: "zero_words",
 * "reduce_partials", "reduce_final", "scan", "histogram", "sort_histogram",
 * "sort_plan", "sort_onesweep", "sort_finish".  Not meant for concurrent use
 * from several threads. */
int32_t ilgpu_hip_profile_enable(int32_t enabled);
int32_t ilgpu_hip_profile_query(const char *kernel_name, int64_t *launches,
                                double *total_ms);

/* ---- radix sort ---------------------------------------------------------
 * Replaces: RadixSort<T,TStride> delegates made by CreateRadixSort
 * (RadixSortExtensions.cs:37-42, 1130-1337), RadixSortPairs delegates made by
 * CreateRadixSortPairs (:56-96, 1017-1118) and the sizing helpers
 * ComputeRadixSortTempStorageSize / ComputeRadixSortPairsTempStorageSize
 * (:384-447).  Sorting is in place and stable; a pairs sort permutes `values`
 * with the keys.
 */

/* Bytes of temp needed to sort n keys of key_type, each with a payload of
 * value_bytes bytes (0 for a keys-only sort).  64-bit arithmetic throughout
 * (the reference's pair sizing multiplies in 32 bits). */
int32_t ilgpu_hip_radix_sort_temp_bytes(int64_t n, int32_t key_type,
                                        int32_t value_bytes,
                                        int64_t *temp_bytes);

/* The same for views with element strides above one: each strided view adds a
 * dense staging copy of its n elements.  ComputeRadixSortTempStorageSize has no
 * stride argument (RadixSortExtensions.cs:419-447: the reference's kernels
 * index through the view), so a binding offers this as an overload that takes
 * the views' strides; sorting a strided view with the dense size returns
 * ILGPU_HIP_ERROR_OUT_OF_RANGE (temp too small). */
int32_t ilgpu_hip_radix_sort_temp_bytes_strided(int64_t n, int32_t key_type,
                                                int32_t value_bytes,
                                                int64_t key_stride,
                                                int64_t value_stride,
                                                int64_t *temp_bytes);

int32_t ilgpu_hip_radix_sort_keys(ilgpu_hip_stream_t stream, void *keys,
                                  int64_t n, int64_t stride, int32_t key_type,
                                  int32_t flags, void *temp,
                                  int64_t temp_bytes);

/* value_bytes in {1, 2, 4, 8, 16}.  With ILGPU_HIP_VALUES_FROM_INDEX (value_bytes
 * 1, 2, 4 or 8) and ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT (2, 4 or 8) the incoming
 * contents of `values` are ignored. */
int32_t ilgpu_hip_radix_sort_pairs(ilgpu_hip_stream_t stream, void *keys,
                                   int64_t key_stride, void *values,
                                   int64_t value_stride, int64_t n,
                                   int32_t key_type, int32_t value_bytes,
                                   int32_t flags, int32_t value_source,
                                   void *temp, int64_t temp_bytes);

/* How many 8-bit passes the last sort that used `temp` ran and how many it
 * found unnecessary (a pass whose digit is the same for every key is skipped:
 * keys below 2^16 run two passes of four, equal keys none).  Same n, key_type
 * and value_bytes (0 for keys only) as that sort, dense views; waits for
 * `stream`.  The reference runs all NumBits / 2 passes whatever the keys
 * (RadixSortExtensions.cs:1276-1334) and has nothing to report. */
int32_t ilgpu_hip_radix_sort_passes(ilgpu_hip_stream_t stream, const void *temp,
                                    int64_t temp_bytes, int64_t n,
                                    int32_t key_type, int32_t value_bytes,
                                    int32_t *executed, int32_t *skipped);

/* Device self-check of the one hardware property the sort's ranking relies
 * on beyond the programming model: the lanes of ONE returning LDS atomic
 * instruction that meet in one address are served in ascending lane order
 * (this is what makes a pass stable at one LDS operation per key).  It has no
 * counterpart in the reference; its place there is taken by the group-wide
 * scans of RadixSortKernel1 (RadixSortExtensions.cs:700-705).  Plays `rows`
 * (1 .. 2^20) ranking rows per wave on every compute unit for six digit
 * distributions and stores the number of lanes found out of order in
 * mismatches[0] (device memory, 8-byte aligned): 0 on gfx950.  Stream-ordered,
 * allocates nothing. */
int32_t ilgpu_hip_selftest_lds_atomic_order(ilgpu_hip_stream_t stream,
                                            int32_t rows, int64_t *mismatches);

/* The same check, once per device and with the answer kept by the library:
 * ILGPU_HIP_SUCCESS for a device whose LDS serves the lanes in order,
 * ILGPU_HIP_ERROR_NOT_SUPPORTED for one that does not.  Every sort entry point
 * calls it first, so no sort runs on a device that has not passed: the first
 * sort on a device plays the check kernels (64 rows) on a counter inside the
 * library (nothing is allocated) and waits for `stream` once; later calls cost
 * one atomic load.  A stream that is being captured cannot be waited for: on a
 * device that has not been asked yet, a sort on such a stream (and this call)
 * returns ILGPU_HIP_ERROR_NOT_SUPPORTED, so callers that capture call this
 * first, outside the capture; accelerator objects of the host layers call it
 * in their constructors.  No counterpart in the reference. */
int32_t ilgpu_hip_sort_check_device(ilgpu_hip_stream_t stream);

/* TEST HOOK, not part of the product surface: process-wide parameters of the
 * sort for the library's own tests and tuning runs.  They are global mutable
 * state (a thread that changes one changes every sort of the process that is
 * launched afterwards), so applications leave them alone and bindings keep
 * them out of their public surface.  A negative value restores the default;
 * none has a counterpart in the reference (its passes are separate kernel
 * launches, RadixSortExtensions.cs:1276-1334).
 *   LOOKBACK_SPIN_LIMIT  how often the look-back of a pass polls the status
 *     word of an earlier tile that has published nothing before it stops
 *     waiting and counts that tile's digit itself from the source keys (tiles
 *     are handed to fixed groups of blocks, so a tile may wait for one whose
 *     group has no resident block; with this bound every block finishes
 *     whatever the others do).  Default 4096; 0 makes every look-back that
 *     meets an empty word take the slow path at once, which is how the tests
 *     exercise it.
 *   LARGE_BLOCK_MIN_TILES_PER_CU  inputs of at least this many 1024-thread
 *     tiles per compute unit are sorted with 1024-thread blocks (longer runs
 *     per digit), smaller ones with 512-thread blocks (more blocks for fewer
 *     keys).  Default 3 for keys, 2 for pairs; 0 = always the large block,
 *     INT32_MAX = never.
 *   ONE_TILE_KERNEL  inputs of at most one 512-thread tile (18432 keys of up
 *     to 4 bytes, fewer for wider keys and for pairs) are sorted by one block
 *     in one launch, without temp memory.  Default 1; 0 sends them through
 *     the passes like longer inputs.
 *   ASSUME_LDS_ATOMIC_ORDER  what ilgpu_hip_sort_check_device answers: 0 = every
 *     device is taken to have failed the check (sorts return
 *     ILGPU_HIP_ERROR_NOT_SUPPORTED before anything is launched), 1 = taken to
 *     have passed, negative (the default) = the devices are asked, anew.
 *   SHORT_TILE_MAX_TILES  keys without values are cut into 512-thread tiles of
 *     a third, a half or two thirds of the usual length (6144, 9216 or 12288
 *     keys of up to 4 bytes), the shortest that makes at most this many tiles:
 *     more compute units at work on a short input.  Default 512, which is also
 *     the most that is taken (temp sizes assume it), and never more than two
 *     per compute unit; 0 = never. */
enum {
  ILGPU_HIP_SORT_PARAM_LOOKBACK_SPIN_LIMIT = 0,
  ILGPU_HIP_SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU = 1,
  ILGPU_HIP_SORT_PARAM_ONE_TILE_KERNEL = 2,
  ILGPU_HIP_SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER = 3,
  ILGPU_HIP_SORT_PARAM_SHORT_TILE_MAX_TILES = 4
};
int32_t ilgpu_hip_sort_set_parameter(int32_t parameter, int32_t value);

/* ---- scan ---------------------------------------------------------------
 * Replaces: Scan<T,TStrideIn,TStrideOut> delegates made by CreateScan(kind)
 * (ScanExtensions.cs:52-61, 930-959) and ComputeScanTempStorageSize (:158-170).
 * elem_type in {I32, I64, U32, U64, F32, F64}.  out_length may exceed
 * in_length (only the first in_length outputs are written, :679-680);
 * shorter is ILGPU_HIP_ERROR_OUT_OF_RANGE.  in and out must not overlap
 * unless they are identical.
 */
int32_t ilgpu_hip_scan_temp_bytes(int64_t n, int32_t elem_type,
                                  int64_t *temp_bytes);

int32_t ilgpu_hip_scan(ilgpu_hip_stream_t stream, const void *in,
                       int64_t in_length, int64_t in_stride, void *out,
                       int64_t out_length, int64_t out_stride,
                       int32_t elem_type, int32_t op, int32_t kind, void *temp,
                       int64_t temp_bytes);

/* The same scan without a temp view, for callers that cannot allocate device
 * memory or carry a temp buffer: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose Scan delegates always take an ArrayView<int> temp,
 * ScanExtensions.cs:52-61).  The tile states live in a device array inside the
 * library (1 MiB + 256 bytes per GPU, held until the process ends), so
 *  - the input may hold at most ILGPU_HIP_SCAN_STATIC_MAX_BYTES bytes
 *    (in_length * element size); more returns ILGPU_HIP_ERROR_STATIC_LIMIT;
 *  - every call on one GPU uses that GPU's array: calls that overlap in time on
 *    the same GPU (two streams, two threads) race and must be serialised by the
 *    caller;
 *  - the call allocates nothing and clears what it needs with a fill kernel
 *    (no memset node), so it may be captured into a graph; the first call on a
 *    device looks up the array's address and should be made outside a capture.
 * Arguments, checks and results are those of ilgpu_hip_scan. */
#define ILGPU_HIP_SCAN_STATIC_MAX_BYTES (1ll << 30)
int32_t ilgpu_hip_scan_static(ilgpu_hip_stream_t stream, const void *in,
                              int64_t in_length, int64_t in_stride, void *out,
                              int64_t out_length, int64_t out_stride,
                              int32_t elem_type, int32_t op, int32_t kind);

/* ---- reduce -------------------------------------------------------------
 * Replaces: Reduction<T,TStride> delegates made by CreateReduction and the
 * Reduce overloads (ReductionExtensions.cs:30-35, 135-216).  out[0] is
 * overwritten with the fold of all inputs (:158-159); out_length >= 1.
 * Integer results are exact (wrapping adds); floating-point Add accumulates
 * in float64 in a fixed order, so repeated calls give identical bits.
 * The reference's delegate has no temp argument: the P/Invoke layer owns a
 * small scratch buffer of ilgpu_hip_reduce_temp_bytes() per delegate.
 */
int32_t ilgpu_hip_reduce_temp_bytes(int64_t n, int32_t elem_type,
                                    int64_t *temp_bytes);

int32_t ilgpu_hip_reduce(ilgpu_hip_stream_t stream, const void *in,
                         int64_t n, int64_t stride, int32_t elem_type,
                         int32_t op, void *out, int64_t out_length, void *temp,
                         int64_t temp_bytes);

/* ---- histogram ----------------------------------------------------------
 * Replaces: Histogram / HistogramUnchecked delegates and launchers
 * (HistogramExtensions.cs:35-59, 293-508; HistogramLaunchers.tt:52-101).
 * bins[locator(v)] += 1 for every input element; bins are ACCUMULATED into,
 * never cleared.  bin_type in {I32, I64, U32, U64, F32, F64}: the reference's
 * AtomicNumericTypes.  A floating-point bin receives its additions of 1.0 one
 * by one in its own precision, as Atomic.Add does, so a float bin stops
 * growing at 2^24 (16777216 + 1 rounds back to 16777216); the result is
 * computed exactly and does not depend on the order of the elements.  If
 * `overflow` is not NULL, overflow[0] |= 1 when some bin's count passed the
 * bin type's MaxValue (an increment found the bin holding MaxValue,
 * HistogramOperations.tt:36-40); NULL selects the unchecked variant.
 * in_type: any ilgpu_hip_type except F16.
 * Floating-point bins must live in ordinary device memory (hipMalloc: coarse
 * grained).  With more bins than LDS holds their single increments go through
 * the hardware's floating-point atomic add in L2, which is exact there; for
 * fine-grained, host-mapped or managed memory the hardware does not promise
 * that, and no reference fixture covers floating-point bins at all.
 */
int32_t ilgpu_hip_histogram(ilgpu_hip_stream_t stream, const void *in,
                            int64_t n, int64_t stride, int32_t in_type,
                            void *bins, int64_t num_bins, int32_t bin_type,
                            int32_t locator, int32_t *overflow);

/* ---- unique -------------------------------------------------------------
 * Replaces: the Unique<T> delegate made by CreateUnique<T, Comparison<T>>, the
 * value-returning Unique and ComputeUniqueTempStorageSize
 * (UniqueExtensions.cs:27-33, 116-209).  Removes consecutive duplicates of
 * input[0..n) in place and writes the new length to new_length[0] (a device
 * int64, the reference's ArrayView<long> output).  Two elements are duplicates
 * if Comparison<T>.Compare yields 0 (ComparisonOperations.tt:30-45): CompareTo,
 * so all NaNs are equal and -0.0 equals +0.0.  elem_type: any of the eleven
 * numeric types.
 */
int32_t ilgpu_hip_unique_temp_bytes(int64_t n, int32_t elem_type,
                                    int64_t *temp_bytes);
int32_t ilgpu_hip_unique(ilgpu_hip_stream_t stream, void *input, int64_t n,
                         int32_t elem_type, int64_t *new_length,
                         int64_t new_length_extent, void *temp,
                         int64_t temp_bytes);

/* ---- initialize, sequence, reorder ----------------------------------------
 * Replace: Initializer delegates and Initialize (InitializeExtensions.cs:26-31,
 * 116-176): view[i] = *value, `value` being a HOST pointer to elem_bytes bytes
 * (1, 2, 4, 8 or 16); the Sequencer, RepeatedSequencer, BatchedSequencer and
 * RepeatedBatchedSequencer delegates (SequenceExtensions.cs:31-123, 238-630)
 * for the identity sequencers (Sequencers.tt:25-37, IndexSequencer):
 * view[i] = (T)((i / batch_length) % sequence_length), where Sequence passes
 * sequence_length = n and batch_length = 1; and Reorder
 * (ReorderExtensions.cs:194-214): target[i] = source[order[i]] for
 * i < order_length, with the reference's checks order_length >= source_length
 * and target_length >= order_length.  Index values are not range-checked.
 */
int32_t ilgpu_hip_initialize(ilgpu_hip_stream_t stream, void *view, int64_t n,
                             int64_t stride, int32_t elem_bytes,
                             const void *value);
int32_t ilgpu_hip_sequence(ilgpu_hip_stream_t stream, void *view, int64_t n,
                           int64_t stride, int32_t elem_type,
                           int64_t sequence_length, int64_t batch_length);
int32_t ilgpu_hip_reorder(ilgpu_hip_stream_t stream, const void *source,
                          int64_t source_length, void *target,
                          int64_t target_length, const int32_t *order,
                          int64_t order_length, int32_t elem_bytes);

/* ---- transform, reorder-transform ----------------------------------------
 * Replace: the Transformer delegates, CreateTransformer and Transform
 * (TransformExtensions.cs:73-115, 255-506): target[i] = f(source[i]) for
 * i < source_length, with the reference's checks source_length >= 1 and
 * target_length >= source_length (:304-317); and ReorderTransformer,
 * CreateReorderTransformer and ReorderTransform (ReorderExtensions.cs:42-52,
 * 143-297): target[i] = f(source[order[i]]) for i < order_length, with the
 * checks of ilgpu_hip_reorder.
 *
 * The reference JIT-compiles any ITransformer<TSource, TTarget> struct
 * (TransformExtensions.cs:24-37).  Here the transformers are a closed set of
 * the form (TTarget)op((TSource)value): op is computed in the source type
 * (integers wrap, as unchecked C#), then converted to the target type by the
 * C# explicit numeric conversion (integers truncate or extend by the source's
 * sign; to and between floating-point types: round to nearest even).  The set
 * covers IdentityTransformer (:42-55) and every transformer of the reference's
 * tests (Generic/AlgorithmsTestData.tt:170-252).  Floating-point sources with
 * integer targets are ILGPU_HIP_ERROR_NOT_SUPPORTED (C# leaves that conversion
 * unspecified for NaN and out-of-range values), and so is BIT_COMPLEMENT of a
 * floating-point source.  `factor` is used by MULTIPLY only, converted to the
 * source type.  A transform with equal source and target types may run in
 * place (source == target, equal strides).
 */
enum ilgpu_hip_transformer {
  ILGPU_HIP_TRANSFORM_CONVERT = 0,        /* (TTarget)value; identity if the types match */
  ILGPU_HIP_TRANSFORM_NEGATE = 1,         /* (TTarget)(-value) */
  ILGPU_HIP_TRANSFORM_BIT_COMPLEMENT = 2, /* (TTarget)(~value), integer sources */
  ILGPU_HIP_TRANSFORM_MULTIPLY = 3        /* (TTarget)(value * (TSource)factor) */
};
int32_t ilgpu_hip_transform(ilgpu_hip_stream_t stream, const void *source,
                            int64_t source_length, int64_t source_stride,
                            int32_t source_type, void *target,
                            int64_t target_length, int64_t target_stride,
                            int32_t target_type, int32_t transformer,
                            int64_t factor);
int32_t ilgpu_hip_reorder_transform(ilgpu_hip_stream_t stream,
                                    const void *source, int64_t source_length,
                                    int32_t source_type, void *target,
                                    int64_t target_length, int32_t target_type,
                                    const int32_t *order, int64_t order_length,
                                    int32_t transformer, int64_t factor);

#ifdef __cplusplus
}
#endif
#endif /* ILGPU_HIP_ALGORITHMS_H */
