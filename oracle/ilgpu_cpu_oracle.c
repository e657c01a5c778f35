/*
 * TEST INFRASTRUCTURE ONLY — see ilgpu_cpu_oracle.h.
 *
 * Plain-C restatement of the algorithms ILGPU's CPUAccelerator runs for the
 * ILGPU.Algorithms primitives.  The structure (virtual groups, 2-bit digits,
 * count -> inclusive counter scan -> scatter; 16-thread group scan; 16 strided
 * reduce threads) follows the reference so that the same code serves as the
 * "CPU path" timing baseline.  Not used by, linked into or imported from the
 * HIP library.
 */
#include "ilgpu_cpu_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ types */

int oracle_elem_size(int type) {
  switch (type) {
    case ORACLE_I8: case ORACLE_U8: return 1;
    case ORACLE_I16: case ORACLE_U16: case ORACLE_F16: return 2;
    case ORACLE_I32: case ORACLE_U32: case ORACLE_F32: return 4;
    case ORACLE_I64: case ORACLE_U64: case ORACLE_F64: return 8;
    default: return -1;
  }
}

static inline void copy_rec(void *dst, const void *src, int size) {
  switch (size) {
    case 1: memcpy(dst, src, 1); break;
    case 2: memcpy(dst, src, 2); break;
    case 4: memcpy(dst, src, 4); break;
    case 8: memcpy(dst, src, 8); break;
    case 12: memcpy(dst, src, 12); break;
    case 16: memcpy(dst, src, 16); break;
    default: memcpy(dst, src, (size_t)size); break;
  }
}

/* --------------------------------------------------------- radix bits
 * RadixSortOperations.tt:52-93.  Each branch below keeps the C# integer
 * promotion rules of the template's expression, not a "cleaned up" version:
 *   signed ints : bits = value ^ (1 << (NumBits-1))   (int / long arithmetic)
 *   unsigned    : bits = value
 *   float/double: signMask = 1 << (NumBits-1);
 *                 onesComplementMask = (~FloatAsInt(v)) >> (NumBits-1);
 *                 FloatAsInt returns an UNSIGNED integer (Interop.cs:170-192),
 *                 so the shift is logical and the mask is 0 or 1;
 *                 bits = FloatAsInt(v) ^ (signMask | onesComplementMask)
 *   Half        : onesComplementMask = ((uint)~FloatAsInt(v)) >> 15 where
 *                 FloatAsInt returns ushort: ~ promotes to int first, so the
 *                 upper 16 bits are all ones before the logical shift.
 *   result      : (int)(bits >> shift) & bitMask
 */
static inline int ascending_bits(int type, const void *value, int shift,
                                 int bit_mask) {
  switch (type) {
    case ORACLE_I8: {
      int8_t v; memcpy(&v, value, 1);
      int32_t bits = (int32_t)v ^ (1 << 7);
      return (bits >> shift) & bit_mask;
    }
    case ORACLE_I16: {
      int16_t v; memcpy(&v, value, 2);
      int32_t bits = (int32_t)v ^ (1 << 15);
      return (bits >> shift) & bit_mask;
    }
    case ORACLE_I32: {
      int32_t v; memcpy(&v, value, 4);
      int32_t bits = v ^ (int32_t)(1u << 31);
      return (bits >> shift) & bit_mask; /* arithmetic shift, as in C# */
    }
    case ORACLE_I64: {
      int64_t v; memcpy(&v, value, 8);
      int64_t bits = v ^ (int64_t)(1ull << 63);
      return (int32_t)(bits >> shift) & bit_mask;
    }
    case ORACLE_U8: {
      uint8_t v; memcpy(&v, value, 1);
      int32_t bits = v;
      return (bits >> shift) & bit_mask;
    }
    case ORACLE_U16: {
      uint16_t v; memcpy(&v, value, 2);
      int32_t bits = v;
      return (bits >> shift) & bit_mask;
    }
    case ORACLE_U32: {
      uint32_t v; memcpy(&v, value, 4);
      return (int32_t)(v >> shift) & bit_mask;
    }
    case ORACLE_U64: {
      uint64_t v; memcpy(&v, value, 8);
      return (int32_t)(v >> shift) & bit_mask;
    }
    case ORACLE_F16: {
      uint16_t raw; memcpy(&raw, value, 2);
      uint32_t sign_mask = 1u << 15;
      uint32_t ones = ((uint32_t)~(int32_t)raw) >> 15;
      uint32_t bits = (uint32_t)raw ^ (sign_mask | ones);
      return (int32_t)(bits >> shift) & bit_mask;
    }
    case ORACLE_F32: {
      uint32_t raw; memcpy(&raw, value, 4);
      uint32_t sign_mask = 1u << 31;
      uint32_t ones = (~raw) >> 31;
      uint32_t bits = raw ^ (sign_mask | ones);
      return (int32_t)(bits >> shift) & bit_mask;
    }
    case ORACLE_F64: {
      uint64_t raw; memcpy(&raw, value, 8);
      uint64_t sign_mask = 1ull << 63;
      uint64_t ones = (~raw) >> 63;
      uint64_t bits = raw ^ (sign_mask | ones);
      return (int32_t)(bits >> shift) & bit_mask;
    }
    default: return 0;
  }
}

int oracle_extract_radix_bits(int type, int descending, const void *value,
                              int shift, int bit_mask) {
  int asc = ascending_bits(type, value, shift, bit_mask);
  /* RadixSortOperations.tt:122-123 */
  return descending ? ((~asc) & bit_mask) : asc;
}

/* --------------------------------------------------------- radix sort
 * Records of rec_size bytes whose first bytes are the key of `type`.
 * Specialization4: UnrollFactor 4, BitIncrement 2 (RadixSortExtensions.cs:988-995).
 */
#define UNROLL 4
#define BIT_INCREMENT 2

/* TileInfo (TileInfo.cs:29-35) with Group.DimX == 1, Group.IdxX == 0. */
static inline void tile_bounds(int64_t n, int64_t iters, int group,
                               int64_t *start, int64_t *max_len) {
  int64_t tile = iters; /* Group.DimX * numIterationsPerGroup */
  *start = (int64_t)group * tile;
  int64_t end = ((int64_t)group + 1) * tile;
  *max_len = n < end ? n : end;
}

/* CPURadixSortKernel1 (RadixSortExtensions.cs:755-826) for one virtual group. */
static void cpu_kernel1(int type, int desc, const char *input, char *output,
                        int32_t *counter, int num_groups, int64_t iters,
                        int64_t n, int rec, int shift, int group) {
  int32_t scan_mem[UNROLL] = {0, 0, 0, 0};
  int32_t add_mem[UNROLL] = {0, 0, 0, 0};
  int64_t start, max_len;
  tile_bounds(n, iters, group, &start, &max_len);

  for (int64_t i = start; i < max_len; ++i)
    ++scan_mem[oracle_extract_radix_bits(type, desc, input + i * rec, shift,
                                         UNROLL - 1)];
  for (int j = 0; j < UNROLL; ++j)
    counter[num_groups * j + group] = scan_mem[j];

  int32_t scanned = 0, previous = scan_mem[0];
  for (int j = 1; j < UNROLL; ++j) {
    scanned += previous;
    previous = scan_mem[j];
    scan_mem[j] = scanned;
  }
  scan_mem[0] = 0;

  for (int64_t i = start; i < max_len; ++i) {
    int bits = oracle_extract_radix_bits(type, desc, input + i * rec, shift,
                                         UNROLL - 1);
    int64_t pos = start;
    pos += add_mem[bits]++;
    pos += scan_mem[bits];
    copy_rec(output + pos * rec, input + i * rec, rec);
  }
}

/* GetExclusiveCount (RadixSortExtensions.cs:835-836). */
static inline int32_t exclusive_count(int64_t index, const int32_t *counter) {
  return index < 1 ? 0 : counter[index - 1];
}

/* CPURadixSortKernel2 (RadixSortExtensions.cs:929-979) for one virtual group. */
static void cpu_kernel2(int type, int desc, const char *input, char *output,
                        const int32_t *counter, int num_groups, int64_t iters,
                        int64_t n, int rec, int shift, int group) {
  int64_t start, max_len;
  tile_bounds(n, iters, group, &start, &max_len);
  for (int64_t i = start; i < max_len; ++i) {
    int bits = oracle_extract_radix_bits(type, desc, input + i * rec, shift,
                                         UNROLL - 1);
    int32_t offset = 0;
    int64_t pos =
        exclusive_count((int64_t)bits * num_groups + group, counter) + i - start;
    for (int w = 0; w < bits; ++w) {
      int64_t address = (int64_t)w * num_groups + group;
      offset += counter[address] - exclusive_count(address, counter);
    }
    pos -= offset;
    copy_rec(output + pos * rec, input + i * rec, rec);
  }
}

/* The per-call loop of the CPU branch (RadixSortExtensions.cs:1168-1227):
 * zero counters, kernel 1, inclusive AddInt32 scan of the counters, kernel 2,
 * for bitIdx = 0, 2, ..., NumBits-2.  Groups run one after another, which is
 * what CPUMultiprocessor.cs:267-304 does with a (16,1) launch on one
 * multiprocessor. */
static int radix_sort_records(int type, int desc, char *data, int64_t n,
                              int rec, int num_groups) {
  if (n < 1 || num_groups < 1 || rec < 1) return -1;
  int num_bits = oracle_elem_size(type) * 8;
  if (num_bits < 1) return -1;
  int64_t iters = (n + num_groups - 1) / num_groups; /* XMath.DivRoundUp */
  int64_t counter_len = (int64_t)num_groups * UNROLL;
  char *temp = (char *)malloc((size_t)n * rec);
  int32_t *counter = (int32_t *)malloc(sizeof(int32_t) * counter_len);
  int32_t *counter2 = (int32_t *)malloc(sizeof(int32_t) * counter_len);
  if (!temp || !counter || !counter2) {
    free(temp); free(counter); free(counter2);
    return -1;
  }
  for (int bit = 0; bit < num_bits; bit += BIT_INCREMENT) {
    memset(counter, 0, sizeof(int32_t) * counter_len);
    for (int g = 0; g < num_groups; ++g)
      cpu_kernel1(type, desc, data, temp, counter, num_groups, iters, n, rec,
                  bit, g);
    int32_t running = 0; /* inclusive scan, wrapping int adds */
    for (int64_t j = 0; j < counter_len; ++j) {
      running = (int32_t)((uint32_t)running + (uint32_t)counter[j]);
      counter2[j] = running;
    }
    for (int g = 0; g < num_groups; ++g)
      cpu_kernel2(type, desc, temp, data, counter2, num_groups, iters, n, rec,
                  bit, g);
  }
  free(temp); free(counter); free(counter2);
  return 0;
}

int oracle_radix_sort(int type, int descending, void *data, int64_t n,
                      int num_groups) {
  int size = oracle_elem_size(type);
  if (size < 0 || !data) return -1;
  return radix_sort_records(type, descending, (char *)data, n, size,
                            num_groups);
}

int oracle_radix_sort_pairs(int key_type, int descending, void *keys,
                            void *values, int value_bytes, int64_t n,
                            int num_groups) {
  int ksize = oracle_elem_size(key_type);
  if (ksize < 0 || !keys || !values || value_bytes < 1 || value_bytes > 16 ||
      n < 1)
    return -1;
  /* RadixSortPair<TKey,TValue> (RadixSortExtensions.cs:477-506): key first. */
  int rec = ksize + value_bytes;
  char *recs = (char *)malloc((size_t)n * rec);
  if (!recs) return -1;
  /* GatherRadixSortPairsKernel (:605-623) with a ViewSourceSequencer. */
  for (int64_t i = 0; i < n; ++i) {
    memcpy(recs + i * rec, (char *)keys + i * ksize, (size_t)ksize);
    memcpy(recs + i * rec + ksize, (char *)values + i * value_bytes,
           (size_t)value_bytes);
  }
  int status = radix_sort_records(key_type, descending, recs, n, rec,
                                  num_groups);
  /* ScatterRadixSortPairsKernel (:625-645). */
  if (status == 0) {
    for (int64_t i = 0; i < n; ++i) {
      memcpy((char *)keys + i * ksize, recs + i * rec, (size_t)ksize);
      memcpy((char *)values + i * value_bytes, recs + i * rec + ksize,
             (size_t)value_bytes);
    }
  }
  free(recs);
  return status;
}

/* ------------------------------------------------------- scan / reduce ops
 * ScanReduceOperations.tt:20-72.  Integer adds wrap (unchecked C#); float and
 * double Max/Min are Math.Max/Math.Min (IntrinsicMath.cs:101-112,197-208):
 * NaN if either operand is NaN, and -0.0 orders below +0.0.
 */
static inline double dotnet_max_f64(double a, double b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == b) return signbit(a) ? b : a;
  return a > b ? a : b;
}
static inline double dotnet_min_f64(double a, double b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == b) return signbit(a) ? a : b;
  return a < b ? a : b;
}
static inline float dotnet_max_f32(float a, float b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == b) return signbit(a) ? b : a;
  return a > b ? a : b;
}
static inline float dotnet_min_f32(float a, float b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == b) return signbit(a) ? a : b;
  return a < b ? a : b;
}

#define DEFINE_INT_OPS(NAME, T, UT, TMIN, TMAX)                                \
  static inline T NAME##_identity(int op) {                                    \
    return op == ORACLE_OP_ADD ? (T)0 : op == ORACLE_OP_MAX ? (TMIN) : (TMAX); \
  }                                                                            \
  static inline T NAME##_apply(int op, T a, T b) {                             \
    if (op == ORACLE_OP_ADD) return (T)((UT)a + (UT)b);                        \
    if (op == ORACLE_OP_MAX) return a > b ? a : b;                             \
    return a < b ? a : b;                                                      \
  }
DEFINE_INT_OPS(i32, int32_t, uint32_t, INT32_MIN, INT32_MAX)
DEFINE_INT_OPS(i64, int64_t, uint64_t, INT64_MIN, INT64_MAX)
DEFINE_INT_OPS(u32, uint32_t, uint32_t, 0u, UINT32_MAX)
DEFINE_INT_OPS(u64, uint64_t, uint64_t, 0ull, UINT64_MAX)

/* float.MinValue / float.MaxValue are -FLT_MAX / +FLT_MAX, not infinities. */
static inline float f32_identity(int op) {
  return op == ORACLE_OP_ADD ? 0.0f
         : op == ORACLE_OP_MAX ? -3.402823466e+38f : 3.402823466e+38f;
}
static inline float f32_apply(int op, float a, float b) {
  if (op == ORACLE_OP_ADD) { volatile float r = a + b; return r; }
  if (op == ORACLE_OP_MAX) return dotnet_max_f32(a, b);
  return dotnet_min_f32(a, b);
}
static inline double f64_identity(int op) {
  return op == ORACLE_OP_ADD ? 0.0
         : op == ORACLE_OP_MAX ? -1.7976931348623157e+308
                               : 1.7976931348623157e+308;
}
static inline double f64_apply(int op, double a, double b) {
  if (op == ORACLE_OP_ADD) return a + b;
  if (op == ORACLE_OP_MAX) return dotnet_max_f64(a, b);
  return dotnet_min_f64(a, b);
}

/* ------------------------------------------------------------------ scan
 * SingleGroupScanKernel (ScanExtensions.cs:407-439): one group of G threads,
 * TileInfo(n, DivRoundUp(n, G)); ComputeTileScan (:340-388) walks the tile G
 * elements at a time.  Each step runs the group scan of
 * IL/ILGroupExtensions.cs:116-145 (thread 0 folds shared memory left to
 * right) and combines it with the running left boundary:
 *   inclusive: result_t = s[t], right = s[G-1],
 *              next left = Apply(left, right)                       (:185-192)
 *   exclusive: result_t = t == 0 ? Identity : s[t-1], right = s[max(0,G-2)],
 *              next left = Apply(Apply(left, right), value of thread G-1)
 *                                                         (:82-91, :158-170)
 * Out-of-range threads contribute Identity (:364-366, :382).
 */
#define DEFINE_SCAN(NAME, T)                                                   \
  static void scan_##NAME(int op, int inclusive, const T *in, T *out,          \
                          int64_t n, int G) {                                  \
    T *s = (T *)malloc(sizeof(T) * (size_t)G);                                 \
    T left = NAME##_identity(op);                                              \
    int64_t tile_end = ((n + G - 1) / G) * G; /* EndIndex = TileSize */        \
    for (int64_t base = 0; base < tile_end; base += G) {                       \
      for (int t = 0; t < G; ++t) {                                            \
        T v = base + t < n ? in[base + t] : NAME##_identity(op);               \
        s[t] = t == 0 ? v : NAME##_apply(op, s[t - 1], v);                     \
      }                                                                        \
      T last_value =                                                           \
          base + G - 1 < n ? in[base + G - 1] : NAME##_identity(op);           \
      for (int t = 0; t < G && base + t < n; ++t) {                            \
        T cur = inclusive ? s[t] : (t == 0 ? NAME##_identity(op) : s[t - 1]);  \
        out[base + t] = NAME##_apply(op, left, cur);                           \
      }                                                                        \
      if (inclusive) {                                                         \
        left = NAME##_apply(op, left, s[G - 1]);                               \
      } else {                                                                 \
        T right = s[G - 2 > 0 ? G - 2 : 0];                                    \
        left = NAME##_apply(op, NAME##_apply(op, left, right), last_value);    \
      }                                                                        \
    }                                                                          \
    free(s);                                                                   \
  }
DEFINE_SCAN(i32, int32_t)
DEFINE_SCAN(i64, int64_t)
DEFINE_SCAN(u32, uint32_t)
DEFINE_SCAN(u64, uint64_t)
DEFINE_SCAN(f32, float)
DEFINE_SCAN(f64, double)

int oracle_scan(int type, int op, int inclusive, const void *in, void *out,
                int64_t n, int group_size) {
  if (!in || !out || n < 1 || group_size < 1 || op < 0 || op > 2) return -1;
  switch (type) {
    case ORACLE_I32: scan_i32(op, inclusive, in, out, n, group_size); return 0;
    case ORACLE_I64: scan_i64(op, inclusive, in, out, n, group_size); return 0;
    case ORACLE_U32: scan_u32(op, inclusive, in, out, n, group_size); return 0;
    case ORACLE_U64: scan_u64(op, inclusive, in, out, n, group_size); return 0;
    case ORACLE_F32: scan_f32(op, inclusive, in, out, n, group_size); return 0;
    case ORACLE_F64: scan_f64(op, inclusive, in, out, n, group_size); return 0;
    default: return -1;
  }
}

/* ---------------------------------------------------------------- reduce
 * ReductionImplementation (ReductionExtensions.cs:52-125) launched with the
 * grid-stride extent of the default CPU device: MaxNumGroupsExtent = (1, 16)
 * (Accelerator.cs:180-183), so 16 threads each fold elements t, t+16, ...
 * (Execute, :104-110).  Finish (:117-124): warp reduce by ShuffleDown tree
 * (PTXWarpExtensions.cs:26-37: offsets warpSize/2 ... 1), first lanes apply
 * atomically into shared memory that starts at Identity
 * (IL/ILGroupExtensions.cs:35-53), then one AtomicApply into output[0] that
 * starts at Identity (:158-159).  The order of the warps' atomics is not
 * fixed in the reference; this restatement uses warp index order.
 */
#define DEFINE_REDUCE(NAME, T)                                                 \
  static void reduce_##NAME(int op, const T *in, int64_t n, T *out, int G,     \
                            int W) {                                           \
    T *acc = (T *)malloc(sizeof(T) * (size_t)G);                               \
    for (int t = 0; t < G; ++t) {                                              \
      T a = NAME##_identity(op);                                               \
      for (int64_t i = t; i < n; i += G) a = NAME##_apply(op, a, in[i]);       \
      acc[t] = a;                                                              \
    }                                                                          \
    T shared = NAME##_identity(op);                                            \
    for (int w = 0; w < G; w += W) {                                           \
      for (int off = W / 2; off > 0; off >>= 1)                                \
        for (int l = 0; l + off < W; ++l)                                      \
          acc[w + l] = NAME##_apply(op, acc[w + l], acc[w + l + off]);         \
      shared = NAME##_apply(op, shared, acc[w]);                               \
    }                                                                          \
    *out = NAME##_apply(op, NAME##_identity(op), shared);                      \
    free(acc);                                                                 \
  }
DEFINE_REDUCE(i32, int32_t)
DEFINE_REDUCE(i64, int64_t)
DEFINE_REDUCE(u32, uint32_t)
DEFINE_REDUCE(u64, uint64_t)
DEFINE_REDUCE(f32, float)
DEFINE_REDUCE(f64, double)

int oracle_reduce(int type, int op, const void *in, int64_t n, void *out,
                  int group_size, int warp_size) {
  if (!in || !out || n < 1 || group_size < 1 || warp_size < 1 ||
      group_size % warp_size != 0 || op < 0 || op > 2)
    return -1;
  switch (type) {
    case ORACLE_I32: reduce_i32(op, in, n, out, group_size, warp_size); return 0;
    case ORACLE_I64: reduce_i64(op, in, n, out, group_size, warp_size); return 0;
    case ORACLE_U32: reduce_u32(op, in, n, out, group_size, warp_size); return 0;
    case ORACLE_U64: reduce_u64(op, in, n, out, group_size, warp_size); return 0;
    case ORACLE_F32: reduce_f32(op, in, n, out, group_size, warp_size); return 0;
    case ORACLE_F64: reduce_f64(op, in, n, out, group_size, warp_size); return 0;
    default: return -1;
  }
}

double oracle_sum_f64(int type, const void *in, int64_t n) {
  double s = 0.0;
  if (type == ORACLE_F32) {
    const float *p = (const float *)in;
    for (int64_t i = 0; i < n; ++i) s += (double)p[i];
  } else if (type == ORACLE_F64) {
    const double *p = (const double *)in;
    for (int64_t i = 0; i < n; ++i) s += p[i];
  } else if (type == ORACLE_I32) {
    const int32_t *p = (const int32_t *)in;
    for (int64_t i = 0; i < n; ++i) s += (double)p[i];
  }
  return s;
}

/* ------------------------------------------------------------- histogram
 * One Atomic.Add(ref bin, 1) per element; overflow when the OLD value equals
 * MaxValue (HistogramOperations.tt:36-40); the add itself wraps.  The flag is
 * OR-ed into histogramOverflow[0] (HistogramExtensions.cs:197).
 */
static int64_t load_as_i64(int type, const void *p, int64_t i, double *as_f) {
  *as_f = 0.0;
  switch (type) {
    case ORACLE_I8: return ((const int8_t *)p)[i];
    case ORACLE_I16: return ((const int16_t *)p)[i];
    case ORACLE_I32: return ((const int32_t *)p)[i];
    case ORACLE_I64: return ((const int64_t *)p)[i];
    case ORACLE_U8: return ((const uint8_t *)p)[i];
    case ORACLE_U16: return ((const uint16_t *)p)[i];
    case ORACLE_U32: return ((const uint32_t *)p)[i];
    case ORACLE_U64: return (int64_t)((const uint64_t *)p)[i];
    case ORACLE_F32: *as_f = ((const float *)p)[i]; return 0;
    case ORACLE_F64: *as_f = ((const double *)p)[i]; return 0;
    default: return 0;
  }
}

/* Bin locators.
 * identity: bin = (int)value — the caller guarantees 0 <= value < numBins.
 * modulo  : the locator of the reference's tests (HistogramTests.tt:83-94):
 *           integers: (int)XMath.Abs(value % (uint)numBins)
 *           floats  : (int)XMath.Abs(XMath.Rem(value, numBins))
 *           C# promotion: an int/sbyte/short operand with a uint operand is
 *           evaluated in long, a long operand stays long, ulong stays ulong;
 *           the remainder has the sign of the dividend.
 */
static int64_t locate_bin(int in_type, int locator, const void *in, int64_t i,
                          int64_t num_bins) {
  double f;
  int64_t v = load_as_i64(in_type, in, i, &f);
  int is_float = in_type == ORACLE_F32 || in_type == ORACLE_F64;
  if (locator == ORACLE_LOCATOR_IDENTITY) return is_float ? (int64_t)f : v;
  if (is_float) {
    double r = in_type == ORACLE_F32
                   ? (double)fmodf((float)f, (float)num_bins)
                   : fmod(f, (double)num_bins);
    return (int64_t)(int32_t)fabs(r);
  }
  if (in_type == ORACLE_U64) {
    uint64_t u = ((const uint64_t *)in)[i];
    return (int64_t)(u % (uint64_t)num_bins);
  }
  int64_t r = v % num_bins;
  return r < 0 ? -r : r;
}

#define DEFINE_HIST(NAME, T, UT, TMAX)                                         \
  static int hist_##NAME(int in_type, int locator, const void *in, int64_t n,  \
                         T *bins, int64_t num_bins, int32_t *overflow) {       \
    int did = 0;                                                               \
    for (int64_t i = 0; i < n; ++i) {                                          \
      int64_t b = locate_bin(in_type, locator, in, i, num_bins);               \
      if (b < 0 || b >= num_bins) return -2;                                   \
      T old = bins[b];                                                         \
      bins[b] = (T)((UT)old + (UT)1);                                          \
      did |= old == (TMAX);                                                    \
    }                                                                          \
    if (overflow) *overflow |= did ? 1 : 0;                                    \
    return 0;                                                                  \
  }
DEFINE_HIST(i32, int32_t, uint32_t, INT32_MAX)
DEFINE_HIST(i64, int64_t, uint64_t, INT64_MAX)
DEFINE_HIST(u32, uint32_t, uint32_t, UINT32_MAX)
DEFINE_HIST(u64, uint64_t, uint64_t, UINT64_MAX)

/* Floating-point bins (HistogramLaunchers.tt:25 over AtomicNumericTypes, which
 * include float and double): Atomic.Add(ref target, 1) adds 1.0 in the bin's
 * own precision, one rounding per element (HistogramOperations.tt:36-40); a
 * float bin therefore stops growing at 2^24.  volatile keeps every addition in
 * the bin's precision. */
#define DEFINE_HIST_FP(NAME, T, TMAX)                                          \
  static int hist_##NAME(int in_type, int locator, const void *in, int64_t n,  \
                         T *bins, int64_t num_bins, int32_t *overflow) {       \
    int did = 0;                                                               \
    for (int64_t i = 0; i < n; ++i) {                                          \
      int64_t b = locate_bin(in_type, locator, in, i, num_bins);               \
      if (b < 0 || b >= num_bins) return -2;                                   \
      volatile T old = bins[b];                                                \
      volatile T next = old + (T)1;                                            \
      bins[b] = next;                                                          \
      did |= old == (TMAX);                                                    \
    }                                                                          \
    if (overflow) *overflow |= did ? 1 : 0;                                    \
    return 0;                                                                  \
  }
DEFINE_HIST_FP(f32, float, FLT_MAX)
DEFINE_HIST_FP(f64, double, DBL_MAX)

int oracle_histogram(int in_type, int bin_type, int locator, const void *in,
                     int64_t n, void *bins, int64_t num_bins,
                     int32_t *overflow) {
  if (!in || !bins || n < 1 || num_bins < 1 || oracle_elem_size(in_type) < 0 ||
      in_type == ORACLE_F16)
    return -1;
  switch (bin_type) {
    case ORACLE_I32: return hist_i32(in_type, locator, in, n, bins, num_bins, overflow);
    case ORACLE_I64: return hist_i64(in_type, locator, in, n, bins, num_bins, overflow);
    case ORACLE_U32: return hist_u32(in_type, locator, in, n, bins, num_bins, overflow);
    case ORACLE_U64: return hist_u64(in_type, locator, in, n, bins, num_bins, overflow);
    case ORACLE_F32: return hist_f32(in_type, locator, in, n, bins, num_bins, overflow);
    case ORACLE_F64: return hist_f64(in_type, locator, in, n, bins, num_bins, overflow);
    default: return -1;
  }
}

/* ----------------------------------------------------------------- unique */

static float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {                       /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* Comparison<T>.Compare(first, second) = first.CompareTo(second)
 * (ComparisonOperations.tt:30-45).  .NET CompareTo on floating-point types
 * orders NaN below everything and equal to NaN; -0.0 equals +0.0. */
static int compare_to_f64(double a, double b) {
  if (a < b) return -1;
  if (a > b) return 1;
  if (a == b) return 0;
  if (a != a) return b != b ? 0 : -1;
  return 1;
}

static int compare_elements(int type, const char *data, int64_t i, int64_t j) {
  switch (type) {
    case ORACLE_I8: { int8_t a = ((const int8_t *)data)[i], b = ((const int8_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_U8: { uint8_t a = ((const uint8_t *)data)[i], b = ((const uint8_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_I16: { int16_t a = ((const int16_t *)data)[i], b = ((const int16_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_U16: { uint16_t a = ((const uint16_t *)data)[i], b = ((const uint16_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_I32: { int32_t a = ((const int32_t *)data)[i], b = ((const int32_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_U32: { uint32_t a = ((const uint32_t *)data)[i], b = ((const uint32_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_I64: { int64_t a = ((const int64_t *)data)[i], b = ((const int64_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_U64: { uint64_t a = ((const uint64_t *)data)[i], b = ((const uint64_t *)data)[j]; return (a > b) - (a < b); }
    case ORACLE_F16: return compare_to_f64(half_bits_to_float(((const uint16_t *)data)[i]),
                                           half_bits_to_float(((const uint16_t *)data)[j]));
    case ORACLE_F32: return compare_to_f64(((const float *)data)[i], ((const float *)data)[j]);
    default: return compare_to_f64(((const double *)data)[i], ((const double *)data)[j]);
  }
}

/* UniqueKernel (UniqueExtensions.cs:59-118) with the groups run one after the
 * other, as its SequentialGroupExecutor enforces: group g owns elements
 * [g * tile, (g + 1) * tile); an element is flagged if it differs from its
 * predecessor, where the first element of a group other than the first is
 * compared with the last element kept so far (input[output[0] - 1]); thread 0
 * then compacts the flagged elements to input[output[0]...] in order. */
int64_t oracle_unique(int type, void *data, int64_t n, int64_t tile) {
  const int size = oracle_elem_size(type);
  if (size < 0 || n < 0 || tile < 1) return -1;
  char *bytes = (char *)data;
  unsigned char *flags = (unsigned char *)malloc((size_t)tile);
  if (!flags) return -1;
  int64_t kept = 0;
  for (int64_t start = 0; start < n; start += tile) {
    const int64_t end = start + tile < n ? start + tile : n;
    for (int64_t i = start; i < end; ++i) {
      if (i == 0) {
        flags[0] = 1;
      } else {
        const int64_t prev = i == start ? kept - 1 : i - 1;
        flags[i - start] = compare_elements(type, bytes, i, prev) != 0;
      }
    }
    for (int64_t i = start; i < end; ++i)
      if (flags[i - start]) {
        memmove(bytes + kept * size, bytes + i * size, (size_t)size);
        ++kept;
      }
  }
  free(flags);
  return kept;
}

/* ------------------------------------------------------------ temp sizes */

/* ScanExtensions.cs:158-170: AcceleratorType.CPU => 1. */
int64_t oracle_scan_temp_ints_cpu(void) { return 1; }

/* RadixSortExtensions.cs:419-447 on the CPU accelerator:
 * numGroups = MaxNumThreads; numIntTElements = DivRoundUp(sizeof(T)*n, 4);
 * result = numGroups * unrollFactor * 2 + numIntTElements + tempScanMemory. */
int64_t oracle_radix_sort_temp_ints_cpu(int elem_bytes, int64_t n,
                                        int max_num_threads) {
  int64_t num_int_t = ((int64_t)elem_bytes * n + 3) / 4;
  return (int64_t)max_num_threads * UNROLL * 2 + num_int_t +
         oracle_scan_temp_ints_cpu();
}

/* TempViewManager.Allocate<T>(length) (TempViewManager.cs:84-112). */
int64_t oracle_temp_view_allocate(int64_t num_ints, int64_t temp_len_ints,
                                  int elem_bytes, int is_primitive,
                                  int64_t length) {
  int64_t view_len = ((int64_t)elem_bytes * length + 3) / 4;
  if (num_ints + view_len > temp_len_ints) return -1;
  if (is_primitive) {
    int64_t byte_offset = num_ints * 4;
    if (elem_bytes > 4 && byte_offset % elem_bytes != 0) return -2;
  }
  return num_ints + view_len;
}
