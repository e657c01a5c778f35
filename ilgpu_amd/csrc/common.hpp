// Shared device/host helpers for the gfx950 kernels: wave64 primitives,
// wide loads, the scan/reduce functors and status plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ilgpu_hip_algorithms.h"

namespace ilgpu_hip {

constexpr int kWaveSize = 64;

// ---- host-side status plumbing ------------------------------------------
void set_last_runtime_error(hipError_t e);

#define ILGPU_HIP_CHECK(expr)                                  \
  do {                                                         \
    hipError_t _e = (expr);                                    \
    if (_e != hipSuccess) {                                    \
      ::ilgpu_hip::set_last_runtime_error(_e);                 \
      return ILGPU_HIP_ERROR_RUNTIME;                          \
    }                                                          \
  } while (0)

inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }
inline int64_t div_up(int64_t a, int64_t b) { return (a + b - 1) / b; }

// The current device's index (-1 if the runtime cannot tell) and its number of
// compute units (cached per device).
constexpr int kMaxCachedDevices = 64;
int current_device();
int device_cu_count();

// Optional per-kernel timing (the library's counterpart of ILGPU's
// ProfilingMarker, ProfilingMarker.cs:19-61): while enabled through
// ilgpu_hip_profile_enable(), every ProfileScope brackets its kernel launch
// with a pair of HIP events on the launch stream.  Off by default; when off a
// scope costs one relaxed atomic load.
class ProfileScope {
 public:
  ProfileScope(hipStream_t stream, const char* name);
  ~ProfileScope();
  ProfileScope(const ProfileScope&) = delete;
  ProfileScope& operator=(const ProfileScope&) = delete;

 private:
  hipStream_t stream_;
  const char* name_;
  hipEvent_t start_;
  bool active_;
};

inline int elem_size(int32_t type) {
  switch (type) {
    case ILGPU_HIP_I8: case ILGPU_HIP_U8: return 1;
    case ILGPU_HIP_I16: case ILGPU_HIP_U16: case ILGPU_HIP_F16: return 2;
    case ILGPU_HIP_I32: case ILGPU_HIP_U32: case ILGPU_HIP_F32: return 4;
    case ILGPU_HIP_I64: case ILGPU_HIP_U64: case ILGPU_HIP_F64: return 8;
    default: return -1;
  }
}

// ---- wave64 primitives --------------------------------------------------
__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Number of set bits of `mask` in lanes below the calling lane.
__device__ __forceinline__ int mbcnt(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

template <typename T>
__device__ __forceinline__ T shfl_up(T v, int delta) {
  if constexpr (sizeof(T) == 8) {
    union { T t; int32_t w[2]; } a, b;
    a.t = v;
    b.w[0] = __shfl_up(a.w[0], delta, kWaveSize);
    b.w[1] = __shfl_up(a.w[1], delta, kWaveSize);
    return b.t;
  } else {
    union { T t; int32_t w; } a, b;
    a.w = 0;
    a.t = v;
    b.w = __shfl_up(a.w, delta, kWaveSize);
    return b.t;
  }
}

template <typename T>
__device__ __forceinline__ T shfl_down(T v, int delta) {
  if constexpr (sizeof(T) == 8) {
    union { T t; int32_t w[2]; } a, b;
    a.t = v;
    b.w[0] = __shfl_down(a.w[0], delta, kWaveSize);
    b.w[1] = __shfl_down(a.w[1], delta, kWaveSize);
    return b.t;
  } else {
    union { T t; int32_t w; } a, b;
    a.w = 0;
    a.t = v;
    b.w = __shfl_down(a.w, delta, kWaveSize);
    return b.t;
  }
}

template <typename T>
__device__ __forceinline__ T shfl(T v, int src_lane) {
  if constexpr (sizeof(T) == 8) {
    union { T t; int32_t w[2]; } a, b;
    a.t = v;
    b.w[0] = __shfl(a.w[0], src_lane, kWaveSize);
    b.w[1] = __shfl(a.w[1], src_lane, kWaveSize);
    return b.t;
  } else {
    union { T t; int32_t w; } a, b;
    a.w = 0;
    a.t = v;
    b.w = __shfl(a.w, src_lane, kWaveSize);
    return b.t;
  }
}

// ---- scan / reduce functors ---------------------------------------------
// Add/Max/Min of ScanReduceOperations.tt:20-72.  Integer adds wrap; float and
// double Max/Min follow Math.Max/Math.Min (NaN wins, -0.0 < +0.0); the
// identities of Max/Min are T.MinValue / T.MaxValue (finite for floats).
template <typename T> struct Limits;
template <> struct Limits<int32_t> {
  static __host__ __device__ constexpr int32_t lowest() { return INT32_MIN; }
  static __host__ __device__ constexpr int32_t highest() { return INT32_MAX; }
};
template <> struct Limits<uint32_t> {
  static __host__ __device__ constexpr uint32_t lowest() { return 0u; }
  static __host__ __device__ constexpr uint32_t highest() { return UINT32_MAX; }
};
template <> struct Limits<int64_t> {
  static __host__ __device__ constexpr int64_t lowest() { return INT64_MIN; }
  static __host__ __device__ constexpr int64_t highest() { return INT64_MAX; }
};
template <> struct Limits<uint64_t> {
  static __host__ __device__ constexpr uint64_t lowest() { return 0ull; }
  static __host__ __device__ constexpr uint64_t highest() { return UINT64_MAX; }
};
template <> struct Limits<float> {
  static __host__ __device__ constexpr float lowest() { return -3.402823466e+38f; }
  static __host__ __device__ constexpr float highest() { return 3.402823466e+38f; }
};
template <> struct Limits<double> {
  static __host__ __device__ constexpr double lowest() { return -1.7976931348623157e+308; }
  static __host__ __device__ constexpr double highest() { return 1.7976931348623157e+308; }
};

template <typename T> struct is_fp { static constexpr bool value = false; };
template <> struct is_fp<float> { static constexpr bool value = true; };
template <> struct is_fp<double> { static constexpr bool value = true; };

template <typename T> struct make_unsigned_t_ { using type = T; };
template <> struct make_unsigned_t_<int32_t> { using type = uint32_t; };
template <> struct make_unsigned_t_<int64_t> { using type = uint64_t; };

template <typename T>
__device__ __forceinline__ bool fp_signbit(T v) {
  if constexpr (sizeof(T) == 4) return (__float_as_uint((float)v) >> 31) != 0;
  else return (((uint64_t)__double_as_longlong((double)v)) >> 63) != 0;
}

template <typename T, int OP> struct Functor;

template <typename T> struct Functor<T, ILGPU_HIP_OP_ADD> {
  static __device__ __forceinline__ T identity() { return T(0); }
  static __device__ __forceinline__ T apply(T a, T b) {
    if constexpr (is_fp<T>::value) return a + b;
    else {
      using U = typename make_unsigned_t_<T>::type;
      return (T)((U)a + (U)b);
    }
  }
};
// Math.Max / Math.Min of the reference's MaxFloat/MinDouble... functors
// (ScanReduceOperations.tt:36-72, IntrinsicMath.cs:111-112, 207-208): a NaN
// operand wins (the first one if both are), and -0.0 < +0.0.  The hardware
// maximum and minimum return the other operand for a NaN; what they return
// for (+0, -0) is not specified by the builtin, so equal operands (that is
// the two zeros, or identical values) are told apart by their sign bit.
template <typename T> __device__ __forceinline__ T fp_hw_max(T a, T b) {
  T m;
  if constexpr (sizeof(T) == 4) m = __builtin_fmaxf(a, b);
  else m = __builtin_fmax(a, b);
  return a == b ? (fp_signbit(a) ? b : a) : m;
}
template <typename T> __device__ __forceinline__ T fp_hw_min(T a, T b) {
  T m;
  if constexpr (sizeof(T) == 4) m = __builtin_fminf(a, b);
  else m = __builtin_fmin(a, b);
  return a == b ? (fp_signbit(a) ? a : b) : m;
}
template <typename T> struct Functor<T, ILGPU_HIP_OP_MAX> {
  static __device__ __forceinline__ T identity() { return Limits<T>::lowest(); }
  static __device__ __forceinline__ T apply(T a, T b) {
    if constexpr (is_fp<T>::value) {
      const T m = fp_hw_max(a, b);
      return a != a ? a : (b != b ? b : m);
    } else {
      return a > b ? a : b;
    }
  }
};
template <typename T> struct Functor<T, ILGPU_HIP_OP_MIN> {
  static __device__ __forceinline__ T identity() { return Limits<T>::highest(); }
  static __device__ __forceinline__ T apply(T a, T b) {
    if constexpr (is_fp<T>::value) {
      const T m = fp_hw_min(a, b);
      return a != a ? a : (b != b ? b : m);
    } else {
      return a < b ? a : b;
    }
  }
};

// A 16-byte vector of T for dwordx4 loads and stores.
template <typename T> struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  using type = T __attribute__((ext_vector_type(16 / sizeof(T))));
};

}  // namespace ilgpu_hip
