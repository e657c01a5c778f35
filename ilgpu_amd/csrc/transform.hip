// Transform and ReorderTransform: target[i] = f(source[i]) and
// target[i] = f(source[order[i]]) for a closed set of transformers.
//
// Stand in for
//   Transformer delegates, Transform   TransformExtensions.cs:73-115, 255-506
//   ReorderTransformer, ReorderTransform ReorderExtensions.cs:42-52, 143-297
// The reference JIT-compiles any C# struct that implements
// ITransformer<TSource, TTarget> (TransformExtensions.cs:24-37) into a
// grid-stride loop (TransformImplementation.Execute, :153-159).  Without a JIT
// the set is closed: every transformer here has the form
//     (TTarget)op((TSource)value)
// with op computed in the source type (wrapping for integers) followed by the
// C# explicit numeric conversion to the target type.  That covers
// IdentityTransformer (:42-55) and the transformers of the reference's own
// tests (Generic/AlgorithmsTestData.tt:170-252): int -> long, uint -> ulong,
// -value, (int)~value, (long)~value, value * 2, Index1D -> T.
//
// Conversions: integer -> integer truncates or extends by the source's sign;
// integer -> floating point and floating point -> floating point round to
// nearest even.  Floating point -> integer is rejected at the C ABI: C# leaves
// its result for NaN and out-of-range values unspecified.
//
// One pass: n * (sizeof(S) + sizeof(T)) bytes (+ 4 n for the order view).
#include "kernels.hpp"

namespace ilgpu_hip {

namespace {

constexpr int kBlock = 256;

inline int64_t grid_for(int64_t work_items) {
  int64_t blocks = div_up(work_items > 0 ? work_items : 1, kBlock);
  const int64_t cap = (int64_t)device_cu_count() * 4096;
  return blocks > cap ? cap : blocks;
}

template <typename T> struct is_float_type { static constexpr bool value = false; };
template <> struct is_float_type<_Float16> { static constexpr bool value = true; };
template <> struct is_float_type<float> { static constexpr bool value = true; };
template <> struct is_float_type<double> { static constexpr bool value = true; };

// op in the source type; integers wrap.
template <typename S>
__device__ __forceinline__ S apply_transformer(S v, int op, int64_t factor) {
  if constexpr (is_float_type<S>::value) {
    switch (op) {
      case ILGPU_HIP_TRANSFORM_NEGATE: return -v;
      case ILGPU_HIP_TRANSFORM_MULTIPLY: return v * (S)factor;
      default: return v;
    }
  } else {
    using U = typename std::make_unsigned<S>::type;
    switch (op) {
      case ILGPU_HIP_TRANSFORM_NEGATE: return (S)(U)(0u - (U)v);
      case ILGPU_HIP_TRANSFORM_BIT_COMPLEMENT: return (S)(U)~(U)v;
      // In 64 bits: 8- and 16-bit operands would be promoted to int, whose
      // product can overflow (0xFFFF * 0xFFFF); the low bits are the same.
      case ILGPU_HIP_TRANSFORM_MULTIPLY:
        return (S)(U)((uint64_t)(U)v * (uint64_t)factor);
      default: return v;
    }
  }
}

template <typename S, typename T>
__device__ __forceinline__ T convert(S v) {
  if constexpr (is_float_type<S>::value || is_float_type<T>::value) {
    return (T)v;  // round to nearest even; float -> integer never instantiated
  } else {
    // Extend by the source's sign to 64 bits, then truncate.
    using Wide = typename std::conditional<std::is_signed<S>::value, int64_t, uint64_t>::type;
    return (T)(typename std::make_unsigned<T>::type)(uint64_t)(Wide)v;
  }
}

// target[i * target_stride] = f(source[index]) with index = order[i] where an
// order view is given and i * source_stride otherwise.
template <typename S, typename T>
__global__ __launch_bounds__(kBlock) void transform_kernel(
    const S* source, int64_t source_stride, T* target, int64_t target_stride,
    const int32_t* __restrict__ order, int64_t n, int op, int64_t factor) {
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    const int64_t index = order != nullptr ? (int64_t)order[i] : i * source_stride;
    target[i * target_stride] =
        convert<S, T>(apply_transformer<S>(source[index], op, factor));
  }
}

// Dense views: K consecutive elements per thread, K chosen so that the wider
// of the two element types moves as one 16-byte vector.  The last n % K
// elements go through the scalar kernel.
template <typename E, int K> struct alignas(sizeof(E) * K) Pack { E v[K]; };

// Streaming (non-temporal) access to a pack as one machine vector of its size:
// dense transforms read and write every byte once (negate of 2^28 int32:
// 0.346 -> 0.33 ms).
template <int BYTES> struct PackBits;
template <> struct PackBits<2> { using type = uint16_t; };
template <> struct PackBits<4> { using type = uint32_t; };
template <> struct PackBits<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct PackBits<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
#ifndef ILGPU_HIP_TRANSFORM_NT
#define ILGPU_HIP_TRANSFORM_NT 1
#endif
template <typename P> __device__ __forceinline__ P load_pack(const P* p) {
  if constexpr (ILGPU_HIP_TRANSFORM_NT) {
    using B = typename PackBits<sizeof(P)>::type;
    const B bits = __builtin_nontemporal_load(reinterpret_cast<const B*>(p));
    P out;
    __builtin_memcpy(&out, &bits, sizeof(P));
    return out;
  } else {
    return *p;
  }
}
template <typename P> __device__ __forceinline__ void store_pack(P* p, const P& value) {
  if constexpr (ILGPU_HIP_TRANSFORM_NT) {
    using B = typename PackBits<sizeof(P)>::type;
    B bits;
    __builtin_memcpy(&bits, &value, sizeof(P));
    __builtin_nontemporal_store(bits, reinterpret_cast<B*>(p));
  } else {
    *p = value;
  }
}

template <typename S, typename T, int K>
__global__ __launch_bounds__(kBlock) void transform_dense_kernel(
    const Pack<S, K>* source, Pack<T, K>* target, int64_t packs, int op, int64_t factor) {
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < packs; i += step) {
    const Pack<S, K> in = load_pack(&source[i]);
    Pack<T, K> out;
#pragma unroll
    for (int k = 0; k < K; ++k)
      out.v[k] = convert<S, T>(apply_transformer<S>(in.v[k], op, factor));
    store_pack(&target[i], out);
  }
}

template <typename S, typename T>
int32_t transform_typed(hipStream_t stream, const TransformArgs& a) {
  if constexpr (is_float_type<S>::value && !is_float_type<T>::value) {
    return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  } else {
    ProfileScope scope(stream, a.order != nullptr ? "reorder_transform" : "transform");
    constexpr int kWide = sizeof(S) > sizeof(T) ? sizeof(S) : sizeof(T);
    constexpr int K = 16 / kWide;
    const bool dense = a.order == nullptr && a.source_stride == 1 && a.target_stride == 1 &&
                       reinterpret_cast<uintptr_t>(a.source) % (sizeof(S) * K) == 0 &&
                       reinterpret_cast<uintptr_t>(a.target) % (sizeof(T) * K) == 0;
    if (K > 1 && dense && a.n >= K) {
      const int64_t packs = a.n / K;
      hipLaunchKernelGGL((transform_dense_kernel<S, T, K>), dim3((unsigned)grid_for(packs)),
                         dim3(kBlock), 0, stream,
                         static_cast<const Pack<S, K>*>(a.source),
                         static_cast<Pack<T, K>*>(a.target), packs, a.transformer, a.factor);
      ILGPU_HIP_CHECK(hipGetLastError());
      const int64_t done = packs * K;
      if (done == a.n) return ILGPU_HIP_SUCCESS;
      hipLaunchKernelGGL((transform_kernel<S, T>), dim3(1), dim3(kBlock), 0, stream,
                         static_cast<const S*>(a.source) + done, (int64_t)1,
                         static_cast<T*>(a.target) + done, (int64_t)1,
                         static_cast<const int32_t*>(nullptr), a.n - done, a.transformer,
                         a.factor);
      ILGPU_HIP_CHECK(hipGetLastError());
      return ILGPU_HIP_SUCCESS;
    }
    hipLaunchKernelGGL((transform_kernel<S, T>), dim3((unsigned)grid_for(a.n)),
                       dim3(kBlock), 0, stream, static_cast<const S*>(a.source),
                       a.source_stride, static_cast<T*>(a.target), a.target_stride,
                       a.order, a.n, a.transformer, a.factor);
    ILGPU_HIP_CHECK(hipGetLastError());
    return ILGPU_HIP_SUCCESS;
  }
}

template <typename S>
int32_t transform_from(hipStream_t stream, const TransformArgs& a) {
  switch (a.target_type) {
    case ILGPU_HIP_I8: return transform_typed<S, int8_t>(stream, a);
    case ILGPU_HIP_U8: return transform_typed<S, uint8_t>(stream, a);
    case ILGPU_HIP_I16: return transform_typed<S, int16_t>(stream, a);
    case ILGPU_HIP_U16: return transform_typed<S, uint16_t>(stream, a);
    case ILGPU_HIP_I32: return transform_typed<S, int32_t>(stream, a);
    case ILGPU_HIP_U32: return transform_typed<S, uint32_t>(stream, a);
    case ILGPU_HIP_I64: return transform_typed<S, int64_t>(stream, a);
    case ILGPU_HIP_U64: return transform_typed<S, uint64_t>(stream, a);
    case ILGPU_HIP_F16: return transform_typed<S, _Float16>(stream, a);
    case ILGPU_HIP_F32: return transform_typed<S, float>(stream, a);
    case ILGPU_HIP_F64: return transform_typed<S, double>(stream, a);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace

int32_t launch_transform(hipStream_t stream, const TransformArgs& a) {
  switch (a.source_type) {
    case ILGPU_HIP_I8: return transform_from<int8_t>(stream, a);
    case ILGPU_HIP_U8: return transform_from<uint8_t>(stream, a);
    case ILGPU_HIP_I16: return transform_from<int16_t>(stream, a);
    case ILGPU_HIP_U16: return transform_from<uint16_t>(stream, a);
    case ILGPU_HIP_I32: return transform_from<int32_t>(stream, a);
    case ILGPU_HIP_U32: return transform_from<uint32_t>(stream, a);
    case ILGPU_HIP_I64: return transform_from<int64_t>(stream, a);
    case ILGPU_HIP_U64: return transform_from<uint64_t>(stream, a);
    case ILGPU_HIP_F16: return transform_from<_Float16>(stream, a);
    case ILGPU_HIP_F32: return transform_from<float>(stream, a);
    case ILGPU_HIP_F64: return transform_from<double>(stream, a);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace ilgpu_hip
