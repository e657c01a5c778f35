// Initialize, Sequence and Reorder: the element-wise neighbours of sort and scan
// in user pipelines (fill a view, write an index sequence, gather by index).
//
// Stand in for
//   Initializer delegates       InitializeExtensions.cs:26-31, 116-176
//   (Repeated)(Batched)Sequencer SequenceExtensions.cs:31-123, 238-630, with the
//                               identity sequencers of Sequencers.tt:25-37 and
//                               IndexSequencer (Sequencer.cs:36-45)
//   Reorder                     ReorderExtensions.cs:194-214 (identity transformer)
// The reference runs each as a grid-stride loop over a JIT-compiled functor;
// here the functor set is closed (a value, the index itself, a gather).
//
// Every kernel is one pass of stores (plus one read for the gather):
// n * sizeof(T) bytes written; 16 bytes per lane where the view is dense.
#include "kernels.hpp"

namespace ilgpu_hip {

namespace {

constexpr int kBlock = 256;

// One work item per thread up to a generous cap: pure store kernels run
// fastest (6.9 TB/s measured for a 1 GiB fill) when the grid is not folded into
// a few long grid-stride loops.
inline int64_t grid_for(int64_t work_items) {
  int64_t blocks = div_up(work_items > 0 ? work_items : 1, kBlock);
  const int64_t cap = (int64_t)device_cu_count() * 4096;
  return blocks > cap ? cap : blocks;
}

struct alignas(16) Bytes16 { uint32_t w[4]; };

// view[i * stride] = value
template <typename E>
__global__ __launch_bounds__(kBlock) void initialize_kernel(E* view, int64_t n,
                                                            int64_t stride, E value) {
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step)
    view[i * stride] = value;
}

// Dense views: 16-byte stores of the replicated value, scalar head and tail.
template <typename E>
__global__ __launch_bounds__(kBlock) void initialize_dense_kernel(E* view, int64_t n,
                                                                  E value) {
  using V = typename Vec16<E>::type;
  constexpr int VN = Vec16<E>::N;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(view);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(E));
  if (head > n) head = n;
  const int64_t nvec = (n - head) / VN;
  const int64_t tail_start = head + nvec * VN;
  V v;
#pragma unroll
  for (int k = 0; k < VN; ++k) v[k] = value;
  V* body = reinterpret_cast<V*>(view + head);
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += step)
    body[i] = v;
  if (blockIdx.x == 0) {
    const int64_t extra = head + (n - tail_start);
    if ((int64_t)threadIdx.x < extra) {
      const int64_t idx = (int64_t)threadIdx.x < head
                              ? (int64_t)threadIdx.x
                              : tail_start + ((int64_t)threadIdx.x - head);
      view[idx] = value;
    }
  }
}

template <typename E>
int32_t initialize_typed(hipStream_t stream, void* view, int64_t n, int64_t stride,
                         const void* value) {
  E v;
  __builtin_memcpy(&v, value, sizeof(E));
  ProfileScope scope(stream, "initialize");
  if constexpr (sizeof(E) < 16) {
    if (stride == 1) {
      hipLaunchKernelGGL((initialize_dense_kernel<E>),
                         dim3((unsigned)grid_for(n / Vec16<E>::N)), dim3(kBlock), 0,
                         stream, static_cast<E*>(view), n, v);
      ILGPU_HIP_CHECK(hipGetLastError());
      return ILGPU_HIP_SUCCESS;
    }
  }
  hipLaunchKernelGGL((initialize_kernel<E>), dim3((unsigned)grid_for(n)), dim3(kBlock), 0,
                     stream, static_cast<E*>(view), n, stride, v);
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

// view[i * stride] = (T)((i / batch_length) % sequence_length)
// (SequenceExtensions.cs:163-171 with ComputeSequenceElement(x) = (T)x).
template <typename T>
__global__ __launch_bounds__(kBlock) void sequence_kernel(T* view, int64_t n,
                                                          int64_t stride,
                                                          int64_t sequence_length,
                                                          int64_t batch_length) {
  const int64_t step = (int64_t)gridDim.x * kBlock;
  const bool plain = batch_length == 1 && sequence_length >= n;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    const int64_t s = plain ? i : (i / batch_length) % sequence_length;
    view[i * stride] = (T)s;
  }
}

// Dense views: 16-byte stores, scalar head and tail (as initialize_dense_kernel).
template <typename T>
__global__ __launch_bounds__(kBlock) void sequence_dense_kernel(T* view, int64_t n,
                                                                int64_t sequence_length,
                                                                int64_t batch_length) {
  using V = typename Vec16<T>::type;
  constexpr int VN = Vec16<T>::N;
  const bool plain = batch_length == 1 && sequence_length >= n;
  auto element = [&](int64_t i) -> T {
    return (T)(plain ? i : (i / batch_length) % sequence_length);
  };
  const uintptr_t addr = reinterpret_cast<uintptr_t>(view);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(T));
  if (head > n) head = n;
  const int64_t nvec = (n - head) / VN;
  const int64_t tail_start = head + nvec * VN;
  V* body = reinterpret_cast<V*>(view + head);
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += step) {
    V v;
#pragma unroll
    for (int k = 0; k < VN; ++k) v[k] = element(head + i * VN + k);
    body[i] = v;
  }
  if (blockIdx.x == 0) {
    const int64_t extra = head + (n - tail_start);
    if ((int64_t)threadIdx.x < extra) {
      const int64_t idx = (int64_t)threadIdx.x < head
                              ? (int64_t)threadIdx.x
                              : tail_start + ((int64_t)threadIdx.x - head);
      view[idx] = element(idx);
    }
  }
}

template <typename T>
int32_t sequence_typed(hipStream_t stream, void* view, int64_t n, int64_t stride,
                       int64_t sequence_length, int64_t batch_length) {
  ProfileScope scope(stream, "sequence");
  if (stride == 1) {
    hipLaunchKernelGGL((sequence_dense_kernel<T>),
                       dim3((unsigned)grid_for(n / Vec16<T>::N)), dim3(kBlock), 0, stream,
                       static_cast<T*>(view), n, sequence_length, batch_length);
    ILGPU_HIP_CHECK(hipGetLastError());
    return ILGPU_HIP_SUCCESS;
  }
  hipLaunchKernelGGL((sequence_kernel<T>), dim3((unsigned)grid_for(n)), dim3(kBlock), 0,
                     stream, static_cast<T*>(view), n, stride, sequence_length,
                     batch_length);
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

// target[i] = source[order[i]]
template <typename E>
__global__ __launch_bounds__(kBlock) void reorder_kernel(const E* __restrict__ source,
                                                         E* __restrict__ target,
                                                         const int32_t* __restrict__ order,
                                                         int64_t n) {
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step)
    target[i] = source[order[i]];
}

template <typename E>
int32_t reorder_typed(hipStream_t stream, const void* source, void* target,
                      const int32_t* order, int64_t n) {
  ProfileScope scope(stream, "reorder");
  hipLaunchKernelGGL((reorder_kernel<E>), dim3((unsigned)grid_for(n)), dim3(kBlock), 0,
                     stream, static_cast<const E*>(source), static_cast<E*>(target),
                     order, n);
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

}  // namespace

int32_t launch_initialize(hipStream_t stream, void* view, int64_t n, int64_t stride,
                          int elem_bytes, const void* value) {
  switch (elem_bytes) {
    case 1: return initialize_typed<uint8_t>(stream, view, n, stride, value);
    case 2: return initialize_typed<uint16_t>(stream, view, n, stride, value);
    case 4: return initialize_typed<uint32_t>(stream, view, n, stride, value);
    case 8: return initialize_typed<uint64_t>(stream, view, n, stride, value);
    case 16: return initialize_typed<Bytes16>(stream, view, n, stride, value);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

int32_t launch_sequence(hipStream_t stream, void* view, int64_t n, int64_t stride,
                        int32_t type, int64_t sequence_length, int64_t batch_length) {
  switch (type) {
    case ILGPU_HIP_I8: return sequence_typed<int8_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_U8: return sequence_typed<uint8_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_I16: return sequence_typed<int16_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_U16: return sequence_typed<uint16_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_I32: return sequence_typed<int32_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_U32: return sequence_typed<uint32_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_I64: return sequence_typed<int64_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_U64: return sequence_typed<uint64_t>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_F16: return sequence_typed<_Float16>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_F32: return sequence_typed<float>(stream, view, n, stride, sequence_length, batch_length);
    case ILGPU_HIP_F64: return sequence_typed<double>(stream, view, n, stride, sequence_length, batch_length);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

int32_t launch_reorder(hipStream_t stream, const void* source, void* target,
                       const int32_t* order, int64_t n, int elem_bytes) {
  switch (elem_bytes) {
    case 1: return reorder_typed<uint8_t>(stream, source, target, order, n);
    case 2: return reorder_typed<uint16_t>(stream, source, target, order, n);
    case 4: return reorder_typed<uint32_t>(stream, source, target, order, n);
    case 8: return reorder_typed<uint64_t>(stream, source, target, order, n);
    case 16: return reorder_typed<Bytes16>(stream, source, target, order, n);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace ilgpu_hip
