// Reduction: out[0] = fold(op, in[0..n)).
//
// Stands in for ReductionImplementation + CreateReduction
// (ReductionExtensions.cs:52-167).  The reference folds per thread in a
// grid-stride loop, reduces the group and issues one global atomic per group;
// here the same fold is a hierarchical wave -> block -> grid reduction with a
// fixed association order, so the result is deterministic:
//
//   kernel 1  every lane streams 16-byte vectors (dwordx4, nontemporal) in a
//             grid-stride loop and folds them into private accumulators, then
//             a wave64 shuffle tree and a small LDS exchange leave one partial
//             per block in `partials[blockIdx]`.  Blocks of 1024 threads, one
//             vector per lane and iteration, 8 blocks per CU measured fastest
//             (wider unrolling or smaller blocks lose 5-15 %);
//   kernel 2  one block folds the partials in index order and writes out[0].
//
// float Add accumulates in float64 (conversion and fp64 adds are free under
// the HBM bound) and rounds once at the end, which keeps the result within
// 1e-5 relative of a float64 host sum even when the sum is close to zero.
//
// Algorithmic HBM traffic: n * sizeof(T) bytes read (partials are < 32 KiB).
#include "common.hpp"

namespace ilgpu_hip {

namespace {

#ifndef ILGPU_HIP_REDUCE_BLOCK
#define ILGPU_HIP_REDUCE_BLOCK 1024
#endif
#ifndef ILGPU_HIP_REDUCE_UNROLL
#define ILGPU_HIP_REDUCE_UNROLL 1
#endif
#ifndef ILGPU_HIP_REDUCE_BLOCKS_PER_CU
#define ILGPU_HIP_REDUCE_BLOCKS_PER_CU 8
#endif
constexpr int kBlock = ILGPU_HIP_REDUCE_BLOCK;
constexpr int kUnroll = ILGPU_HIP_REDUCE_UNROLL;
constexpr int kMaxBlocks = 4096;  // upper bound on partials, fixes the temp size
constexpr int kBlocksPerCu = ILGPU_HIP_REDUCE_BLOCKS_PER_CU;
constexpr int64_t kSingleBlockElements = 32768;  // inputs up to here: one block, one launch

template <typename T, int OP> struct AccType { using type = T; };
template <> struct AccType<float, ILGPU_HIP_OP_ADD> { using type = double; };

template <typename A, int OP>
__device__ __forceinline__ A block_fold(A v, A* lds) {
  using F = Functor<A, OP>;
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1)
    v = F::apply(v, shfl_down(v, off));
  const int wave = threadIdx.x / kWaveSize;
  if ((threadIdx.x & (kWaveSize - 1)) == 0) lds[wave] = v;
  __syncthreads();
  A r = lds[0];
#pragma unroll
  for (int w = 1; w < kBlock / kWaveSize; ++w) r = F::apply(r, lds[w]);
  return r;
}

template <typename T, int OP>
__global__ __launch_bounds__(kBlock) void reduce_partials_kernel(
    const T* __restrict__ in, int64_t n, int64_t in_stride,
    typename AccType<T, OP>::type* __restrict__ partials, T* __restrict__ result) {
  using A = typename AccType<T, OP>::type;
  using F = Functor<A, OP>;
  using V = typename Vec16<T>::type;
  constexpr int VN = Vec16<T>::N;
  __shared__ A lds[kBlock / kWaveSize];

  if (in_stride != 1) {
    // Stride1D.General with an element stride above one: element i lives at
    // in[i * in_stride]; one scalar load per element.
    A acc = F::identity();
    const int64_t step = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step)
      acc = F::apply(acc, (A)in[i * in_stride]);
    A r = block_fold<A, OP>(acc, lds);
    if (threadIdx.x == 0) {
      if (result != nullptr) result[0] = (T)r;
      else partials[blockIdx.x] = r;
    }
    return;
  }

  // Split [0,n) into an unaligned head, a body of whole 16-byte vectors and a
  // tail; head and tail together hold fewer than 2*VN elements.
  const uintptr_t addr = reinterpret_cast<uintptr_t>(in);
  int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(T));
  if (head > n) head = n;
  const V* body = reinterpret_cast<const V*>(in + head);
  const int64_t nvec = (n - head) / VN;
  const int64_t tail_start = head + nvec * VN;

  A acc[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) acc[u] = F::identity();

  const int64_t stride = (int64_t)gridDim.x * kBlock;
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  for (; i + (kUnroll - 1) * stride < nvec; i += kUnroll * stride) {
    V v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      v[u] = __builtin_nontemporal_load(&body[i + u * stride]);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int k = 0; k < VN; ++k) acc[u] = F::apply(acc[u], (A)v[u][k]);
  }
  for (; i < nvec; i += stride) {
    V v = __builtin_nontemporal_load(&body[i]);
#pragma unroll
    for (int k = 0; k < VN; ++k) acc[0] = F::apply(acc[0], (A)v[k]);
  }
  if (blockIdx.x == 0) {
    const int64_t extra = head + (n - tail_start);
    if ((int64_t)threadIdx.x < extra) {
      const int64_t idx = (int64_t)threadIdx.x < head
                              ? (int64_t)threadIdx.x
                              : tail_start + ((int64_t)threadIdx.x - head);
      acc[0] = F::apply(acc[0], (A)in[idx]);
    }
  }
#pragma unroll
  for (int u = 1; u < kUnroll; ++u) acc[0] = F::apply(acc[0], acc[u]);
  A r = block_fold<A, OP>(acc[0], lds);
  if (threadIdx.x == 0) {
    // A launch of one block is the whole reduction: no second kernel.
    if (result != nullptr) result[0] = (T)r;
    else partials[blockIdx.x] = r;
  }
}

template <typename T, int OP>
__global__ __launch_bounds__(kBlock) void reduce_final_kernel(
    const typename AccType<T, OP>::type* __restrict__ partials,
    int num_partials, T* __restrict__ out) {
  using A = typename AccType<T, OP>::type;
  using F = Functor<A, OP>;
  __shared__ A lds[kBlock / kWaveSize];
  A acc = F::identity();
  for (int i = threadIdx.x; i < num_partials; i += kBlock)
    acc = F::apply(acc, partials[i]);
  A r = block_fold<A, OP>(acc, lds);
  if (threadIdx.x == 0) out[0] = (T)r;
}

template <typename T, int OP>
int32_t launch_typed(hipStream_t stream, const void* in, int64_t n,
                     int64_t in_stride, void* out, void* temp) {
  using A = typename AccType<T, OP>::type;
  const int64_t nvec = n / Vec16<T>::N;
  int64_t blocks = div_up(nvec > 0 ? nvec : 1, kBlock);
  const int64_t cap = (int64_t)device_cu_count() * kBlocksPerCu;
  if (blocks > cap) blocks = cap;
  if (blocks > kMaxBlocks) blocks = kMaxBlocks;
  if (blocks < 1) blocks = 1;
  // Short inputs: one block folds everything and writes the result itself (a
  // second launch costs more than the first block's extra elements).
  if (n <= kSingleBlockElements) blocks = 1;
  A* partials = reinterpret_cast<A*>(align_up((int64_t)(uintptr_t)temp, 16));
  {
    ProfileScope scope(stream, "reduce_partials");
    hipLaunchKernelGGL((reduce_partials_kernel<T, OP>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, stream, static_cast<const T*>(in), n,
                       in_stride, partials,
                       blocks == 1 ? static_cast<T*>(out) : static_cast<T*>(nullptr));
  }
  ILGPU_HIP_CHECK(hipGetLastError());
  if (blocks == 1) return ILGPU_HIP_SUCCESS;
  {
    ProfileScope scope(stream, "reduce_final");
    hipLaunchKernelGGL((reduce_final_kernel<T, OP>), dim3(1), dim3(kBlock), 0,
                       stream, partials, (int)blocks, static_cast<T*>(out));
  }
  ILGPU_HIP_CHECK(hipGetLastError());
  return ILGPU_HIP_SUCCESS;
}

template <typename T>
int32_t launch_op(hipStream_t stream, const void* in, int64_t n,
                  int64_t in_stride, int32_t op, void* out, void* temp) {
  switch (op) {
    case ILGPU_HIP_OP_ADD:
      return launch_typed<T, ILGPU_HIP_OP_ADD>(stream, in, n, in_stride, out, temp);
    case ILGPU_HIP_OP_MAX:
      return launch_typed<T, ILGPU_HIP_OP_MAX>(stream, in, n, in_stride, out, temp);
    case ILGPU_HIP_OP_MIN:
      return launch_typed<T, ILGPU_HIP_OP_MIN>(stream, in, n, in_stride, out, temp);
    default:
      return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace

int64_t reduce_temp_bytes() { return (int64_t)kMaxBlocks * 8 + 16; }

int32_t launch_reduce(hipStream_t stream, const void* in, int64_t n,
                      int64_t in_stride, int32_t type, int32_t op, void* out,
                      void* temp) {
  switch (type) {
    case ILGPU_HIP_I32: return launch_op<int32_t>(stream, in, n, in_stride, op, out, temp);
    case ILGPU_HIP_U32: return launch_op<uint32_t>(stream, in, n, in_stride, op, out, temp);
    case ILGPU_HIP_I64: return launch_op<int64_t>(stream, in, n, in_stride, op, out, temp);
    case ILGPU_HIP_U64: return launch_op<uint64_t>(stream, in, n, in_stride, op, out, temp);
    case ILGPU_HIP_F32: return launch_op<float>(stream, in, n, in_stride, op, out, temp);
    case ILGPU_HIP_F64: return launch_op<double>(stream, in, n, in_stride, op, out, temp);
    default: return ILGPU_HIP_ERROR_NOT_SUPPORTED;
  }
}

}  // namespace ilgpu_hip
