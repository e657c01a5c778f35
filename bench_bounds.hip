// Micro-benchmarks that bound the kernels of libilgpu_hip_algorithms on one MI355X.
//
// Each section measures one hardware rate that a kernel of the library cannot
// beat, with the access pattern of that kernel and nothing else around it:
//
//   copy     read, write and copy rates of 1 GiB for the shapes the kernels
//            use (grid-stride vectors; one tile per block held in registers,
//            wave-contiguous or block-strided): the ceiling of scan, unique,
//            transform, sequence and reduce.
//   scatter  the sort pass's write pattern by itself: every tile reads its
//            keys linearly and writes 256 runs, each directly behind the run
//            of the previous tile in that digit's region; against the same
//            kernel writing linearly.
//   lds      LDS instructions per cycle and compute unit (atomics with and
//            without replicas, loads, stores), and LDS atomics next to a key
//            stream from memory: the ceiling of the histogram kernels.
//   latency  time until a batch of N status-row loads has returned to one
//            wave, on an idle device and on a compute unit that is streaming
//            keys: what a look-back step costs.
//
//   tiles    blocks per microsecond with and without a ticket, and a tile-shaped
//            read of 1 GiB behind it: what scan and unique pay per tile before
//            any arithmetic.
//
// Usage: bench_bounds [copy|scatter|lds|latency|tiles|all]   (default all)
// Built by `python -m ilgpu_amd.build` into ilgpu_amd/lib/bench_bounds.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CK(expr)                                                                  \
  do {                                                                            \
    hipError_t e_ = (expr);                                                       \
    if (e_ != hipSuccess) {                                                       \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);  \
      std::exit(1);                                                               \
    }                                                                             \
  } while (0)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

static int g_cus = 256;

template <typename F>
static float time_ms(F launch, int iters = 20) {
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 3; ++i) launch();
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(a));
  for (int i = 0; i < iters; ++i) launch();
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms = 0;
  CK(hipEventElapsedTime(&ms, a, b));
  CK(hipEventDestroy(a));
  CK(hipEventDestroy(b));
  return ms / iters;
}

// ---------------------------------------------------------------- copy ----
template <int BLOCK, int UNROLL>
__global__ __launch_bounds__(BLOCK) void read_stride(const u32x4* __restrict__ in,
                                                     uint32_t* __restrict__ out, int64_t nvec) {
  const int64_t stride = (int64_t)gridDim.x * BLOCK;
  uint32_t acc = 0;
  int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
  for (; i + (UNROLL - 1) * stride < nvec; i += UNROLL * stride) {
    u32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(&in[i + u * stride]);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc += v[u].x + v[u].y + v[u].z + v[u].w;
  }
  for (; i < nvec; i += stride) acc += in[i].x;
  if (acc == 0x12345678u) out[0] = acc;
}

// One vector per thread, one block per 4 KiB.
__global__ __launch_bounds__(256) void write_one_vector(u32x4* __restrict__ out, int64_t nvec) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const u32x4 v = {1u, 2u, 3u, (uint32_t)threadIdx.x};
  if (i < nvec) __builtin_nontemporal_store(v, &out[i]);
}

// One 16-byte vector per thread, one block per 4 KiB.
__global__ __launch_bounds__(256) void copy_one_vector(const u32x4* __restrict__ in,
                                                       u32x4* __restrict__ out, int64_t nvec) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < nvec) __builtin_nontemporal_store(__builtin_nontemporal_load(&in[i]), &out[i]);
}

template <int BLOCK, int UNROLL>
__global__ __launch_bounds__(BLOCK) void copy_stride(const u32x4* __restrict__ in,
                                                     u32x4* __restrict__ out, int64_t nvec) {
  const int64_t stride = (int64_t)gridDim.x * BLOCK;
  int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
  for (; i + (UNROLL - 1) * stride < nvec; i += UNROLL * stride) {
    u32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(&in[i + u * stride]);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) __builtin_nontemporal_store(v[u], &out[i + u * stride]);
  }
  for (; i < nvec; i += stride) out[i] = in[i];
}

// The scan kernel's shape: a block holds one tile of BLOCK * VECS vectors in
// registers, loads all of it, then stores all of it.  WAVE_CONTIGUOUS: every
// wave owns VECS consecutive KiB; otherwise vector j of the block is one
// contiguous stretch of BLOCK vectors.
template <int BLOCK, int VECS, bool WAVE_CONTIGUOUS>
__global__ __launch_bounds__(BLOCK) void copy_tile(const u32x4* __restrict__ in,
                                                   u32x4* __restrict__ out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t tile = (int64_t)blockIdx.x * BLOCK * VECS;
  u32x4 v[VECS];
#pragma unroll
  for (int j = 0; j < VECS; ++j) {
    const int64_t i = WAVE_CONTIGUOUS ? tile + ((int64_t)wave * VECS + j) * 64 + lane
                                      : tile + (int64_t)j * BLOCK + threadIdx.x;
    v[j] = __builtin_nontemporal_load(&in[i]);
  }
#pragma unroll
  for (int j = 0; j < VECS; ++j) {
    const int64_t i = WAVE_CONTIGUOUS ? tile + ((int64_t)wave * VECS + j) * 64 + lane
                                      : tile + (int64_t)j * BLOCK + threadIdx.x;
    __builtin_nontemporal_store(v[j], &out[i]);
  }
}

template <int BLOCK, int VECS, bool WC>
static void run_copy_tile(const u32x4* a, u32x4* b, int64_t nvec) {
  const int grid = (int)(nvec / (BLOCK * VECS));
  const float ms = time_ms([&] { hipLaunchKernelGGL((copy_tile<BLOCK, VECS, WC>), dim3(grid), dim3(BLOCK), 0, 0, a, b); });
  std::printf("  copy, tile in registers, %4d threads x %2d vectors, %s: %.4f ms  %.0f GB/s\n", BLOCK,
              VECS, WC ? "wave-contiguous" : "block-strided  ", ms, 2.0 * nvec * 16 / ms / 1e6);
}

static void section_copy() {
  const int64_t nvec = (int64_t)1 << 26;  // 1 GiB
  const double bytes = (double)nvec * 16;
  u32x4 *a, *b;
  uint32_t* o;
  CK(hipMalloc(&a, nvec * 16));
  CK(hipMalloc(&b, nvec * 16));
  CK(hipMalloc(&o, 4));
  CK(hipMemset(a, 1, nvec * 16));
  CK(hipMemset(b, 0, nvec * 16));
  std::printf("copy: 1 GiB, non-temporal loads and stores, mean of 20 launches\n");
  float ms;
  ms = time_ms([&] { hipLaunchKernelGGL((read_stride<1024, 4>), dim3(g_cus * 2), dim3(1024), 0, 0, a, o, nvec); });
  std::printf("  read, grid-stride, 1024 threads x 4 vectors, 2 blocks per CU: %.4f ms  %.0f GB/s\n", ms, bytes / ms / 1e6);
  ms = time_ms([&] { hipLaunchKernelGGL((read_stride<512, 2>), dim3(g_cus * 4), dim3(512), 0, 0, a, o, nvec); });
  std::printf("  read, grid-stride,  512 threads x 2 vectors, 4 blocks per CU: %.4f ms  %.0f GB/s\n", ms, bytes / ms / 1e6);
  ms = time_ms([&] { hipLaunchKernelGGL(write_one_vector, dim3((unsigned)(nvec / 256)), dim3(256), 0, 0, b, nvec); });
  std::printf("  write, one vector per thread, 256-thread blocks: %.4f ms  %.0f GB/s\n", ms, bytes / ms / 1e6);
  ms = time_ms([&] { (void)hipMemsetAsync(b, 0, nvec * 16, 0); });
  std::printf("  hipMemsetAsync: %.4f ms  %.0f GB/s\n", ms, bytes / ms / 1e6);
  ms = time_ms([&] { hipLaunchKernelGGL(copy_one_vector, dim3((unsigned)(nvec / 256)), dim3(256), 0, 0, a, b, nvec); });
  std::printf("  copy, one vector per thread, 256-thread blocks: %.4f ms  %.0f GB/s\n", ms, 2 * bytes / ms / 1e6);
  ms = time_ms([&] { hipLaunchKernelGGL((copy_stride<256, 4>), dim3(g_cus * 8), dim3(256), 0, 0, a, b, nvec); });
  std::printf("  copy, grid-stride, 256 threads x 4 vectors, 8 blocks per CU: %.4f ms  %.0f GB/s\n", ms, 2 * bytes / ms / 1e6);
  run_copy_tile<256, 1, true>(a, b, nvec);
  run_copy_tile<256, 2, true>(a, b, nvec);
  run_copy_tile<256, 4, true>(a, b, nvec);
  run_copy_tile<256, 8, true>(a, b, nvec);
  run_copy_tile<1024, 1, true>(a, b, nvec);
  run_copy_tile<1024, 2, true>(a, b, nvec);
  run_copy_tile<1024, 4, true>(a, b, nvec);
  run_copy_tile<512, 16, true>(a, b, nvec);
  run_copy_tile<512, 16, false>(a, b, nvec);
  run_copy_tile<1024, 8, true>(a, b, nvec);
  run_copy_tile<256, 16, true>(a, b, nvec);
  run_copy_tile<512, 8, true>(a, b, nvec);
  ms = time_ms([&] { (void)hipMemcpyAsync(b, a, nvec * 16, hipMemcpyDeviceToDevice, 0); });
  std::printf("  hipMemcpyAsync device to device: %.4f ms  %.0f GB/s\n", ms, 2 * bytes / ms / 1e6);
  CK(hipFree(a));
  CK(hipFree(b));
  CK(hipFree(o));
}

// ------------------------------------------------------------- scatter ----
// MODE 0: runs behind the previous tile's runs; 1: the same kernel writing its
// tile linearly; 2: as 0, but every store instruction covers one 256-byte
// aligned window of one run (lanes before the run's start are idle) and reads
// what it stores from LDS; 10: as 2 with chunks of 8; C = 8, 16, 32: as 0, with chunks of C consecutive
// tiles kept on one XCD (blocks are dealt to the eight XCDs round-robin).
template <int BLOCK, int KPT, int MODE>
__global__ __launch_bounds__(BLOCK) void scatter_runs(const uint32_t* __restrict__ src,
                                                      uint32_t* __restrict__ dst,
                                                      const uint32_t* __restrict__ start,
                                                      const uint16_t* __restrict__ len) {
  extern __shared__ uint32_t lds[];
  uint32_t* s_digit = lds;                 // digit of every staged position
  uint32_t* s_off = lds + KPT * BLOCK;     // global start - local start, per digit
  uint32_t* s_pre = s_off + 256;
  uint32_t* s_len = s_pre + 256;
  uint32_t* s_start = s_len + 256;
  int t = blockIdx.x;
  if (MODE >= 8) {
    constexpr int C = MODE == 10 ? 8 : MODE;
    const int xcd = blockIdx.x % 8, k = blockIdx.x / 8;
    const int tt = (8 * (k / C) + xcd) * C + k % C;
    if ((int)blockIdx.x < (int)(gridDim.x / (8 * C)) * 8 * C) t = tt;
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t key[KPT];
  const uint32_t* in = src + (size_t)t * BLOCK * KPT;
#pragma unroll
  for (int j = 0; j < KPT; ++j) key[j] = in[j * BLOCK + tid];
  if (tid < 256) {
    s_len[tid] = len[(size_t)t * 256 + tid];
    s_start[tid] = start[(size_t)t * 256 + tid];
  }
  __syncthreads();
  if (tid < 64) {  // exclusive scan of the 256 run lengths by one wave
    const uint32_t a = s_len[tid * 4], b = s_len[tid * 4 + 1], c = s_len[tid * 4 + 2], d = s_len[tid * 4 + 3];
    const uint32_t sum = a + b + c + d;
    uint32_t inc = sum;
    for (int s = 1; s < 64; s <<= 1) {
      const uint32_t o = __shfl_up(inc, s, 64);
      if (lane >= s) inc += o;
    }
    const uint32_t ex = inc - sum;
    s_pre[tid * 4] = ex;
    s_pre[tid * 4 + 1] = ex + a;
    s_pre[tid * 4 + 2] = ex + a + b;
    s_pre[tid * 4 + 3] = ex + a + b + c;
  }
  __syncthreads();
  if (tid < 256) s_off[tid] = s_start[tid] - s_pre[tid];
  for (int d = wave; d < 256; d += BLOCK / 64) {
    const uint32_t p = s_pre[d], n = s_len[d];
    for (uint32_t i = lane; i < n; i += 64) s_digit[p + i] = d;
  }
  __syncthreads();
  if (MODE == 2 || MODE == 10) {
    // every wave takes digits; its lanes sit on 256-byte windows of the destination
    for (int d = wave; d < 256; d += BLOCK / 64) {
      const uint32_t b = s_start[d], e = b + s_len[d];
      for (uint32_t p = (b & ~63u) + lane; p < e; p += 64)
        if (p >= b) dst[p] = key[0] + s_digit[p - s_off[d]];
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < KPT; ++j) {
    const int p = j * BLOCK + tid;
    const uint32_t d = s_digit[p];
    if (MODE == 1) dst[(size_t)t * BLOCK * KPT + p] = key[j] + d + s_off[d];
    else dst[s_off[d] + p] = key[j] + d;
  }
}

template <int BLOCK, int KPT>
static void run_scatter(const char* name, int spread, const uint32_t* src, uint32_t* dst, size_t n) {
  const int tile_keys = BLOCK * KPT;
  const int tiles = (int)(n / tile_keys);
  const int mean = tile_keys / 256;
  std::vector<uint32_t> start((size_t)256 * tiles);
  std::vector<uint16_t> len((size_t)256 * tiles);
  std::vector<uint32_t> pos(256);
  uint64_t x = 88172645463325252ull;
  for (int d = 0; d < 256; ++d) pos[d] = (uint32_t)((n / 256) * d);
  for (int t = 0; t < tiles; ++t) {
    int left = tile_keys;
    for (int d = 0; d < 256; ++d) {
      x ^= x << 13; x ^= x >> 7; x ^= x << 17;
      int l = mean + (spread ? (int)(x % (2 * spread + 1)) - spread : 0);
      if (d == 255 || l > left) l = left;  // the runs of a tile add up to the tile
      if (pos[d] + l > (n / 256) * (d + 1) + (1 << 16)) l = 0;
      start[(size_t)t * 256 + d] = pos[d];
      len[(size_t)t * 256 + d] = (uint16_t)l;
      pos[d] += l;
      left -= l;
    }
  }
  uint32_t* dstart;
  uint16_t* dlen;
  CK(hipMalloc(&dstart, start.size() * 4));
  CK(hipMalloc(&dlen, len.size() * 2));
  CK(hipMemcpy(dstart, start.data(), start.size() * 4, hipMemcpyHostToDevice));
  CK(hipMemcpy(dlen, len.data(), len.size() * 2, hipMemcpyHostToDevice));
  const size_t lds = (size_t)(tile_keys + 4 * 256) * 4;
  CK(hipFuncSetAttribute((const void*)scatter_runs<BLOCK, KPT, 0>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  CK(hipFuncSetAttribute((const void*)scatter_runs<BLOCK, KPT, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  CK(hipFuncSetAttribute((const void*)scatter_runs<BLOCK, KPT, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  CK(hipFuncSetAttribute((const void*)scatter_runs<BLOCK, KPT, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  CK(hipFuncSetAttribute((const void*)scatter_runs<BLOCK, KPT, 10>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  CK(hipFuncSetAttribute((const void*)scatter_runs<BLOCK, KPT, 16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  CK(hipFuncSetAttribute((const void*)scatter_runs<BLOCK, KPT, 32>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  const double bytes = 2.0 * (double)tiles * tile_keys * 4;
  for (int mode : {1, 0, 2, 8, 10, 16, 32}) {
    const float ms = time_ms([&] {
      if (mode == 0) hipLaunchKernelGGL((scatter_runs<BLOCK, KPT, 0>), dim3(tiles), dim3(BLOCK), lds, 0, src, dst, dstart, dlen);
      else if (mode == 1) hipLaunchKernelGGL((scatter_runs<BLOCK, KPT, 1>), dim3(tiles), dim3(BLOCK), lds, 0, src, dst, dstart, dlen);
      else if (mode == 2) hipLaunchKernelGGL((scatter_runs<BLOCK, KPT, 2>), dim3(tiles), dim3(BLOCK), lds, 0, src, dst, dstart, dlen);
      else if (mode == 10) hipLaunchKernelGGL((scatter_runs<BLOCK, KPT, 10>), dim3(tiles), dim3(BLOCK), lds, 0, src, dst, dstart, dlen);
      else if (mode == 8) hipLaunchKernelGGL((scatter_runs<BLOCK, KPT, 8>), dim3(tiles), dim3(BLOCK), lds, 0, src, dst, dstart, dlen);
      else if (mode == 16) hipLaunchKernelGGL((scatter_runs<BLOCK, KPT, 16>), dim3(tiles), dim3(BLOCK), lds, 0, src, dst, dstart, dlen);
      else hipLaunchKernelGGL((scatter_runs<BLOCK, KPT, 32>), dim3(tiles), dim3(BLOCK), lds, 0, src, dst, dstart, dlen);
    }, 5);
    char what[64];
    if (mode == 1) std::snprintf(what, sizeof what, "linear write");
    else if (mode == 0) std::snprintf(what, sizeof what, "256 runs per tile");
    else if (mode == 2) std::snprintf(what, sizeof what, "256 runs per tile, aligned windows");
    else if (mode == 10) std::snprintf(what, sizeof what, "256 runs, 8 per XCD, aligned windows");
    else std::snprintf(what, sizeof what, "256 runs, %d consecutive tiles per XCD", mode);
    std::printf("  %-38s %-40s %.3f ms  %.0f GB/s\n", name, what, ms, bytes / ms / 1e6);
  }
  CK(hipFree(dstart));
  CK(hipFree(dlen));
}

static void section_scatter() {
  const size_t n = (size_t)1 << 28;
  uint32_t *src, *dst;
  CK(hipMalloc(&src, n * 4 + (1 << 24)));
  CK(hipMalloc(&dst, n * 4 + (1 << 24)));
  CK(hipMemset(src, 1, n * 4));
  CK(hipMemset(dst, 0, n * 4));
  std::printf("scatter: 2^28 u32 keys read linearly, written as the sort pass writes them (read + write bytes)\n");
  run_scatter<512, 36>("tile 18432 keys, runs of 72 +- 12", 12, src, dst, n);
  run_scatter<960, 36>("tile 34560 keys, runs of 135 +- 16", 16, src, dst, n);
  run_scatter<960, 36>("tile 34560 keys, runs of 135 exactly", 0, src, dst, n);
  CK(hipFree(src));
  CK(hipFree(dst));
}

// ----------------------------------------------------------------- lds ----
constexpr int kLdsIters = 2048;
// MODE 0: add, 32 replicas (bin * 32 + lane % 32); 1: add, 16 replicas; 2: add, no
// replicas; 3: returning add, 32 replicas; 4: store; 5: load; 6: 64-bit add;
// 7: add to a fixed address per lane (no address arithmetic).
template <int MODE>
__global__ void lds_rate(uint32_t* out, int active_lanes) {
  extern __shared__ uint32_t s[];
  for (int i = threadIdx.x; i < 8192; i += blockDim.x) s[i] = 0;
  __syncthreads();
  const int lane = threadIdx.x & 63;
  uint32_t x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  uint32_t acc = 0;
  if (lane < active_lanes) {
    for (int it = 0; it < kLdsIters; ++it) {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if ((k & 3) == 0) { x ^= x << 13; x ^= x >> 17; x ^= x << 5; }
        const uint32_t bin = (x >> (8 * (k & 3))) & 255u;
        if constexpr (MODE == 0) atomicAdd(&s[(bin << 5) + (lane & 31)], 1u);
        if constexpr (MODE == 1) atomicAdd(&s[(bin << 4) + (lane & 15)], 1u);
        if constexpr (MODE == 2) atomicAdd(&s[bin], 1u);
        if constexpr (MODE == 3) acc += atomicAdd(&s[(bin << 5) + (lane & 31)], 1u);
        if constexpr (MODE == 4) s[(bin << 5) + (lane & 31)] = x;
        if constexpr (MODE == 5) acc += s[(bin << 5) + (lane & 31)];
        if constexpr (MODE == 6)
          atomicAdd(reinterpret_cast<unsigned long long*>(&s[((bin & 127) << 6) + 2 * (lane & 31)]), 1ull);
        if constexpr (MODE == 7) atomicAdd(&s[lane], 1u);
      }
    }
  }
  __syncthreads();
  if (acc == 0x12345678u || s[threadIdx.x] == 0xFFFFFFFFu) out[0] = acc;
}

template <int MODE>
static void run_lds_rate(const char* name, int block, int blocks_per_cu, int active, uint32_t* out) {
  const int grid = g_cus * blocks_per_cu;
  const float ms = time_ms([&] { hipLaunchKernelGGL(lds_rate<MODE>, dim3(grid), dim3(block), 32768, 0, out, active); }, 3);
  const double per_cu = (double)blocks_per_cu * (block / 64) * kLdsIters * 8;
  std::printf("  %-30s %2d waves per CU, %2d lanes: %.3f ms, one wave instruction per %.2f ns and CU\n", name,
              blocks_per_cu * block / 64, active, ms, ms * 1e6 / per_cu);
}

// Digit histogram of 2^28 u32 keys as the sort's histogram kernel counts them:
// four LDS atomics per key into 16 replicas.  SOURCE 0: keys made in registers;
// 1: keys loaded (non-temporal when NT); 2: keys loaded, nothing counted.
template <int SOURCE, bool NT>
__global__ __launch_bounds__(512) void lds_beside_stream(const u32x4* __restrict__ keys, int64_t nvec,
                                                         uint32_t* out, unsigned long long* clocks) {
  extern __shared__ uint32_t s[];
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) s[i] = 0;
  __syncthreads();
  const long long c0 = clock64(), w0 = wall_clock64();
  const uint32_t lane_base = (threadIdx.x & 15) * 4u;
  char* counters = reinterpret_cast<char*>(s);
  uint32_t x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  uint32_t acc = 0;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // two vectors per round, as the kernel (nvec is a multiple of 2 * stride here)
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i + stride < nvec; i += 2 * stride) {
    u32x4 v[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if constexpr (SOURCE == 0) {
        x ^= x << 13; x ^= x >> 17; x ^= x << 5; v[u].x = x;
        x ^= x << 13; x ^= x >> 17; x ^= x << 5; v[u].y = x;
        x ^= x << 13; x ^= x >> 17; x ^= x << 5; v[u].z = x;
        x ^= x << 13; x ^= x >> 17; x ^= x << 5; v[u].w = x;
      } else {
        v[u] = NT ? __builtin_nontemporal_load(&keys[i + u * stride]) : keys[i + u * stride];
      }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if constexpr (SOURCE == 2) {
        acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
      } else {
        const uint32_t k[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
          for (int p = 0; p < 4; ++p) {
            const uint32_t d = (k[q] >> (8 * p)) & 255u;
            atomicAdd(reinterpret_cast<uint32_t*>(counters + ((d << 6) + lane_base + p * 16384u)), 1u);
          }
        }
      }
    }
  }
  __syncthreads();
  const long long c1 = clock64(), w1 = wall_clock64();
  if (threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
  if (acc == 0x12345678u || s[threadIdx.x] == 0xFFFFFFFFu) out[0] = acc;
}

template <int SOURCE, bool NT>
static void run_lds_beside(const char* name, const u32x4* keys, int64_t nvec, uint32_t* out,
                           unsigned long long* clocks) {
  const int grid = g_cus * 2;
  const float ms = time_ms([&] { hipLaunchKernelGGL((lds_beside_stream<SOURCE, NT>), dim3(grid), dim3(512), 65536, 0, keys, nvec, out, clocks); }, 5);
  std::vector<unsigned long long> h(2 * grid);
  CK(hipMemcpy(h.data(), clocks, h.size() * 8, hipMemcpyDeviceToHost));
  double c = 0, w = 0;
  for (int i = 0; i < grid; ++i) { c += (double)h[2 * i]; w += (double)h[2 * i + 1]; }
  std::printf("  %-46s %.4f ms  (shader clock %.0f MHz; key bytes %.0f GB/s)\n", name, ms, c / w * 100.0,
              nvec * 16.0 / ms / 1e6);
}

static void section_lds() {
  uint32_t* out;
  CK(hipMalloc(&out, 4));
  std::printf("lds: 2048 x 8 LDS instructions per wave, addresses from a register generator, no memory traffic\n");
  run_lds_rate<0>("add, 32 replicas", 512, 1, 64, out);
  run_lds_rate<0>("add, 32 replicas", 512, 2, 64, out);
  run_lds_rate<0>("add, 32 replicas", 512, 4, 64, out);
  run_lds_rate<0>("add, 32 replicas", 512, 2, 32, out);
  run_lds_rate<0>("add, 32 replicas", 512, 2, 16, out);
  run_lds_rate<1>("add, 16 replicas", 512, 2, 64, out);
  run_lds_rate<2>("add, no replicas", 512, 2, 64, out);
  run_lds_rate<3>("returning add, 32 replicas", 512, 2, 64, out);
  run_lds_rate<4>("store", 512, 2, 64, out);
  run_lds_rate<5>("load", 512, 2, 64, out);
  run_lds_rate<6>("64-bit add", 512, 2, 64, out);
  run_lds_rate<7>("add, fixed address per lane", 512, 2, 64, out);

  const int64_t nvec = ((int64_t)1 << 28) / 4;
  u32x4* keys;
  unsigned long long* clocks;
  CK(hipMalloc(&keys, nvec * 16));
  CK(hipMalloc(&clocks, 4096 * 16));
  {
    std::vector<uint32_t> h(1 << 24);
    uint32_t x = 12345;
    for (auto& v : h) { x = x * 1664525u + 1013904223u; v = x ^ (x >> 15); }
    for (int64_t off = 0; off < nvec * 16; off += (int64_t)h.size() * 4)
      CK(hipMemcpy((char*)keys + off, h.data(), h.size() * 4, hipMemcpyHostToDevice));
  }
  std::printf("lds beside a key stream: 2^28 u32 keys, four LDS atomics per key (2^30 in all), 16 waves per CU\n");
  run_lds_beside<0, false>("keys from registers, counted", keys, nvec, out, clocks);
  run_lds_beside<2, false>("keys loaded, not counted", keys, nvec, out, clocks);
  run_lds_beside<2, true>("keys loaded non-temporally, not counted", keys, nvec, out, clocks);
  run_lds_beside<1, false>("keys loaded, counted", keys, nvec, out, clocks);
  run_lds_beside<1, true>("keys loaded non-temporally, counted", keys, nvec, out, clocks);
  CK(hipFree(keys));
  CK(hipFree(clocks));
  CK(hipFree(out));
}

// ------------------------------------------------------------- latency ----
// A batch of N loads per wave from status rows 1 KiB apart.  WIDE 0: 4 bytes per
// lane with an agent-scope atomic load (a wave covers a quarter of a row);
// WIDE 1: 16 bytes per lane with a device-coherent buffer load (a whole row).
template <int N, int WIDE>
__global__ void row_latency(uint32_t* rows, int nrows, unsigned long long* out, int reps) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned long long total = 0;
  uint32_t acc = 0;
  int t = blockIdx.x * 4096 + wave * 64;
  __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(rows, 0, nrows * 1024, 0x00027000);
  for (int r = 0; r < reps; ++r) {
    const unsigned long long t0 = wall_clock64();
    if (WIDE) {
      u32x4 s[N];
#pragma unroll
      for (int u = 0; u < N; ++u)
        s[u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ((t + u) % nrows) * 1024 + lane * 16, 0, 16);
#pragma unroll
      for (int u = 0; u < N; ++u) acc += s[u].x + s[u].w;
    } else {
      uint32_t s[N];
#pragma unroll
      for (int u = 0; u < N; ++u)
        s[u] = __hip_atomic_load(&rows[(size_t)((t + u) % nrows) * 256 + (wave & 3) * 64 + lane],
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int u = 0; u < N; ++u) acc += s[u];
    }
    asm volatile("" ::"v"(acc));
    total += wall_clock64() - t0;
    t += N;
  }
  if (threadIdx.x == 0) out[blockIdx.x] = total;
  if (acc == 0x12345) out[1000] = acc;
}

// Streams 1 GiB through every compute unit it is resident on, `reps` times.
__global__ __launch_bounds__(256) void stream_copy(const u32x4* __restrict__ a, u32x4* __restrict__ b,
                                                   size_t n, int reps) {
  for (int r = 0; r < reps; ++r)
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) b[i] = a[i];
}

template <int N, int WIDE>
static void run_latency(hipStream_t st, uint32_t* rows, int nrows, unsigned long long* out, int threads) {
  const int reps = 200;
  hipLaunchKernelGGL((row_latency<N, WIDE>), dim3(1), dim3(threads), 0, st, rows, nrows, out, reps);
  CK(hipStreamSynchronize(st));
  unsigned long long h;
  CK(hipMemcpy(&h, out, 8, hipMemcpyDeviceToHost));
  std::printf("  %s per lane, %2d loads per wave, %2d waves: %.2f us per batch\n", WIDE ? "16 B" : " 4 B", N,
              threads / 64, (double)h / reps / 100.0);
}

static void section_latency() {
  const int nrows = 1 << 14;
  uint32_t* rows;
  unsigned long long* out;
  u32x4 *a, *b;
  const size_t nbig = (size_t)1 << 26;
  CK(hipMalloc(&rows, (size_t)nrows * 1024));
  CK(hipMalloc(&out, 8192 * 8));
  CK(hipMalloc(&a, nbig * 16));
  CK(hipMalloc(&b, nbig * 16));
  CK(hipMemset(rows, 1, (size_t)nrows * 1024));
  CK(hipMemset(a, 1, nbig * 16));
  hipStream_t s1, s2;
  CK(hipStreamCreateWithFlags(&s1, hipStreamNonBlocking));
  CK(hipStreamCreateWithFlags(&s2, hipStreamNonBlocking));
  std::printf("latency: one block reads status rows (wall clock around issue and arrival of a batch)\n");
  for (int busy = 0; busy < 2; ++busy) {
    std::printf(busy == 0 ? " idle device\n" : " while the device streams a copy (the reading block shares its compute unit with copying blocks)\n");
    if (busy) hipLaunchKernelGGL(stream_copy, dim3((g_cus - 6) * 8), dim3(256), 0, s2, a, b, nbig, 200);
    for (int threads : {64, 1024}) {
      run_latency<4, 0>(s1, rows, nrows, out, threads);
      run_latency<8, 0>(s1, rows, nrows, out, threads);
      run_latency<16, 0>(s1, rows, nrows, out, threads);
      run_latency<24, 0>(s1, rows, nrows, out, threads);
      run_latency<32, 0>(s1, rows, nrows, out, threads);
      run_latency<4, 1>(s1, rows, nrows, out, threads);
      run_latency<8, 1>(s1, rows, nrows, out, threads);
    }
    CK(hipDeviceSynchronize());
  }
  CK(hipStreamDestroy(s1));
  CK(hipStreamDestroy(s2));
  CK(hipFree(rows));
  CK(hipFree(out));
  CK(hipFree(a));
  CK(hipFree(b));
}

// --------------------------------------------------------------- tiles ----
// What a single-pass kernel pays per tile before any arithmetic: the dispatch
// of a 512-thread block, the ticket that orders the tiles (one returning atomic
// on one address, which the whole block waits for) and the tile's loads.
template <bool TICKET, int VECS>
__global__ __launch_bounds__(512) void tile_read(const u32x4* __restrict__ in, uint32_t* ticket,
                                                 uint32_t* sink) {
  __shared__ uint32_t s_tile;
  uint32_t tile = blockIdx.x;
  if (TICKET) {
    if (threadIdx.x == 0) s_tile = atomicAdd(ticket, 1u);
    __syncthreads();
    tile = s_tile;
  }
  if (VECS == 0) return;
  const u32x4* base = in + (size_t)tile * (512 * (VECS > 0 ? VECS : 1));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  u32x4 v[VECS > 0 ? VECS : 1];
#pragma unroll
  for (int j = 0; j < VECS; ++j)
    v[j] = __builtin_nontemporal_load(&base[(wave * VECS + j) * 64 + lane]);
  uint32_t x = 0;
#pragma unroll
  for (int j = 0; j < VECS; ++j) x ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  if (x == 0x9E3779B9u) sink[0] = x;  // never true for the data used: keeps the loads
}

template <bool TICKET, int VECS>
static void run_tile_read(const u32x4* in, uint32_t* ticket, uint32_t* sink, int tiles) {
  const float ms = time_ms([&] {
    if (TICKET) CK(hipMemsetAsync(ticket, 0, 4));
    hipLaunchKernelGGL((tile_read<TICKET, VECS>), dim3(tiles), dim3(512), 0, 0, in, ticket, sink);
  });
  if (VECS == 0)
    std::printf("  %6d blocks, %-9s no loads                : %.4f ms  %5.1f blocks per us\n", tiles,
                TICKET ? "ticket," : "no ticket,", ms, tiles / ms / 1e3);
  else
    std::printf("  %6d blocks, %-9s %2d vectors per thread    : %.4f ms  %5.1f blocks per us  %5.0f GB/s\n",
                tiles, TICKET ? "ticket," : "no ticket,", VECS, ms, tiles / ms / 1e3,
                (double)tiles * 512 * VECS * 16 / ms / 1e6);
}

static void section_tiles() {
  const size_t nvec = (size_t)1 << 26;  // 1 GiB
  u32x4* in;
  uint32_t *ticket, *sink;
  CK(hipMalloc(&in, nvec * 16));
  CK(hipMalloc(&ticket, 256));
  CK(hipMalloc(&sink, 256));
  CK(hipMemset(in, 1, nvec * 16));
  std::printf("tiles: 512-thread blocks that draw a ticket and read one tile of 1 GiB each (memset of the ticket included)\n");
  run_tile_read<false, 0>(in, ticket, sink, 8192);
  run_tile_read<true, 0>(in, ticket, sink, 8192);
  run_tile_read<false, 0>(in, ticket, sink, 16384);
  run_tile_read<true, 0>(in, ticket, sink, 16384);
  run_tile_read<false, 16>(in, ticket, sink, (int)(nvec / (512 * 16)));
  run_tile_read<true, 16>(in, ticket, sink, (int)(nvec / (512 * 16)));
  run_tile_read<false, 12>(in, ticket, sink, (int)(nvec / (512 * 12)));
  run_tile_read<true, 12>(in, ticket, sink, (int)(nvec / (512 * 12)));
  run_tile_read<false, 8>(in, ticket, sink, (int)(nvec / (512 * 8)));
  run_tile_read<true, 8>(in, ticket, sink, (int)(nvec / (512 * 8)));
  CK(hipFree(in));
  CK(hipFree(ticket));
  CK(hipFree(sink));
}

int main(int argc, char** argv) {
  const char* which = argc > 1 ? argv[1] : "all";
  hipDeviceProp_t prop;
  CK(hipGetDeviceProperties(&prop, 0));
  g_cus = prop.multiProcessorCount;
  std::printf("device: %s, %d compute units\n", prop.gcnArchName, g_cus);
  const bool all = std::strcmp(which, "all") == 0;
  if (all || std::strcmp(which, "copy") == 0) section_copy();
  if (all || std::strcmp(which, "scatter") == 0) section_scatter();
  if (all || std::strcmp(which, "lds") == 0) section_lds();
  if (all || std::strcmp(which, "latency") == 0) section_latency();
  if (all || std::strcmp(which, "tiles") == 0) section_tiles();
  std::fflush(stdout);
  return 0;
}
