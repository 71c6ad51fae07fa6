// Yardstick kernels (see dfa3d_measure.h): bare access patterns of the DFA3D kernels, for bench.py.
#include <hip/hip_runtime.h>

#include "dfa3d_measure.h"

namespace {

__global__ __launch_bounds__(256) void stream_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                          size_t n16) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

__global__ void xcd_map_kernel(int32_t *__restrict__ out, int spin_clocks) {
  unsigned id;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(id));
  const long long t0 = clock64();
  while (clock64() - t0 < spin_clocks) {}          // bounded: the clock always advances
  if (threadIdx.x == 0) out[blockIdx.x] = (int32_t)(id & 0xF);
}

__device__ __forceinline__ unsigned next_random(unsigned a) { return a * 1664525u + 1013904223u; }

template <int LANES, int U>
__global__ __launch_bounds__(256) void row_gather_kernel(const uint4 *__restrict__ src, size_t rows, int iters,
                                                         uint4 *__restrict__ sink) {
  const int lane = threadIdx.x % LANES;
  const size_t g = ((size_t)blockIdx.x * 256 + threadIdx.x) / LANES;
  unsigned a = (unsigned)(g * 2654435761u) + 12345u;
  uint4 acc = make_uint4(0, 0, 0, 0);
  for (int it = 0; it < iters; ++it) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      a = next_random(a);
      const size_t r = (size_t)(a >> 4) & (rows - 1);
      v[u] = src[r * LANES + lane];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) { acc.x |= v[u].x; acc.y |= v[u].y; acc.z |= v[u].z; acc.w |= v[u].w; }
  }
  if ((acc.x | acc.y | acc.z | acc.w) == 0x12345678u) sink[0] = acc;      // the source holds zeros: never taken
}

template <int U>
__global__ __launch_bounds__(256) void pair_gather_kernel(const uint2 *__restrict__ src, size_t pairs, int iters,
                                                          uint4 *__restrict__ sink) {
  unsigned a = (unsigned)(((size_t)blockIdx.x * 256 + threadIdx.x) * 2654435761u) + 777u;
  uint2 acc = make_uint2(0, 0);
  for (int it = 0; it < iters; ++it) {
    uint2 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      a = next_random(a);
      v[u] = src[(size_t)(a >> 3) & (pairs - 1)];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) { acc.x |= v[u].x; acc.y |= v[u].y; }
  }
  if ((acc.x | acc.y) == 0x12345678u) sink[0] = make_uint4(acc.x, acc.y, 0, 0);
}

template <int MODE>
__global__ __launch_bounds__(256) void lds_atomics_kernel(int iters, uint4 *__restrict__ sink) {
  __shared__ float sf[8192];
  __shared__ int si[8192];
  for (int i = threadIdx.x; i < 8192; i += 256) { sf[i] = 0; si[i] = 0; }
  __syncthreads();
  const int lane = threadIdx.x;
  unsigned a = (unsigned)((blockIdx.x * 256 + lane) * 2654435761u) + 99u;
  int acc = 0;
  for (int it = 0; it < iters; ++it) {
    int addr;
    if (MODE == 0) addr = ((lane & ~63) + (lane & 63) + it * 64) & 8191;      // a lane stays in its own bank
    else if (MODE == 2) addr = it & 8191;
    else { a = next_random(a); addr = (a >> 8) & 8191; }
    if (MODE == 3) acc += atomicAdd(&si[addr], 1);
    else if (MODE == 4) atomicAdd(&si[addr], 1);
    else if (MODE == 5) acc += atomicExch(&si[addr], it);
    else atomicAdd(&sf[addr], 1.0f);
  }
  __syncthreads();
  if (lane == 0 && sf[5] + (float)si[7] + (float)acc == -1.f) sink[0] = make_uint4(1, 2, 3, 4);
}

int launched() { return (int)hipGetLastError(); }

bool pow2(size_t x) { return x != 0 && (x & (x - 1)) == 0; }

}  // namespace

extern "C" {

int dfa3d_measure_stream_copy(void *dst, const void *src, size_t bytes, void *stream) {
  if (dst == nullptr || src == nullptr || bytes == 0 || bytes % 16 != 0 || ((uintptr_t)dst | (uintptr_t)src) % 16 != 0)
    return -1;
  const size_t n16 = bytes / 16;
  size_t blocks = (n16 + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint4 *)src,
                     (uint4 *)dst, n16);
  return launched();
}

int dfa3d_measure_xcd_map(int32_t *out, int blocks, int threads, int spin_clocks, void *stream) {
  if (out == nullptr || blocks <= 0 || threads <= 0 || threads > 1024 || threads % 64 != 0 || spin_clocks < 0 ||
      spin_clocks > 10000000)
    return -1;
  hipLaunchKernelGGL(xcd_map_kernel, dim3(blocks), dim3(threads), 0, (hipStream_t)stream, out, spin_clocks);
  return launched();
}

int dfa3d_measure_row_gather(const void *src, size_t rows, int row_bytes, int in_flight, int blocks, int iters,
                             void *sink, void *stream) {
  if (src == nullptr || sink == nullptr || !pow2(rows) || blocks <= 0 || iters <= 0) return -1;
  const uint4 *s = (const uint4 *)src;
  uint4 *k = (uint4 *)sink;
  hipStream_t st = (hipStream_t)stream;
#define ROW_CASE(B, L, U) \
  if (row_bytes == B && in_flight == U) { \
    hipLaunchKernelGGL((row_gather_kernel<L, U>), dim3(blocks), dim3(256), 0, st, s, rows, iters, k); \
    return launched(); \
  }
  ROW_CASE(64, 4, 1) ROW_CASE(64, 4, 2) ROW_CASE(64, 4, 4) ROW_CASE(64, 4, 8)
  ROW_CASE(128, 8, 1) ROW_CASE(128, 8, 2) ROW_CASE(128, 8, 4) ROW_CASE(128, 8, 8)
  ROW_CASE(256, 16, 1) ROW_CASE(256, 16, 2) ROW_CASE(256, 16, 4) ROW_CASE(256, 16, 8)
#undef ROW_CASE
  return -1;
}

int dfa3d_measure_pair_gather(const void *src, size_t bytes, int in_flight, int blocks, int iters, void *sink,
                              void *stream) {
  if (src == nullptr || sink == nullptr || !pow2(bytes) || bytes < 8 || blocks <= 0 || iters <= 0) return -1;
  const uint2 *s = (const uint2 *)src;
  uint4 *k = (uint4 *)sink;
  hipStream_t st = (hipStream_t)stream;
#define PAIR_CASE(U) \
  if (in_flight == U) { \
    hipLaunchKernelGGL((pair_gather_kernel<U>), dim3(blocks), dim3(256), 0, st, s, bytes / 8, iters, k); \
    return launched(); \
  }
  PAIR_CASE(1) PAIR_CASE(2) PAIR_CASE(4) PAIR_CASE(8)
#undef PAIR_CASE
  return -1;
}

int dfa3d_measure_lds_atomics(int mode, int blocks, int iters, void *sink, void *stream) {
  if (sink == nullptr || blocks <= 0 || iters <= 0) return -1;
  uint4 *k = (uint4 *)sink;
  hipStream_t st = (hipStream_t)stream;
#define LDS_CASE(M) \
  if (mode == M) { hipLaunchKernelGGL((lds_atomics_kernel<M>), dim3(blocks), dim3(256), 0, st, iters, k); return launched(); }
  LDS_CASE(0) LDS_CASE(1) LDS_CASE(2) LDS_CASE(3) LDS_CASE(4) LDS_CASE(5)
#undef LDS_CASE
  return -1;
}

}  // extern "C"
