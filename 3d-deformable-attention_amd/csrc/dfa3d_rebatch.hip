// Camera re-batching around the DFA3D operator for gfx950.
//
// DFA3D-BEVFormer's spatial cross-attention lets every camera attend only with the BEV queries that
// project into it: it copies those queries (and their reference points) into a per-camera batch
// before the operator and adds the per-camera results back into the BEV slots afterwards, in python
// loops over batch x cameras with one indexing kernel each
// (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:716-722 and
// :741-748).  Here each direction is one kernel, and neither uses atomics:
//
//   rebatch_gather_kernel   dst[j, i, k, :] = scale[j, q] * src[i, j, q, :]   with q = index[i, k]
//                           (zeros where index[i, k] < 0); also the backward of the combine
//   rebatch_combine_kernel  dst[j, q, :] = scale[j, q] * sum over cameras i with pos[i, q] >= 0 of
//                           src[j, i, pos[i, q], :]; also the backward of the gather
//
// index (cams, max_len) lists the queries of each camera, pos (cams, Nq) is its inverse
// (position of query q in camera i's list, or -1).  Rows are E contiguous elements; a lane moves
// 16 bytes when the row length allows it.  Pure streaming: bound by HBM bandwidth.
#include "../../include/dfa3d.h"
#include "dfa3d_launch.h"

namespace dfa3d {

constexpr int kRebatchBlock = 256;

template <typename T, int VEC> struct Pack { T v[VEC]; };

template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> load_pack(const T *p) {
  Pack<T, VEC> r;
  if (VEC * sizeof(T) == 16) {
    const uint4 t = *reinterpret_cast<const uint4 *>(p);
    __builtin_memcpy(&r, &t, 16);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.v[i] = p[i];
  }
  return r;
}
template <typename T, int VEC>
__device__ __forceinline__ void store_pack(T *p, const Pack<T, VEC> &r) {
  if (VEC * sizeof(T) == 16) {
    uint4 t;
    __builtin_memcpy(&t, &r, 16);
    *reinterpret_cast<uint4 *>(p) = t;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[i] = r.v[i];
  }
}

// one thread per VEC elements of a destination row; rows = bs * cams * max_len
template <typename T, int VEC>
__global__ __launch_bounds__(kRebatchBlock) void rebatch_gather_kernel(
    const T *__restrict__ src, long long cam_stride, long long batch_stride, const int *__restrict__ index,
    const T *__restrict__ scale, T *__restrict__ dst, int bs, int cams, int max_len, int Nq, int E) {
  const int per_row = E / VEC;
  const long long total = (long long)bs * cams * max_len * per_row;
  for (long long t = (long long)blockIdx.x * kRebatchBlock + threadIdx.x; t < total;
       t += (long long)gridDim.x * kRebatchBlock) {
    const long long row = t / per_row;
    const int e = (int)(t - row * per_row) * VEC;
    const int k = (int)(row % max_len);
    const long long ji = row / max_len;
    const int i = (int)(ji % cams), j = (int)(ji / cams);
    const int q = index[(long long)i * max_len + k];
    Pack<T, VEC> r;
#pragma unroll
    for (int c = 0; c < VEC; ++c) r.v[c] = 0;
    if (q >= 0 && q < Nq) {
      r = load_pack<T, VEC>(src + i * cam_stride + j * batch_stride + (long long)q * E + e);
      if (scale != nullptr) {
        const T s = scale[(long long)j * Nq + q];
#pragma unroll
        for (int c = 0; c < VEC; ++c) r.v[c] *= s;
      }
    }
    store_pack<T, VEC>(dst + row * E + e, r);
  }
}

// one thread per VEC elements of a destination row; rows = bs * Nq
template <typename T, int VEC>
__global__ __launch_bounds__(kRebatchBlock) void rebatch_combine_kernel(
    const T *__restrict__ src, const int *__restrict__ pos, const T *__restrict__ scale, T *__restrict__ dst,
    int bs, int cams, int max_len, int Nq, int E) {
  const int per_row = E / VEC;
  const long long total = (long long)bs * Nq * per_row;
  for (long long t = (long long)blockIdx.x * kRebatchBlock + threadIdx.x; t < total;
       t += (long long)gridDim.x * kRebatchBlock) {
    const long long row = t / per_row;
    const int e = (int)(t - row * per_row) * VEC;
    const int q = (int)(row % Nq), j = (int)(row / Nq);
    Pack<T, VEC> acc;
#pragma unroll
    for (int c = 0; c < VEC; ++c) acc.v[c] = 0;
    for (int i = 0; i < cams; ++i) {                       // cameras in order: a fixed summation order
      const int k = pos[(long long)i * Nq + q];
      if (k >= 0 && k < max_len) {
        const Pack<T, VEC> r = load_pack<T, VEC>(src + (((long long)j * cams + i) * max_len + k) * E + e);
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc.v[c] += r.v[c];
      }
    }
    if (scale != nullptr) {
      const T s = scale[row];
#pragma unroll
      for (int c = 0; c < VEC; ++c) acc.v[c] *= s;
    }
    store_pack<T, VEC>(dst + row * E + e, acc);
  }
}

static unsigned rebatch_grid(long long threads) {
  long long blocks = (threads + kRebatchBlock - 1) / kRebatchBlock;
  if (blocks < 1) blocks = 1;
  if (blocks > (1 << 20)) blocks = 1 << 20;
  return (unsigned)blocks;
}

template <typename T>
static hipError_t gather_typed(const void *src, long long cam_stride, long long batch_stride, const int *index,
                               const void *scale, void *dst, int bs, int cams, int max_len, int Nq, int E,
                               bool aligned, hipStream_t stream) {
  constexpr int W = 16 / (int)sizeof(T);
  const long long rows = (long long)bs * cams * max_len;
  if (aligned && E % W == 0 && cam_stride % W == 0 && batch_stride % W == 0) {
    hipLaunchKernelGGL((rebatch_gather_kernel<T, W>), dim3(rebatch_grid(rows * (E / W))), dim3(kRebatchBlock), 0, stream,
                       (const T *)src, cam_stride, batch_stride, index, (const T *)scale, (T *)dst, bs, cams, max_len,
                       Nq, E);
  } else {
    hipLaunchKernelGGL((rebatch_gather_kernel<T, 1>), dim3(rebatch_grid(rows * E)), dim3(kRebatchBlock), 0, stream,
                       (const T *)src, cam_stride, batch_stride, index, (const T *)scale, (T *)dst, bs, cams, max_len,
                       Nq, E);
  }
  return hipGetLastError();
}

template <typename T>
static hipError_t combine_typed(const void *src, const int *pos, const void *scale, void *dst, int bs, int cams,
                                int max_len, int Nq, int E, bool aligned, hipStream_t stream) {
  constexpr int W = 16 / (int)sizeof(T);
  const long long rows = (long long)bs * Nq;
  if (aligned && E % W == 0) {
    hipLaunchKernelGGL((rebatch_combine_kernel<T, W>), dim3(rebatch_grid(rows * (E / W))), dim3(kRebatchBlock), 0,
                       stream, (const T *)src, pos, (const T *)scale, (T *)dst, bs, cams, max_len, Nq, E);
  } else {
    hipLaunchKernelGGL((rebatch_combine_kernel<T, 1>), dim3(rebatch_grid(rows * E)), dim3(kRebatchBlock), 0, stream,
                       (const T *)src, pos, (const T *)scale, (T *)dst, bs, cams, max_len, Nq, E);
  }
  return hipGetLastError();
}

hipError_t launch_rebatch_gather(const void *src, long long cam_stride, long long batch_stride, const int *index,
                                 const void *scale, void *dst, int bs, int cams, int max_len, int Nq, int E,
                                 int dtype, hipStream_t stream) {
  const bool aligned = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
  if (dtype == DFA3D_F32)
    return gather_typed<float>(src, cam_stride, batch_stride, index, scale, dst, bs, cams, max_len, Nq, E, aligned, stream);
  if (dtype == DFA3D_F64)
    return gather_typed<double>(src, cam_stride, batch_stride, index, scale, dst, bs, cams, max_len, Nq, E, aligned, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_rebatch_combine(const void *src, const int *pos, const void *scale, void *dst, int bs, int cams,
                                  int max_len, int Nq, int E, int dtype, hipStream_t stream) {
  const bool aligned = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
  if (dtype == DFA3D_F32) return combine_typed<float>(src, pos, scale, dst, bs, cams, max_len, Nq, E, aligned, stream);
  if (dtype == DFA3D_F64) return combine_typed<double>(src, pos, scale, dst, bs, cams, max_len, Nq, E, aligned, stream);
  return hipErrorInvalidValue;
}

}  // namespace dfa3d
