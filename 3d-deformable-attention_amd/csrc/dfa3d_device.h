// Device-side building blocks shared by the forward and backward kernels of the DFA3D
// operator on gfx950 (wave64).
//
// Work decomposition used by every kernel in this library:
//   * a "unit" is one (batch b, query q, head m): L*P sampling points that are contiguous
//     in the location / attention / score tensors and all gather from head m of batch b;
//   * phase A ("lanes over points"): each lane of a wavefront owns one sampling point, does
//     the index arithmetic, the depth-bin gathers and the coalesced reads/writes of the
//     per-point tensors, and leaves one (row byte offset, weight) task per corner in LDS;
//   * phase B ("lanes over channels"): the wavefront walks those tasks; LPR lanes of VEC
//     channels each cover one value row, so one vector load instruction fetches 64/LPR rows,
//     each fully coalesced.
// The semantics (pixel coordinates, skip predicates, zero padding per corner and per depth
// bin, corner slot order LT,RT,RB,LB) are those of the reference kernels
//   DFA3D/dfa3D/ops/csrc/common/cuda/ms_depth_score_sample_cuda_kernel.cuh:24-148 and
//   DFA3D/dfa3D/ops/csrc/common/cuda/wms_deform_attn_cuda_kernel.cuh:24-80,240-303.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "../../include/dfa3d.h"

namespace dfa3d {

// Development builds (-DDFA3D_EXPERIMENT) can cut parts out of the backward kernels to see what they cost;
// in the library as shipped the switches are constant zero and the compiler drops them.
#ifdef DFA3D_EXPERIMENT
#define DFA3D_DIAG(diag, bits) (((diag) & (bits)) != 0)
#define DFA3D_DIAG_PARAM , int diag          // last kernel parameter, development builds only
#define DFA3D_DIAG_ARG(a) , (a).diag
#else
#define DFA3D_DIAG(diag, bits) false
#define DFA3D_DIAG_PARAM
#define DFA3D_DIAG_ARG(a)
#endif

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWave * kWavesPerBlock;

// ---------------------------------------------------------------------------------------
// element access: storage type T -> arithmetic type A
// ---------------------------------------------------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float ld(const float *p) { return *p; }
  static __device__ __forceinline__ void st(float *p, float v) { *p = v; }
};
template <> struct Elem<double> {
  static __device__ __forceinline__ double ld(const double *p) { return *p; }
  static __device__ __forceinline__ void st(double *p, double v) { *p = v; }
};
template <> struct Elem<__hip_bfloat16> {
  static __device__ __forceinline__ float ld(const __hip_bfloat16 *p) {
    return __uint_as_float(((uint32_t) * reinterpret_cast<const uint16_t *>(p)) << 16);
  }
  static __device__ __forceinline__ void st(__hip_bfloat16 *p, float v) { *p = __float2bfloat16(v); }
};

// ---------------------------------------------------------------------------------------
// Buffer-addressed access.  One batch element of value / dist / grad_value / grad_dist is
// described by a raw buffer resource (base, size in bytes); gathers and scatter-adds then take
// a 32-bit byte offset, and an offset at or beyond the size reads as zero / drops the atomic in
// hardware.  Tasks that have nothing to gather carry kNoRow as their offset, so phase B needs
// no branches and can keep many gathers in flight; the same range check means no offset, however
// wrong, can touch memory outside the tensor.
// ---------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kNoRow = 0x80000000u;    // offset of a task with nothing to gather
constexpr uint32_t kNoChan = 0x40000000u;   // channel offset of a lane beyond the last channel
// With every tensor slice below 2^30 bytes, kNoRow + x and row + kNoChan are out of range for
// every in-range row offset and channel offset x (no 32-bit wrap-around).
constexpr long long kMaxSliceBytes = 1LL << 30;

__device__ __forceinline__ rsrc_t make_rsrc(const void *base, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }

// one element at byte offset `off`
template <typename T> struct BufElem;
template <> struct BufElem<float> {
  static __device__ __forceinline__ float ld(rsrc_t r, uint32_t off) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
  }
};
template <> struct BufElem<double> {
  static __device__ __forceinline__ double ld(rsrc_t r, uint32_t off) {
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    return __hiloint2double((int)t.y, (int)t.x);
  }
};
template <> struct BufElem<__hip_bfloat16> {
  static __device__ __forceinline__ float ld(rsrc_t r, uint32_t off) {
    return bf16_bits_to_float(__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0));
  }
};

// VEC consecutive elements of a row at byte offset `off` (aligned to VEC elements)
template <typename T, typename A, int VEC> struct RowVec;
template <typename A> struct RowVec<float, A, 1> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[1]) { v[0] = BufElem<float>::ld(r, off); }
  static __device__ __forceinline__ void st(float *p, const A (&v)[1]) { p[0] = v[0]; }
};
template <typename A> struct RowVec<float, A, 2> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[2]) {
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y);
  }
  static __device__ __forceinline__ void st(float *p, const A (&v)[2]) {
    *reinterpret_cast<float2 *>(p) = make_float2(v[0], v[1]);
  }
};
template <typename A> struct RowVec<float, A, 4> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[4]) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y);
    v[2] = __uint_as_float(t.z); v[3] = __uint_as_float(t.w);
  }
  static __device__ __forceinline__ void st(float *p, const A (&v)[4]) {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <typename A> struct RowVec<float, A, 8> {      // loads only: used by the tile kernels
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[8]) {
    const u32x4 t0 = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    const u32x4 t1 = __builtin_amdgcn_raw_buffer_load_b128(r, off + 16, 0, 0);
    v[0] = __uint_as_float(t0.x); v[1] = __uint_as_float(t0.y); v[2] = __uint_as_float(t0.z); v[3] = __uint_as_float(t0.w);
    v[4] = __uint_as_float(t1.x); v[5] = __uint_as_float(t1.y); v[6] = __uint_as_float(t1.z); v[7] = __uint_as_float(t1.w);
  }
};
template <typename A> struct RowVec<double, A, 1> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[1]) { v[0] = BufElem<double>::ld(r, off); }
  static __device__ __forceinline__ void st(double *p, const A (&v)[1]) { p[0] = v[0]; }
};
template <typename A> struct RowVec<double, A, 2> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[2]) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    v[0] = __hiloint2double((int)t.y, (int)t.x); v[1] = __hiloint2double((int)t.w, (int)t.z);
  }
  static __device__ __forceinline__ void st(double *p, const A (&v)[2]) {
    *reinterpret_cast<double2 *>(p) = make_double2(v[0], v[1]);
  }
};
template <typename A> struct RowVec<double, A, 4> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[4]) {
    const u32x4 t0 = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    const u32x4 t1 = __builtin_amdgcn_raw_buffer_load_b128(r, off + 16, 0, 0);
    v[0] = __hiloint2double((int)t0.y, (int)t0.x); v[1] = __hiloint2double((int)t0.w, (int)t0.z);
    v[2] = __hiloint2double((int)t1.y, (int)t1.x); v[3] = __hiloint2double((int)t1.w, (int)t1.z);
  }
  static __device__ __forceinline__ void st(double *p, const A (&v)[4]) {
    reinterpret_cast<double2 *>(p)[0] = make_double2(v[0], v[1]);
    reinterpret_cast<double2 *>(p)[1] = make_double2(v[2], v[3]);
  }
};
template <typename A> struct RowVec<__hip_bfloat16, A, 1> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[1]) {
    v[0] = BufElem<__hip_bfloat16>::ld(r, off);
  }
  static __device__ __forceinline__ void st(__hip_bfloat16 *p, const A (&v)[1]) { p[0] = __float2bfloat16(v[0]); }
};
template <typename A> struct RowVec<__hip_bfloat16, A, 2> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[2]) {
    const uint32_t t = __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0);
    v[0] = __uint_as_float(t << 16);
    v[1] = __uint_as_float(t & 0xFFFF0000u);
  }
  static __device__ __forceinline__ void st(__hip_bfloat16 *p, const A (&v)[2]) {
    p[0] = __float2bfloat16(v[0]);
    p[1] = __float2bfloat16(v[1]);
  }
};
template <typename A> struct RowVec<__hip_bfloat16, A, 4> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[4]) {
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    v[0] = __uint_as_float(t.x << 16);
    v[1] = __uint_as_float(t.x & 0xFFFF0000u);
    v[2] = __uint_as_float(t.y << 16);
    v[3] = __uint_as_float(t.y & 0xFFFF0000u);
  }
  static __device__ __forceinline__ void st(__hip_bfloat16 *p, const A (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = __float2bfloat16(v[i]);
  }
};

template <typename A> struct RowVec<__hip_bfloat16, A, 8> {      // loads only: used by the tile kernels
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, A (&v)[8]) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xFFFF0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xFFFF0000u);
    v[4] = __uint_as_float(t.z << 16); v[5] = __uint_as_float(t.z & 0xFFFF0000u);
    v[6] = __uint_as_float(t.w << 16); v[7] = __uint_as_float(t.w & 0xFFFF0000u);
  }
};

// Hardware floating-point scatter-add (no compare-and-swap loop) at byte offset `off` of a
// gradient slice; an out-of-range offset drops the update.
__device__ __forceinline__ void scatter_add(rsrc_t r, float *, uint32_t off, float v) {
  __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(v, r, off, 0, 0);
}
__device__ __forceinline__ void scatter_add(rsrc_t, double *base, uint32_t off, double v) {
  if (off < kNoChan) unsafeAtomicAdd(reinterpret_cast<double *>(reinterpret_cast<char *>(base) + off), v);
}

// bfloat16 gradient storage (DFA3D_BF16G): two values rounded to nearest even and packed, and the
// hardware's packed bfloat16 add on device memory (each add rounds the stored sum to bfloat16 again).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  bf16x2_t v;
  v.x = (__bf16)a; v.y = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ void atomic_add_bf16x2(void *p, float a, float b) {
  bf16x2_t v;
  v.x = (__bf16)a; v.y = (__bf16)b;
  __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<bf16x2_t *>(p), v);
}

// ---------------------------------------------------------------------------------------
// wave-private LDS hand-over between phases: LDS operations of one wavefront execute in
// program order, so only the compiler has to be kept from moving accesses across the point.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ void wave_lds_handover() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------------------
// level table in LDS: H, W, Dd, first key; a level whose extent does not fit in the S keys
// (or has a non-positive size) is disabled so that no access can leave the tensors.
// ---------------------------------------------------------------------------------------
struct LevelTable {
  int H[DFA3D_MAX_LEVELS];
  int W[DFA3D_MAX_LEVELS];
  int Dd[DFA3D_MAX_LEVELS];
  int start[DFA3D_MAX_LEVELS];
  int cell[DFA3D_MAX_LEVELS + 1];   // packed distributions only (load_cell_starts): first cell of each level, total
};

__device__ __forceinline__ void load_level_table(LevelTable &tab, const int64_t *shapes, int shape_stride,
                                                 const int64_t *level_start, int L, int S, int D) {
  if ((int)threadIdx.x < L) {
    const int l = threadIdx.x;
    const int64_t H = shapes[l * shape_stride], W = shapes[l * shape_stride + 1];
    const int64_t Dd = (shape_stride > 2 && D > 0) ? shapes[l * shape_stride + 2] : 1;   // D <= 0: depth extent unused
    const int64_t st = level_start[l];
    const bool ok = H > 0 && W > 0 && st >= 0 && H <= S && W <= S && st + H * W <= (int64_t)S &&
                    Dd > 0 && (D <= 0 || Dd <= D);
    tab.H[l] = ok ? (int)H : 0;
    tab.W[l] = ok ? (int)W : 0;
    tab.Dd[l] = ok ? (int)Dd : 0;
    tab.start[l] = ok ? (int)st : 0;
  }
  __syncthreads();
}

// A packed distribution (dfa3d_pack_dist) holds, for every base pixel (h0, w0) with -1 <= h0 < H and
// -1 <= w0 < W of every level (a "cell") and every depth bin d, the distribution values of the four pixels
// around it in slot order LT,RT,RB,LB (zero outside the map): 4 elements per (cell, bin), bins consecutive.
// Cells are numbered level by level, (h0 + 1) * (W + 1) + (w0 + 1) within a level.
__device__ __forceinline__ void load_cell_starts(LevelTable &tab, int L) {
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int l = 0; l < L; ++l) {
      tab.cell[l] = acc;
      acc += (tab.H[l] + 1) * (tab.W[l] + 1);
    }
    tab.cell[L] = acc;
  }
  __syncthreads();
}

// Cells the host sizes a packed table for: levels that share no keys have sum (H + 1)(W + 1) <= 2 S + 2 L of them.
__host__ __device__ inline long long packed_cell_capacity(int S, int L) { return 2LL * S + 2LL * L; }

// bins (d, d + 1) of one cell: 8 elements, 32 bytes (16 for bfloat16), one cache line access
template <typename T> struct PackedTap;
template <> struct PackedTap<float> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, float (&x)[4], float (&y)[4]) {
    const u32x4 t0 = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    const u32x4 t1 = __builtin_amdgcn_raw_buffer_load_b128(r, off == kNoRow ? kNoRow : off + 16, 0, 0);
    x[0] = __uint_as_float(t0.x); x[1] = __uint_as_float(t0.y); x[2] = __uint_as_float(t0.z); x[3] = __uint_as_float(t0.w);
    y[0] = __uint_as_float(t1.x); y[1] = __uint_as_float(t1.y); y[2] = __uint_as_float(t1.z); y[3] = __uint_as_float(t1.w);
  }
};
template <> struct PackedTap<__hip_bfloat16> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, float (&x)[4], float (&y)[4]) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    x[0] = __uint_as_float(t.x << 16); x[1] = __uint_as_float(t.x & 0xFFFF0000u);
    x[2] = __uint_as_float(t.y << 16); x[3] = __uint_as_float(t.y & 0xFFFF0000u);
    y[0] = __uint_as_float(t.z << 16); y[1] = __uint_as_float(t.z & 0xFFFF0000u);
    y[2] = __uint_as_float(t.w << 16); y[3] = __uint_as_float(t.w & 0xFFFF0000u);
  }
};
template <> struct PackedTap<double> {      // not offered (the launcher never passes a packed table of doubles)
  static __device__ __forceinline__ void ld(rsrc_t, uint32_t, double (&x)[4], double (&y)[4]) {
    for (int k = 0; k < 4; ++k) { x[k] = 0; y[k] = 0; }
  }
};

// ---------------------------------------------------------------------------------------
// geometry of one sampling point
// ---------------------------------------------------------------------------------------
// Pixel coordinate of a normalised location.  The reference evaluates
// "loc * size - 0.5" with a separately rounded product (the product is typed float before the
// double literal promotes the subtraction), so fused multiply-add contraction is switched off:
// floor() and the skip predicates must see exactly that value.
template <typename A> __device__ __forceinline__ A to_pixel(A loc, int size) {
#pragma clang fp contract(off)
  const A prod = loc * (A)size;
  const A im = prod - (A)0.5;
  return im;
}

// The reference floors with floorf() for every scalar type (a double is rounded to float first).
template <typename A> __device__ __forceinline__ int floor_index(A x) { return (int)floorf((float)x); }

template <typename A> struct Point2D {
  A lh, lw, hh, hw;      // fractional parts and complements along h and w
  int key[4];            // key index (level start + h*W + w) of slots LT,RT,RB,LB; -1 outside the map
  int h0, w0;            // floor of the pixel coordinates (meaningful when `inside`)
  bool inside;           // stage-2 predicate: -1 < h_im < H and -1 < w_im < W
  __device__ __forceinline__ A bil(int k) const {
    return k == 0 ? hh * hw : k == 1 ? hh * lw : k == 2 ? lh * lw : lh * hw;
  }
};

template <typename A>
__device__ __forceinline__ Point2D<A> locate_2d(A x, A y, int H, int W, int start) {
  Point2D<A> g;
  const A h_im = to_pixel(y, H), w_im = to_pixel(x, W);
  g.inside = h_im > -1 && w_im > -1 && h_im < H && w_im < W;
  // a point that fails the range test (NaN and infinite coordinates do) gets harmless geometry: nothing
  // non-finite may reach a product with a masked, zero operand
  const int h0 = g.inside ? floor_index(h_im) : 0, w0 = g.inside ? floor_index(w_im) : 0;
  g.h0 = h0;
  g.w0 = w0;
  g.lh = g.inside ? h_im - h0 : (A)0;
  g.lw = g.inside ? w_im - w0 : (A)0;
  g.hh = 1 - g.lh;
  g.hw = 1 - g.lw;
  const bool h_lo = h0 >= 0 && h0 <= H - 1, h_hi = h0 + 1 >= 0 && h0 + 1 <= H - 1;
  const bool w_lo = w0 >= 0 && w0 <= W - 1, w_hi = w0 + 1 >= 0 && w0 + 1 <= W - 1;
  const int base = start + h0 * W + w0;
  g.key[0] = (g.inside && h_lo && w_lo) ? base : -1;
  g.key[1] = (g.inside && h_lo && w_hi) ? base + 1 : -1;
  g.key[2] = (g.inside && h_hi && w_hi) ? base + W + 1 : -1;
  g.key[3] = (g.inside && h_hi && w_lo) ? base + W : -1;
  return g;
}

template <typename A> struct DepthTap {
  A ld, hd;              // fractional part along depth and complement
  int d0;                // lower bin
  bool lo_ok, hi_ok;     // bins d0 / d0+1 inside [0, Dd-1]
  bool inside;           // -1 < d_im < Dd
};

template <typename A> __device__ __forceinline__ DepthTap<A> locate_depth(A z, int Dd) {
  DepthTap<A> t;
  const A d_im = to_pixel(z, Dd);
  t.inside = d_im > -1 && d_im < Dd;
  t.d0 = t.inside ? floor_index(d_im) : 0;
  t.ld = t.inside ? d_im - t.d0 : (A)0;       // outside (NaN included): both weights 0, not NaN * 0
  t.hd = t.inside ? 1 - t.ld : (A)0;
  t.lo_ok = t.inside && t.d0 >= 0 && t.d0 <= Dd - 1;
  t.hi_ok = t.inside && t.d0 + 1 >= 0 && t.d0 + 1 <= Dd - 1;
  return t;
}

// Two consecutive elements at byte offset `off` (element-aligned) with ONE load instruction where
// the hardware allows it: the vector L1 handles roughly one cache line per four clocks whatever the
// number of bytes used, so the pair costs one line access instead of two.
template <typename T> struct BufPair;
template <> struct BufPair<float> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, float &x, float &y) {
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    x = __uint_as_float(t.x); y = __uint_as_float(t.y);
  }
};
template <> struct BufPair<double> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, double &x, double &y) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    x = __hiloint2double((int)t.y, (int)t.x); y = __hiloint2double((int)t.w, (int)t.z);
  }
};
template <> struct BufPair<__hip_bfloat16> {
  // two 2-byte loads: rows of an odd number of bins
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, float &x, float &y) {
    x = BufElem<__hip_bfloat16>::ld(r, off);
    y = BufElem<__hip_bfloat16>::ld(r, off == kNoRow ? kNoRow : off + 2);
  }
  // One 8-byte load from the 4-byte boundary at or below the pair: it holds the pair whichever half of its
  // first word the pair starts in.  The load may reach up to four bytes past the buffer's end; the hardware
  // checks the range word by word, so the words inside come back and the one outside reads as zero.  Needs a
  // buffer whose size is a multiple of 4 bytes (an even number of bins per row), or the last word could be
  // cut in the middle and dropped.
  static __device__ __forceinline__ void ld_word_aligned(rsrc_t r, uint32_t off, float &x, float &y) {
    const uint32_t shift = (off & 2u) << 3;              // 0 or 16 bits into the first word
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, off == kNoRow ? kNoRow : (off & ~3u), 0, 0);
    const unsigned long long v = (((unsigned long long)t.y << 32) | t.x) >> shift;
    x = bf16_bits_to_float((uint32_t)v & 0xFFFFu);
    y = bf16_bits_to_float((uint32_t)(v >> 16) & 0xFFFFu);
  }
  // Rows that start on 8-byte boundaries (D % 4 == 0): one 8-byte load of the aligned group of four bins
  // holds the pair unless it starts at the group's last bin (then one extra 2-byte load).  Two instructions,
  // but every access is naturally aligned: faster where the lines are already in the L1 (the tile kernels).
  static __device__ __forceinline__ void ld_aligned4(rsrc_t r, uint32_t off, float &x, float &y) {
    const bool none = off == kNoRow;
    const uint32_t idx = (off >> 1) & 3;
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, none ? kNoRow : (off & ~7u), 0, 0);
    const uint32_t extra = __builtin_amdgcn_raw_buffer_load_b16(r, (none || idx != 3) ? kNoRow : off + 2, 0, 0);
    const unsigned long long v = (((unsigned long long)t.y << 32) | t.x) >> (16 * idx);
    x = bf16_bits_to_float((uint32_t)v & 0xFFFFu);
    y = bf16_bits_to_float(idx == 3 ? (extra & 0xFFFFu) : ((uint32_t)(v >> 16) & 0xFFFFu));
  }
};

// score of a corner from its two taps, written so that every kernel rounds it the same way
__device__ __forceinline__ float depth_lerp(float lo, float hi, float hd, float ld) { return __builtin_fmaf(hi, ld, lo * hd); }
__device__ __forceinline__ double depth_lerp(double lo, double hi, double hd, double ld) { return __builtin_fma(hi, ld, lo * hd); }

// LOCAL: the caller's taps mostly hit lines its workgroup has just used (tile kernels)
template <typename T, bool LOCAL> struct PairLoader {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, int, T &x, T &y) { BufPair<T>::ld(r, off, x, y); }
};
template <bool LOCAL> struct PairLoader<__hip_bfloat16, LOCAL> {
  static __device__ __forceinline__ void ld(rsrc_t r, uint32_t off, int D, float &x, float &y) {
    if (LOCAL && (D & 3) == 0) BufPair<__hip_bfloat16>::ld_aligned4(r, off, x, y);
    else if ((D & 1) == 0) BufPair<__hip_bfloat16>::ld_word_aligned(r, off, x, y);
    else BufPair<__hip_bfloat16>::ld(r, off, x, y);
  }
};

// Depth scores of the four corners of one point: linear interpolation along depth of the
// distribution stored at each corner pixel, zero outside the map / outside [0, Dd-1].
// `dist_r` describes batch element b of dist; lo/hi return the two taps per corner.
template <typename T, typename A, bool LOCAL = false>
__device__ __forceinline__ void corner_scores(rsrc_t dist_r, const int (&key)[4], const DepthTap<A> &tap, int m, int M,
                                              int D, A (&score)[4], A (&lo)[4], A (&hi)[4]) {
  if (D >= 2) {
    // bins (db, db+1) with db clamped into the row always hold both taps that exist
    const int db = min(max(tap.d0, 0), D - 2);
    const bool lo_x = tap.lo_ok && tap.d0 == db, lo_y = tap.lo_ok && tap.d0 == db + 1;
    const bool hi_x = tap.hi_ok && tap.d0 + 1 == db, hi_y = tap.hi_ok && tap.d0 + 1 == db + 1;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t row = (uint32_t)(((key[k] * M + m) * D + db) * (int)sizeof(T));
      A x, y;
      PairLoader<T, LOCAL>::ld(dist_r, (key[k] >= 0 && tap.inside) ? row : kNoRow, D, x, y);
      lo[k] = lo_x ? x : lo_y ? y : (A)0;
      hi[k] = hi_x ? x : hi_y ? y : (A)0;
    }
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t row = (uint32_t)(((key[k] * M + m) * D + tap.d0) * (int)sizeof(T));
      const bool on = key[k] >= 0;
      lo[k] = BufElem<T>::ld(dist_r, (on && tap.lo_ok) ? row : kNoRow);
      hi[k] = BufElem<T>::ld(dist_r, (on && tap.hi_ok) ? row + (uint32_t)sizeof(T) : kNoRow);
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) score[k] = depth_lerp(lo[k], hi[k], tap.hd, tap.ld);
}

// one task of phase B: byte offset of a value row inside the batch element (kNoRow = nothing
// to gather) and the weight the row is multiplied with
template <typename A> struct Task;
template <> struct __align__(8) Task<float> { uint32_t off; float w; };
template <> struct __align__(16) Task<double> { uint32_t off; uint32_t pad; double w; };

// how a wavefront maps onto units and points
struct WaveShape {
  int LP;          // points per unit
  int upw;         // units handled together by one wavefront (1 when LP > 64)
  int chunks;      // 64-point chunks per group of units
};
__host__ __device__ inline WaveShape wave_shape(int L, int P) {
  WaveShape s;
  s.LP = L * P;
  s.upw = s.LP >= kWave ? 1 : kWave / s.LP;
  if (s.upw > 8) s.upw = 8;
  s.chunks = (s.upw * s.LP + kWave - 1) / kWave;
  return s;
}

}  // namespace dfa3d
