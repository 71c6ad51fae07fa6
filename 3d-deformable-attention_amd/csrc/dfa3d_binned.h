// Declarations shared by the kernels of the binned backward (dfa3d_backward_binned.hip, dfa3d_backward_cells.hip):
// the bin plan and workspace the binning kernels leave behind, the work queues of the tile workgroups, and the
// small wavefront / LDS helpers they use.
#pragma once

#include "dfa3d_device.h"
#include "dfa3d_launch.h"

namespace dfa3d {

constexpr int kClasses = 8;         // work queues: one per XCD (workgroup id % 8 with round-robin placement)
constexpr int kQueueStride = 16;    // ints between queue counters: one 64-byte line each
constexpr int kQueueInts = kClasses * kQueueStride + 32;   // + room for the optional phase timers
constexpr int kBinQueries = 32;     // bin_points_kernel: queries of one (batch, head) per block step (16, 64, 128 time worse)
constexpr int kHistCap = 8192;      // bins of one (batch, head) that fit the LDS histogram

struct BinPlan {
  int H[DFA3D_MAX_LEVELS], W[DFA3D_MAX_LEVELS], Dd[DFA3D_MAX_LEVELS], start[DFA3D_MAX_LEVELS];
  int tiles_x[DFA3D_MAX_LEVELS], level_base[DFA3D_MAX_LEVELS];
  int bins_per_bm;     // tiles over all levels of one (batch, head)
  int total_bins;      // slots * bins_per_bm
  int bins_per_class;  // total_bins / kClasses
  int class_start[kClasses + 1];   // first work item of each head class (written by the scan)
  int ty, tx;          // tile edge in pixels
  int chunk;           // points of a bin handled by one work item
  int total_chunks;    // work items (written by the scan)
};

// Bins are numbered slot * bins_per_bm + tile, where the slot of (batch b, head m) puts the heads with the
// same m % 8 next to each other: class c = m % 8 owns the slots [c, c + 1) * head_groups(M) * B.  The
// binning blocks and the tile workgroups of class c run on XCD c, so everything written and read for one
// head (records, gradients per point, tiles) goes through one L2.
__host__ __device__ inline int head_groups(int M) { return (M + kClasses - 1) / kClasses; }
__host__ __device__ inline int slot_count(int B, int M) { return kClasses * head_groups(M) * B; }
__device__ __forceinline__ int slot_of(int b, int m, int B, int M) {
  return ((m % kClasses) * head_groups(M) + m / kClasses) * B + b;
}
__device__ __forceinline__ void slot_decode(int slot, int B, int M, int &b, int &m) {
  b = slot % B;
  const int hm = slot / B, G = head_groups(M);
  m = (hm % G) * kClasses + hm / G;
}

// pixel (y, x) lies inside an H x W map (a tile's first row and column may be pixel -1)
__device__ __forceinline__ bool in_map(int y, int x, int H, int W) { return (unsigned)y < (unsigned)H && (unsigned)x < (unsigned)W; }

// Workgroup barrier that orders LDS accesses only.  __syncthreads() also waits for every global load and store the
// wavefront has in flight (one counter covers both on this part); the tile workgroups hand work to each other
// through LDS alone, so their loads may stay in flight across a barrier and their stores may drain behind it.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

struct BinWorkspace {      // device pointers into the caller's workspace
  BinPlan *plan;
  int *queues;             // kClasses counters, kQueueStride ints apart
  int *counts;             // points per bin
  int *cursor;             // begin of each bin's segment after the scan, end after the fill
  int4 *items;             // work items: (bin, begin of its points, number of points, work items of the bin)
  int4 *geom;              // the items' bins decoded: (batch | head << 16, level, pixel row, pixel column of the tile's row 0)
  uint32_t *entries;       // point indices grouped by bin
  float4 *recs;            // (x, y, z, attention weight) of the same points, same order
};

// Inclusive prefix sum over the 64 lanes with DPP moves: shifts by 1, 2, 4, 8 inside rows of 16 lanes, then
// lane 15 of a row to the next row, then lane 31 to the upper half.
__device__ __forceinline__ int wave_inclusive_scan(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false);   // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false);   // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false);   // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false);   // row_shr:8
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);   // row_bcast:15 into rows 1 and 3
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);   // row_bcast:31 into rows 2 and 3
  return x;
}

// Optional phase timing of the tile kernel (development builds only, -DDFA3D_TILE_TIMING): thread 0
// of every workgroup accumulates shader-clock ticks per phase and adds them to 64-bit counters that
// live in the padding behind the queue counter.
#ifdef DFA3D_TILE_TIMING
#define TT_DECL unsigned long long tt_acc[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0}; unsigned long long tt_last = clock64();
#define TT_MARK(i) do { if (threadIdx.x == 0) { const unsigned long long tt_now = clock64(); tt_acc[i] += tt_now - tt_last; tt_last = tt_now; } } while (0)
#define TT_FLUSH() do { if (threadIdx.x == 0) { unsigned long long *tt_g = reinterpret_cast<unsigned long long *>(ws.queues + kClasses * kQueueStride); for (int i = 0; i < 10; ++i) atomicAdd(tt_g + i, tt_acc[i]); } } while (0)
#else
#define TT_DECL
#define TT_MARK(i) do { } while (0)
#define TT_FLUSH() do { } while (0)
#endif

// Thread 0 of a tile workgroup: next work item, from the queue of the workgroup's own class first and
// from the other classes once that is empty; -1 when every queue is drained.
__device__ __forceinline__ int pop_item(const BinWorkspace &ws, const BinPlan &p, int home, int &classes_done) {
  while (classes_done < kClasses) {
    const int c = (home + classes_done) % kClasses;
    const int lo = p.class_start[c], hi = p.class_start[c + 1];
    if (lo < hi) {
      // from the end: the bins of the coarsest level, which hold the most points, come last in a (batch, head)
      // and should not be what the kernel's last workgroups are left with
      const int w = hi - 1 - atomicAdd(&ws.queues[c * kQueueStride], 1);
      if (w >= lo) return w;
    }
    ++classes_done;
  }
  return -1;
}

// Thread 0's pipeline of work items: the item taken now was popped two items ago and its record requested
// one item ago, so neither the queue atomic nor the record's load is waited for.
struct ItemFetch {
  int classes_done, w_next;
  int4 rec;
  __device__ __forceinline__ int4 load(const BinWorkspace &ws, int w) const {
    return w >= 0 ? ws.items[w] : make_int4(-1, 0, 0, 0);
  }
  __device__ __forceinline__ void start(const BinWorkspace &ws, const BinPlan &p, int home) {
    classes_done = 0;
    const int w = pop_item(ws, p, home, classes_done);
    rec = load(ws, w);
    w_next = w >= 0 ? pop_item(ws, p, home, classes_done) : -1;
  }
  __device__ __forceinline__ void advance(const BinWorkspace &ws, const BinPlan &p, int home, int4 *out) {
    *out = rec;
    rec = load(ws, w_next);
    w_next = w_next >= 0 ? pop_item(ws, p, home, classes_done) : -1;
  }
};

__device__ __forceinline__ float dpp_xadd(float x, int pick) {
  const int xi = __float_as_int(x);
  int r;
  switch (pick) {
    case 0: r = __builtin_amdgcn_mov_dpp(xi, 0xB1, 0xF, 0xF, true); break;    // quad_perm [1,0,3,2]
    case 1: r = __builtin_amdgcn_mov_dpp(xi, 0x4E, 0xF, 0xF, true); break;    // quad_perm [2,3,0,1]
    case 2: r = __builtin_amdgcn_mov_dpp(xi, 0x141, 0xF, 0xF, true); break;   // row_half_mirror
    default: r = __builtin_amdgcn_mov_dpp(xi, 0x140, 0xF, 0xF, true); break;  // row_mirror
  }
  return x + __int_as_float(r);
}
template <int LPR> __device__ __forceinline__ float row_sum_f(float x) {
  if (LPR >= 2) x = dpp_xadd(x, 0);
  if (LPR >= 4) x = dpp_xadd(x, 1);
  if (LPR >= 8) x = dpp_xadd(x, 2);
  if (LPR >= 16) x = dpp_xadd(x, 3);
  if (LPR >= 32) x += __shfl_xor(x, 16, kWave);
  if (LPR >= 64) x += __shfl_xor(x, 32, kWave);
  return x;
}

// VEC consecutive floats of an LDS row, moved with one instruction (the address is VEC-float
// aligned: rows start on 16-byte boundaries and a lane's first channel is a multiple of VEC)
template <int VEC> struct LdsVec;
template <> struct LdsVec<1> {
  static __device__ __forceinline__ void ld(const float *p, float (&v)[1]) { v[0] = p[0]; }
  static __device__ __forceinline__ void st(float *p, const float (&v)[1]) { p[0] = v[0]; }
};
template <> struct LdsVec<2> {
  static __device__ __forceinline__ void ld(const float *p, float (&v)[2]) {
    const float2 t = *reinterpret_cast<const float2 *>(p);
    v[0] = t.x; v[1] = t.y;
  }
  static __device__ __forceinline__ void st(float *p, const float (&v)[2]) {
    *reinterpret_cast<float2 *>(p) = make_float2(v[0], v[1]);
  }
};
template <> struct LdsVec<4> {
  static __device__ __forceinline__ void ld(const float *p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4 *>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  static __device__ __forceinline__ void st(float *p, const float (&v)[4]) {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct LdsVec<8> {
  static __device__ __forceinline__ void ld(const float *p, float (&v)[8]) {
    const float4 t0 = reinterpret_cast<const float4 *>(p)[0], t1 = reinterpret_cast<const float4 *>(p)[1];
    v[0] = t0.x; v[1] = t0.y; v[2] = t0.z; v[3] = t0.w; v[4] = t1.x; v[5] = t1.y; v[6] = t1.z; v[7] = t1.w;
  }
  static __device__ __forceinline__ void st(float *p, const float (&v)[8]) {
    reinterpret_cast<float4 *>(p)[0] = make_float4(v[0], v[1], v[2], v[3]);
    reinterpret_cast<float4 *>(p)[1] = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <int VEC> __device__ __forceinline__ void lds_ld(const float *p, float (&v)[VEC]) { LdsVec<VEC>::ld(p, v); }

// The cell-owned tile kernel (dfa3d_backward_cells.hip): rows of 32 channels, tiles of at most 64 pixels.
bool cell_kernel_applies(int C, int D, int ty, int tx, bool fused);
size_t cell_kernel_lds_bytes(int ty, int tx, int D);
size_t cell_kernel_half_cu_lds();      // the most dynamic LDS with which two of its workgroups fit a CU
const void *cell_kernel_symbol(int dtype, bool fused);
hipError_t launch_cell_kernel(const BwdArgs &a, int dtype, const BinWorkspace &ws, size_t lds, int grid, float *gd_heads,
                              hipStream_t stream);

}  // namespace dfa3d
