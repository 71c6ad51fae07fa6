// Tile kernel of the binned backward for rows of 32 channels: cell-owned lane groups and two kinds of wavefronts.
//
// The bins, work items and queues are those of dfa3d_backward_binned.hip; only the work inside a tile differs.
// A tile of TY x TX pixels (at most 64) is seen as its "cells": the points whose base pixel (upper left of the
// four pixels around the location) is that pixel.  All points of a cell touch the same four value rows, so
//   * a group of 4 lanes (8 channels each) owns a cell for the whole work item: the four value rows and the four
//     accumulators of weight * grad_out live in its registers, every point's grad_out row is read from LDS
//     once, the four dot products and the four weighted sums are formed from it, and nothing is added to an LDS
//     tile during the passes (the accumulators of the cells are put together once, when the item ends);
//   * a pass sorts its 256 points by cell: one integer LDS atomic per point.
// (Base pixels run from -1, for a location within half a pixel of the map's upper or left edge, to H - 1 / W - 1;
// the tiles are laid over that range, so a cell's upper or left pixels may lie outside the map like its lower or
// right ones: such corners carry weight zero, their value rows read as zero and their sums are never written.)
//
// The 8 wavefronts of a workgroup have two roles.  "Walkers" (wavefronts 0-3, 16 cells each) stage the grad_out
// rows of a pass in LDS and walk the cells' lists; "pointers" (wavefronts 4-7, one point of the pass per thread)
// do everything that is per point: geometry, depth taps, corner weights, the sort, and afterwards the point's
// gradients and its grad_dist taps into the LDS depth tile.  The two roles meet at two barriers per pass and
// otherwise overlap: while the walkers walk pass i the pointers prepare pass i + 1, while the walkers stage pass
// i + 1 the pointers finish pass i.
//   phase X(t):  walkers: walk(t-1)                 pointers: late taps of pass t-2, then prepare(t)
//   phase Y(t):  walkers: stage(t)                  pointers: place(t) (scan + sorted records), finish(t-1)
// grad_dist taps go to the LDS tile as in the row-owned kernel: the first tap at an address in a pass adds with a
// plain read-modify-write, later ones use the LDS float atomic one phase later; who is first is decided by an
// integer atomic on a bitmap with one bit per tile address.
//
// Semantics are those of bwd_attention_kernel (dfa3d_backward.hip holds the formulas and the reference lines).
#include "dfa3d_binned.h"

namespace dfa3d {

constexpr int kCellBlock = 512;       // threads: wavefronts 0-3 walk, 4-7 own the points
constexpr int kCellPass = 256;        // points per pass: one per pointer thread
constexpr int kCellC = 32;            // channels: 4 lanes of 8
constexpr int kCellMax = 64;          // cells per tile: 4 walker wavefronts of 16 groups
#ifndef DFA3D_CELL_GPITCH
#define DFA3D_CELL_GPITCH 32
#endif
constexpr int kGPitch = DFA3D_CELL_GPITCH;       // words between staged grad_out rows
// the row of zeros behind the staged rows must also lie behind the accumulators that take their place when an item ends
static_assert(kCellMax * 4 * kCellC <= kCellPass * kGPitch, "accumulators would overwrite the row of zeros");

#ifdef DFA3D_TILE_TIMING
// thread 0 (a walker) clocks slots 0-7, thread 256 (a pointer) slots 8-15
#define CT_DECL unsigned long long ct_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}; unsigned long long ct_last = clock64();
#define CT_MARK(i) do { if ((threadIdx.x & 255) == 0) { const unsigned long long ct_now = clock64(); ct_acc[(i) & 7] += ct_now - ct_last; ct_last = ct_now; } } while (0)
#define CT_FLUSH() do { if ((threadIdx.x & 255) == 0) { unsigned long long *ct_g = reinterpret_cast<unsigned long long *>(ws.queues + kClasses * kQueueStride) + (threadIdx.x ? 8 : 0); for (int i = 0; i < 8; ++i) atomicAdd(ct_g + i, ct_acc[i]); } } while (0)
#else
#define CT_DECL
#define CT_MARK(i) do { } while (0)
#define CT_FLUSH() do { } while (0)
#endif

struct CellLds {      // offsets (in 4-byte words) into the dynamic LDS block
  int gd, bits, gstage, sw, sslot, dots, cnt, offs, goff, total;
};
__host__ __device__ inline CellLds cell_lds_layout(int ty, int tx, int D) {
  CellLds o;
  const int R = (ty + 1) * (tx + 1);
  o.gd = 0;
  o.bits = (o.gd + R * D + 3) & ~3;
  o.gstage = (o.bits + (R * D + 31) / 32 + 3) & ~3;          // 16-byte aligned rows
  // kCellPass staged rows and a row of zeros; when the item ends the same words hold the cells' accumulators
  const int stage_words = (kCellPass + 1) * kGPitch, acc_words = kCellMax * 4 * kCellC;
  o.sw = o.gstage + (stage_words > acc_words ? stage_words : acc_words);
  o.sslot = o.sw + kCellPass * 4;
  o.dots = o.sslot + kCellPass / 2;                          // 16-bit point slots
  o.cnt = o.dots + kCellPass * 4;
  o.offs = o.cnt + 2 * kCellMax;
  o.goff = o.offs + kCellMax + 1;
  o.total = o.goff + kCellPass;
  return o;
}

size_t cell_kernel_lds_bytes(int ty, int tx, int D) { return (size_t)cell_lds_layout(ty, tx, D).total * 4; }

// what a pointer thread keeps of its point between the phases
struct PointState {
  uint32_t gp;                // index of the point
  float a, sc[4], hl[4];      // attention weight; corner scores; upper minus lower depth tap per corner
  float lh, lw, ld;           // fractional parts along h, w, depth
  unsigned bits;              // bit k: corner k inside the map; 4: depth inside; 5, 6: lower, upper tap exists; 7: live;
                              // 8-13: the point's cell; 16-31: lower depth bin + 1
};
// the taps of a finished point that found their address taken: added atomically one phase later
struct LateTaps {
  float gs[4], hd, ld;        // gradient at each corner's score; weights of the lower and the upper bin
  unsigned pack;              // bit j: tap j (corner j / 2, lower / upper bin) is still to be added; 8-13: cell; 16-31: lower bin + 1
};
// Queue state of the thread that fetches the work items: the item taken now was popped two items ago and its two
// records asked for one item ago, so neither the queue atomic nor the loads are waited for.
struct CellFetch {
  int classes_done, w_next;
  int4 rec, geo;
  __device__ __forceinline__ void load(const BinWorkspace &ws, int w) {
    rec = w >= 0 ? ws.items[w] : make_int4(-1, 0, 0, 0);
    geo = w >= 0 ? ws.geom[w] : make_int4(0, 0, 0, 0);
  }
  __device__ __forceinline__ void start(const BinWorkspace &ws, const BinPlan &p, int home) {
    classes_done = 0;
    const int w = pop_item(ws, p, home, classes_done);
    load(ws, w);
    w_next = w >= 0 ? pop_item(ws, p, home, classes_done) : -1;
  }
  __device__ __forceinline__ void advance(const BinWorkspace &ws, const BinPlan &p, int home, int4 *r, int4 *g) {
    *r = rec; *g = geo;
    load(ws, w_next);
    w_next = w_next >= 0 ? pop_item(ws, p, home, classes_done) : -1;
  }
};
// a work item, decoded
struct ItemGeom { int bin, seg, n_item, chunks, b, m, H, W, Dd, start, y0, x0; };
// what the kernel declares as static LDS (level tables, the fetching thread's state, three item records): the dynamic
// block of each of two workgroups on a CU may be half of the CU's 160 KB less this
constexpr size_t kCellStaticLds = 4 * DFA3D_MAX_LEVELS * sizeof(int) + sizeof(CellFetch) + 3 * sizeof(ItemGeom);
size_t cell_kernel_half_cu_lds() { return 80 * 1024 - kCellStaticLds; }
// an item record read from LDS is the same in every lane: keep it in scalar registers
__device__ __forceinline__ ItemGeom uniform(const ItemGeom &g) {
  ItemGeom u;
  u.bin = __builtin_amdgcn_readfirstlane(g.bin); u.seg = __builtin_amdgcn_readfirstlane(g.seg);
  u.n_item = __builtin_amdgcn_readfirstlane(g.n_item); u.chunks = __builtin_amdgcn_readfirstlane(g.chunks);
  u.b = __builtin_amdgcn_readfirstlane(g.b); u.m = __builtin_amdgcn_readfirstlane(g.m);
  u.H = __builtin_amdgcn_readfirstlane(g.H); u.W = __builtin_amdgcn_readfirstlane(g.W);
  u.Dd = __builtin_amdgcn_readfirstlane(g.Dd); u.start = __builtin_amdgcn_readfirstlane(g.start);
  u.y0 = __builtin_amdgcn_readfirstlane(g.y0); u.x0 = __builtin_amdgcn_readfirstlane(g.x0);
  return u;
}

// Four partial sums per lane (one per corner) over the four lanes of a group: lane c gets the whole sum of corner c.
// Two exchange steps in which every lane passes on the two (then one) partial sums its partner collects.
__device__ __forceinline__ float quad_corner_sum(float d0, float d1, float d2, float d3, bool odd, bool upper) {
  const float keep_a = odd ? d1 : d0, send_a = odd ? d0 : d1, keep_b = odd ? d3 : d2, send_b = odd ? d2 : d3;
  const float a = keep_a + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(send_a), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  const float b = keep_b + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(send_b), 0xB1, 0xF, 0xF, true));
  const float keep = upper ? b : a, send = upper ? a : b;
  return keep + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(send), 0x4E, 0xF, 0xF, true));               // quad_perm [2,3,0,1]
}

// FUSED: both stages (depth scores recomputed from dist, grad_dist and the z gradient produced).
// !FUSED: stage 2 alone: scores read from score_in, their gradient written to grad_score_out, no depth tile
// (the launcher passes D = 0), grad_loc has gl_stride components of which x, y are written.
template <typename T, bool FUSED>
__global__ __launch_bounds__(kCellBlock, 4) void cell_backward_kernel(
    BinWorkspace ws, const T *__restrict__ value, const T *__restrict__ dist, const T *__restrict__ score_in,
    const T *__restrict__ grad_out, const T *__restrict__ grad_score_in,
    void *__restrict__ grad_value, void *__restrict__ grad_dist, float *__restrict__ grad_loc, int gl_stride,
    float *__restrict__ grad_attn, float *__restrict__ grad_score_out, const float *__restrict__ grad_wu, int Md,
    int Mg, int B, int S, int M, int D, int L, int Q, int P, int grad16 DFA3D_DIAG_PARAM) {
  // grad16: bit 0 = grad_value is bfloat16, bit 1 = grad_dist is bfloat16 (else float)
  // Md: heads stored in dist (M, or 1 = shared by all heads); Mg: heads of the grad_dist buffer written here
  constexpr int C = kCellC, PP = kCellPass, VEC = 8, LPR = 4;
  extern __shared__ __align__(16) float smem[];
  __shared__ int s_lv[4][DFA3D_MAX_LEVELS];              // the plan's level tables: H, W, Dd, first key
  __shared__ CellFetch s_fetch;                           // the fetching thread's queue state, between its turns
  __shared__ ItemGeom s_geom[3];                         // the item before, this one and the next, decoded by the thread that fetches them

  const BinPlan &p = *ws.plan;
  const int nb = p.bins_per_bm;
  if (nb == 0) return;
  const int TY = p.ty, TX = p.tx, TW = TX + 1, R = (TY + 1) * TW, n_cells = TY * TX;
  const CellLds lay = cell_lds_layout(TY, TX, D);
  const int tid = threadIdx.x, lane = tid % kWave;
  // The role is decided by a scalar, so that the compiler branches on it uniformly: a wavefront must never run
  // through the other role's code with all lanes switched off, because barriers count wavefronts, not lanes.
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const bool walker = wave < 4;
  const int pslot = tid - PP;                              // pointers: the point slot of this thread
  float *gd = smem + lay.gd, *gstage = smem + lay.gstage, *dots = smem + lay.dots;
  uint32_t *bitmap = reinterpret_cast<uint32_t *>(smem + lay.bits);
  float4 *s_w = reinterpret_cast<float4 *>(smem + lay.sw);
  uint16_t *s_slot = reinterpret_cast<uint16_t *>(smem + lay.sslot);
  int *cnt = reinterpret_cast<int *>(smem + lay.cnt), *offs = reinterpret_cast<int *>(smem + lay.offs);
  uint32_t *goff = reinterpret_cast<uint32_t *>(smem + lay.goff);
  const int cl = lane % LPR;
  const int cell = wave * (kWave / LPR) + lane / LPR;      // walkers: the cell of this lane group
  const int LP = L * P;
  const int n_bit_words = (R * D + 31) / 32;
  const bool gv16 = (grad16 & 1) != 0, gd16 = (grad16 & 2) != 0;          // uniform

  for (int i = tid; i < lay.gstage; i += kCellBlock) smem[i] = 0;                   // depth tile and bitmap
  for (int i = tid; i < 2 * kCellMax; i += kCellBlock) cnt[i] = 0;
  if (tid < DFA3D_MAX_LEVELS) {      // decoding an item then costs no dependent loads from device memory
    s_lv[0][tid] = p.H[tid]; s_lv[1][tid] = p.W[tid]; s_lv[2][tid] = p.Dd[tid]; s_lv[3][tid] = p.start[tid];
  }
  __syncthreads();
  CT_DECL

  // four consecutive elements at element index `e` of a batch slice of a gradient: stored, or added atomically
  auto put4 = [&](char *base, rsrc_t r, bool is16, uint32_t e, const float4 &val, bool store, bool every) {
    if (!is16) {
      float *fb = reinterpret_cast<float *>(base);
      if (store) {
        *reinterpret_cast<float4 *>(fb + e) = val;                              // zeros too: full lines
      } else {
        if (every || val.x != 0) scatter_add(r, fb, e * 4, val.x);
        if (every || val.y != 0) scatter_add(r, fb, e * 4 + 4, val.y);
        if (every || val.z != 0) scatter_add(r, fb, e * 4 + 8, val.z);
        if (every || val.w != 0) scatter_add(r, fb, e * 4 + 12, val.w);
      }
    } else {
      char *dst = base + (size_t)e * 2;
      if (store) {
        *reinterpret_cast<uint2 *>(dst) = make_uint2(pack_bf16x2(val.x, val.y), pack_bf16x2(val.z, val.w));
      } else {
        if (val.x != 0 || val.y != 0) atomic_add_bf16x2(dst, val.x, val.y);
        if (val.z != 0 || val.w != 0) atomic_add_bf16x2(dst + 4, val.z, val.w);
      }
    }
  };

  // The depth tile of the item in slot `which` goes out and is left zeroed: threads first, first + step, ... of the
  // float4 groups (both roles share the work in the one phase in which nobody adds to the tile).
  auto flush_gd = [&](int which, int first, int step) {
const ItemGeom q = uniform(s_geom[which]);
    const int mg = Mg == 1 ? 0 : q.m;
    char *gdist_b = static_cast<char *>(grad_dist) + (size_t)q.b * S * Mg * D * (gd16 ? 2 : 4);
    const rsrc_t gdist_r = make_rsrc(gdist_b, (size_t)S * Mg * D * sizeof(float));
    const bool sole_d = q.chunks == 1 && Mg == M;       // a gradient shared by the heads collects from all of them
    const int d4n = D >> 2;
    for (int i0 = first; i0 < R * d4n; i0 += step) {
      int i = i0;
      asm volatile("" : "+v"(i));                 // not to be worked out ahead of the loop and kept in registers
      const int r = i / d4n, d = (i - r * d4n) << 2;
      float4 val = *reinterpret_cast<float4 *>(gd + r * D + d);
      const bool nz = val.x != 0 || val.y != 0 || val.z != 0 || val.w != 0;
      if (nz) *reinterpret_cast<float4 *>(gd + r * D + d) = make_float4(0, 0, 0, 0);
      const int ry = r / TW, rx = r - ry * TW;
      const int y = q.y0 + ry, x = q.x0 + rx;
      if (in_map(y, x, q.H, q.W) && !DFA3D_DIAG(diag, 4)) {
        const uint32_t e = (uint32_t)(((q.start + y * q.W + x) * Mg + mg) * D + d);
        const bool store = sole_d && ry >= 1 && ry < TY && rx >= 1 && rx < TX;
        if (store || nz) put4(gdist_b, gdist_r, gd16, e, val, store, false);
      }
    }
  };
  // Work items follow one another without a pause.  An item of n passes takes n + 1 turns of two phases (X, Y: one
  // barrier after each); what is left of it when its last turn ends is dealt with beside the first turns of the item
  // after it: its accumulators (handed over in LDS in its last phase Y) go out in phase X of turn 0, the late taps of
  // its last pass come in that same phase, and its depth tile goes out in phase X of turn 1, before the new item's
  // first finish touches the tile.  When the queues are drained one more item of zero passes does the same for the
  // last real one.
  //   X(t)  walkers: t = 0: value rows of the item, accumulators of the item before; else walk pass t - 1
  //         pointers: late taps of the pass finished last; prepare pass t; t = 1: depth tile of the item before
  //   Y(t)  walkers: stage pass t, or (t = n) hand over the accumulators
  //         pointers: place pass t; finish pass t - 1; ask for the records of the next pass
  // The two roles run the same sequence of items, turns and barriers, each in a loop of its own: what a role keeps in
  // registers from turn to turn then never competes with the other role's registers.
  if (walker) {
    // =========================== walkers ===========================
    float v[4][VEC], acc[4][VEC];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) { v[k][i] = 0; acc[k][i] = 0; }
    }
    const uint32_t chan_off = (uint32_t)(cl * VEC * sizeof(T));
    auto decode = [&](const int4 &item, const int4 &geo) {
      ItemGeom g;
      g.bin = item.x; g.seg = item.y; g.n_item = item.z; g.chunks = item.w;
      g.b = geo.x & 0xFFFF; g.m = geo.x >> 16;
      const int l = geo.y;
      g.H = s_lv[0][l]; g.W = s_lv[1][l]; g.Dd = s_lv[2][l]; g.start = s_lv[3][l];
      g.y0 = geo.z; g.x0 = geo.w;                            // pixel of the tile's row 0
      return g;
    };
    if (tid == 0) {
      CellFetch fetch;
      int4 rec, geo;
      fetch.start(ws, p, blockIdx.x % kClasses);
      fetch.advance(ws, p, blockIdx.x % kClasses, &rec, &geo);
      s_geom[0] = decode(rec, geo);
      s_fetch = fetch;
    }
    __syncthreads();                                        // the first item's record is there
    for (int it = 0;; ++it) {
      const ItemGeom g = uniform(s_geom[it % 3]);
      const bool have_prev = it > 0, done = g.bin < 0;
      if (done && !have_prev) break;
      const int n_pass = done ? 0 : (g.n_item + PP - 1) / PP;
      CT_MARK(0);
      // The record of the item after this one, first of all: here the walkers hold nothing in registers (the
      // accumulators were handed over, the value rows are about to be replaced), and nobody reads the slot before
      // this item's last phase Y.
      if (tid == 0 && !done) {
        CellFetch fetch = s_fetch;
        int4 rec, geo;
        fetch.advance(ws, p, blockIdx.x % kClasses, &rec, &geo);
        s_geom[(it + 1) % 3] = decode(rec, geo);
        s_fetch = fetch;
      }
      const rsrc_t value_r = make_rsrc(value + (size_t)g.b * S * M * C, (size_t)S * M * C * sizeof(T));
      const rsrc_t go_r = make_rsrc(grad_out + (size_t)g.b * Q * M * C, (size_t)Q * M * C * sizeof(T));
      for (int turn = 0; turn <= n_pass; ++turn) {          // uniform over the workgroup
        // ---------------- phase X ----------------
        for (int i = tid; i < n_bit_words; i += PP) bitmap[i] = 0;                 // last used in the phase Y before
        if (turn >= 1 && tid < kCellMax) cnt[((turn - 1) & 1) * kCellMax + tid] = 0;   // the sort of pass turn - 1 is over
        if (turn == 0) {
          // the four value rows of this group's cell (zero outside the map, or when the cell is not part of the
          // tile), asked for first: they arrive while the accumulators of the item before go out
          {
            const int cy = cell / TX, cx = cell - cy * TX;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int y = g.y0 + cy + (k >= 2 ? 1 : 0), x = g.x0 + cx + ((k == 1 || k == 2) ? 1 : 0);
              const bool ok = !done && cell < n_cells && in_map(y, x, g.H, g.W) && !DFA3D_DIAG(diag, 8);
              RowVec<T, float, VEC>::ld(value_r, (ok ? (uint32_t)(((g.start + y * g.W + x) * M + g.m) * C * (int)sizeof(T)) : kNoRow) + chan_off, v[k]);
            }
          }
          if (have_prev) {
            // Pixel (ry, rx) of the tile collects corner 0 of cell (ry, rx), corner 1 of (ry, rx - 1), corner 2 of
            // (ry - 1, rx - 1) and corner 3 of (ry - 1, rx), four floats per lane.  Pixels 1..TY-1 x 1..TX-1 belong to
            // no neighbour's halo; when the item held all the points of its bin nobody else adds to them, so they are
            // stored instead of added atomically (grad_value is zero on entry, or the binning launches cleared what is
            // added to).
            const ItemGeom q = uniform(s_geom[(it + 2) % 3]);
            char *gvalue_b = static_cast<char *>(grad_value) + (size_t)q.b * S * M * C * (gv16 ? 2 : 4);
            const rsrc_t gvalue_r = make_rsrc(gvalue_b, (size_t)S * M * C * sizeof(float));
            constexpr int c4n = C >> 2;
            for (int i0 = tid; i0 < R * c4n; i0 += PP) {
              int i = i0;
              asm volatile("" : "+v"(i));             // not to be worked out ahead of the loop and kept in registers
              const int r = i / c4n, c = (i - r * c4n) << 2;
              const int ry = r / TW, rx = r - ry * TW;
              float4 val = make_float4(0, 0, 0, 0);
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                const int cy = ry - (k >= 2 ? 1 : 0), cx = rx - ((k == 1 || k == 2) ? 1 : 0);
                if (cy >= 0 && cy < TY && cx >= 0 && cx < TX) {
                  const float4 t = *reinterpret_cast<const float4 *>(gstage + ((cy * TX + cx) * 4 + k) * C + c);
                  val.x += t.x; val.y += t.y; val.z += t.z; val.w += t.w;
                }
              }
              const bool nz = val.x != 0 || val.y != 0 || val.z != 0 || val.w != 0;
              const int y = q.y0 + ry, x = q.x0 + rx;
              if (in_map(y, x, q.H, q.W) && !DFA3D_DIAG(diag, 4)) {
                const uint32_t e = (uint32_t)(((q.start + y * q.W + x) * M + q.m) * C + c);
                const bool store = q.chunks == 1 && ry >= 1 && ry < TY && rx >= 1 && rx < TX;
                if (store || nz) put4(gvalue_b, gvalue_r, gv16, e, val, store, true);
              }
            }
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[k][i] = 0;
          }
        } else if (!DFA3D_DIAG(diag, 16)) {
          // walk the lists of pass turn - 1
          const int beg = cell < n_cells ? offs[cell] : 0, end = cell < n_cells ? offs[cell + 1] : 0;
          if (beg < end) {                                  // lanes leave the loop as their cell's list ends
            // One point per step; the next step's grad_out row is asked for while this step's sums are formed, so
            // that no LDS round trip is waited for with nothing to do.
            const float *g_lane = gstage + cl * VEC;
            int s_cur = s_slot[beg];
            float g_cur[VEC];
            lds_ld<VEC>(g_lane + s_cur * kGPitch, g_cur);
            for (int t = beg; t < end; ++t) {
              const int s_nxt = s_slot[t + 1 < end ? t + 1 : t];
              const float4 w_cur = s_w[t];
              float d[4];
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                d[k] = 0;
#pragma unroll
                for (int i = 0; i < VEC; ++i) d[k] += v[k][i] * g_cur[i];
              }
              float g_nxt[VEC];
              lds_ld<VEC>(g_lane + s_nxt * kGPitch, g_nxt);
              const float wk[4] = {w_cur.x, w_cur.y, w_cur.z, w_cur.w};
#pragma unroll
              for (int k = 0; k < 4; ++k) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[k][i] += wk[k] * g_cur[i];
              }
              dots[s_cur * 4 + cl] = quad_corner_sum(d[0], d[1], d[2], d[3], (cl & 1) != 0, (cl & 2) != 0);   // lane c reports corner c
              s_cur = s_nxt;
#pragma unroll
              for (int i = 0; i < VEC; ++i) g_cur[i] = g_nxt[i];
            }
          }
        }
        if (turn == 1) {
          // the depth tile of the item before: complete since the late taps of turn 0, not touched again before this
          // item's first finish in phase Y of this turn
          if (FUSED && have_prev) flush_gd((it + 2) % 3, tid, kCellBlock);
        }
        CT_MARK(1);
        lds_barrier();
        CT_MARK(2);
        // ---------------- phase Y ----------------
        if (turn < n_pass) {
          // stage the grad_out rows of pass turn
          constexpr int RPI = kWave / LPR, kRows = PP / 4;      // rows per load instruction, rows per walker wavefront
#pragma unroll
          for (int j = 0; j < kRows; j += RPI) {
            const int slot = wave * kRows + j + lane / LPR;
            float gg[VEC];
            if (DFA3D_DIAG(diag, 256)) { for (int i = 0; i < VEC; ++i) gg[i] = 1.f; } else   // cost of the grad_out loads
            RowVec<T, float, VEC>::ld(go_r, goff[slot] + chan_off, gg);
            LdsVec<VEC>::st(gstage + slot * kGPitch + cl * VEC, gg);
          }
        } else if (done) {
          if (FUSED && have_prev) flush_gd((it + 2) % 3, tid, PP);   // the last item's depth tile: nothing follows
        } else {
          // the item's last walk is over: the cells' accumulators go where the staged rows were
          if (cell < n_cells) {
#pragma unroll
            for (int k = 0; k < 4; ++k) LdsVec<VEC>::st(gstage + (cell * 4 + k) * C + cl * VEC, acc[k]);
          }
        }
        CT_MARK(3);
        lds_barrier();
        CT_MARK(4);
      }
      if (done) break;
    }
  } else {
    // =========================== pointers ===========================
    PointState cur, nxt;
    LateTaps late;
    uint32_t pre_gp = 0;                                    // index and record of the point this thread prepares next
    float4 pre_rec = make_float4(0, 0, 0, 0);
    cur.bits = 0; nxt.bits = 0; late.pack = 0; late.hd = late.ld = 0;
    cur.gp = nxt.gp = 0; cur.a = nxt.a = 0; cur.lh = cur.lw = cur.ld = nxt.lh = nxt.lw = nxt.ld = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) { cur.sc[k] = cur.hl[k] = nxt.sc[k] = nxt.hl[k] = 0; late.gs[k] = 0; }
    __syncthreads();                                        // the first item's record is there
    {
      const ItemGeom g0 = uniform(s_geom[0]);
      if (g0.bin >= 0 && pslot < g0.n_item) {
        pre_gp = ws.entries[g0.seg + pslot];
        pre_rec = ws.recs[g0.seg + pslot];
      }
    }
    for (int it = 0;; ++it) {
      const ItemGeom g = uniform(s_geom[it % 3]);
      const bool have_prev = it > 0, done = g.bin < 0;
      if (done && !have_prev) break;
      const int n_pass = done ? 0 : (g.n_item + PP - 1) / PP;
      CT_MARK(0);
      const int md = Md == 1 ? 0 : g.m;
      const rsrc_t dist_r = make_rsrc(FUSED ? dist + (size_t)g.b * S * Md * D : nullptr, FUSED ? (size_t)S * Md * D * sizeof(T) : 0);
      const rsrc_t go_r = make_rsrc(grad_out + (size_t)g.b * Q * M * C, (size_t)Q * M * C * sizeof(T));
      for (int turn = 0; turn <= n_pass; ++turn) {          // uniform over the workgroup
        // ---------------- phase X: late taps of the pass finished last, then prepare pass turn ----------------
        if (FUSED && (late.pack & 0xFFu)) {
          const int lcell = (late.pack >> 8) & 63, lcy = lcell / TX, lcx = lcell - lcy * TX, ld0 = (int)(late.pack >> 16) - 1;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            if (late.pack >> j & 1) {
              const int k = j >> 1, row = (lcy + (k >= 2 ? 1 : 0)) * TW + lcx + ((k == 1 || k == 2) ? 1 : 0);
              atomicAdd(gd + row * D + ld0 + (j & 1), ((j & 1) ? late.ld : late.hd) * late.gs[k]);
            }
          }
          late.pack = 0;
        }
        CT_MARK(1);
        float4 pw = make_float4(0, 0, 0, 0);               // corner weights of this thread's point
        int my_cell = -1, my_rank = 0;
        if (turn < n_pass) {
          const int base = turn * PP;
          const bool live = pslot < g.n_item - base;
          Point2D<float> pg;
          DepthTap<float> tap;
          size_t gp = 0;
          float a = 0, wk[4] = {0, 0, 0, 0};
          unsigned on_bits = 0;
#pragma unroll
          for (int k = 0; k < 4; ++k) { nxt.sc[k] = 0; nxt.hl[k] = 0; pg.key[k] = -1; }
          pg.inside = false; pg.lh = pg.lw = pg.hh = pg.hw = 0; pg.h0 = pg.w0 = 0;
          tap.inside = tap.lo_ok = tap.hi_ok = false; tap.d0 = 0; tap.ld = tap.hd = 0;
          uint32_t my_goff = kNoRow, touch = 0;
          if (live) {
            gp = pre_gp;                                     // asked for one phase ago
            const float4 rec = pre_rec;
            const size_t unit = gp / LP;
            a = rec.w;
            my_goff = (uint32_t)((unit - (size_t)g.b * Q * M) * C * sizeof(T));
            // ask for the point's grad_out row now, so that the walkers' staging loads of the next phase find it in the L2
            touch = __builtin_amdgcn_raw_buffer_load_b32(go_r, my_goff, 0, 0);
            pg = locate_2d<float>(rec.x, rec.y, g.H, g.W, g.start);
            if (FUSED) {
              tap = locate_depth<float>(rec.z, g.Dd);
              if (DFA3D_DIAG(diag, 32)) { for (int k = 0; k < 4; ++k) { nxt.sc[k] = 0.5f; nxt.hl[k] = 0.1f; } } else   // cost of the depth taps
              {
                float lo[4], hi[4];
                corner_scores<T, float, true>(dist_r, pg.key, tap, md, Md, D, nxt.sc, lo, hi);
#pragma unroll
                for (int k = 0; k < 4; ++k) nxt.hl[k] = hi[k] - lo[k];
              }
            } else {
              const T *si = score_in + gp * 4;
#pragma unroll
              for (int k = 0; k < 4; ++k) nxt.sc[k] = score_in != nullptr ? Elem<T>::ld(si + k) : 1.f;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              if (pg.key[k] >= 0) {
                on_bits |= 1u << k;
                wk[k] = pg.bil(k) * nxt.sc[k] * a;
              }
            }
            if (pg.inside) {
              // the cell: the base pixel within the tile (the binning put the point into this tile by it)
              const int cy = min(max(pg.h0 - g.y0, 0), TY - 1), cx = min(max(pg.w0 - g.x0, 0), TX - 1);
              my_cell = cy * TX + cx;
              my_rank = atomicAdd(cnt + (turn & 1) * kCellMax + my_cell, 1);
            }
          }
          if (touch == 0x7FC12345u) my_goff = kNoRow;      // never (a NaN payload no gradient carries): keeps the load alive
          goff[pslot] = my_goff;
          pw = make_float4(wk[0], wk[1], wk[2], wk[3]);
          nxt.gp = (uint32_t)gp; nxt.a = a; nxt.lh = pg.lh; nxt.lw = pg.lw; nxt.ld = tap.ld;
          nxt.bits = on_bits | (tap.inside ? 16u : 0u) | (tap.lo_ok ? 32u : 0u) | (tap.hi_ok ? 64u : 0u) |
                     ((live && my_cell >= 0) ? 128u : 0u) | ((unsigned)max(my_cell, 0) << 8) | ((unsigned)(tap.d0 + 1) << 16);
        }
        if (FUSED && have_prev && turn == 1) flush_gd((it + 2) % 3, tid, kCellBlock);     // the walkers take the other half
        CT_MARK(2);
        lds_barrier();
        CT_MARK(3);
        // ---------------- phase Y: place pass turn, finish pass turn - 1 ----------------
        if (turn < n_pass) {
          // exclusive prefix of the cell counters; every pointer wavefront computes it and writes the same numbers,
          // so it can go on with its own copy without waiting for the others
          const int c = cnt[(turn & 1) * kCellMax + lane];
          const int inc = wave_inclusive_scan(c);
          offs[lane] = inc - c;
          if (lane == kWave - 1) offs[kCellMax] = inc;
          if (my_cell >= 0) {
            const int pos = offs[my_cell] + my_rank;
            s_slot[pos] = (uint16_t)pslot;
            s_w[pos] = pw;
          }
        }
        CT_MARK(4);
        if (turn >= 1 && (cur.bits & 128u) && !DFA3D_DIAG(diag, 512)) {       // (development builds: cost of phase C)
          Point2D<float> pg;
          DepthTap<float> tap;
          pg.lh = cur.lh; pg.lw = cur.lw; pg.hh = 1 - cur.lh; pg.hw = 1 - cur.lw;
          tap.inside = (cur.bits & 16u) != 0; tap.lo_ok = (cur.bits & 32u) != 0; tap.hi_ok = (cur.bits & 64u) != 0;
          tap.d0 = (int)(cur.bits >> 16) - 1; tap.ld = cur.ld; tap.hd = tap.inside ? 1 - cur.ld : 0.f;
          const unsigned on_bits = cur.bits & 15u;
          const int ccell = (cur.bits >> 8) & 63, ccy = ccell / TX, ccx = ccell - ccy * TX;
          const float a = cur.a;
          const size_t gp = cur.gp;
          const float4 d4 = *reinterpret_cast<const float4 *>(dots + pslot * 4);
          const float dc[4] = {d4.x, d4.y, d4.z, d4.w};
          float gs[4], sk[4], ga = 0;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const bool on = on_bits >> k & 1;
            const float bk = pg.bil(k);
            gs[k] = on ? bk * a * dc[k] : 0.f;
            sk[k] = on ? cur.sc[k] * dc[k] : 0.f;
            ga += bk * sk[k];
          }
          const float gx = (float)g.W * a * (pg.hh * (sk[1] - sk[0]) + pg.lh * (sk[2] - sk[3]));
          const float gy = (float)g.H * a * (pg.hw * (sk[3] - sk[0]) + pg.lw * (sk[2] - sk[1]));
          float *gl = grad_loc + gp * gl_stride;
          if (!FUSED) { gl[0] = gx; gl[1] = gy; }
          if (FUSED) {
            if (grad_score_in != nullptr) {
              const T *gi = grad_score_in + gp * 4;
#pragma unroll
              for (int k = 0; k < 4; ++k) gs[k] += Elem<T>::ld(gi + k);
            }
            if (grad_wu != nullptr) {       // weight_update = sum over points of attn * mean corner score
              const float gw = grad_wu[gp / LP] * 0.25f;
              ga += gw * (cur.sc[0] + cur.sc[1] + cur.sc[2] + cur.sc[3]);
#pragma unroll
              for (int k = 0; k < 4; ++k) gs[k] += gw * a;
            }
            float gz = 0;
            unsigned want = 0;                          // bit j: tap j exists
            int at4[4];                                 // tile address of each corner's lower tap
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const bool corner_in = (on_bits >> k & 1) && tap.inside;     // a corner inside the map lies inside the tile
              if (!corner_in) gs[k] = 0.f;
              const bool taps = corner_in && gs[k] != 0 && !DFA3D_DIAG(diag, 2);
              at4[k] = ((ccy + (k >= 2 ? 1 : 0)) * TW + ccx + ((k == 1 || k == 2) ? 1 : 0)) * D + tap.d0;
              if (taps && tap.lo_ok) want |= 1u << (2 * k);
              if (taps && tap.hi_ok) want |= 2u << (2 * k);
              gz += gs[k] * cur.hl[k];
              late.gs[k] = gs[k];
            }
            late.hd = tap.hd; late.ld = tap.ld;
            gl[0] = gx; gl[1] = gy; gl[2] = gz * (float)g.Dd;      // one 12-byte store
            grad_attn[gp] = ga;                       // all stores before the tile updates: they complete slowly
            // Who is first at a tile address in this pass: the bit of the address in the bitmap, set with an integer
            // atomic.  The first adds at once with a plain read-modify-write (nobody else touches the address before
            // the next barrier); the others add atomically in the next phase.
            unsigned first = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              if (want >> j & 1) {
                const int at = at4[j >> 1] + (j & 1);
                const uint32_t bit = 1u << (at & 31);
                if (DFA3D_DIAG(diag, 1024) || (atomicOr(&bitmap[at >> 5], bit) & bit)) {} else first |= 1u << j;
              }
            }
            float cur8[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) cur8[j] = (first >> j & 1) ? gd[at4[j >> 1] + (j & 1)] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (first >> j & 1) gd[at4[j >> 1] + (j & 1)] = cur8[j] + ((j & 1) ? tap.ld : tap.hd) * gs[j >> 1];
            late.pack = (want & ~first) | (cur.bits & 0xFFFF3F00u);
          } else if (grad_score_out != nullptr) {
            float *go4 = grad_score_out + gp * 4;
#pragma unroll
            for (int k = 0; k < 4; ++k) go4[k] = gs[k];
            grad_attn[gp] = ga;
          } else {
            grad_attn[gp] = ga;
          }
        }
        // the records of the next pass's points (of this item, or of the first pass of the item after it, whose record
        // was written in phase X of turn 1): they arrive while the workgroup waits at the barrier
        if (!done) {
          const bool last = turn >= n_pass;
          const ItemGeom ng = uniform(s_geom[(it + 1) % 3]);
          const int next_seg = last ? ng.seg : g.seg, next_base = last ? 0 : (turn + 1) * PP;
          const int next_n = last ? (ng.bin >= 0 ? ng.n_item : 0) : g.n_item;
          if ((!last || turn >= 1) && pslot < next_n - next_base) {
            pre_gp = ws.entries[next_seg + next_base + pslot];
            pre_rec = ws.recs[next_seg + next_base + pslot];
          }
        }
        cur = nxt;
        nxt.bits = 0;
        CT_MARK(5);
        lds_barrier();
        CT_MARK(6);
      }
      if (done) break;
    }
  }
  CT_FLUSH();
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
// The kernel takes rows of 32 channels on tiles of at most 64 pixels whose rows and depth rows are whole
// 16-byte groups; everything else stays with the row-owned tile kernel.
bool cell_kernel_applies(int C, int D, int ty, int tx, bool fused) {
  return C == kCellC && ty * tx <= kCellMax && ty >= 1 && tx >= 1 && (!fused || (D & 3) == 0);
}

template <typename T>
static hipError_t launch_cell_typed(const BwdArgs &a, const BinWorkspace &ws, size_t lds, int grid, float *gd_heads,
                                    hipStream_t stream) {
  if (a.dist != nullptr) {
    hipLaunchKernelGGL((cell_backward_kernel<T, true>), dim3(grid), dim3(kCellBlock), lds, stream, ws, (const T *)a.value,
                       (const T *)a.dist, (const T *)nullptr, (const T *)a.grad_out, (const T *)a.grad_score_in,
                       a.grad_value, gd_heads != nullptr ? (void *)gd_heads : a.grad_dist, (float *)a.grad_loc,
                       a.grad_loc_stride, (float *)a.grad_attn, (float *)nullptr, (const float *)a.grad_weight_update,
                       a.dist_heads == 1 ? 1 : a.M, (a.dist_heads == 1 && gd_heads == nullptr) ? 1 : a.M, a.B, a.S, a.M,
                       a.D, a.L, a.Q, a.P, (a.grad_bf16 ? 1 : 0) | ((a.grad_bf16 && gd_heads == nullptr) ? 2 : 0)
                       DFA3D_DIAG_ARG(a));
  } else {
    hipLaunchKernelGGL((cell_backward_kernel<T, false>), dim3(grid), dim3(kCellBlock), lds, stream, ws, (const T *)a.value,
                       (const T *)nullptr, (const T *)a.score_in, (const T *)a.grad_out, (const T *)nullptr,
                       a.grad_value, (void *)nullptr, (float *)a.grad_loc, a.grad_loc_stride, (float *)a.grad_attn,
                       (float *)a.grad_score_out, (const float *)nullptr, a.M, a.M, a.B, a.S, a.M, 0, a.L, a.Q, a.P, 0
                       DFA3D_DIAG_ARG(a));
  }
  return hipGetLastError();
}

const void *cell_kernel_symbol(int dtype, bool fused) {
  if (dtype == DFA3D_F32)
    return fused ? reinterpret_cast<const void *>(cell_backward_kernel<float, true>)
                 : reinterpret_cast<const void *>(cell_backward_kernel<float, false>);
  return fused ? reinterpret_cast<const void *>(cell_backward_kernel<__hip_bfloat16, true>)
               : reinterpret_cast<const void *>(cell_backward_kernel<__hip_bfloat16, false>);
}

hipError_t launch_cell_kernel(const BwdArgs &a, int dtype, const BinWorkspace &ws, size_t lds, int grid, float *gd_heads,
                              hipStream_t stream) {
  return dtype == DFA3D_F32 ? launch_cell_typed<float>(a, ws, lds, grid, gd_heads, stream)
                            : launch_cell_typed<__hip_bfloat16>(a, ws, lds, grid, gd_heads, stream);
}

}  // namespace dfa3d
