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
constexpr int kGPitch = kCellC;       // words between staged grad_out rows
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
  o.dots = o.sslot + kCellPass;
  o.cnt = o.dots + kCellPass * 4 + kWave;                    // + one scrap word per lane
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
  int d0;                     // lower depth bin
  uint32_t tr01, tr23;        // tile rows of the corners, 16 bits each, 0xFFFF = none
  unsigned bits;              // bit k: corner k inside the map; 4: depth inside; 5, 6: lower, upper tap exists; 7: live
};
// the taps of a finished point that found their address taken: added atomically one phase later
struct LateTaps {
  float v[8];                 // value of tap j (corner j / 2, lower / upper bin)
  int at[4];                  // tile address of each corner's lower tap, -1 = none
  unsigned late;              // bit j: tap j is still to be added
};

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
  __shared__ int4 s_item;

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
  int *s_slot = reinterpret_cast<int *>(smem + lay.sslot);
  int *cnt = reinterpret_cast<int *>(smem + lay.cnt), *offs = reinterpret_cast<int *>(smem + lay.offs);
  uint32_t *goff = reinterpret_cast<uint32_t *>(smem + lay.goff);
  const int cl = lane % LPR;
  const int cell = wave * (kWave / LPR) + lane / LPR;      // walkers: the cell of this lane group
  const int LP = L * P;
  const int n_bit_words = (R * D + 31) / 32;

  for (int i = tid; i < lay.gstage; i += kCellBlock) smem[i] = 0;                   // depth tile and bitmap
  for (int i = tid; i < C; i += kCellBlock) gstage[PP * kGPitch + i] = 0;           // the row idle lanes read
  for (int i = tid; i < 2 * kCellMax; i += kCellBlock) cnt[i] = 0;
  CT_DECL

  ItemFetch fetch;
  if (tid == 0) fetch.start(ws, p, blockIdx.x % kClasses);
  for (;;) {
    // ---- next work item: (bin, chunk of its points), in bin order
    __syncthreads();
    if (tid == 0) fetch.advance(ws, p, blockIdx.x % kClasses, &s_item);
    __syncthreads();
    const int4 item = s_item;
    const int bin = item.x, seg = item.y, n_item = item.z, chunks_here = item.w;
    if (bin < 0) break;                                   // queues drained: every wave leaves
    CT_MARK(0);
    const int bm = bin / nb, local = bin - bm * nb;
    int b, m;
    slot_decode(bm, B, M, b, m);
    int l = 0;
    while (l + 1 < L && local >= p.level_base[l + 1]) ++l;
    const int tile = local - p.level_base[l];
    const int H = p.H[l], W = p.W[l], Dd = p.Dd[l], start = p.start[l];
    const int y0 = (tile / p.tiles_x[l]) * TY - 1, x0 = (tile % p.tiles_x[l]) * TX - 1;      // pixel of the tile's row 0
    const int n_pass = (n_item + PP - 1) / PP;

    if (walker) {
      // =========================== walkers ===========================
      const rsrc_t value_r = make_rsrc(value + (size_t)b * S * M * C, (size_t)S * M * C * sizeof(T));
      const rsrc_t go_r = make_rsrc(grad_out + (size_t)b * Q * M * C, (size_t)Q * M * C * sizeof(T));
      const uint32_t chan_off = (uint32_t)(cl * VEC * sizeof(T));
      // the four value rows of this group's cell (zero outside the map, or when the cell is not part of the tile)
      float v[4][VEC], acc[4][VEC];
      {
        const int cy = cell / TX, cx = cell - cy * TX;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int y = y0 + cy + (k >= 2 ? 1 : 0), x = x0 + cx + ((k == 1 || k == 2) ? 1 : 0);
          const bool ok = cell < n_cells && in_map(y, x, H, W) && !DFA3D_DIAG(diag, 8);
          RowVec<T, float, VEC>::ld(value_r, (ok ? (uint32_t)(((start + y * W + x) * M + m) * C * (int)sizeof(T)) : kNoRow) + chan_off, v[k]);
#pragma unroll
          for (int i = 0; i < VEC; ++i) acc[k][i] = 0;
        }
      }
      for (int turn = 0; turn <= n_pass + 1; ++turn) {      // uniform over the workgroup
        // ---------------- phase X: walk the lists of pass turn - 1 ----------------
        for (int i = tid; i < n_bit_words; i += 4 * kWave) bitmap[i] = 0;          // last used in phase Y before
        if (turn >= 1) {
          int *c_old = cnt + ((turn - 1) & 1) * kCellMax;                          // the sort of pass turn - 1 is over
          if (tid < kCellMax) c_old[tid] = 0;
        }
        if (turn >= 1 && turn <= n_pass && !DFA3D_DIAG(diag, 16)) {
          const int beg = cell < n_cells ? offs[cell] : 0, end = cell < n_cells ? offs[cell + 1] : 0;
          constexpr int UT = 2;
          const float *g_lane = gstage + cl * VEC;
          for (int t = beg; t < end; t += UT) {
            int sl[UT];
            float4 w4[UT];
            float gg[UT][VEC];
#pragma unroll
            for (int j = 0; j < UT; ++j) {
              const bool on = t + j < end;
              const int idx = min(t + j, PP - 1);
              const int s = s_slot[idx];
              const float4 w = s_w[idx];
              sl[j] = on ? s : PP;                              // an idle step reads the row of zeros, weight zero
              w4[j] = on ? w : make_float4(0, 0, 0, 0);
            }
#pragma unroll
            for (int j = 0; j < UT; ++j) lds_ld<VEC>(g_lane + sl[j] * kGPitch, gg[j]);
#pragma unroll
            for (int j = 0; j < UT; ++j) {
              float d[4];
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                d[k] = 0;
#pragma unroll
                for (int i = 0; i < VEC; ++i) d[k] += v[k][i] * gg[j][i];
              }
#pragma unroll
              for (int k = 0; k < 4; ++k) d[k] = row_sum_f<LPR>(d[k]);
              const float wk[4] = {w4[j].x, w4[j].y, w4[j].z, w4[j].w};
#pragma unroll
              for (int k = 0; k < 4; ++k) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[k][i] += wk[k] * gg[j][i];
              }
              // lane c of the group reports corner c's dot; an idle step's goes to a scrap word
              const float mine_d = cl == 0 ? d[0] : cl == 1 ? d[1] : cl == 2 ? d[2] : d[3];
              dots[sl[j] < PP ? sl[j] * 4 + cl : PP * 4 + lane] = mine_d;
            }
          }
        }
        CT_MARK(1);
        __syncthreads();
        CT_MARK(2);
        if (turn > n_pass) break;
        // ---------------- phase Y: stage the grad_out rows of pass turn ----------------
        if (turn < n_pass) {
          constexpr int RPI = kWave / LPR, kRows = PP / 4;      // rows per load instruction, rows per walker wavefront
#pragma unroll
          for (int j = 0; j < kRows; j += RPI) {
            const int slot = wave * kRows + j + lane / LPR;
            float gg[VEC];
            if (DFA3D_DIAG(diag, 256)) { for (int i = 0; i < VEC; ++i) gg[i] = 1.f; } else   // cost of the grad_out loads
            RowVec<T, float, VEC>::ld(go_r, goff[slot] + chan_off, gg);
            LdsVec<VEC>::st(gstage + slot * kGPitch + cl * VEC, gg);
          }
        } else {
          // the item's last walk is over: the cells' accumulators go where the staged rows were
          if (cell < n_cells) {
#pragma unroll
            for (int k = 0; k < 4; ++k) LdsVec<VEC>::st(gstage + (cell * 4 + k) * C + cl * VEC, acc[k]);
          }
        }
        CT_MARK(3);
        __syncthreads();
        CT_MARK(4);
      }
    } else {
      // =========================== pointers ===========================
      const int md = Md == 1 ? 0 : m;
      const rsrc_t dist_r = make_rsrc(FUSED ? dist + (size_t)b * S * Md * D : nullptr, FUSED ? (size_t)S * Md * D * sizeof(T) : 0);
      PointState cur, nxt;
      LateTaps late;
      cur.bits = 0; nxt.bits = 0; late.late = 0;
      cur.gp = nxt.gp = 0; cur.a = nxt.a = 0; cur.lh = cur.lw = cur.ld = nxt.lh = nxt.lw = nxt.ld = 0; cur.d0 = nxt.d0 = 0;
      cur.tr01 = cur.tr23 = nxt.tr01 = nxt.tr23 = 0xFFFFFFFFu;
#pragma unroll
      for (int k = 0; k < 4; ++k) { cur.sc[k] = cur.hl[k] = nxt.sc[k] = nxt.hl[k] = 0; late.at[k] = -1; }
#pragma unroll
      for (int j = 0; j < 8; ++j) late.v[j] = 0;
      for (int turn = 0; turn <= n_pass + 1; ++turn) {      // uniform over the workgroup
        // ---------------- phase X: late taps of pass turn - 2, then prepare pass turn ----------------
        if (FUSED && late.late) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (late.late >> j & 1) atomicAdd(gd + late.at[j >> 1] + (j & 1), late.v[j]);
          late.late = 0;
        }
        CT_MARK(1);
        float4 pw = make_float4(0, 0, 0, 0);               // corner weights in the order of the cell's corners
        int my_cell = -1, my_rank = 0;
        if (turn < n_pass) {
          const int base = turn * PP;
          const bool live = pslot < n_item - base;
          Point2D<float> g;
          DepthTap<float> tap;
          size_t gp = 0;
          float a = 0, wk[4] = {0, 0, 0, 0};
          int tr[4] = {-1, -1, -1, -1};
          unsigned on_bits = 0;
#pragma unroll
          for (int k = 0; k < 4; ++k) { nxt.sc[k] = 0; nxt.hl[k] = 0; g.key[k] = -1; }
          g.inside = false; g.lh = g.lw = g.hh = g.hw = 0; g.h0 = g.w0 = 0;
          tap.inside = tap.lo_ok = tap.hi_ok = false; tap.d0 = 0; tap.ld = tap.hd = 0;
          uint32_t my_goff = kNoRow;
          if (live) {
            gp = ws.entries[seg + base + pslot];
            const float4 rec = ws.recs[seg + base + pslot];
            const size_t unit = gp / LP;
            a = rec.w;
            g = locate_2d<float>(rec.x, rec.y, H, W, start);
            if (FUSED) {
              tap = locate_depth<float>(rec.z, Dd);
              if (DFA3D_DIAG(diag, 32)) { for (int k = 0; k < 4; ++k) { nxt.sc[k] = 0.5f; nxt.hl[k] = 0.1f; } } else   // cost of the depth taps
              {
                float lo[4], hi[4];
                corner_scores<T, float, true>(dist_r, g.key, tap, md, Md, D, nxt.sc, lo, hi);
#pragma unroll
                for (int k = 0; k < 4; ++k) nxt.hl[k] = hi[k] - lo[k];
              }
            } else {
              const T *si = score_in + gp * 4;
#pragma unroll
              for (int k = 0; k < 4; ++k) nxt.sc[k] = score_in != nullptr ? Elem<T>::ld(si + k) : 1.f;
            }
            my_goff = (uint32_t)((unit - (size_t)b * Q * M) * C * sizeof(T));
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              if (g.key[k] >= 0) {
                on_bits |= 1u << k;
                const int ry = g.h0 + (k >= 2 ? 1 : 0) - y0, rx = g.w0 + ((k == 1 || k == 2) ? 1 : 0) - x0;
                if (ry >= 0 && ry <= TY && rx >= 0 && rx <= TX) {
                  tr[k] = ry * TW + rx;
                  wk[k] = g.bil(k) * nxt.sc[k] * a;
                }
              }
            }
            if (g.inside) {
              // the cell: the base pixel within the tile (the binning put the point into this tile by it)
              const int cy = min(max(g.h0 - y0, 0), TY - 1), cx = min(max(g.w0 - x0, 0), TX - 1);
              my_cell = cy * TX + cx;
              my_rank = atomicAdd(cnt + (turn & 1) * kCellMax + my_cell, 1);
            }
          }
          goff[pslot] = my_goff;
          pw = make_float4(wk[0], wk[1], wk[2], wk[3]);
          nxt.gp = (uint32_t)gp; nxt.a = a; nxt.lh = g.lh; nxt.lw = g.lw; nxt.ld = tap.ld; nxt.d0 = tap.d0;
          nxt.tr01 = ((uint32_t)tr[0] & 0xFFFFu) | ((uint32_t)tr[1] << 16);
          nxt.tr23 = ((uint32_t)tr[2] & 0xFFFFu) | ((uint32_t)tr[3] << 16);
          nxt.bits = on_bits | (tap.inside ? 16u : 0u) | (tap.lo_ok ? 32u : 0u) | (tap.hi_ok ? 64u : 0u) |
                     ((live && my_cell >= 0) ? 128u : 0u);
        }
        CT_MARK(2);
        __syncthreads();
        CT_MARK(3);
        if (turn > n_pass) break;
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
            s_slot[pos] = pslot;
            s_w[pos] = pw;
          }
        }
        CT_MARK(4);
        if (turn >= 1 && (cur.bits & 128u) && !DFA3D_DIAG(diag, 512)) {       // (development builds: cost of phase C)
          Point2D<float> g;
          DepthTap<float> tap;
          g.lh = cur.lh; g.lw = cur.lw; g.hh = 1 - cur.lh; g.hw = 1 - cur.lw;
          tap.inside = (cur.bits & 16u) != 0; tap.lo_ok = (cur.bits & 32u) != 0; tap.hi_ok = (cur.bits & 64u) != 0;
          tap.d0 = cur.d0; tap.ld = cur.ld; tap.hd = tap.inside ? 1 - cur.ld : 0.f;
          int trc[4] = {(int)(int16_t)(cur.tr01 & 0xFFFFu), (int)(int16_t)(cur.tr01 >> 16),
                        (int)(int16_t)(cur.tr23 & 0xFFFFu), (int)(int16_t)(cur.tr23 >> 16)};
          const unsigned on_bits = cur.bits & 15u;
          const float a = cur.a;
          const size_t gp = cur.gp;
          const float4 d4 = *reinterpret_cast<const float4 *>(dots + pslot * 4);
          const float dc[4] = {d4.x, d4.y, d4.z, d4.w};
          float gs[4], s[4], ga = 0;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const float dk = dc[k];
            const bool on = on_bits >> k & 1;
            const float bk = g.bil(k);
            gs[k] = on ? bk * a * dk : 0.f;
            s[k] = on ? cur.sc[k] * dk : 0.f;
            ga += bk * s[k];
          }
          const float gx = (float)W * a * (g.hh * (s[1] - s[0]) + g.lh * (s[2] - s[3]));
          const float gy = (float)H * a * (g.hw * (s[3] - s[0]) + g.lw * (s[2] - s[1]));
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
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const bool corner_in = (on_bits >> k & 1) && tap.inside;
              const bool taps = trc[k] >= 0 && tap.inside && gs[k] != 0 && !DFA3D_DIAG(diag, 2);
              late.at[k] = taps ? trc[k] * D + tap.d0 : -1;
              if (taps && tap.lo_ok) want |= 1u << (2 * k);
              if (taps && tap.hi_ok) want |= 2u << (2 * k);
              if (!corner_in) gs[k] = 0.f;
              gz += gs[k] * cur.hl[k];
              late.v[2 * k] = tap.hd * gs[k];
              late.v[2 * k + 1] = tap.ld * gs[k];
            }
            gl[0] = gx; gl[1] = gy; gl[2] = gz * (float)Dd;      // one 12-byte store
            grad_attn[gp] = ga;                       // all stores before the tile updates: they complete slowly
            // Who is first at a tile address in this pass: the bit of the address in the bitmap, set with an integer
            // atomic.  The first adds at once with a plain read-modify-write (nobody else touches the address before
            // the next barrier); the others add atomically in the next phase.
            unsigned first = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              if (want >> j & 1) {
                const int at = late.at[j >> 1] + (j & 1);
                const uint32_t bit = 1u << (at & 31);
                if (DFA3D_DIAG(diag, 1024) || (atomicOr(&bitmap[at >> 5], bit) & bit)) {} else first |= 1u << j;
              }
            }
            float cur8[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) cur8[j] = (first >> j & 1) ? gd[late.at[j >> 1] + (j & 1)] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (first >> j & 1) gd[late.at[j >> 1] + (j & 1)] = cur8[j] + late.v[j];
            late.late = want & ~first;
          } else if (grad_score_out != nullptr) {
            float *go4 = grad_score_out + gp * 4;
#pragma unroll
            for (int k = 0; k < 4; ++k) go4[k] = gs[k];
            grad_attn[gp] = ga;
          } else {
            grad_attn[gp] = ga;
          }
        }
        cur = nxt;
        nxt.bits = 0;
        CT_MARK(5);
        __syncthreads();
        CT_MARK(6);
      }
    }
    // Both roles have passed the same barriers; the last one came after the late taps of the final pass, so the
    // depth tile is complete, and the cells' accumulators lie in LDS.

    // ---------------- flush the tile (and leave the depth tile zeroed for the next item) ----------------
    const bool gv16 = (grad16 & 1) != 0, gd16 = (grad16 & 2) != 0;          // uniform
    const int mg = Mg == 1 ? 0 : m;
    char *gvalue_b = static_cast<char *>(grad_value) + (size_t)b * S * M * C * (gv16 ? 2 : 4);
    char *gdist_b = FUSED ? static_cast<char *>(grad_dist) + (size_t)b * S * Mg * D * (gd16 ? 2 : 4) : nullptr;
    const rsrc_t gvalue_r = make_rsrc(gvalue_b, (size_t)S * M * C * sizeof(float));
    const rsrc_t gdist_r = make_rsrc(gdist_b, FUSED ? (size_t)S * Mg * D * sizeof(float) : 0);
    // Pixels 1..TY-1 x 1..TX-1 of the tile belong to no neighbour's halo; when this item holds all the
    // points of its bin nobody else adds to them, so they are stored instead of added atomically
    // (grad_value and grad_dist are zero on entry).
    const bool sole = chunks_here == 1;
    const bool sole_d = sole && Mg == M;                 // a gradient shared by the heads collects from all of them
    // four consecutive elements at element index `e` of a batch slice: stored, or added atomically
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
    // grad_value: pixel (ry, rx) of the tile collects corner 0 of cell (ry, rx), corner 1 of (ry, rx - 1), corner 2
    // of (ry - 1, rx - 1) and corner 3 of (ry - 1, rx), four floats per lane
    constexpr int c4n = C >> 2;
    const int d4n = D >> 2;
    for (int i = tid; i < R * c4n; i += kCellBlock) {
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
      const int y = y0 + ry, x = x0 + rx;
      if (in_map(y, x, H, W) && !DFA3D_DIAG(diag, 4)) {
        const uint32_t e = (uint32_t)(((start + y * W + x) * M + m) * C + c);
        const bool store = sole && ry >= 1 && ry < TY && rx >= 1 && rx < TX;
        if (store || nz) put4(gvalue_b, gvalue_r, gv16, e, val, store, true);
      }
    }
    if (FUSED) {
      for (int i = tid; i < R * d4n; i += kCellBlock) {
        const int r = i / d4n, d = (i - r * d4n) << 2;
        float4 val = *reinterpret_cast<float4 *>(gd + r * D + d);
        const bool nz = val.x != 0 || val.y != 0 || val.z != 0 || val.w != 0;
        if (nz) *reinterpret_cast<float4 *>(gd + r * D + d) = make_float4(0, 0, 0, 0);
        const int ry = r / TW, rx = r - ry * TW;
        const int y = y0 + ry, x = x0 + rx;
        if (in_map(y, x, H, W) && !DFA3D_DIAG(diag, 4)) {
          const uint32_t e = (uint32_t)(((start + y * W + x) * Mg + mg) * D + d);
          const bool store = sole_d && ry >= 1 && ry < TY && rx >= 1 && rx < TX;
          if (store || nz) put4(gdist_b, gdist_r, gd16, e, val, store, false);
        }
      }
    }
    CT_MARK(7);
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
