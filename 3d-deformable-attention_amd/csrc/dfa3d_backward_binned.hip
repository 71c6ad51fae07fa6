// Binned backward of the fused DFA3D operator for gfx950: no floating-point atomics on device
// memory in the hot loop.
//
// Why: device-memory atomics retire at roughly 10^10 cache-line requests per second on this part,
// and the straightforward backward (bwd_attention_kernel) needs 4 row updates of grad_value and 8
// scalar updates of grad_dist per sampling point.  So the points are first binned by the image tile they
// fall in, and one workgroup per tile accumulates that tile of grad_value and grad_dist in LDS and writes it
// out once: grad_value rows without any atomics (a lane group owns each tile row), grad_dist taps with
// plain LDS updates handed out by integer tickets (LDS floating-point atomics only for the few taps that
// meet another one of the same pass at their address).
//
//   plan_and_clear_kernel       validates the level table, lays out the tiles (bins), clears counters
//   bin_count_kernel            points per bin (LDS histogram per block, one atomic per touched bin)
//   bin_scan_kernel             exclusive prefix over bins, work items (bin, chunk of its points); its further
//                               blocks clear gradient rows for callers that did not zero them (options.clear)
//   bin_fill_sorted_kernel      writes each point's index and record into its bin's segment, a block's points
//                               sorted by bin in LDS first so that runs of records leave together; zero
//                               gradients for points the operator skips
//   bin_points_kernel<0>, <1>   count and fill for shapes the two above do not take (more than 2048 tiles per
//                               (batch, head), more than 2048 points per unit): every record straight to its slot
//   tile_backward_kernel        persistent workgroups pull work items from per-XCD queues; per item: LDS
//                               tiles of (TY+1) x (TX+1) pixels (one-pixel halo to the right/bottom, so
//                               all four corners of a point of this bin land in the tile), the phases
//                               described above the kernel, then one flush of the tile.  FUSED=false:
//                               stage 2 alone
//   tile_depth_backward_kernel  stage 1 alone on the same bins
//   fill_zero / head_sum        a distribution shared by the heads: grad_dist per head, then summed
//
// A point belongs to the tile that holds its base pixel (h0, w0) = floor of its pixel coordinates, -1 <= h0 < H,
// -1 <= w0 < W; the tiles are laid over that range, so the first tile of a level starts at pixel -1.
// Semantics are those of bwd_attention_kernel (see dfa3d_backward.hip for the formulas and the
// reference lines they restate).
#include <map>
#include <mutex>
#include <utility>

#include "dfa3d_binned.h"

namespace dfa3d {

#ifdef DFA3D_TILE_SYNCTHREADS
#define TILE_BARRIER() __syncthreads()
#else
#define TILE_BARRIER() lds_barrier()
#endif


// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void plan_and_clear_kernel(
    BinWorkspace ws, const int64_t *__restrict__ shapes, int shape_stride, const int64_t *__restrict__ level_start, int L,
    int S, int D,
    int B, int M, int ty, int tx, int chunk, int max_bins_per_bm) {
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    BinPlan p;
    int base = 0;
    for (int l = 0; l < DFA3D_MAX_LEVELS; ++l) {
      int64_t H = 0, W = 0, Dd = 0, st = 0;
      bool ok = false;
      if (l < L) {
        H = shapes[l * shape_stride]; W = shapes[l * shape_stride + 1];
        Dd = (shape_stride > 2 && D > 0) ? shapes[l * shape_stride + 2] : 1; st = level_start[l];
        ok = H > 0 && W > 0 && st >= 0 && H <= S && W <= S && st + H * W <= (int64_t)S && Dd > 0 &&
             (D <= 0 || Dd <= D);
      }
      p.H[l] = ok ? (int)H : 0; p.W[l] = ok ? (int)W : 0; p.Dd[l] = ok ? (int)Dd : 0; p.start[l] = ok ? (int)st : 0;
      // tiles are laid over the base pixels of the points, which run from -1 (a location within half a pixel of
      // the map's upper / left edge) to H - 1 / W - 1: the first tile starts at pixel -1
      const int nx = ok ? ((int)W + tx) / tx : 0, ny = ok ? ((int)H + ty) / ty : 0;
      p.tiles_x[l] = nx;
      p.level_base[l] = base;
      base += nx * ny;
    }
    // the host sized the counters from an upper bound of the tile count; never exceed it
    if (base > max_bins_per_bm) base = 0;
    p.bins_per_bm = base;
    p.total_bins = base * slot_count(B, M);
    p.bins_per_class = base * head_groups(M) * B;
    for (int c = 0; c <= kClasses; ++c) p.class_start[c] = 0;
    p.ty = ty; p.tx = tx;
    p.chunk = chunk; p.total_chunks = 0;
    *ws.plan = p;
  }
  const size_t n = (size_t)max_bins_per_bm * slot_count(B, M);
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    ws.counts[i] = 0;
    ws.cursor[i] = 0;
  }
  if (blockIdx.x == 0 && threadIdx.x < kQueueInts) ws.queues[threadIdx.x] = 0;    // the counters and their padding
}

// bin (within one (batch, head)) of a point that the operator does not skip: the tile that holds its base pixel
// (h0, w0), -1 <= h0 < H, -1 <= w0 < W; tile (i, j) covers base pixels [i ty - 1, (i + 1) ty - 1) x [j tx - 1, ...)
__device__ __forceinline__ int bin_of(const BinPlan &p, int l, const Point2D<float> &g) {
  return p.level_base[l] + ((g.h0 + 1) / p.ty) * p.tiles_x[l] + (g.w0 + 1) / p.tx;
}

// The bins of the work items decoded (batch, head, level, pixel of the tile's row 0), so that the tile workgroups
// need no divisions to find their tile: block `block` of `n_blocks` of a fill launch takes its share of the items.
__device__ __forceinline__ void decode_items(const BinWorkspace &ws, int B, int M, int L, int block, int n_blocks) {
  const BinPlan &p = *ws.plan;
  const int n = p.total_chunks;
  for (int w = block * (int)blockDim.x + (int)threadIdx.x; w < n; w += n_blocks * (int)blockDim.x) {
    const int bin = ws.items[w].x;
    const int bm = bin / p.bins_per_bm, local = bin - bm * p.bins_per_bm;
    int b, m, l = 0;
    slot_decode(bm, B, M, b, m);
    while (l + 1 < L && local >= p.level_base[l + 1]) ++l;
    const int tile = local - p.level_base[l];
    ws.geom[w] = make_int4(b | (m << 16), l, (tile / p.tiles_x[l]) * p.ty - 1, (tile % p.tiles_x[l]) * p.tx - 1);
  }
}

// The fill comes in two forms.  bin_fill_sorted_kernel (few enough bins and points per unit): a block sorts its
// kStage points by bin in LDS and writes each bin's run of records to consecutive addresses, so a wavefront's
// store touches a handful of lines instead of 64.  bin_points_kernel<1>: every point's record goes straight to
// its slot.
constexpr int kSortedBins = 2048;   // bins of one (batch, head) the sorted fill holds counters for
constexpr int kStage = 2048;        // points a block of the sorted fill stages (1024: 0.39 ms, 4096: 0.36 ms against 0.32 ms)
constexpr int kFillThreads = 1024;  // 256 / 512 threads: 0.49 / 0.38 ms
__host__ __device__ inline bool sorted_fill_applies(int bins_per_bm, int LP) { return bins_per_bm <= kSortedBins && LP <= kStage; }
constexpr size_t kSortedFillLds = (size_t)kStage * (16 + 4 + 4) + (size_t)(3 * kSortedBins + 1) * 4;

// MODE 0: count.  MODE 1: fill (needs the scanned cursor).
template <int MODE>
__global__ __launch_bounds__(256) void bin_points_kernel(
    BinWorkspace ws, const float *__restrict__ loc, int loc_stride, const float *__restrict__ attn,
    float *__restrict__ grad_loc, int gl_stride, float *__restrict__ grad_attn, float *__restrict__ grad_score,
    int B, int M, int L, int Q, int P, int q_blocks, int n_blocks, int hist_cap DFA3D_DIAG_PARAM) {
  extern __shared__ int s_hist[];          // [0, nb): counts, then for MODE 1 [nb, 2 nb): segment bases
  const BinPlan &p = *ws.plan;
  const int nb = p.bins_per_bm;
  if (nb == 0) return;
  if (sorted_fill_applies(nb, L * P)) return;                   // bin_count_kernel / bin_fill_sorted_kernel do it
  const bool use_lds = nb <= hist_cap;
  if (MODE == 1) decode_items(ws, B, M, L, blockIdx.x, gridDim.x);
  // The launch is a few thousand workgroups that walk the n_blocks blocks of work (so that it costs next to nothing
  // when the kernel steps aside).  head = block % M: with the round-robin placement of workgroups on the 8 XCDs
  // and a grid that is a multiple of 8, the records of one (batch, head) are written through one XCD's L2.
  for (int blk = blockIdx.x; blk < n_blocks; blk += gridDim.x) {
  __syncthreads();                          // the previous block's LDS histogram is no longer in use
  const int m = blk % M, rest = blk / M;
  const int qb = rest % q_blocks, b = rest / q_blocks;
  const int bm = slot_of(b, m, B, M);
  const int LP = L * P;
  const int q0 = qb * kBinQueries, nq = min(kBinQueries, Q - q0);
  const int npts = nq * LP;
  int *gcount = ws.counts + (size_t)bm * nb;
  int *gcursor = ws.cursor + (size_t)bm * nb;

  if (use_lds) {
    for (int i = threadIdx.x; i < nb * (MODE == 1 ? 2 : 1); i += blockDim.x) s_hist[i] = 0;
    __syncthreads();
  }
  // pass 1: histogram of this block's points; the fill keeps the bins of its first kKept rounds in registers
  constexpr int kKept = 4;
  int kept[kKept];
#pragma unroll
  for (int k = 0; k < kKept; ++k) kept[k] = -1;
  int round = 0;
  for (int i = threadIdx.x; i < npts; i += blockDim.x, ++round) {
    const int qi = i / LP, lp = i - qi * LP, l = lp / P;
    const size_t gp = ((size_t)(b * (size_t)Q + q0 + qi) * M + m) * LP + lp;
    const Point2D<float> g = locate_2d<float>(loc[gp * loc_stride], loc[gp * loc_stride + 1], p.H[l], p.W[l], p.start[l]);
    if (g.inside && p.tiles_x[l] > 0) {
      const int bin = bin_of(p, l, g);
      if (MODE == 1) {
#pragma unroll
        for (int k = 0; k < kKept; ++k) kept[k] = round == k ? bin : kept[k];
      }
      if (use_lds) atomicAdd(&s_hist[bin], 1);
      else if (MODE == 0) atomicAdd(&gcount[bin], 1);
    } else if (MODE == 1) {
      // skipped by the operator: all its gradients are zero, and no tile will visit it
      for (int i = 0; i < gl_stride; ++i) grad_loc[gp * gl_stride + i] = 0;
      if (grad_attn != nullptr) grad_attn[gp] = 0;
      if (grad_score != nullptr) {
        for (int k = 0; k < 4; ++k) grad_score[gp * 4 + k] = 0;
      }
    }
  }
  if (use_lds) {
    __syncthreads();
    for (int i = threadIdx.x; i < nb; i += blockDim.x) {
      const int c = s_hist[i];
      if (c > 0) {
        if (MODE == 0) atomicAdd(&gcount[i], c);
        else s_hist[nb + i] = atomicAdd(&gcursor[i], c);     // reserve a run of the bin's segment
      }
      if (MODE == 1) s_hist[i] = 0;                          // reused as the running rank
    }
    __syncthreads();
  }
  if (MODE == 1) {
    // pass 2: place the points
    round = 0;
    for (int i = threadIdx.x; i < npts; i += blockDim.x, ++round) {
      const int qi = i / LP, lp = i - qi * LP, l = lp / P;
      const size_t gp = ((size_t)(b * (size_t)Q + q0 + qi) * M + m) * LP + lp;
      int bin = -1;
      if (round < kKept) {
#pragma unroll
        for (int k = 0; k < kKept; ++k) bin = round == k ? kept[k] : bin;
      } else {
        const Point2D<float> g = locate_2d<float>(loc[gp * loc_stride], loc[gp * loc_stride + 1], p.H[l], p.W[l], p.start[l]);
        if (g.inside && p.tiles_x[l] > 0) bin = bin_of(p, l, g);
      }
      if (bin >= 0) {
        const int slot = use_lds ? s_hist[nb + bin] + atomicAdd(&s_hist[bin], 1) : atomicAdd(&gcursor[bin], 1);
        if (!DFA3D_DIAG(diag, 128)) ws.entries[slot] = (uint32_t)gp;
        if (!DFA3D_DIAG(diag, 64))
          ws.recs[slot] = make_float4(loc[gp * loc_stride], loc[gp * loc_stride + 1],
                                      loc_stride > 2 ? loc[gp * loc_stride + 2] : 0.f, attn != nullptr ? attn[gp] : 0.f);
      }
    }
  }
  }
}

// Count in the same shape as the sorted fill: 1024 threads, kStage points per block, all loads of a thread issued
// before its first LDS atomic.
__global__ __launch_bounds__(kFillThreads) void bin_count_kernel(
    BinWorkspace ws, const float *__restrict__ loc, int loc_stride, int B, int M, int L, int Q, int P, int nq_block,
    int q_blocks) {
  __shared__ int s_cnt[kSortedBins];
  const BinPlan &p = *ws.plan;
  const int nb = p.bins_per_bm;
  const int LP = L * P;
  if (nb == 0 || !sorted_fill_applies(nb, LP)) return;
  const int tid = threadIdx.x;
  const int m = blockIdx.x % M, rest = blockIdx.x / M;
  const int qb = rest % q_blocks, b = rest / q_blocks;
  const int bm = slot_of(b, m, B, M);
  const int q0 = qb * nq_block, nq = min(nq_block, Q - q0);      // any split of the queries gives the same counts
  const int npts = nq * LP;
  constexpr int kPer = kStage / kFillThreads;
  for (int i = tid; i < nb; i += kFillThreads) s_cnt[i] = 0;
  float x[kPer], y[kPer];
  int lv[kPer];
#pragma unroll
  for (int r = 0; r < kPer; ++r) {
    const int i = tid + kFillThreads * r;
    lv[r] = -1; x[r] = y[r] = 0;
    if (i < npts) {
      const int qi = i / LP, lp = i - qi * LP;
      const size_t gp = ((size_t)(b * (size_t)Q + q0 + qi) * M + m) * LP + lp;
      x[r] = loc[gp * loc_stride]; y[r] = loc[gp * loc_stride + 1];
      lv[r] = lp / P;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kPer; ++r) {
    if (lv[r] >= 0) {
      const int l = lv[r];
      const Point2D<float> g = locate_2d<float>(x[r], y[r], p.H[l], p.W[l], p.start[l]);
      if (g.inside && p.tiles_x[l] > 0) atomicAdd(&s_cnt[bin_of(p, l, g)], 1);
    }
  }
  __syncthreads();
  int *gcount = ws.counts + (size_t)bm * nb;
  for (int i = tid; i < nb; i += kFillThreads) {
    const int c = s_cnt[i];
    if (c > 0) atomicAdd(&gcount[i], c);
  }
}

__global__ __launch_bounds__(kFillThreads) void bin_fill_sorted_kernel(
    BinWorkspace ws, const float *__restrict__ loc, int loc_stride, const float *__restrict__ attn,
    float *__restrict__ grad_loc, int gl_stride, float *__restrict__ grad_attn, float *__restrict__ grad_score,
    int B, int M, int L, int Q, int P, int q_blocks) {
  extern __shared__ __align__(16) unsigned char s_raw[];        // kSortedFillLds bytes
  uint4 *s_rec = reinterpret_cast<uint4 *>(s_raw);               // staged records, grouped by bin
  uint32_t *s_gp = reinterpret_cast<uint32_t *>(s_rec + kStage);
  int *s_dst = reinterpret_cast<int *>(s_gp + kStage);
  int *s_cnt = s_dst + kStage;                                   // points of this block per bin
  int *s_lofs = s_cnt + kSortedBins;                             // first staged slot of each bin; [kSortedBins]: total
  int *s_base = s_lofs + kSortedBins + 1;                        // first slot of this block's run in the bin's segment
  __shared__ int s_wave[kFillThreads / kWave];
  const BinPlan &p = *ws.plan;
  const int nb = p.bins_per_bm;
  const int LP = L * P;
  if (nb == 0 || !sorted_fill_applies(nb, LP)) return;
  decode_items(ws, B, M, L, blockIdx.x, gridDim.x);
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int m = blockIdx.x % M, rest = blockIdx.x / M;          // head = block % M, as in bin_points_kernel
  const int qb = rest % q_blocks, b = rest / q_blocks;
  const int bm = slot_of(b, m, B, M);
  // A block takes every q_blocks-th query, not a run of consecutive ones.  Consecutive queries of a model look at
  // neighbouring places (BEV pillars in raster order), so a run of them would put a compact patch of points into a
  // bin, the tile kernel's passes (consecutive points of a bin) would each hit a few tile rows only, and its rows
  // phase, which takes as long as the longest row's list, would slow down (measured: 1.74 -> 2.25 ms).  Spread
  // over the whole query range a block's points cover each bin's area evenly, whatever the order of the queries.
  const int nq = (Q - qb + q_blocks - 1) / q_blocks;             // <= kStage / LP, of which q_blocks is the ceiling quotient
  const int npts = nq * LP;                                      // <= kStage
  int *gcursor = ws.cursor + (size_t)bm * nb;
  constexpr int kPer = kStage / kFillThreads;                             // points per thread

  for (int i = tid; i < nb; i += kFillThreads) s_cnt[i] = 0;
  __syncthreads();
  // 1. every point: its bin and its rank among this block's points of that bin
  int bin[kPer], rank[kPer];
  uint4 rec[kPer];
  uint32_t gpi[kPer];
#pragma unroll
  for (int r = 0; r < kPer; ++r) {
    const int i = tid + kFillThreads * r;
    bin[r] = -1; rank[r] = 0;
    if (i < npts) {
      const int qi = i / LP, lp = i - qi * LP, l = lp / P;
      const size_t gp = ((size_t)(b * (size_t)Q + qb + (size_t)qi * q_blocks) * M + m) * LP + lp;
      const float x = loc[gp * loc_stride], y = loc[gp * loc_stride + 1];
      const Point2D<float> g = locate_2d<float>(x, y, p.H[l], p.W[l], p.start[l]);
      if (g.inside && p.tiles_x[l] > 0) {
        bin[r] = bin_of(p, l, g);
        rank[r] = atomicAdd(&s_cnt[bin[r]], 1);
        rec[r] = make_uint4(__float_as_uint(x), __float_as_uint(y),
                            loc_stride > 2 ? __float_as_uint(loc[gp * loc_stride + 2]) : 0u,
                            attn != nullptr ? __float_as_uint(attn[gp]) : 0u);
        gpi[r] = (uint32_t)gp;
      } else {
        // skipped by the operator: all its gradients are zero, and no tile will visit it
        for (int c = 0; c < gl_stride; ++c) grad_loc[gp * gl_stride + c] = 0;
        if (grad_attn != nullptr) grad_attn[gp] = 0;
        if (grad_score != nullptr) {
          for (int k = 0; k < 4; ++k) grad_score[gp * 4 + k] = 0;
        }
      }
    }
  }
  __syncthreads();
  // 2. runs: reserve this block's run in every touched bin's segment; staged order = bins in order (exclusive scan)
  {
    constexpr int kBinsPer = kSortedBins / kFillThreads;                  // consecutive bins per thread
    int c[kBinsPer], sum = 0;
#pragma unroll
    for (int j = 0; j < kBinsPer; ++j) {
      const int i = tid * kBinsPer + j;
      c[j] = i < nb ? s_cnt[i] : 0;
      sum += c[j];
      if (c[j] > 0) s_base[i] = atomicAdd(&gcursor[i], c[j]);
    }
    const int inc = wave_inclusive_scan(sum);
    if (lane == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    int run = inc - sum;
    for (int w = 0; w < wave; ++w) run += s_wave[w];
#pragma unroll
    for (int j = 0; j < kBinsPer; ++j) {
      const int i = tid * kBinsPer + j;
      if (i < nb) s_lofs[i] = run;
      run += c[j];
    }
    if (tid == kFillThreads - 1) s_lofs[kSortedBins] = run;                   // number of staged points
  }
  __syncthreads();
  // 3. stage
#pragma unroll
  for (int r = 0; r < kPer; ++r) {
    if (bin[r] >= 0) {
      const int pos = s_lofs[bin[r]] + rank[r];
      s_rec[pos] = rec[r];
      s_gp[pos] = gpi[r];
      s_dst[pos] = s_base[bin[r]] + rank[r];
    }
  }
  __syncthreads();
  // 4. write out: consecutive staged slots of one bin go to consecutive addresses
  const int total = s_lofs[kSortedBins];
  for (int i = tid; i < total; i += kFillThreads) {
    const int dst = s_dst[i];
    ws.recs[dst] = *reinterpret_cast<const float4 *>(&s_rec[i]);
    ws.entries[dst] = s_gp[i];
  }
}

// What the tile kernel adds to instead of storing, cleared for a caller that did not zero grad_value / grad_dist
// (options.clear).  The tile kernel stores the rows of the pixels that lie inside a tile (not on its first row or
// column, which are the halo of its upper and left neighbours) when that tile's points fit one work item and the
// rows are whole 16-byte groups; every other row of the two tensors only ever receives atomic adds, or nothing:
// pixels on tile rims, pixels of tiles without points or with several work items, keys outside every level.
// A lane decides for one (batch, key, head) row; the wavefront then clears its 64 consecutive rows together, 16 bytes
// per lane on consecutive addresses (the heads of a key share their fate, so whole lines go out).
__device__ __forceinline__ void clear_rows_of_wave(char *base, size_t first_row, int row_bytes, bool clear_mine, int lane) {
  char *dst = base + first_row * row_bytes;
  if ((row_bytes & 15) == 0) {
    const int n16 = row_bytes >> 4;
    for (int c = lane; c < kWave * n16; c += kWave) {
      const int r = c / n16;
      if (__shfl((int)clear_mine, r, kWave)) *reinterpret_cast<uint4 *>(dst + (size_t)c * 16) = make_uint4(0, 0, 0, 0);
    }
  } else {
    const int n4 = row_bytes >> 2;
    for (int c = lane; c < kWave * n4; c += kWave) {
      const int r = c / n4;
      if (__shfl((int)clear_mine, r, kWave)) *reinterpret_cast<uint32_t *>(dst + (size_t)c * 4) = 0;
    }
  }
}

struct ClearArgs {
  char *grad_value, *grad_dist;     // either may be nullptr: not that one
  int value_row_bytes, dist_row_bytes, B, S, M, L, stores;
};
__device__ __forceinline__ void clear_unstored(const BinWorkspace &ws, const ClearArgs &ca, unsigned block, unsigned n_blocks) {
  char *grad_value = ca.grad_value, *grad_dist = ca.grad_dist;
  const int value_row_bytes = ca.value_row_bytes, dist_row_bytes = ca.dist_row_bytes;
  const int B = ca.B, S = ca.S, M = ca.M, L = ca.L, stores = ca.stores;
  const BinPlan &p = *ws.plan;
  const int nb = p.bins_per_bm, TY = p.ty, TX = p.tx, ch = p.chunk;
  const size_t rows = (size_t)B * S * M;
  const int lane = threadIdx.x % kWave;
  // every wavefront takes 64 consecutive rows per turn; all its lanes stay in the loop (shuffles)
  for (size_t i0 = ((size_t)block * blockDim.x + threadIdx.x) - lane; i0 < rows; i0 += (size_t)n_blocks * blockDim.x) {
    const size_t i = i0 + lane;
    bool clear_mine = i < rows;
    if (clear_mine && stores && nb > 0) {
      const int m = (int)(i % M);
      const size_t bs = i / M;
      const int s = (int)(bs % S), b = (int)(bs / S);
      for (int l = 0; l < L; ++l) {
        const int local = s - p.start[l];
        if (p.H[l] > 0 && local >= 0 && local < p.H[l] * p.W[l]) {
          const int y = local / p.W[l], x = local - y * p.W[l];
          if ((y + 1) % TY != 0 && (x + 1) % TX != 0) {       // the first tile starts at pixel -1
            const int bin = slot_of(b, m, B, M) * nb + p.level_base[l] + ((y + 1) / TY) * p.tiles_x[l] + (x + 1) / TX;
            const int c = ws.counts[bin];
            clear_mine = !(c > 0 && c <= ch);                 // exactly one work item: it stores this row
          }
          break;
        }
      }
    }
    if (grad_value != nullptr) clear_rows_of_wave(grad_value, i0, value_row_bytes, clear_mine, lane);
    if (grad_dist != nullptr) clear_rows_of_wave(grad_dist, i0, dist_row_bytes, clear_mine, lane);
  }
}

// work items of a bin with c points (most bins fit one item, which saves the division)
__device__ __forceinline__ int items_of_bin(int c, int ch) { return c <= ch ? (c > 0 ? 1 : 0) : (c + ch - 1) / ch; }

// The first `scan_blocks` blocks scan, 1024 bins each (in turns if there are more bins than that).  A block needs no
// word from the blocks before it: it adds up the counts of all bins before its own (a few dozen loads per thread for
// tens of thousands of bins), which is cheaper than one workgroup walking all bins and writing every work item from
// one CU.  Further blocks, if any, clear the gradient rows that need it meanwhile (both kinds only read the counts);
// the kernel is held to 64 registers so that two such workgroups fit a CU.
__global__ __launch_bounds__(1024, 8) void bin_scan_kernel(BinWorkspace ws, ClearArgs ca, int scan_blocks) {
  if ((int)blockIdx.x >= scan_blocks) {
    clear_unstored(ws, ca, blockIdx.x - scan_blocks, gridDim.x - scan_blocks);
    return;
  }
  __shared__ int s_pts[16], s_chk[16], s_bp[16], s_bc[16];
  const int n = ws.plan->total_bins, ch = ws.plan->chunk, per_class = ws.plan->bins_per_class;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  for (int base = (int)blockIdx.x * 1024; base < n; base += scan_blocks * 1024) {
    // points and work items of the bins before this block's: every thread its share, summed over the wavefront
    int bp = 0, bc = 0;
#pragma unroll 4
    for (int i = threadIdx.x; i < base; i += 1024) {
      const int c = ws.counts[i];
      bp += c;
      bc += items_of_bin(c, ch);
    }
    bp = __builtin_amdgcn_readlane(wave_inclusive_scan(bp), kWave - 1);
    bc = __builtin_amdgcn_readlane(wave_inclusive_scan(bc), kWave - 1);
    const int i = base + (int)threadIdx.x;
    const int c = i < n ? ws.counts[i] : 0, k = items_of_bin(c, ch);
    const int ip = wave_inclusive_scan(c), ic = wave_inclusive_scan(k);      // inclusive scans within the wavefront
    __syncthreads();                                         // the tables of the turn before have been read
    if (lane == kWave - 1) { s_pts[wave] = ip; s_chk[wave] = ic; }
    if (lane == 0) { s_bp[wave] = bp; s_bc[wave] = bc; }
    __syncthreads();
    int run_p = ip - c, run_c = ic - k;
    for (int w = 0; w < 16; ++w) {
      run_p += s_bp[w] + (w < wave ? s_pts[w] : 0);
      run_c += s_bc[w] + (w < wave ? s_chk[w] : 0);
    }
    if (i < n) {
      if (i % per_class == 0) ws.plan->class_start[i / per_class] = run_c;
      ws.cursor[i] = run_p;
      for (int t = 0; t < k; ++t)
        ws.items[run_c + t] = make_int4(i, run_p + t * ch, min(ch, c - t * ch), k);
      if (i == n - 1) {
        ws.plan->total_chunks = run_c + k;
        ws.plan->class_start[kClasses] = run_c + k;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Tile workgroups.
//
// A work item is one bin (image tile of one batch element, head and level) and up to `chunk` of
// its points.  The points are taken PP (128 or 256) at a time, one per thread:
//   phase A  thread = point: geometry, depth taps, corner weights; every corner becomes a task
//            (tile row, weight, point slot); the point's grad_out row is staged in LDS
//   sort     tasks are grouped by tile row (counting sort in LDS, integer counters)
//   rows     a group of LPR lanes owns a tile row: it loads the value row once, then for each of the
//            row's tasks takes the staged grad_out row, leaves the dot product for phase C and
//            accumulates weight * grad_out in registers; the row sum is added to the LDS tile with a
//            plain read-modify-write (nobody else touches that row during the pass)
//   phase C  thread = point: per-point gradients from the four dots; the 8 grad_dist taps of a point go
//            to the LDS tile (first taker of an address: plain update, later ones: atomics)
// After the item's last pass the tile is flushed to memory once: stores for the inner rows of an item that
// holds all the points of its bin, atomic adds for the rest (the chunks of one bin overlap, and so do the
// rims of neighbouring bins).
// ---------------------------------------------------------------------------------------


struct TileLds {      // offsets (in 4-byte words) into the dynamic LDS block
  int gv, gd, gstage, tasks, dots, cnt, offs, goff, total;
};
__host__ __device__ inline TileLds tile_lds_layout(int ty, int tx, int C, int D, int PP) {
  TileLds o;
  const int R = (ty + 1) * (tx + 1);
  o.gv = 0;
  o.gd = o.gv + R * C;
  o.gstage = (o.gd + R * D + 3) & ~3;              // 16-byte aligned rows
  o.tasks = (o.gstage + (PP + 1) * C + 1) & ~1;    // PP staged rows and one row of zeros; 8-byte records
  o.dots = o.tasks + PP * 4 * 2;
  o.cnt = o.dots + PP * 4 + kWave;                 // + one scrap word per lane
  o.offs = o.cnt + R;
  o.goff = o.offs + R + 1;
  o.total = o.goff + PP;
  return o;
}


struct RowTask { float w; uint32_t who; };   // who = point slot * 4 + corner: the index of the task's dot


// FUSED: both stages (depth scores recomputed from dist, grad_dist and the z gradient produced).
// !FUSED: stage 2 alone: scores read from score_in, their gradient written to grad_score_out, no
// depth tile (the launcher passes D = 0), grad_loc has gl_stride components of which x, y are written.
template <typename T, int VEC, int LPR, bool FUSED>
__global__ __launch_bounds__(512, 4) void tile_backward_kernel(
    BinWorkspace ws, const T *__restrict__ value, const T *__restrict__ dist, const T *__restrict__ score_in,
    const T *__restrict__ grad_out, const T *__restrict__ grad_score_in,
    void *__restrict__ grad_value, void *__restrict__ grad_dist, float *__restrict__ grad_loc, int gl_stride,
    float *__restrict__ grad_attn, float *__restrict__ grad_score_out, const float *__restrict__ grad_wu, int Md,
    int Mg, int B, int S, int M, int C, int D, int L, int Q, int P, int PP, int grad16 DFA3D_DIAG_PARAM) {
  // grad16: bit 0 = grad_value is bfloat16, bit 1 = grad_dist is bfloat16 (else float)
  // Md: heads stored in dist (M, or 1 = shared by all heads); Mg: heads of the grad_dist buffer written here
  constexpr int RPI = kWave / LPR;                  // row groups per wavefront
  extern __shared__ __align__(16) float smem[];
  __shared__ int4 s_item;

  const BinPlan &p = *ws.plan;
  const int nb = p.bins_per_bm;
  if (nb == 0) return;
  const int TY = p.ty, TX = p.tx, TW = TX + 1, R = (TY + 1) * TW;
  const TileLds lay = tile_lds_layout(TY, TX, C, D, PP);
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int n_thr = blockDim.x, n_waves = n_thr / kWave;
  const int kGroups = n_waves * RPI;                   // row groups in the workgroup
  const int stage_per_wave = PP / n_waves;             // grad_out rows each wavefront stages
  float *gv = smem + lay.gv, *gd = smem + lay.gd, *gstage = smem + lay.gstage, *dots = smem + lay.dots;
  RowTask *tasks = reinterpret_cast<RowTask *>(smem + lay.tasks);
  int *cnt = reinterpret_cast<int *>(smem + lay.cnt), *offs = reinterpret_cast<int *>(smem + lay.offs);
  uint32_t *goff = reinterpret_cast<uint32_t *>(smem + lay.goff);
  const int group = wave * RPI + lane / LPR, cl = lane % LPR;
  const int passes = (C + VEC * LPR - 1) / (VEC * LPR);
  const int LP = L * P;
  const int my_set = tid / PP, slot = tid % PP;         // the workgroup has at least 2 PP threads; halves 0 and 1
                                                        // own alternate passes, further threads none

  for (int i = tid; i < R * (C + D); i += n_thr) smem[i] = 0;   // gv and gd are adjacent
  for (int i = tid; i < C; i += n_thr) gstage[PP * C + i] = 0;  // the row that idle lanes of the rows phase read
  TT_DECL

  ItemFetch fetch;
  if (tid == 0) fetch.start(ws, p, blockIdx.x % kClasses);
  int pass_tag = 0x5EED0000;                               // changes with every pass of this workgroup
  for (;;) {
    // ---- next work item: (bin, chunk of its points), in bin order
    TILE_BARRIER();
    if (tid == 0) fetch.advance(ws, p, blockIdx.x % kClasses, &s_item);
    TILE_BARRIER();
    const int4 item = s_item;
    const int bin = item.x, seg = item.y, n_item = item.z, chunks_here = item.w;
    if (bin < 0) break;                                   // queues drained: every wave leaves
    TT_MARK(0);
    const int bm = bin / nb, local = bin - bm * nb;
    int b, m;
    slot_decode(bm, B, M, b, m);
    int l = 0;
    while (l + 1 < L && local >= p.level_base[l + 1]) ++l;
    const int tile = local - p.level_base[l];
    const int H = p.H[l], W = p.W[l], Dd = p.Dd[l], start = p.start[l];
    const int y0 = (tile / p.tiles_x[l]) * TY - 1, x0 = (tile % p.tiles_x[l]) * TX - 1;      // pixel of the tile's row 0

    const rsrc_t value_r = make_rsrc(value + (size_t)b * S * M * C, (size_t)S * M * C * sizeof(T));
    const int md = Md == 1 ? 0 : m;
    const rsrc_t dist_r = make_rsrc(FUSED ? dist + (size_t)b * S * Md * D : nullptr, FUSED ? (size_t)S * Md * D * sizeof(T) : 0);
    const rsrc_t go_r = make_rsrc(grad_out + (size_t)b * Q * M * C, (size_t)Q * M * C * sizeof(T));

    // Per-point state of the pass a thread owns.  With twice as many threads as points per pass the two halves
    // of the workgroup own alternate passes: while one half runs phase C of pass i, the other runs phase A of
    // pass i + 1 (two dependent memory round trips), which then costs no time of its own.
    // What phase C needs of a point, kept small: it stays in registers through the rows phase, where every
    // register counts.  Complements (1 - lh, ...) are formed again where they are used.
    uint32_t st_gp = 0;                                 // index of the point
    float st_a = 0, sc[4], hl[4];                       // weight; corner scores; upper minus lower depth tap per corner
    float st_lh = 0, st_lw = 0, st_ld = 0;              // fractional parts along h, w, depth
    int st_d0 = 0;                                      // lower depth bin
    uint32_t st_tr01 = 0xFFFFFFFFu, st_tr23 = 0xFFFFFFFFu;   // tile rows of the corners, 16 bits each, 0xFFFF = none
    unsigned st_bits = 0;            // bit k: corner k inside the map; 4: depth inside; 5, 6: lower, upper tap exists; 7: live
    // ---------------- phase A: one thread per point ----------------
    auto phase_a = [&](int base, int (&tr)[4], float (&wk)[4]) {
      for (int i = slot; i < R; i += PP) cnt[i] = 0;
      const bool live = slot < n_item - base;
      Point2D<float> g;
      DepthTap<float> tap;
      size_t gp = 0;
      float a = 0;
      unsigned on_bits = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) { sc[k] = 0; hl[k] = 0; g.key[k] = -1; }
      g.inside = false; g.lh = g.lw = g.hh = g.hw = 0; g.h0 = g.w0 = 0;
      tap.inside = tap.lo_ok = tap.hi_ok = false; tap.d0 = 0; tap.ld = tap.hd = 0;
      uint32_t my_goff = kNoRow;
      if (live) {
        gp = ws.entries[seg + base + slot];
        const float4 rec = ws.recs[seg + base + slot];
        const size_t unit = gp / LP;
        a = rec.w;
        g = locate_2d<float>(rec.x, rec.y, H, W, start);
        if (FUSED) {
          tap = locate_depth<float>(rec.z, Dd);
          if (DFA3D_DIAG(diag, 32)) { for (int k = 0; k < 4; ++k) { sc[k] = 0.5f; hl[k] = 0.1f; } } else   // cost of the depth taps
          {
            float lo[4], hi[4];
            corner_scores<T, float, true>(dist_r, g.key, tap, md, Md, D, sc, lo, hi);
#pragma unroll
            for (int k = 0; k < 4; ++k) hl[k] = hi[k] - lo[k];
          }
        } else {
          const T *si = score_in + gp * 4;
#pragma unroll
          for (int k = 0; k < 4; ++k) sc[k] = score_in != nullptr ? Elem<T>::ld(si + k) : 1.f;
        }
        my_goff = (uint32_t)((unit - (size_t)b * Q * M) * C * sizeof(T));
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (g.key[k] >= 0) {
            on_bits |= 1u << k;
            const int ry = g.h0 + (k >= 2 ? 1 : 0) - y0, rx = g.w0 + ((k == 1 || k == 2) ? 1 : 0) - x0;
            if (ry >= 0 && ry <= TY && rx >= 0 && rx <= TX) {
              tr[k] = ry * TW + rx;
              wk[k] = g.bil(k) * sc[k] * a;
            }
          }
        }
      }
      goff[slot] = my_goff;
      st_gp = (uint32_t)gp; st_a = a; st_lh = g.lh; st_lw = g.lw; st_ld = tap.ld; st_d0 = tap.d0;
      st_tr01 = ((uint32_t)tr[0] & 0xFFFFu) | ((uint32_t)tr[1] << 16);
      st_tr23 = ((uint32_t)tr[2] & 0xFFFFu) | ((uint32_t)tr[3] << 16);
      st_bits = on_bits | (tap.inside ? 16u : 0u) | (tap.lo_ok ? 32u : 0u) | (tap.hi_ok ? 64u : 0u) | (live ? 128u : 0u);
    };
    // The loop is rotated: a turn runs phase C of the previous pass on the half that owns it and, meanwhile,
    // phase A of this pass on the other half; then sort and rows of this pass on everybody.  One extra turn
    // finishes the last pass.
    for (int pass_idx = 0;; ++pass_idx) {                        // uniform over the workgroup
      const int base = pass_idx * PP;
      const bool has = base < n_item;
      const bool mine = has && my_set == (pass_idx & 1);         // this thread's half owns the pass
      const bool prev_mine = pass_idx > 0 && my_set == ((pass_idx - 1) & 1);
      int tr[4] = {-1, -1, -1, -1};                               // of this pass: used until its tasks are placed
      float wk[4] = {0, 0, 0, 0};
      if (mine) phase_a(base, tr, wk);

      // ---------------- phase C: per-point gradients, grad_dist taps into the LDS tile ----------------
      // LDS floating-point atomics retire about 0.3 lanes per clock per CU on this part, integer ones more
      // than twenty times as many.  So every tap first swaps this pass's tag into a word that belongs to its
      // tile address (the words live where the grad_out rows were staged: the rows phase is over).  Whoever
      // gets something else than the tag back is the first at that address and adds at once with a plain
      // read-modify-write: nobody else touches the address before the barrier below.  Only the others (under
      // a fifth of the taps at 256 points per pass) use the floating-point atomic, after that barrier.  Stale
      // words cannot do harm: one that happens to equal the tag just sends its address's taps to the atomics.
      int *tickets = reinterpret_cast<int *>(gstage);
      const bool ticketed = FUSED && R * D <= PP * C && !DFA3D_DIAG(diag, 1024);     // uniform over the workgroup
      ++pass_tag;
      // the previous pass's points as phase A left them
      Point2D<float> g;
      DepthTap<float> tap;
      g.lh = st_lh; g.lw = st_lw; g.hh = 1 - st_lh; g.hw = 1 - st_lw;
      tap.inside = (st_bits & 16u) != 0; tap.lo_ok = (st_bits & 32u) != 0; tap.hi_ok = (st_bits & 64u) != 0;
      tap.d0 = st_d0; tap.ld = st_ld; tap.hd = tap.inside ? 1 - st_ld : 0.f;
      int trc[4] = {(int)(int16_t)(st_tr01 & 0xFFFFu), (int)(int16_t)(st_tr01 >> 16),
                    (int)(int16_t)(st_tr23 & 0xFFFFu), (int)(int16_t)(st_tr23 >> 16)};
      const unsigned on_bits = st_bits & 15u;
      const bool live = (st_bits & 128u) != 0;
      const float a = st_a;
      const size_t gp = st_gp;
      float gs[4] = {0, 0, 0, 0};
      unsigned first_mask = 0;              // bit 2k / 2k+1: this thread took the first ticket of corner k's lower / upper tap
      if (prev_mine && live && !DFA3D_DIAG(diag, 512)) {               // (development builds: cost of phase C)
        float s[4], ga = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float dk = dots[slot * 4 + k];
          const bool on = on_bits >> k & 1;
          const float bk = g.bil(k);
          gs[k] = on ? bk * a * dk : 0.f;
          s[k] = on ? sc[k] * dk : 0.f;
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
            ga += gw * (sc[0] + sc[1] + sc[2] + sc[3]);
#pragma unroll
            for (int k = 0; k < 4; ++k) gs[k] += gw * a;
          }
          float gz = 0;
          int at8[8];                               // tile address of each of the eight taps, -1 = no tap
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const bool taps = trc[k] >= 0 && tap.inside && gs[k] != 0 && !DFA3D_DIAG(diag, 2);
            const int at = trc[k] * D + tap.d0;
            at8[2 * k] = (taps && tap.lo_ok) ? at : -1;
            at8[2 * k + 1] = (taps && tap.hi_ok) ? at + 1 : -1;
            if (!taps) {
              gs[k] = ((on_bits >> k & 1) && tap.inside) ? gs[k] : 0.f;      // no taps below for this corner
              if (!(trc[k] >= 0 && tap.inside) || DFA3D_DIAG(diag, 2)) trc[k] = -1;
            }
            gz += ((on_bits >> k & 1) && tap.inside) ? gs[k] * hl[k] : 0.f;
          }
          gl[0] = gx; gl[1] = gy; gl[2] = gz * (float)Dd;      // one 12-byte store
          grad_attn[gp] = ga;                       // all stores before the tile updates: they complete slowly
          if (ticketed) {
            // the eight swaps back to back, then the reads of the first takers, then their writes: one LDS
            // round trip each instead of one per tap (a thread's eight addresses are all different)
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (at8[j] >= 0 && atomicExch(&tickets[at8[j]], pass_tag) != pass_tag) first_mask |= 1u << j;
            float cur8[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) cur8[j] = (first_mask >> j & 1) ? gd[at8[j]] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (first_mask >> j & 1) gd[at8[j]] = cur8[j] + ((j & 1) ? tap.ld : tap.hd) * gs[j >> 1];
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (at8[j] >= 0) atomicAdd(gd + at8[j], ((j & 1) ? tap.ld : tap.hd) * gs[j >> 1]);
          }
        } else if (grad_score_out != nullptr) {
          float *go4 = grad_score_out + gp * 4;
#pragma unroll
          for (int k = 0; k < 4; ++k) go4[k] = gs[k];
          grad_attn[gp] = ga;
        } else {
          grad_attn[gp] = ga;
        }
      }
      if (ticketed && pass_idx > 0) {
        TILE_BARRIER();                                 // plain updates done before the atomic ones start
        if (prev_mine && live) {
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            if (trc[k] >= 0 && gs[k] != 0) {
              float *dst = gd + trc[k] * D + tap.d0;
              if (tap.lo_ok && !(first_mask & (1u << (2 * k)))) atomicAdd(dst, tap.hd * gs[k]);
              if (tap.hi_ok && !(first_mask & (2u << (2 * k)))) atomicAdd(dst + 1, tap.ld * gs[k]);
            }
          }
        }
      }
      TT_MARK(5);
      if (!has) break;
      TILE_BARRIER();                                   // counters cleared, goff visible
      TT_MARK(1);
      int rank[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) rank[k] = (mine && tr[k] >= 0) ? atomicAdd(&cnt[tr[k]], 1) : 0;
      // stage the grad_out rows of this wavefront's 64 points (lanes over channels)
      for (int pass = 0; pass < passes; ++pass) {
        const int chan = (pass * LPR + cl) * VEC;
        const uint32_t chan_off = chan < C ? (uint32_t)(chan * sizeof(T)) : kNoChan;
#pragma unroll 4
        for (int j = 0; j < stage_per_wave; j += RPI) {
          // a wavefront with fewer rows to stage than row groups (short passes, few lanes per row) leaves the
          // groups beyond its share idle: their slots belong to the next wavefront, or lie past the last one
          const int sub = j + lane / LPR;
          const bool slot_ok = sub < stage_per_wave;
          const int slot = wave * stage_per_wave + min(sub, stage_per_wave - 1);
          float gg[VEC];
          if (DFA3D_DIAG(diag, 256)) { for (int i = 0; i < VEC; ++i) gg[i] = 1.f; } else   // cost of the grad_out loads
          RowVec<T, float, VEC>::ld(go_r, goff[slot] + chan_off, gg);
          if (slot_ok && chan < C) LdsVec<VEC>::st(gstage + slot * C + chan, gg);
        }
      }
      TILE_BARRIER();                                   // counts complete
      TT_MARK(2);
      // Exclusive prefix of the row counters.  Every wavefront that places tasks computes it, two rows per
      // lane and 128 rows per step, and writes the same numbers: it can go on with its own copy without
      // waiting for the others.
      if (mine) {                                        // whole wavefronts
        int run = 0;
        for (int r0 = 0; r0 < R; r0 += 2 * kWave) {
          const int r = r0 + 2 * lane;
          const int c0 = r < R ? cnt[r] : 0, c1 = r + 1 < R ? cnt[r + 1] : 0;
          const int inc = wave_inclusive_scan(c0 + c1);
          if (r < R) offs[r] = run + inc - c0 - c1;
          if (r + 1 < R) offs[r + 1] = run + inc - c1;
          run += __builtin_amdgcn_readlane(inc, kWave - 1);
        }
        if (lane == 0) offs[R] = run;
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (!mine) {
        } else if (tr[k] >= 0) {
          RowTask t;
          t.w = wk[k];
          t.who = (uint32_t)(slot * 4 + k);
          tasks[offs[tr[k]] + rank[k]] = t;
        } else {
          dots[slot * 4 + k] = 0;                        // no row will write this dot
        }
      }
      TILE_BARRIER();                                   // tasks grouped by row, grad_out rows staged
      TT_MARK(3);

      // ---------------- rows: one group of LPR lanes per tile row ----------------
      for (int pass = 0; pass < passes; ++pass) {
        const int chan = (pass * LPR + cl) * VEC;
        const bool chan_ok = chan < C;
        const uint32_t chan_off = chan_ok ? (uint32_t)(chan * sizeof(T)) : kNoChan;
        float v_next[VEC];
        {
          const int r = group;
          const int y = y0 + r / TW, x = x0 + r % TW;
          const bool ld_ok = r < R && offs[min(r, R - 1) + 1] > offs[min(r, R - 1)] && in_map(y, x, H, W) && !DFA3D_DIAG(diag, 8);
          RowVec<T, float, VEC>::ld(value_r, (ld_ok ? (uint32_t)(((start + y * W + x) * M + m) * C * (int)sizeof(T)) : kNoRow) + chan_off, v_next);
        }
        for (int r0 = 0; r0 < R; r0 += kGroups) {        // uniform over the workgroup
          const int r = r0 + group;
          const bool row_ok = r < R;
          const int beg = row_ok ? offs[r] : 0;
          const int n_r = row_ok ? offs[r + 1] - beg : 0;
          int n_max = n_r;                               // longest list among this wavefront's groups
#pragma unroll
          for (int off = LPR; off < kWave; off <<= 1) n_max = max(n_max, __shfl_xor(n_max, off, kWave));
          const int y = y0 + r / TW, x = x0 + r % TW;
          const bool pix_ok = row_ok && n_r > 0 && in_map(y, x, H, W);
          float v[VEC], acc[VEC];
#pragma unroll
          for (int i = 0; i < VEC; ++i) { v[i] = v_next[i]; acc[i] = 0; }
          {                                              // value row of this group's next round
            const int rn = r + kGroups;
            const int yn = y0 + rn / TW, xn = x0 + rn % TW;
            const bool ld_ok = rn < R && offs[min(rn, R - 1) + 1] > offs[min(rn, R - 1)] && in_map(yn, xn, H, W) && !DFA3D_DIAG(diag, 8);
            RowVec<T, float, VEC>::ld(value_r, (ld_ok ? (uint32_t)(((start + yn * W + xn) * M + m) * C * (int)sizeof(T)) : kNoRow) + chan_off, v_next);
          }
          if (DFA3D_DIAG(diag, 16)) n_max = 0;                      // cost of the task loop
          if (n_max == 0) continue;                      // wave-uniform
          // tasks in flight per group: registers decide (measured: 4 with four channels per lane, 1 with eight;
          // one more costs 1 % .. 10 % of the kernel's time)
          constexpr int UT = VEC >= 8 ? 1 : 4;
          const RowTask *row_tasks = tasks + beg;
          const int last_task = PP * 4 - 1 - beg;         // reads past a short list stay inside the array
          const float *g_lane = gstage + (chan_ok ? chan : 0);
          const int dummy = PP * 4 + lane;                // private scrap word for lanes with nothing to report
          for (int t0 = 0; t0 < n_max; t0 += UT) {
            RowTask tk[UT];
            float gg[UT][VEC], part[UT];
            // A group whose list is shorter than the wavefront's longest one idles on a task of weight zero that
            // points at the row of zeros: nothing another point staged (a non-finite gradient, say) and no
            // stale word is ever multiplied in.
#pragma unroll
            for (int j = 0; j < UT; ++j) {
              const RowTask t = row_tasks[min(t0 + j, last_task)];
              const bool on = t0 + j < n_r;
              tk[j].w = on ? t.w : 0.f;
              tk[j].who = on ? t.who : (uint32_t)(PP * 4);
            }
#pragma unroll
            for (int j = 0; j < UT; ++j) lds_ld<VEC>(g_lane + (tk[j].who >> 2) * C, gg[j]);
#pragma unroll
            for (int j = 0; j < UT; ++j) {
              part[j] = 0;
#pragma unroll
              for (int i = 0; i < VEC; ++i) part[j] += v[i] * gg[j][i];
            }
#pragma unroll
            for (int j = 0; j < UT; ++j) part[j] = row_sum_f<LPR>(part[j]);
#pragma unroll
            for (int j = 0; j < UT; ++j) {
#pragma unroll
              for (int i = 0; i < VEC; ++i) acc[i] += tk[j].w * gg[j][i];
              const int di = cl == 0 ? (int)tk[j].who : dummy;     // an idle task's dot lands in the scrap words
              if (pass == 0) dots[di] = part[j];          // uniform branch
              else dots[di] += part[j];
            }
          }
          if (pix_ok && chan_ok && !DFA3D_DIAG(diag, 1)) {
            float *dst = gv + r * C + chan;
            float cur[VEC];
            LdsVec<VEC>::ld(dst, cur);
#pragma unroll
            for (int i = 0; i < VEC; ++i) cur[i] += acc[i];
            LdsVec<VEC>::st(dst, cur);
          }
        }
      }
      TILE_BARRIER();                                   // dots complete
      TT_MARK(4);
    }
    TILE_BARRIER();                                     // the tile is complete

    // ---------------- flush the tile (and leave it zeroed for the next item) ----------------
    const bool gv16 = (grad16 & 1) != 0, gd16 = (grad16 & 2) != 0;          // uniform
    const int mg = Mg == 1 ? 0 : m;
    char *gvalue_b = static_cast<char *>(grad_value) + (size_t)b * S * M * C * (gv16 ? 2 : 4);
    char *gdist_b = FUSED ? static_cast<char *>(grad_dist) + (size_t)b * S * Mg * D * (gd16 ? 2 : 4) : nullptr;
    const rsrc_t gvalue_r = make_rsrc(gvalue_b, (size_t)S * M * C * sizeof(float));
    const rsrc_t gdist_r = make_rsrc(gdist_b, FUSED ? (size_t)S * Mg * D * sizeof(float) : 0);
    // Rows 1..TY-1 x 1..TX-1 of the tile belong to no neighbour's halo; when this item holds all the
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
    if (((C | D) & 3) == 0) {
      // four floats per lane: whole 128-byte lines leave each row group at once
      const int c4n = C >> 2, d4n = D >> 2;
      for (int i = tid; i < R * c4n; i += n_thr) {
        const int r = i / c4n, c = (i - r * c4n) << 2;
        float4 val = *reinterpret_cast<float4 *>(gv + r * C + c);
        const bool nz = val.x != 0 || val.y != 0 || val.z != 0 || val.w != 0;
        if (nz) *reinterpret_cast<float4 *>(gv + r * C + c) = make_float4(0, 0, 0, 0);
        const int ry = r / TW, rx = r - ry * TW;
        const int y = y0 + ry, x = x0 + rx;
        if (in_map(y, x, H, W) && !DFA3D_DIAG(diag, 4)) {
          const uint32_t e = (uint32_t)(((start + y * W + x) * M + m) * C + c);
          const bool store = sole && ry >= 1 && ry < TY && rx >= 1 && rx < TX;
          if (store || nz) put4(gvalue_b, gvalue_r, gv16, e, val, store, true);
        }
      }
      for (int i = tid; i < R * d4n; i += n_thr) {
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
    } else {                                                    // float gradients only (the launcher sees to it)
      float *gvalue_f = reinterpret_cast<float *>(gvalue_b), *gdist_f = reinterpret_cast<float *>(gdist_b);
      for (int i = tid; i < R * C; i += n_thr) {
        const float val = gv[i];
        if (val != 0) {
          gv[i] = 0;
          const int r = i / C, c = i - r * C;
          const int ry = r / TW, rx = r % TW;
          const int y = y0 + ry, x = x0 + rx;
          if (in_map(y, x, H, W) && !DFA3D_DIAG(diag, 4))
            scatter_add(gvalue_r, gvalue_f, (uint32_t)((((start + y * W + x) * M + m) * C + c) * 4), val);
        }
      }
      for (int i = tid; i < R * D; i += n_thr) {
        const float val = gd[i];
        if (val != 0) {
          gd[i] = 0;
          const int r = i / D, d = i - r * D;
          const int ry = r / TW, rx = r % TW;
          const int y = y0 + ry, x = x0 + rx;
          if (in_map(y, x, H, W) && !DFA3D_DIAG(diag, 4))
            scatter_add(gdist_r, gdist_f, (uint32_t)((((start + y * W + x) * Mg + mg) * D + d) * 4), val);
        }
      }
    }
    TT_MARK(6);
  }
  TT_MARK(7);
  TT_FLUSH();
}

// ---------------------------------------------------------------------------------------
// Stage-1 backward alone on the same bins: the gradient with respect to the four depth scores of
// each point is given; grad_dist is accumulated in an LDS tile, the z gradient written per point.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void tile_depth_backward_kernel(
    BinWorkspace ws, const T *__restrict__ dist, const T *__restrict__ grad_score, float *__restrict__ grad_dist,
    float *__restrict__ grad_loc3, int B, int S, int M, int D, int L, int Q, int P) {
  extern __shared__ __align__(16) float smem[];
  __shared__ int4 s_item;
  const BinPlan &p = *ws.plan;
  const int nb = p.bins_per_bm;
  if (nb == 0) return;
  const int TY = p.ty, TX = p.tx, TW = TX + 1, R = (TY + 1) * TW;
  const int tid = threadIdx.x, n_thr = blockDim.x;
  float *gd = smem;
  // 16-bit ticket counters, one per tile address, behind the tile (see the fused kernel's phase C: integer
  // LDS atomics are more than twenty times faster than floating-point ones).  Zero between rounds: whoever
  // takes the first ticket of an address resets it after use.
  uint32_t *tickets = reinterpret_cast<uint32_t *>(smem + ((R * D + 3) & ~3));
  for (int i = tid; i < R * D; i += n_thr) gd[i] = 0;
  for (int i = tid; i < (R * D + 1) / 2; i += n_thr) tickets[i] = 0;
  ItemFetch fetch;
  if (tid == 0) fetch.start(ws, p, blockIdx.x % kClasses);
  for (;;) {
    TILE_BARRIER();
    if (tid == 0) fetch.advance(ws, p, blockIdx.x % kClasses, &s_item);
    TILE_BARRIER();
    const int4 item = s_item;
    const int bin = item.x, seg = item.y, n_item = item.z;
    if (bin < 0) break;                                   // queues drained: every wave leaves
    const int bm = bin / nb, local = bin - bm * nb;
    int b, m;
    slot_decode(bm, B, M, b, m);
    int l = 0;
    while (l + 1 < L && local >= p.level_base[l + 1]) ++l;
    const int tile = local - p.level_base[l];
    const int H = p.H[l], W = p.W[l], Dd = p.Dd[l], start = p.start[l];
    const int y0 = (tile / p.tiles_x[l]) * TY - 1, x0 = (tile % p.tiles_x[l]) * TX - 1;      // pixel of the tile's row 0
    const rsrc_t dist_r = make_rsrc(dist + (size_t)b * S * M * D, (size_t)S * M * D * sizeof(T));

    // n_thr points per round (fewer than 2^16 tickets per address and round)
    for (int base = 0; base < n_item; base += n_thr) {       // uniform over the workgroup
      const int i = base + tid;
      int at[4] = {-1, -1, -1, -1};                          // tile address of each corner's UPPER tap (bin d0 + 1 >= 0)
      float gk[4] = {0, 0, 0, 0};
      unsigned first_mask = 0;
      DepthTap<float> tap;
      tap.inside = tap.lo_ok = tap.hi_ok = false; tap.d0 = 0; tap.ld = tap.hd = 0;
      if (i < n_item) {
        const size_t gp = ws.entries[seg + i];
        const float4 rec = ws.recs[seg + i];
        const Point2D<float> g = locate_2d<float>(rec.x, rec.y, H, W, start);
        tap = locate_depth<float>(rec.z, Dd);
        float sc[4], lo[4], hi[4];
        corner_scores<T, float, true>(dist_r, g.key, tap, m, M, D, sc, lo, hi);
        const T *gi = grad_score + gp * 4;
        float gz = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (g.key[k] >= 0 && tap.inside) {
            gk[k] = Elem<T>::ld(gi + k);
            const int ry = g.h0 + (k >= 2 ? 1 : 0) - y0, rx = g.w0 + ((k == 1 || k == 2) ? 1 : 0) - x0;
            if (ry >= 0 && ry <= TY && rx >= 0 && rx <= TX && gk[k] != 0) {
              at[k] = (ry * TW + rx) * D + tap.d0 + 1;
              if (tap.lo_ok) {
                const int sh = 16 * ((at[k] - 1) & 1);
                if (((atomicAdd(&tickets[(at[k] - 1) >> 1], 1u << sh) >> sh) & 0xFFFFu) == 0) first_mask |= 1u << (2 * k);
              }
              if (tap.hi_ok) {
                const int sh = 16 * (at[k] & 1);
                if (((atomicAdd(&tickets[at[k] >> 1], 1u << sh) >> sh) & 0xFFFFu) == 0) first_mask |= 2u << (2 * k);
              }
            }
            gz += gk[k] * (hi[k] - lo[k]);
          }
        }
        float *gl = grad_loc3 + gp * 3;
        gl[0] = 0; gl[1] = 0; gl[2] = gz * (float)Dd;
      }
      TILE_BARRIER();                                     // every ticket of the round taken
      uint16_t *ticket16 = reinterpret_cast<uint16_t *>(tickets);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (at[k] >= 0) {
          if (first_mask & (1u << (2 * k))) { gd[at[k] - 1] += tap.hd * gk[k]; ticket16[at[k] - 1] = 0; }
          if (first_mask & (2u << (2 * k))) { gd[at[k]] += tap.ld * gk[k]; ticket16[at[k]] = 0; }
        }
      }
      TILE_BARRIER();                                     // plain updates done before the atomic ones start
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (at[k] >= 0) {
          if (tap.lo_ok && !(first_mask & (1u << (2 * k)))) atomicAdd(gd + at[k] - 1, tap.hd * gk[k]);
          if (tap.hi_ok && !(first_mask & (2u << (2 * k)))) atomicAdd(gd + at[k], tap.ld * gk[k]);
        }
      }
    }
    TILE_BARRIER();
    float *gdist_b = grad_dist + (size_t)b * S * M * D;
    const rsrc_t gdist_r = make_rsrc(gdist_b, (size_t)S * M * D * sizeof(float));
    for (int i = tid; i < R * D; i += n_thr) {
      const float val = gd[i];
      if (val != 0) {
        gd[i] = 0;
        const int r = i / D, d = i - r * D;
        const int y = y0 + r / TW, x = x0 + r % TW;
        if (in_map(y, x, H, W)) scatter_add(gdist_r, gdist_b, (uint32_t)((((start + y * W + x) * M + m) * D + d) * 4), val);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
static int max_bins_per_bm(int S, int L, int ty, int tx) {
  // tiles of a level = ((H + ty) / ty) ((W + tx) / tx) <= (H/ty + 1) (W/tx + 1) <= HW/(ty tx) + H/ty + W/tx + 1
  // and H + W <= HW + 1
  const int e = ty < tx ? ty : tx;
  const long long v = (long long)S / (ty * tx) + ((long long)S + L) / e + 2LL * L + 1;
  return (int)v;
}

constexpr int kMinChunk = 64;        // smallest accepted points-per-item
// Points of a bin per work item.  A bin that fits one item is flushed with stores instead of atomic adds, so
// large items pay; the queues are served from their ends so that the heavy bins of the coarse levels do not
// come last.  Measured at the BEVFormer-base shape: 1024 -> 2.01 ms, 2048 -> 1.87, 4096 -> 1.83, 8192 -> 1.92.
constexpr int kDefaultChunk = 4096;
// only the fused entry point sets dist_heads
static bool shared_dist(const BwdArgs &a) { return a.dist_heads == 1 && a.M > 1; }

__global__ __launch_bounds__(256) void fill_zero_kernel(float4 *__restrict__ dst, size_t n4) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256)
    dst[i] = make_float4(0, 0, 0, 0);
}
__global__ __launch_bounds__(64) void fill_zero_words_kernel(uint32_t *__restrict__ dst, size_t n) {
  for (size_t i = threadIdx.x; i < n; i += 64) dst[i] = 0;
}

hipError_t launch_zero_fill(void *dst, size_t bytes, hipStream_t stream) {
  if (dst == nullptr || (bytes & 3) != 0 || ((uintptr_t)dst & 3) != 0) return hipErrorInvalidValue;
  char *p = static_cast<char *>(dst);
  const size_t head = ((uintptr_t)p & 15) ? 16 - ((uintptr_t)p & 15) : 0;        // bytes before the first 16-byte boundary
  const size_t lead = head < bytes ? head : bytes, body = (bytes - lead) & ~(size_t)15, tail = bytes - lead - body;
  if (lead) hipLaunchKernelGGL(fill_zero_words_kernel, dim3(1), dim3(64), 0, stream, reinterpret_cast<uint32_t *>(p), lead / 4);
  if (body) hipLaunchKernelGGL(fill_zero_kernel, dim3(2048), dim3(256), 0, stream, reinterpret_cast<float4 *>(p + lead), body / 16);
  if (tail) hipLaunchKernelGGL(fill_zero_words_kernel, dim3(1), dim3(64), 0, stream, reinterpret_cast<uint32_t *>(p + lead + body), tail / 4);
  return hipGetLastError();
}

// dst[r, :] = sum over heads m of src[r, m, :], rows of D floats, heads in order; dst is float, or bfloat16
// when dst16 is set (then D is a multiple of 4)
__global__ __launch_bounds__(256) void head_sum_kernel(const float *__restrict__ src, void *__restrict__ dst,
                                                       size_t rows, int M, int D, int dst16) {
  if ((D & 3) == 0) {
    const int d4 = D >> 2;
    const size_t n = rows * d4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
      const size_t r = i / d4;
      const int d = (int)(i - r * d4) << 2;
      float4 acc = make_float4(0, 0, 0, 0);
      for (int m = 0; m < M; ++m) {
        const float4 t = *reinterpret_cast<const float4 *>(src + (r * M + m) * D + d);
        acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
      }
      if (dst16)
        *reinterpret_cast<uint2 *>(static_cast<char *>(dst) + (r * D + d) * 2) =
            make_uint2(pack_bf16x2(acc.x, acc.y), pack_bf16x2(acc.z, acc.w));
      else
        *reinterpret_cast<float4 *>(static_cast<float *>(dst) + r * D + d) = acc;
    }
  } else {
    const size_t n = rows * D;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
      const size_t r = i / D;
      const int d = (int)(i - r * D);
      float acc = 0;
      for (int m = 0; m < M; ++m) acc += src[(r * M + m) * D + d];
      static_cast<float *>(dst)[i] = acc;
    }
  }
}
struct BinLayout { size_t plan, queues, counts, cursor, items, geom, entries, recs, gd_heads, total; };
static BinLayout bin_layout(const BwdArgs &a, int ty, int tx) {
  BinLayout o;
  const size_t nbins = (size_t)max_bins_per_bm(a.S, a.L, ty, tx) * slot_count(a.B, a.M);
  const size_t npts = (size_t)a.B * a.Q * a.M * a.L * a.P;
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  o.plan = 0;
  o.queues = up(o.plan + sizeof(BinPlan));
  o.counts = up(o.queues + kQueueInts * sizeof(int));
  o.cursor = up(o.counts + nbins * sizeof(int));
  // work items: at most one partial chunk per bin plus the full chunks
  o.items = up(o.cursor + nbins * sizeof(int));
  o.geom = up(o.items + (nbins + npts / kMinChunk + 1) * sizeof(int4));
  o.entries = up(o.geom + (nbins + npts / kMinChunk + 1) * sizeof(int4));
  o.recs = up(o.entries + npts * sizeof(uint32_t));
  // a distribution shared by the heads: grad_dist per head first (stores, as with a distribution per head),
  // summed over the heads afterwards; eight XCDs adding atomically into one shared tile cost twice as much
  o.gd_heads = up(o.recs + npts * sizeof(float4));
  const size_t per_head = shared_dist(a) ? (size_t)a.B * a.S * a.M * a.D * sizeof(float) : 0;
  o.total = up(o.gd_heads + per_head);
  return o;
}

#ifdef DFA3D_EXPERIMENT
// development builds: where in a workspace the tile kernel's phase clocks live (ten 64-bit counters)
size_t tile_timer_offset() {
  return ((sizeof(BinPlan) + 255) & ~(size_t)255) + (size_t)kClasses * kQueueStride * sizeof(int);
}
#endif

// Launch shape of the tile kernels: tile edge, threads per workgroup, points per pass.
struct TileConfig { int ty, tx, block, pp; size_t lds; bool cells; };      // cells: the cell-owned kernel takes the launch

// kind 0: both stages, 1: stage 2 alone (no depth tile), 2: stage 1 alone (depth tile only)
static size_t tile_lds_bytes(int kind, int ty, int tx, int C, int D, int pp) {
  if (kind == 2) {       // depth tile + 16-bit tickets
    const size_t n = (size_t)(ty + 1) * (tx + 1) * D;
    return ((n + 3) & ~(size_t)3) * 4 + ((n + 1) / 2) * 4;
  }
  return (size_t)tile_lds_layout(ty, tx, C, kind == 1 ? 0 : D, pp).total * 4;
}

// Defaults: 512 threads; the tile and the points per pass (pp) follow from what fits in LDS, in an order of
// preference taken from measurements on rows of 32 .. 256 channels and 64 .. 256 depth bins:
//   * two workgroups per CU (79 KB each) beat one, and one per CU on a 4x8 tile beats tiles under 4x4 pixels by
//     far (256 channels: 3.2 ms against 11.9 ms);
//   * tiles above 8x16 pixels lose (the rows phase needs several rounds); passes of 64 points lose to 128 and 256;
//   * an 8x8 tile at pp 128 beats a 4x8 tile at pp 256 (128 bins: 0.68 against 0.74 ms for 2.56 M points) unless
//     most tiles take several passes (`dense`: the dense BEV workload, 41 points per pixel, 7.0 against 8.9 ms).
static TileConfig pick_tile_config(int kind, int C, int D, int tile_hint, int block_hint, int pass_hint, bool dense,
                                   bool cells_wanted) {
  TileConfig c;
  c.cells = false;
  if (cells_wanted && kind != 2 && (block_hint == 0 || block_hint == 512) && (pass_hint == 0 || pass_hint == 256)) {
    // The cell-owned kernel (rows of 32 channels): the largest tile of at most 64 pixels whose depth tile leaves
    // room for two workgroups per CU, else for one.
    static const int order[][2] = {{8, 8}, {6, 8}, {4, 8}, {4, 4}, {2, 4}, {2, 2}, {1, 1}};
    const int hy = tile_hint / 100, hx = tile_hint % 100;
    // two workgroups per CU: half of the 160 KB less the kernel's static LDS (a depth tile of 112 bins on 8x8 pixels
    // just fits; 128 bins would fit on 8x7 pixels, which is no faster than 6x8 on the dense workload: 5.66 against 5.65 ms)
    for (size_t budget : {cell_kernel_half_cu_lds(), (size_t)150 * 1024}) {
      for (auto &t : order) {
        const int ty = tile_hint > 0 ? hy : t[0], tx = tile_hint > 0 ? hx : t[1];
        const int Dk = kind == 1 ? 0 : D;
        if (cell_kernel_applies(C, Dk, ty, tx, kind == 0) && cell_kernel_lds_bytes(ty, tx, Dk) <= budget) {
          c.cells = true; c.block = 512; c.pp = 256; c.ty = ty; c.tx = tx; c.lds = cell_kernel_lds_bytes(ty, tx, Dk);
          return c;
        }
      }
    }
  }
  c.block = kind == 2 ? 256 : (block_hint == 256 ? 256 : 512);
  const int pp_max = kind == 2 ? c.block : c.block / 2;      // the fused tile kernel wants two halves of pp threads
  auto clamp_pp = [&](int pp) { return pp > pp_max ? pp_max : pp; };
  const size_t two_per_cu = kind == 2 ? 40 * 1024 : 79 * 1024, one_per_cu = 150 * 1024;
  const int hy = tile_hint / 100, hx = tile_hint % 100;
  const bool tile_given = tile_hint > 0 && hy >= 1 && hx >= 1 && hy <= 64 && hx <= 64;
  const bool pass_given = pass_hint == 64 || pass_hint == 128 || pass_hint == 256;
  auto fits = [&](int ty, int tx, int pp, size_t budget) { return tile_lds_bytes(kind, ty, tx, C, D, clamp_pp(pp)) <= budget; };
  auto done = [&](int ty, int tx, int pp) {
    c.ty = ty; c.tx = tx; c.pp = clamp_pp(pp);
    c.lds = tile_lds_bytes(kind, c.ty, c.tx, C, D, c.pp);
    return c;
  };
  struct Pref { int ty, tx, pp; };
  static const Pref sparse_order[] = {{8, 16, 256}, {8, 8, 256}, {8, 8, 128}, {4, 8, 256}, {4, 8, 128}, {4, 4, 256},
                                      {4, 4, 128}, {8, 8, 64}, {4, 8, 64}, {4, 4, 64}};
  static const Pref dense_order[] = {{8, 16, 256}, {8, 8, 256}, {4, 8, 256}, {4, 4, 256}, {8, 8, 128}, {4, 8, 128},
                                     {4, 4, 128}, {8, 8, 64}, {4, 8, 64}, {4, 4, 64}};
  const Pref *order = dense ? dense_order : sparse_order;
  for (size_t budget : {two_per_cu, one_per_cu}) {
    for (int i = 0; i < 10; ++i) {
      const int ty = tile_given ? hy : order[i].ty, tx = tile_given ? hx : order[i].tx;
      const int pp = pass_given ? pass_hint : order[i].pp;
      if (fits(ty, tx, pp, budget)) return done(ty, tx, pp);
    }
  }
  // nothing of at least 4x4 pixels fits: whatever the caller fixed, else the largest small tile with short passes
  const int pp = pass_given ? pass_hint : 64;
  if (tile_given) return done(hy, hx, pp);
  const int small[][2] = {{2, 4}, {2, 2}, {1, 1}};
  for (auto &t : small)
    if (fits(t[0], t[1], pp, one_per_cu)) return done(t[0], t[1], pp);
  return done(1, 1, pp);
}

static int bwd_kind(const BwdArgs &a) { return a.dist != nullptr ? 0 : 1; }
static TileConfig tile_config_of(const BwdArgs &a, int kind) {
  const double per_pixel = (double)a.Q * a.L * a.P / (a.S > 0 ? a.S : 1);      // sampling points per pixel of a (batch, head)
  // a caller that names the channels per lane asks for the row-owned kernel, whose tiling that is
  return pick_tile_config(kind, a.C, a.D, a.tile_hint, a.block_hint, a.pass_hint, per_pixel >= 16.0, a.vec_hint == 0);
}

static size_t workspace_bytes_for(const BwdArgs &a, int kind, int dtype) {
  if (dtype == DFA3D_F64) return 0;
  if ((size_t)a.B * a.Q * a.M * a.L * a.P >= (1ull << 31)) return 0;          // point indices and segment offsets are 32-bit
  if (kind != 2 && (size_t)a.Q * a.M * a.C * 4 >= (size_t)kMaxSliceBytes) return 0;   // grad_out rows are buffer-addressed per batch element
  if (a.grad_bf16 && (kind != 0 || ((a.C | a.D) & 3) != 0)) return 0;          // bfloat16 gradients: whole 8-byte groups
  const TileConfig c = tile_config_of(a, kind);
  if (c.lds > 150 * 1024) return 0;                                            // rows too long for LDS tiles
  return bin_layout(a, c.ty, c.tx).total;
}

// kind as in tile_lds_bytes; `a.dist != nullptr` is not consulted here, so dimension-only queries work
size_t binned_backward_workspace_bytes(const BwdArgs &a, int kind, int dtype) { return workspace_bytes_for(a, kind, dtype); }

// Per-device facts and per-kernel attributes are looked up once and remembered (a launch then costs no
// runtime queries).
static std::mutex g_launch_mutex;
static int g_cu_count[64];                                           // 0 = not asked yet
static std::map<std::pair<const void *, int>, size_t> g_lds_allowed;  // (kernel, device) -> dynamic LDS bytes granted

static int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  return dev;
}

static int tile_grid(size_t lds, int block) {
  const int dev = current_device();
  int cus;
  {
    std::lock_guard<std::mutex> lock(g_launch_mutex);
    if (g_cu_count[dev] == 0) {
      int n = 0;
      if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
      g_cu_count[dev] = n;
    }
    cus = g_cu_count[dev];
  }
  const size_t per_cu = lds > 0 ? (160 * 1024) / lds : 8;
  int wg_per_cu = (int)(per_cu < 1 ? 1 : per_cu > 8 ? 8 : per_cu);
  const int by_waves = 32 / (block / kWave);
  if (wg_per_cu > by_waves) wg_per_cu = by_waves < 1 ? 1 : by_waves;
  return cus * wg_per_cu;
}

static hipError_t allow_lds(const void *fn, size_t lds) {
  if (lds <= 64 * 1024) return hipSuccess;
  const std::pair<const void *, int> key(fn, current_device());
  std::lock_guard<std::mutex> lock(g_launch_mutex);
  auto it = g_lds_allowed.find(key);
  if (it != g_lds_allowed.end() && it->second >= lds) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e == hipSuccess) g_lds_allowed[key] = lds;
  return e;
}
template <typename K> static hipError_t allow_lds(K kern, size_t lds) {
  return allow_lds(reinterpret_cast<const void *>(kern), lds);
}

template <typename T, int VEC, int LPR>
static hipError_t launch_tile_cfg(const BwdArgs &a, const BinWorkspace &ws, const TileConfig &c, float *gd_heads,
                                  hipStream_t stream) {
  // gd_heads != nullptr: the kernel writes grad_dist per head there instead of into a.grad_dist
  const int grid = tile_grid(c.lds, c.block);
  if (a.dist != nullptr) {
    auto kern = tile_backward_kernel<T, VEC, LPR, true>;
    if (hipError_t e = allow_lds(kern, c.lds)) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(c.block), c.lds, stream, ws, (const T *)a.value, (const T *)a.dist,
                       (const T *)nullptr, (const T *)a.grad_out, (const T *)a.grad_score_in, a.grad_value,
                       gd_heads != nullptr ? (void *)gd_heads : a.grad_dist, (float *)a.grad_loc, a.grad_loc_stride, (float *)a.grad_attn,
                       (float *)nullptr, (const float *)a.grad_weight_update, a.dist_heads == 1 ? 1 : a.M,
                       (a.dist_heads == 1 && gd_heads == nullptr) ? 1 : a.M, a.B, a.S, a.M, a.C, a.D, a.L, a.Q, a.P, c.pp,
                       (a.grad_bf16 ? 1 : 0) | ((a.grad_bf16 && gd_heads == nullptr) ? 2 : 0) DFA3D_DIAG_ARG(a));
  } else {
    auto kern = tile_backward_kernel<T, VEC, LPR, false>;
    if (hipError_t e = allow_lds(kern, c.lds)) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(c.block), c.lds, stream, ws, (const T *)a.value, (const T *)nullptr,
                       (const T *)a.score_in, (const T *)a.grad_out, (const T *)nullptr, a.grad_value,
                       (void *)nullptr, (float *)a.grad_loc, a.grad_loc_stride, (float *)a.grad_attn,
                       (float *)a.grad_score_out, (const float *)nullptr, a.M, a.M, a.B, a.S, a.M, a.C, 0, a.L, a.Q,
                       a.P, c.pp, 0 DFA3D_DIAG_ARG(a));
  }
  return hipGetLastError();
}

static hipError_t allow_lds(const void *fn, size_t lds);

template <typename T>
static hipError_t launch_tile_typed(const BwdArgs &a, const BinWorkspace &ws, const TileConfig &c, float *gd_heads,
                                    hipStream_t stream) {
  if (c.cells) {
    const int dtype = sizeof(T) == 4 ? DFA3D_F32 : DFA3D_BF16;
    if (hipError_t e = allow_lds(cell_kernel_symbol(dtype, a.dist != nullptr), c.lds)) return e;
    return launch_cell_kernel(a, dtype, ws, c.lds, tile_grid(c.lds, c.block), gd_heads, stream);
  }
  // Eight channels per lane when the tile has more rows than four-channel row groups (a 9x9 tile against 64
  // groups of 8 lanes): 128 groups of 4 lanes then cover it in one round with fewer instructions per corner
  // task.  Smaller tiles would leave most of those groups idle.
  const int groups4 = (c.block / 64) * 8;
  if (((a.vec_hint == 0 && (c.ty + 1) * (c.tx + 1) > groups4) || a.vec_hint == 8) && sizeof(T) <= 4) {
    if (a.C == 32) return launch_tile_cfg<T, 8, 4>(a, ws, c, gd_heads, stream);
    if (a.C == 64) return launch_tile_cfg<T, 8, 8>(a, ws, c, gd_heads, stream);
  }
  const RowTiling rt = pick_row_tiling(a.C, (int)sizeof(T), a.vec_hint);
#define DFA3D_CASE(V, R) \
  if (rt.vec == V && rt.lpr == R) return launch_tile_cfg<T, V, R>(a, ws, c, gd_heads, stream);
  DFA3D_ROW_TILINGS(DFA3D_CASE)
#undef DFA3D_CASE
  return hipErrorInvalidValue;
}

static BinWorkspace carve_workspace(void *workspace, const BinLayout &lay) {
  char *base = static_cast<char *>(workspace);
  BinWorkspace ws;
  ws.plan = reinterpret_cast<BinPlan *>(base + lay.plan);
  ws.queues = reinterpret_cast<int *>(base + lay.queues);
  ws.counts = reinterpret_cast<int *>(base + lay.counts);
  ws.cursor = reinterpret_cast<int *>(base + lay.cursor);
  ws.items = reinterpret_cast<int4 *>(base + lay.items);
  ws.geom = reinterpret_cast<int4 *>(base + lay.geom);
  ws.entries = reinterpret_cast<uint32_t *>(base + lay.entries);
  ws.recs = reinterpret_cast<float4 *>(base + lay.recs);
  return ws;
}

// plan, count, scan, fill.  `a` supplies dimensions, shapes, locations and the per-point gradient
// buffers that receive zeros for points the operator skips.
static hipError_t run_binning(const BwdArgs &a, const BinWorkspace &ws, int ty, int tx, float *gd_heads, hipStream_t stream) {
  const int mb = max_bins_per_bm(a.S, a.L, ty, tx);
  hipLaunchKernelGGL(plan_and_clear_kernel, dim3(64), dim3(256), 0, stream, ws, a.shapes, a.shape_stride, a.level_start,
                     a.L, a.S, (a.dist != nullptr || a.C == 0) ? a.D : 0, a.B, a.M, ty, tx, a.chunk_hint > 0 ? a.chunk_hint : kDefaultChunk, mb);
  const int q_blocks = (a.Q + kBinQueries - 1) / kBinQueries;
  const long long blocks = (long long)a.B * a.M * q_blocks;
  if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  const int hist_cap = mb < kHistCap ? mb : kHistCap;
  const unsigned grid = blocks < 2048 ? (unsigned)blocks : 2048u;
  hipLaunchKernelGGL(bin_points_kernel<0>, dim3(grid), dim3(256), (size_t)hist_cap * 4, stream, ws,
                     (const float *)a.loc, a.loc_stride, (const float *)a.attn, (float *)a.grad_loc, a.grad_loc_stride,
                     (float *)a.grad_attn, (float *)a.grad_score_out, a.B, a.M, a.L, a.Q, a.P, q_blocks, (int)blocks, hist_cap DFA3D_DIAG_ARG(a));
  const int LP = a.L * a.P;
  const int nq_block = LP <= kStage ? kStage / LP : 1;
  const int q_blocks2 = (a.Q + nq_block - 1) / nq_block;
  const long long blocks2 = (long long)a.B * a.M * q_blocks2;
  if (blocks2 > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  if (LP <= kStage)                         // steps aside if there turn out to be too many bins, as the one above does if not
    hipLaunchKernelGGL(bin_count_kernel, dim3((unsigned)blocks2), dim3(kFillThreads), 0, stream, ws, (const float *)a.loc,
                       a.loc_stride, a.B, a.M, a.L, a.Q, a.P, nq_block, q_blocks2);
  // What further blocks of the scan's launch clear meanwhile: for a caller that did not zero them (options.clear),
  // the rows of grad_value / grad_dist that the tile kernel adds to rather than stores; and always, for a
  // distribution shared by the heads, those rows of the per-head grad_dist in the workspace (the head sum then
  // writes all of the caller's grad_dist).
  ClearArgs ca{};
  unsigned clear_blocks = 0;
  if (a.clear_grads || gd_heads != nullptr) {            // launch_backward_binned has checked that this applies
    const int ge = a.grad_bf16 ? 2 : 4;
    ca.grad_value = a.clear_grads ? static_cast<char *>(a.grad_value) : nullptr;
    ca.value_row_bytes = a.C * ge;
    if (gd_heads != nullptr) { ca.grad_dist = reinterpret_cast<char *>(gd_heads); ca.dist_row_bytes = a.D * 4; }
    else if (a.dist != nullptr) { ca.grad_dist = static_cast<char *>(a.grad_dist); ca.dist_row_bytes = a.D * ge; }
    ca.B = a.B; ca.S = a.S; ca.M = a.M; ca.L = a.L;
    ca.stores = ((a.C | (a.dist != nullptr ? a.D : 0)) & 3) == 0 ? 1 : 0;        // the tile kernel's own condition
    const size_t rows = (size_t)a.B * a.S * a.M;
    clear_blocks = (unsigned)((rows + 1023) / 1024 < 4096 ? (rows + 1023) / 1024 : 4096);
  }
  // scanning blocks for the most bins there can be (the plan kernel knows how many there are), 64 at most
  const size_t max_bins = (size_t)mb * slot_count(a.B, a.M);
  const unsigned scan_blocks = (max_bins + 1023) / 1024 < 64 ? (unsigned)((max_bins + 1023) / 1024) : 64u;
  hipLaunchKernelGGL(bin_scan_kernel, dim3(scan_blocks + clear_blocks), dim3(1024), 0, stream, ws, ca, (int)scan_blocks);
  if (LP <= kStage) {
    if (hipError_t e = allow_lds(bin_fill_sorted_kernel, kSortedFillLds)) return e;
    hipLaunchKernelGGL(bin_fill_sorted_kernel, dim3((unsigned)blocks2), dim3(kFillThreads), kSortedFillLds, stream, ws, (const float *)a.loc,
                       a.loc_stride, (const float *)a.attn, (float *)a.grad_loc, a.grad_loc_stride, (float *)a.grad_attn,
                       (float *)a.grad_score_out, a.B, a.M, a.L, a.Q, a.P, q_blocks2);
  }
  hipLaunchKernelGGL(bin_points_kernel<1>, dim3(grid), dim3(256), (size_t)hist_cap * 8, stream, ws,
                     (const float *)a.loc, a.loc_stride, (const float *)a.attn, (float *)a.grad_loc, a.grad_loc_stride,
                     (float *)a.grad_attn, (float *)a.grad_score_out, a.B, a.M, a.L, a.Q, a.P, q_blocks, (int)blocks, hist_cap DFA3D_DIAG_ARG(a));
  return hipGetLastError();
}

// Binned backward of both stages (a.dist given) or of stage 2 alone (a.dist == nullptr, a.score_in /
// a.grad_score_out given).  Returns hipErrorNotSupported when the binned path does not apply and the
// caller should use launch_backward instead.
hipError_t launch_backward_binned(const BwdArgs &a, int dtype, void *workspace, size_t workspace_bytes,
                                  hipStream_t stream) {
  const int kind = bwd_kind(a);
  if (dtype == DFA3D_F64) return hipErrorNotSupported;
  if (kind == 0 && (a.loc_stride != 3 || a.grad_loc_stride != 3 || a.shape_stride != 3)) return hipErrorNotSupported;
  const size_t need = workspace_bytes_for(a, kind, dtype);
  if (need == 0 || workspace == nullptr || workspace_bytes < need || ((uintptr_t)workspace & 255) != 0)
    return hipErrorNotSupported;
  if (a.clear_grads) {
    if (kind == 2) return hipErrorInvalidValue;            // the depth-only tile kernel stores nothing
    // clear_unstored writes 16-byte groups where a row is made of them: buffers on 16-byte boundaries,
    // or the direct kernels (which clear everything) take the call
    if ((((uintptr_t)a.grad_value | (uintptr_t)a.grad_dist) & 15) != 0) return hipErrorNotSupported;
  }
  const TileConfig cfg = tile_config_of(a, kind);
  const BinLayout lay = bin_layout(a, cfg.ty, cfg.tx);
  const BinWorkspace ws = carve_workspace(workspace, lay);
  float *gd_heads = shared_dist(a) ? reinterpret_cast<float *>(static_cast<char *>(workspace) + lay.gd_heads) : nullptr;
#ifdef DFA3D_EXPERIMENT
  const int stage = a.stage;                     // development builds: 1 = binning launches only, 2 = tile kernel only
#else
  constexpr int stage = 0;
#endif
  if (stage == 0 || stage == 1) {
    if (hipError_t e = run_binning(a, ws, cfg.ty, cfg.tx, gd_heads, stream)) return e;
  }
  if (a.event_binned != nullptr) {
    if (hipError_t e = hipEventRecord((hipEvent_t)a.event_binned, stream)) return e;
  }
  if (stage == 1) return hipSuccess;
  if (gd_heads != nullptr && stage == 2)
    hipLaunchKernelGGL(fill_zero_kernel, dim3(2048), dim3(256), 0, stream, reinterpret_cast<float4 *>(gd_heads),
                       ((size_t)a.B * a.S * a.M * a.D + 3) / 4);
  if (a.grad_bf16 && dtype != DFA3D_BF16) return hipErrorInvalidValue;
  const hipError_t e = dtype == DFA3D_F32 ? launch_tile_typed<float>(a, ws, cfg, gd_heads, stream)
                                          : launch_tile_typed<__hip_bfloat16>(a, ws, cfg, gd_heads, stream);
  if (e != hipSuccess || gd_heads == nullptr) return e;
  hipLaunchKernelGGL(head_sum_kernel, dim3(2048), dim3(256), 0, stream, gd_heads, a.grad_dist,
                     (size_t)a.B * a.S, a.M, a.D, a.grad_bf16 ? 1 : 0);
  return hipGetLastError();
}

// Binned backward of stage 1 alone.
size_t binned_depth_score_backward_workspace_bytes(const DepthScoreBwdArgs &d, int dtype, int tile_hint) {
  BwdArgs a{};
  a.B = d.B; a.S = d.S; a.M = d.M; a.C = 0; a.D = d.D; a.L = d.L; a.Q = d.Q; a.P = d.P; a.tile_hint = tile_hint;
  return workspace_bytes_for(a, 2, dtype);
}

hipError_t launch_depth_score_backward_binned(const DepthScoreBwdArgs &d, int dtype, void *workspace,
                                              size_t workspace_bytes, int tile_hint, int chunk_hint,
                                              void *event_binned, hipStream_t stream) {
  if (dtype == DFA3D_F64) return hipErrorNotSupported;
  BwdArgs a{};
  a.B = d.B; a.S = d.S; a.M = d.M; a.C = 0; a.D = d.D; a.L = d.L; a.Q = d.Q; a.P = d.P;
  a.shapes = d.shapes3; a.shape_stride = 3; a.level_start = d.level_start; a.loc = d.loc3; a.loc_stride = 3;
  a.attn = nullptr; a.grad_loc = d.grad_loc3; a.grad_loc_stride = 3; a.grad_attn = nullptr; a.grad_score_out = nullptr;
  a.tile_hint = tile_hint; a.chunk_hint = chunk_hint;
  const size_t need = workspace_bytes_for(a, 2, dtype);
  if (need == 0 || workspace == nullptr || workspace_bytes < need || ((uintptr_t)workspace & 255) != 0)
    return hipErrorNotSupported;
  const TileConfig cfg = tile_config_of(a, 2);
  const BinWorkspace ws = carve_workspace(workspace, bin_layout(a, cfg.ty, cfg.tx));
  if (hipError_t e = run_binning(a, ws, cfg.ty, cfg.tx, nullptr, stream)) return e;
  if (event_binned != nullptr) {
    if (hipError_t e = hipEventRecord((hipEvent_t)event_binned, stream)) return e;
  }
  const int grid = tile_grid(cfg.lds, cfg.block);
  if (hipError_t e = dtype == DFA3D_F32 ? allow_lds(tile_depth_backward_kernel<float>, cfg.lds)
                                        : allow_lds(tile_depth_backward_kernel<__hip_bfloat16>, cfg.lds))
    return e;
  if (dtype == DFA3D_F32) {
    hipLaunchKernelGGL(tile_depth_backward_kernel<float>, dim3(grid), dim3(cfg.block), cfg.lds, stream, ws,
                       (const float *)d.dist, (const float *)d.grad_score, (float *)d.grad_dist, (float *)d.grad_loc3,
                       d.B, d.S, d.M, d.D, d.L, d.Q, d.P);
  } else {
    hipLaunchKernelGGL(tile_depth_backward_kernel<__hip_bfloat16>, dim3(grid), dim3(cfg.block), cfg.lds, stream, ws,
                       (const __hip_bfloat16 *)d.dist, (const __hip_bfloat16 *)d.grad_score, (float *)d.grad_dist,
                       (float *)d.grad_loc3, d.B, d.S, d.M, d.D, d.L, d.Q, d.P);
  }
  return hipGetLastError();
}

}  // namespace dfa3d
