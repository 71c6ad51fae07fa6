// Forward kernels of the DFA3D operator for gfx950.
//
//   fwd_attention_kernel<..., FUSED=true>   depth-score sampling + weighted attention in one pass
//                                           (the reference runs two kernels and two slice copies:
//                                           multi_scale_3ddeformable_attn_function.py:279-303)
//   fwd_attention_kernel<..., FUSED=false>  stage 2 alone, scores given
//                                           (wms_deform_attn_cuda_kernel.cuh:240-303)
//   depth_score_kernel                      stage 1 alone
//                                           (ms_depth_score_sample_cuda_kernel.cuh:94-148)
#include "dfa3d_device.h"
#include "dfa3d_launch.h"

namespace dfa3d {

// Phase B of the forward pass: acc += sum over tasks [t_begin, t_end) of w * row, the wavefront
// covering 64/LPR rows per step with LPR lanes of VEC channels per row.  `chan_off` is the lane's
// byte offset inside a row (kNoChan for a lane beyond the last channel).
template <typename T, typename A, int VEC, int LPR>
__device__ __forceinline__ void gather_rows(rsrc_t value_r, const Task<A> *tasks, int t_begin, int t_end, int row_slot,
                                            uint32_t chan_off, A (&acc)[VEC]) {
  constexpr int RPI = kWave / LPR;
  constexpr int U = 8;
  int t0 = t_begin;
  for (; t0 + RPI * U <= t_end; t0 += RPI * U) {
    Task<A> e[U];
#pragma unroll
    for (int j = 0; j < U; ++j) e[j] = tasks[t0 + j * RPI + row_slot];
    A v[U][VEC];
#pragma unroll
    for (int j = 0; j < U; ++j) RowVec<T, A, VEC>::ld(value_r, e[j].off + chan_off, v[j]);
#pragma unroll
    for (int j = 0; j < U; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] += e[j].w * v[j][i];
    }
  }
  for (; t0 < t_end; t0 += RPI) {
    const int t = t0 + row_slot;
    const Task<A> e = tasks[min(t, kWave * 4 - 1)];
    const bool in = t < t_end;
    A v[VEC];
    RowVec<T, A, VEC>::ld(value_r, (in ? e.off : kNoRow) + chan_off, v);
    const A w = in ? e.w : (A)0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] += w * v[i];
  }
}

// ---------------------------------------------------------------------------------------
// Fused / stage-2 forward.
// grid: M * B * ceil(Q / queries_per_block) blocks; block id % M = head, so that with the
// round-robin placement of workgroups on the 8 XCDs each XCD's L2 serves one head (M = 8).
// ---------------------------------------------------------------------------------------
template <typename T, typename A, int VEC, int LPR, bool FUSED>
__global__ __launch_bounds__(kBlock) void fwd_attention_kernel(
    const T *__restrict__ value, const T *__restrict__ dist, const int64_t *__restrict__ shapes, int shape_stride,
    const int64_t *__restrict__ level_start, const A *__restrict__ loc, int loc_stride,
    const A *__restrict__ attn, const T *__restrict__ score_in, T *__restrict__ out, T *__restrict__ score_out,
    A *__restrict__ weight_update, const T *__restrict__ packed_arg, int Md, int B, int S, int M, int C, int D, int L,
    int Q, int P, int iters, int q_blocks) {
  // packed: the head-shared distribution as dfa3d_pack_dist lays it out (D >= 2), or nullptr
  __shared__ LevelTable tab;
  __shared__ Task<A> s_tasks[kWavesPerBlock][kWave * 4];

  load_level_table(tab, shapes, shape_stride, level_start, L, S, FUSED ? D : 0);
  if (FUSED && packed_arg != nullptr) load_cell_starts(tab, L);      // uniform
  // The packed table was sized on the host for levels that share no keys (at most 2 S + 2 L cells).  A level
  // table whose levels overlap can ask for more: then the table is not used (nor was it written) and the taps
  // come from dist itself.
  const T *packed = (FUSED && packed_arg != nullptr && tab.cell[L] <= packed_cell_capacity(S, L)) ? packed_arg : nullptr;

  const WaveShape ws = wave_shape(L, P);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int m = blockIdx.x % M;
  const int rest = blockIdx.x / M;
  const int qb = rest % q_blocks, b = rest / q_blocks;
  const int row_slot = lane / LPR, cl = lane % LPR;
  const int passes = (C + VEC * LPR - 1) / (VEC * LPR);
  Task<A> *tasks = s_tasks[wave];

  const rsrc_t value_r = make_rsrc(value + (size_t)b * S * M * C, (size_t)S * M * C * sizeof(T));
  const rsrc_t dist_r = make_rsrc(FUSED ? dist + (size_t)b * S * Md * D : nullptr,
                                  FUSED ? (size_t)S * Md * D * sizeof(T) : 0);
  const int md = Md == 1 ? 0 : m;                                    // head whose distribution this head reads
  const size_t packed_slice = (FUSED && packed != nullptr) ? (size_t)tab.cell[L] * D * 4 : 0;   // elements per batch element
  const rsrc_t packed_r = make_rsrc(packed_slice ? packed + (size_t)b * packed_slice : nullptr, packed_slice * sizeof(T));
  const int q_per_iter = kWavesPerBlock * ws.upw;

  for (int it = 0; it < iters; ++it) {
    const int q0 = (qb * iters + it) * q_per_iter + wave * ws.upw;   // first query of this wave's group
    if (q0 >= Q) break;                                              // wave-uniform
    A wu_unit = 0;                                                   // upw == 1: the unit's sum over its chunks
    for (int pass = 0; pass < passes; ++pass) {
      const int chan = (pass * LPR + cl) * VEC;
      const bool chan_ok = chan < C;
      const uint32_t chan_off = chan_ok ? (uint32_t)(chan * sizeof(T)) : kNoChan;
      A acc[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] = 0;

      for (int chunk = 0; chunk < ws.chunks; ++chunk) {
        // ---------------- phase A: one lane per sampling point ----------------
        const int pt = chunk * kWave + lane;                 // point within the group of units
        const int ul = pt / ws.LP, lp = pt - ul * ws.LP;     // unit within group, point within unit
        const int q = q0 + ul;
        const bool live = ul < ws.upw && q < Q;
        Task<A> t4[4];
        A wu = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) { t4[k].off = kNoRow; t4[k].w = 0; }
        if (live) {
          const int l = lp / P;
          const size_t gp = ((size_t)(b * (size_t)Q + q) * M + m) * ws.LP + lp;   // global point index
          const A *pl = loc + gp * loc_stride;
          // locations, weights and scores pass through once: non-temporal, so that they do not push the value
          // rows and distributions that the gathers keep coming back to out of the L2
          const A x = __builtin_nontemporal_load(pl), y = __builtin_nontemporal_load(pl + 1);
          const A a = __builtin_nontemporal_load(attn + gp);
          const Point2D<A> g = locate_2d<A>(x, y, tab.H[l], tab.W[l], tab.start[l]);
          A sc[4];
          if (FUSED) {
            A lo[4], hi[4];
            const DepthTap<A> tap = locate_depth<A>(__builtin_nontemporal_load(pl + 2), tab.Dd[l]);
            if (packed != nullptr) {                                // uniform: all eight taps from one line
              const int db = min(max(tap.d0, 0), D - 2);
              const bool lo_x = tap.lo_ok && tap.d0 == db, lo_y = tap.lo_ok && tap.d0 == db + 1;
              const bool hi_x = tap.hi_ok && tap.d0 + 1 == db, hi_y = tap.hi_ok && tap.d0 + 1 == db + 1;
              const int cell = tab.cell[l] + (g.h0 + 1) * (tab.W[l] + 1) + g.w0 + 1;
              A x4[4], y4[4];
              PackedTap<T>::ld(packed_r, (g.inside && tap.inside) ? (uint32_t)((cell * D + db) * 4 * (int)sizeof(T)) : kNoRow,
                               x4, y4);
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                lo[k] = lo_x ? x4[k] : lo_y ? y4[k] : (A)0;
                hi[k] = hi_x ? x4[k] : hi_y ? y4[k] : (A)0;
                sc[k] = depth_lerp(lo[k], hi[k], tap.hd, tap.ld);
              }
            } else {
              corner_scores<T, A>(dist_r, g.key, tap, md, Md, D, sc, lo, hi);
            }
            if (score_out != nullptr && pass == 0) {
              T *so = score_out + gp * 4;
              if constexpr (sizeof(T) == 4) {                     // one 16-byte store
                typedef float f4 __attribute__((ext_vector_type(4)));
                f4 v4 = {(float)sc[0], (float)sc[1], (float)sc[2], (float)sc[3]};
                __builtin_nontemporal_store(v4, reinterpret_cast<f4 *>(so));
              } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) Elem<T>::st(so + k, sc[k]);
              }
            }
            wu = a * ((sc[0] + sc[1] + sc[2] + sc[3]) * (A)0.25);
          } else {
            const T *si = score_in + gp * 4;        // no scores given: plain deformable attention
#pragma unroll
            for (int k = 0; k < 4; ++k) sc[k] = score_in != nullptr ? Elem<T>::ld(si + k) : (A)1;
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            if (g.key[k] >= 0) {
              t4[k].off = (uint32_t)((g.key[k] * M + m) * C * (int)sizeof(T));
              t4[k].w = g.bil(k) * sc[k] * a;
            }
          }
        }
        if (FUSED && weight_update != nullptr && pass == 0) {      // wave-uniform
          // sum over the lanes of each unit: lane i gathers lanes [i, i + 2^k) of its own unit
          const int seg = ws.upw == 1 ? kWave : ws.LP, pos = ws.upw == 1 ? lane : lp;
          for (int off = 1; off < seg; off <<= 1) {
            const A up = __shfl_down(wu, off, kWave);
            if (pos + off < seg) wu += up;
          }
          if (ws.upw == 1) {
            wu_unit += wu;                                         // lane 0 holds the chunk's sum
            if (chunk == ws.chunks - 1 && lane == 0) weight_update[((size_t)b * Q + q0) * M + m] = wu_unit;
          } else if (live && lp == 0) {
            weight_update[((size_t)b * Q + q) * M + m] = wu;
          }
        }
        wave_lds_handover();     // previous phase B has consumed the task list
#pragma unroll
        for (int k = 0; k < 4; ++k) tasks[lane * 4 + k] = t4[k];
        wave_lds_handover();

        // ---------------- phase B: lanes over channels ----------------
        if (ws.upw == 1) {
          const int n_pts = min(kWave, ws.LP - chunk * kWave);
          gather_rows<T, A, VEC, LPR>(value_r, tasks, 0, n_pts * 4, row_slot, chan_off, acc);
        } else {
          // several whole units in this chunk: finish each one here
          for (int u = 0; u < ws.upw; ++u) {
            if (q0 + u >= Q) break;
            A au[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) au[i] = 0;
            gather_rows<T, A, VEC, LPR>(value_r, tasks, u * ws.LP * 4, (u + 1) * ws.LP * 4, row_slot, chan_off, au);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
#pragma unroll
              for (int off = LPR; off < kWave; off <<= 1) au[i] += __shfl_xor(au[i], off, kWave);
            }
            if (row_slot == 0 && chan_ok) {
              const size_t unit = ((size_t)b * Q + (q0 + u)) * M + m;
              RowVec<T, A, VEC>::st(out + unit * C + chan, au);
            }
          }
        }
      }
      if (ws.upw == 1) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
#pragma unroll
          for (int off = LPR; off < kWave; off <<= 1) acc[i] += __shfl_xor(acc[i], off, kWave);
        }
        if (row_slot == 0 && chan_ok) {
          const size_t unit = ((size_t)b * Q + q0) * M + m;
          RowVec<T, A, VEC>::st(out + unit * C + chan, acc);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Stage 1 alone: one lane per sampling point.  Block id -> (head, batch, block of kDsQueries
// queries) with head = block % M, as in the attention kernels: the distributions one XCD's L2
// sees are those of one head.
// ---------------------------------------------------------------------------------------
constexpr int kDsQueries = 32;
template <typename T, typename A>
__global__ __launch_bounds__(kBlock) void depth_score_kernel(
    const T *__restrict__ dist, const int64_t *__restrict__ shapes3, const int64_t *__restrict__ level_start,
    const A *__restrict__ loc3, T *__restrict__ score, int B, int S, int M, int D, int L, int Q, int P) {
  __shared__ LevelTable tab;
  load_level_table(tab, shapes3, 3, level_start, L, S, D);
  const int LP = L * P;
  const int m = blockIdx.x % M;
  const int rest = blockIdx.x / M;
  const int q_blocks = (Q + kDsQueries - 1) / kDsQueries;
  const int qb = rest % q_blocks, b = rest / q_blocks;
  const int q0 = qb * kDsQueries, nq = min(kDsQueries, Q - q0);
  const rsrc_t dist_r = make_rsrc(dist + (size_t)b * S * M * D, (size_t)S * M * D * sizeof(T));
  for (int i = threadIdx.x; i < nq * LP; i += kBlock) {
    const int ql = i / LP, lp = i - ql * LP;
    const size_t gp = (((size_t)b * Q + q0 + ql) * M + m) * LP + lp;
    const int l = lp / P;
    const A *pl = loc3 + gp * 3;
    const Point2D<A> g = locate_2d<A>(pl[0], pl[1], tab.H[l], tab.W[l], tab.start[l]);
    const DepthTap<A> tap = locate_depth<A>(pl[2], tab.Dd[l]);
    A sc[4], lo[4], hi[4];
    corner_scores<T, A>(dist_r, g.key, tap, m, M, D, sc, lo, hi);
    T *so = score + gp * 4;
#pragma unroll
    for (int k = 0; k < 4; ++k) Elem<T>::st(so + k, sc[k]);
  }
}

// ---------------------------------------------------------------------------------------
// Packs a head-shared distribution (B,S,1,D) for the forward's depth taps: see load_cell_starts for the layout.
// One thread per (cell, bin): four gathered values, one 16-byte (bfloat16: 8-byte) store; consecutive threads
// write consecutive addresses.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void pack_dist_kernel(
    const T *__restrict__ dist, const int64_t *__restrict__ shapes3, const int64_t *__restrict__ level_start,
    T *__restrict__ packed, int B, int S, int D, int L) {
  __shared__ LevelTable tab;
  load_level_table(tab, shapes3, 3, level_start, L, S, D);
  load_cell_starts(tab, L);
  if (tab.cell[L] > packed_cell_capacity(S, L)) return;       // overlapping levels: more cells than the table holds; the forward then ignores it
  const size_t cells = (size_t)tab.cell[L];
  const size_t n = (size_t)B * cells * D;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const int d = (int)(i % D);
    const size_t bc = i / D;
    const int cell = (int)(bc % cells), b = (int)(bc / cells);
    int l = 0;
    while (l + 1 < L && cell >= tab.cell[l + 1]) ++l;
    const int H = tab.H[l], W = tab.W[l], local = cell - tab.cell[l];
    const int h0 = local / (W + 1) - 1, w0 = local % (W + 1) - 1;
    const T *lvl = dist + ((size_t)b * S + tab.start[l]) * D + d;
    T v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int h = h0 + (k >= 2 ? 1 : 0), w = w0 + ((k == 1 || k == 2) ? 1 : 0);      // slots LT, RT, RB, LB
      const bool in = h >= 0 && h < H && w >= 0 && w < W;
      v[k] = in ? lvl[(size_t)(h * W + w) * D] : T(0.f);
    }
    T *dst = packed + i * 4;
#pragma unroll
    for (int k = 0; k < 4; ++k) dst[k] = v[k];
  }
}

template <typename T>
static hipError_t launch_pack_typed(const void *dist, const int64_t *shapes3, const int64_t *level_start, void *packed,
                                    int B, int S, int D, int L, hipStream_t stream) {
  hipLaunchKernelGGL((pack_dist_kernel<T>), dim3(256 * 16), dim3(256), 0, stream, (const T *)dist, shapes3, level_start,
                     (T *)packed, B, S, D, L);
  return hipGetLastError();
}

hipError_t launch_pack_dist(const void *dist, const int64_t *shapes3, const int64_t *level_start, void *packed, int B,
                            int S, int D, int L, int dtype, hipStream_t stream) {
  switch (dtype) {
    case DFA3D_F32: return launch_pack_typed<float>(dist, shapes3, level_start, packed, B, S, D, L, stream);
    case DFA3D_BF16: return launch_pack_typed<__hip_bfloat16>(dist, shapes3, level_start, packed, B, S, D, L, stream);
  }
  return hipErrorInvalidValue;
}

// ---------------------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------------------
template <typename T, typename A, int VEC, int LPR>
static hipError_t launch_fwd_cfg(const FwdArgs &a, hipStream_t stream) {
  const WaveShape ws = wave_shape(a.L, a.P);
  const int q_per_iter = kWavesPerBlock * ws.upw;
  const int iters = a.iters > 0 ? a.iters : 1;
  const int q_blocks = (a.Q + q_per_iter * iters - 1) / (q_per_iter * iters);
  const long long blocks = (long long)a.M * a.B * q_blocks;
  if (blocks <= 0 || blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  if (a.dist != nullptr) {
    hipLaunchKernelGGL((fwd_attention_kernel<T, A, VEC, LPR, true>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                       (const T *)a.value, (const T *)a.dist, a.shapes, a.shape_stride, a.level_start,
                       (const A *)a.loc, a.loc_stride, (const A *)a.attn, (const T *)nullptr, (T *)a.out,
                       (T *)a.score_out, (A *)a.weight_update, (const T *)a.packed_dist, a.dist_heads == 1 ? 1 : a.M, a.B,
                       a.S, a.M, a.C, a.D, a.L, a.Q, a.P, iters, q_blocks);
  } else {
    hipLaunchKernelGGL((fwd_attention_kernel<T, A, VEC, LPR, false>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                       (const T *)a.value, (const T *)nullptr, a.shapes, a.shape_stride, a.level_start,
                       (const A *)a.loc, a.loc_stride, (const A *)a.attn, (const T *)a.score_in, (T *)a.out,
                       (T *)nullptr, (A *)nullptr, (const T *)nullptr, a.M, a.B, a.S, a.M, a.C, a.D, a.L, a.Q, a.P, iters,
                       q_blocks);
  }
  return hipGetLastError();
}

template <typename T, typename A>
static hipError_t launch_fwd_typed(const FwdArgs &a, hipStream_t stream) {
  const RowTiling rt = pick_row_tiling(a.C, (int)sizeof(T), a.vec_hint);
#define DFA3D_CASE(V, R) \
  if (rt.vec == V && rt.lpr == R) return launch_fwd_cfg<T, A, V, R>(a, stream);
  DFA3D_ROW_TILINGS(DFA3D_CASE)
#undef DFA3D_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_forward(const FwdArgs &a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case DFA3D_F32: return launch_fwd_typed<float, float>(a, stream);
    case DFA3D_F64: return launch_fwd_typed<double, double>(a, stream);
    case DFA3D_BF16: return launch_fwd_typed<__hip_bfloat16, float>(a, stream);
  }
  return hipErrorInvalidValue;
}

template <typename T, typename A>
static hipError_t launch_ds_typed(const DepthScoreArgs &a, hipStream_t stream) {
  const long long blocks = (long long)a.M * a.B * ((a.Q + kDsQueries - 1) / kDsQueries);
  if (blocks <= 0 || blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((depth_score_kernel<T, A>), dim3((unsigned)blocks), dim3(kBlock), 0, stream, (const T *)a.dist,
                     a.shapes3, a.level_start, (const A *)a.loc3, (T *)a.score, a.B, a.S, a.M, a.D, a.L, a.Q, a.P);
  return hipGetLastError();
}

hipError_t launch_depth_score(const DepthScoreArgs &a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case DFA3D_F32: return launch_ds_typed<float, float>(a, stream);
    case DFA3D_F64: return launch_ds_typed<double, double>(a, stream);
    case DFA3D_BF16: return launch_ds_typed<__hip_bfloat16, float>(a, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dfa3d
