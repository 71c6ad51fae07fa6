// Backward kernels of the DFA3D operator for gfx950.
//
//   bwd_attention_kernel<..., FUSED=true>   backward of both stages in one pass; the depth scores
//                                           and their gradient never touch memory (the reference
//                                           runs two kernels, six zero fills and a host
//                                           synchronisation: multi_scale_3ddeformable_attn_function.py:306-352)
//   bwd_attention_kernel<..., FUSED=false>  stage-2 backward alone
//                                           (wms_deform_attn_cuda_kernel.cuh:82-159, 305-419)
//   depth_score_bwd_kernel                  stage-1 backward alone
//                                           (ms_depth_score_sample_cuda_kernel.cuh:150-327)
//
// Every gradient other than grad_value is a function of the four per-corner dot products
//   dot_k = sum_c value[corner k, c] * grad_out[c]:
//   grad_attn       = sum_k bil_k * score_k * dot_k
//   grad_score_k    = bil_k * attn * dot_k
//   grad_x          = W * attn * (-s0*hh*dot0 + s1*hh*dot1 + s2*lh*dot2 - s3*lh*dot3)
//   grad_y          = H * attn * (-s0*hw*dot0 - s1*lw*dot1 + s2*lw*dot2 + s3*hw*dot3)
//   grad_dist[k,d0] += hd * grad_score_k,  grad_dist[k,d0+1] += ld * grad_score_k
//   grad_z          = Dd * sum_k grad_score_k * (dist[k,d0+1] - dist[k,d0])
// (slots k = LT,RT,RB,LB).  Phase B produces the dots with a lane reduction per value row and
// issues the grad_value atomics; phase C, one lane per point again, turns the dots into the
// per-point gradients with coalesced stores and the grad_dist atomics.
#include "dfa3d_device.h"
#include "dfa3d_launch.h"

namespace dfa3d {

// ---- sum over the LPR lanes that share a value row; every lane ends up with the total ----
__device__ __forceinline__ float dpp_add(float x, int ctrl_pick) {
  // ctrl_pick: 0 quad xor 1, 1 quad xor 2, 2 half-row mirror, 3 row mirror
  int r;
  const int xi = __float_as_int(x);
  switch (ctrl_pick) {
    case 0: r = __builtin_amdgcn_mov_dpp(xi, 0xB1, 0xF, 0xF, true); break;    // quad_perm [1,0,3,2]
    case 1: r = __builtin_amdgcn_mov_dpp(xi, 0x4E, 0xF, 0xF, true); break;    // quad_perm [2,3,0,1]
    case 2: r = __builtin_amdgcn_mov_dpp(xi, 0x141, 0xF, 0xF, true); break;   // row_half_mirror
    default: r = __builtin_amdgcn_mov_dpp(xi, 0x140, 0xF, 0xF, true); break;  // row_mirror
  }
  return x + __int_as_float(r);
}

template <int LPR> __device__ __forceinline__ float row_sum(float x) {
  if (LPR >= 2) x = dpp_add(x, 0);
  if (LPR >= 4) x = dpp_add(x, 1);
  if (LPR >= 8) x = dpp_add(x, 2);
  if (LPR >= 16) x = dpp_add(x, 3);
  if (LPR >= 32) x += __shfl_xor(x, 16, kWave);
  if (LPR >= 64) x += __shfl_xor(x, 32, kWave);
  return x;
}
template <int LPR> __device__ __forceinline__ double row_sum(double x) {
#pragma unroll
  for (int off = 1; off < LPR; off <<= 1) x += __shfl_xor(x, off, kWave);
  return x;
}

// Phase B of the backward pass over tasks [t_begin, t_end): per task the dot product of the value
// row with grad_out (left in dots[t]) and the scatter-add of w * grad_out into grad_value.
//   chan_off   lane's byte offset inside a value row (kNoChan beyond the last channel)
//   GSHIFT     log2(sizeof(A) / sizeof(T)): a gradient row offset is the value row offset << GSHIFT
template <typename T, typename A, int VEC, int LPR>
__device__ __forceinline__ void dots_and_scatter(rsrc_t value_r, rsrc_t gvalue_r, A *gvalue_b, const Task<A> *tasks,
                                                 A *dots, int t_begin, int t_end, int row_slot, int cl,
                                                 uint32_t chan_off, const A (&go)[VEC], bool first_pass) {
  constexpr int RPI = kWave / LPR;
  constexpr int U = 4;
  constexpr int GSHIFT = sizeof(A) == sizeof(T) ? 0 : 1;
  static_assert(sizeof(A) == sizeof(T) || sizeof(A) == 2 * sizeof(T), "gradient element is 1x or 2x the storage element");
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
      // a zero weight adds nothing: drop the update instead of sending it to memory
      const uint32_t goff = ((e[j].w != 0 && e[j].off != kNoRow) ? (e[j].off << GSHIFT) : kNoRow) +
                            (chan_off == kNoChan ? kNoChan : (chan_off << GSHIFT));
#pragma unroll
      for (int i = 0; i < VEC; ++i) scatter_add(gvalue_r, gvalue_b, goff + i * (uint32_t)sizeof(A), e[j].w * go[i]);
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      A part = 0;
#pragma unroll
      for (int i = 0; i < VEC; ++i) part += v[j][i] * go[i];
      part = row_sum<LPR>(part);
      const int t = t0 + j * RPI + row_slot;
      if (cl == 0) dots[t] = first_pass ? part : dots[t] + part;
    }
  }
  for (; t0 < t_end; t0 += RPI) {
    const int t = t0 + row_slot;
    const bool in = t < t_end;
    const Task<A> e = tasks[min(t, kWave * 4 - 1)];
    const uint32_t off = in ? e.off : kNoRow;
    A v[VEC];
    RowVec<T, A, VEC>::ld(value_r, off + chan_off, v);
    const uint32_t goff = ((e.w != 0 && off != kNoRow) ? (off << GSHIFT) : kNoRow) +
                          (chan_off == kNoChan ? kNoChan : (chan_off << GSHIFT));
    A part = 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      scatter_add(gvalue_r, gvalue_b, goff + i * (uint32_t)sizeof(A), e.w * go[i]);
      part += v[i] * go[i];
    }
    part = row_sum<LPR>(part);
    if (cl == 0 && in) dots[t] = first_pass ? part : dots[t] + part;
  }
}

// ---------------------------------------------------------------------------------------
// Fused / stage-2 backward.  Same grid and wave layout as the forward kernel.
//   gradient inputs (grad_out, grad_score_in) have the forward outputs' type T;
//   gradient outputs have the arithmetic type A.
// ---------------------------------------------------------------------------------------
template <typename T, typename A, int VEC, int LPR, bool FUSED>
__global__ __launch_bounds__(kBlock) void bwd_attention_kernel(
    const T *__restrict__ value, const T *__restrict__ dist, const int64_t *__restrict__ shapes, int shape_stride,
    const int64_t *__restrict__ level_start, const A *__restrict__ loc, int loc_stride,
    const A *__restrict__ attn, const T *__restrict__ score_in, const T *__restrict__ grad_out,
    const T *__restrict__ grad_score_in, A *__restrict__ grad_value, A *__restrict__ grad_dist,
    A *__restrict__ grad_loc, int gl_stride, A *__restrict__ grad_attn, A *__restrict__ grad_score_out,
    const A *__restrict__ grad_wu, int Md,
    int B, int S, int M, int C, int D, int L, int Q, int P, int iters, int q_blocks DFA3D_DIAG_PARAM) {
  __shared__ LevelTable tab;
  __shared__ Task<A> s_tasks[kWavesPerBlock][kWave * 4];
  __shared__ A s_dots[kWavesPerBlock][kWave * 4];

  load_level_table(tab, shapes, shape_stride, level_start, L, S, FUSED ? D : 0);

  const WaveShape ws = wave_shape(L, P);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int m = blockIdx.x % M;
  const int rest = blockIdx.x / M;
  const int qb = rest % q_blocks, b = rest / q_blocks;
  const int row_slot = lane / LPR, cl = lane % LPR;
  const int passes = (C + VEC * LPR - 1) / (VEC * LPR);
  Task<A> *tasks = s_tasks[wave];
  A *dots = s_dots[wave];

  A *gvalue_b = grad_value + (size_t)b * S * M * C;
  A *gdist_b = FUSED ? grad_dist + (size_t)b * S * Md * D : nullptr;
  const int md = Md == 1 ? 0 : m;
  const rsrc_t value_r = make_rsrc(value + (size_t)b * S * M * C, (size_t)S * M * C * sizeof(T));
  const rsrc_t gvalue_r = make_rsrc(gvalue_b, DFA3D_DIAG(diag, 1) ? 0 : (size_t)S * M * C * sizeof(A));
  const rsrc_t dist_r = make_rsrc(FUSED ? dist + (size_t)b * S * Md * D : nullptr,
                                  FUSED ? (size_t)S * Md * D * sizeof(T) : 0);
  const rsrc_t gdist_r = make_rsrc(gdist_b, (FUSED && !DFA3D_DIAG(diag, 2)) ? (size_t)S * Md * D * sizeof(A) : 0);
  const int q_per_iter = kWavesPerBlock * ws.upw;

  for (int it = 0; it < iters; ++it) {
    const int q0 = (qb * iters + it) * q_per_iter + wave * ws.upw;
    if (q0 >= Q) break;   // wave-uniform
    for (int chunk = 0; chunk < ws.chunks; ++chunk) {
      // ---------------- phase A: one lane per sampling point ----------------
      const int pt = chunk * kWave + lane;
      const int ul = pt / ws.LP, lp = pt - ul * ws.LP;
      const int q = q0 + ul;
      const bool live = ul < ws.upw && q < Q;
      size_t gp = 0;
      int l = 0;
      Point2D<A> g;
      DepthTap<A> tap;
      A a = 0, sc[4], lo[4], hi[4];
      Task<A> t4[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        t4[k].off = kNoRow; t4[k].w = 0;
        sc[k] = 0; lo[k] = 0; hi[k] = 0; g.key[k] = -1;
      }
      g.inside = false; tap.inside = false; tap.lo_ok = false; tap.hi_ok = false; tap.d0 = 0;
      g.lh = g.lw = g.hh = g.hw = 0; tap.ld = tap.hd = 0;
      if (live) {
        l = lp / P;
        gp = ((size_t)(b * (size_t)Q + q) * M + m) * ws.LP + lp;
        const A *pl = loc + gp * loc_stride;
        a = attn[gp];
        g = locate_2d<A>(pl[0], pl[1], tab.H[l], tab.W[l], tab.start[l]);
        if (FUSED) {
          tap = locate_depth<A>(pl[2], tab.Dd[l]);
          corner_scores<T, A>(dist_r, g.key, tap, md, Md, D, sc, lo, hi);
        } else {
          const T *si = score_in + gp * 4;
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
      wave_lds_handover();
#pragma unroll
      for (int k = 0; k < 4; ++k) tasks[lane * 4 + k] = t4[k];
      wave_lds_handover();

      // ---------------- phase B: dots and grad_value scatter-adds ----------------
      for (int pass = 0; pass < passes; ++pass) {
        const int chan = (pass * LPR + cl) * VEC;
        const bool chan_ok = chan < C;
        const uint32_t chan_off = chan_ok ? (uint32_t)(chan * sizeof(T)) : kNoChan;
        for (int u = 0; u < ws.upw; ++u) {
          if (q0 + u >= Q) break;
          const int t_begin = ws.upw == 1 ? 0 : u * ws.LP * 4;
          const int t_end = ws.upw == 1 ? min(kWave, ws.LP - chunk * kWave) * 4 : t_begin + ws.LP * 4;
          const size_t unit = ((size_t)b * Q + (q0 + u)) * M + m;
          A go[VEC];
#pragma unroll
          for (int i = 0; i < VEC; ++i) go[i] = 0;
          if (chan_ok) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) go[i] = Elem<T>::ld(grad_out + unit * C + chan + i);
          }
          dots_and_scatter<T, A, VEC, LPR>(value_r, gvalue_r, gvalue_b, tasks, dots, t_begin, t_end, row_slot, cl,
                                           chan_off, go, pass == 0);
        }
      }
      wave_lds_handover();

      // ---------------- phase C: one lane per point again ----------------
      if (live) {
        A dot[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) dot[k] = dots[lane * 4 + k];
        A gs[4], s[4];
        A ga = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const bool on = g.key[k] >= 0;
          const A bk = g.bil(k);
          gs[k] = on ? bk * a * dot[k] : (A)0;
          s[k] = on ? sc[k] * dot[k] : (A)0;
          ga += bk * s[k];
        }
        A gx = 0, gy = 0;
        if (g.inside) {
          gx = (A)tab.W[l] * a * (g.hh * (s[1] - s[0]) + g.lh * (s[2] - s[3]));
          gy = (A)tab.H[l] * a * (g.hw * (s[3] - s[0]) + g.lw * (s[2] - s[1]));
        }
        A *gl = grad_loc + gp * gl_stride;
        gl[0] = gx;
        gl[1] = gy;
        grad_attn[gp] = ga;
        if (FUSED) {
          if (grad_score_in != nullptr) {
            const T *gi = grad_score_in + gp * 4;
#pragma unroll
            for (int k = 0; k < 4; ++k) gs[k] += Elem<T>::ld(gi + k);
          }
          if (grad_wu != nullptr) {       // weight_update = sum over points of attn * mean corner score
            const A gw = grad_wu[gp / ws.LP] * (A)0.25;
            grad_attn[gp] = ga + gw * (sc[0] + sc[1] + sc[2] + sc[3]);
#pragma unroll
            for (int k = 0; k < 4; ++k) gs[k] += gw * a;
          }
          A gz = 0;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const bool on = g.key[k] >= 0 && gs[k] != 0;
            const uint32_t row = (uint32_t)(((g.key[k] * Md + md) * D + tap.d0) * (int)sizeof(A));
            scatter_add(gdist_r, gdist_b, (on && tap.lo_ok) ? row : kNoRow, tap.hd * gs[k]);
            scatter_add(gdist_r, gdist_b, (on && tap.hi_ok) ? row + (uint32_t)sizeof(A) : kNoRow, tap.ld * gs[k]);
            gz += (g.key[k] >= 0 && tap.inside) ? gs[k] * (hi[k] - lo[k]) : (A)0;
          }
          gl[2] = gz * (A)tab.Dd[l];
        } else if (grad_score_out != nullptr) {
          A *go4 = grad_score_out + gp * 4;
#pragma unroll
          for (int k = 0; k < 4; ++k) go4[k] = gs[k];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Stage-1 backward alone: one lane per sampling point, block id -> (head, batch, query block)
// as in the forward.
// ---------------------------------------------------------------------------------------
constexpr int kDsQueries = 32;
template <typename T, typename A>
__global__ __launch_bounds__(kBlock) void depth_score_bwd_kernel(
    const T *__restrict__ dist, const int64_t *__restrict__ shapes3, const int64_t *__restrict__ level_start,
    const A *__restrict__ loc3, const T *__restrict__ grad_score, A *__restrict__ grad_dist,
    A *__restrict__ grad_loc3, int B, int S, int M, int D, int L, int Q, int P) {
  __shared__ LevelTable tab;
  load_level_table(tab, shapes3, 3, level_start, L, S, D);
  const int LP = L * P;
  const int m = blockIdx.x % M;
  const int rest = blockIdx.x / M;
  const int q_blocks = (Q + kDsQueries - 1) / kDsQueries;
  const int qb = rest % q_blocks, b = rest / q_blocks;
  const int q0 = qb * kDsQueries, nq = min(kDsQueries, Q - q0);
  const rsrc_t dist_r = make_rsrc(dist + (size_t)b * S * M * D, (size_t)S * M * D * sizeof(T));
  A *gdist_b = grad_dist + (size_t)b * S * M * D;
  const rsrc_t gdist_r = make_rsrc(gdist_b, (size_t)S * M * D * sizeof(A));
  for (int i = threadIdx.x; i < nq * LP; i += kBlock) {
    const int ql = i / LP, lp = i - ql * LP;
    const size_t gp = (((size_t)b * Q + q0 + ql) * M + m) * LP + lp;
    const int l = lp / P;
    const A *pl = loc3 + gp * 3;
    const Point2D<A> g = locate_2d<A>(pl[0], pl[1], tab.H[l], tab.W[l], tab.start[l]);
    const DepthTap<A> tap = locate_depth<A>(pl[2], tab.Dd[l]);
    A sc[4], lo[4], hi[4];
    corner_scores<T, A>(dist_r, g.key, tap, m, M, D, sc, lo, hi);
    const T *gi = grad_score + gp * 4;
    A gz = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool on = g.key[k] >= 0 && tap.inside;
      const A gk = Elem<T>::ld(gi + k);
      const uint32_t row = (uint32_t)(((g.key[k] * M + m) * D + tap.d0) * (int)sizeof(A));
      scatter_add(gdist_r, gdist_b, (on && tap.lo_ok) ? row : kNoRow, tap.hd * gk);
      scatter_add(gdist_r, gdist_b, (on && tap.hi_ok) ? row + (uint32_t)sizeof(A) : kNoRow, tap.ld * gk);
      gz += on ? gk * (hi[k] - lo[k]) : (A)0;
    }
    gz *= (A)tab.Dd[l];
    A *gl = grad_loc3 + gp * 3;
    gl[0] = 0;
    gl[1] = 0;
    gl[2] = gz;
  }
}

// ---------------------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------------------
template <typename T, typename A, int VEC, int LPR>
static hipError_t launch_bwd_cfg(const BwdArgs &a, hipStream_t stream) {
  const WaveShape ws = wave_shape(a.L, a.P);
  const int q_per_iter = kWavesPerBlock * ws.upw;
  const int iters = a.iters > 0 ? a.iters : 1;
  const int q_blocks = (a.Q + q_per_iter * iters - 1) / (q_per_iter * iters);
  const long long blocks = (long long)a.M * a.B * q_blocks;
  if (blocks <= 0 || blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  if (a.dist != nullptr) {
    hipLaunchKernelGGL((bwd_attention_kernel<T, A, VEC, LPR, true>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                       (const T *)a.value, (const T *)a.dist, a.shapes, a.shape_stride, a.level_start,
                       (const A *)a.loc, a.loc_stride, (const A *)a.attn, (const T *)nullptr,
                       (const T *)a.grad_out, (const T *)a.grad_score_in, (A *)a.grad_value, (A *)a.grad_dist,
                       (A *)a.grad_loc, a.grad_loc_stride, (A *)a.grad_attn, (A *)nullptr,
                       (const A *)a.grad_weight_update, a.dist_heads == 1 ? 1 : a.M, a.B, a.S, a.M, a.C, a.D,
                       a.L, a.Q, a.P, iters, q_blocks DFA3D_DIAG_ARG(a));
  } else {
    hipLaunchKernelGGL((bwd_attention_kernel<T, A, VEC, LPR, false>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                       (const T *)a.value, (const T *)nullptr, a.shapes, a.shape_stride, a.level_start,
                       (const A *)a.loc, a.loc_stride, (const A *)a.attn, (const T *)a.score_in,
                       (const T *)a.grad_out, (const T *)nullptr, (A *)a.grad_value, (A *)nullptr, (A *)a.grad_loc,
                       a.grad_loc_stride, (A *)a.grad_attn, (A *)a.grad_score_out, (const A *)nullptr, a.M, a.B, a.S,
                       a.M, a.C, a.D, a.L, a.Q, a.P, iters, q_blocks DFA3D_DIAG_ARG(a));
  }
  return hipGetLastError();
}

template <typename T, typename A>
static hipError_t launch_bwd_typed(const BwdArgs &a, hipStream_t stream) {
  const RowTiling rt = pick_row_tiling(a.C, (int)sizeof(T), a.vec_hint, true);
#define DFA3D_CASE(V, R) \
  if (rt.vec == V && rt.lpr == R) return launch_bwd_cfg<T, A, V, R>(a, stream);
  DFA3D_ROW_TILINGS(DFA3D_CASE)
#undef DFA3D_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_backward(const BwdArgs &a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case DFA3D_F32: return launch_bwd_typed<float, float>(a, stream);
    case DFA3D_F64: return launch_bwd_typed<double, double>(a, stream);
    case DFA3D_BF16: return launch_bwd_typed<__hip_bfloat16, float>(a, stream);
  }
  return hipErrorInvalidValue;
}

template <typename T, typename A>
static hipError_t launch_dsb_typed(const DepthScoreBwdArgs &a, hipStream_t stream) {
  const long long blocks = (long long)a.M * a.B * ((a.Q + kDsQueries - 1) / kDsQueries);
  if (blocks <= 0 || blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((depth_score_bwd_kernel<T, A>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                     (const T *)a.dist, a.shapes3, a.level_start, (const A *)a.loc3, (const T *)a.grad_score,
                     (A *)a.grad_dist, (A *)a.grad_loc3, a.B, a.S, a.M, a.D, a.L, a.Q, a.P);
  return hipGetLastError();
}

hipError_t launch_depth_score_backward(const DepthScoreBwdArgs &a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case DFA3D_F32: return launch_dsb_typed<float, float>(a, stream);
    case DFA3D_F64: return launch_dsb_typed<double, double>(a, stream);
    case DFA3D_BF16: return launch_dsb_typed<__hip_bfloat16, float>(a, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dfa3d
