/*
 * TEST INFRASTRUCTURE ONLY - scalar CPU restatement of the DFA3D operator, one
 * precision per inclusion.  Included by dfa3d_oracle.c with
 *   REAL   = float  / double
 *   FN(x)  = x##_f32 / x##_f64
 * and a third time as x##_f64g32: double arithmetic on the float path's pixel
 * coordinates (DFA3D_ORACLE_FLOAT_GEOMETRY), the yardstick for float summation error.
 *
 * Every routine states the reference lines it restates.  Paths are relative to
 * the reference checkout; "ms.cuh" is
 *   DFA3D/dfa3D/ops/csrc/common/cuda/ms_depth_score_sample_cuda_kernel.cuh
 * and "wms.cuh" is
 *   DFA3D/dfa3D/ops/csrc/common/cuda/wms_deform_attn_cuda_kernel.cuh
 *
 * Corner numbering used for the depth-score slots (ms.cuh:89-92, wms.cuh:51-72):
 *   slot 0 = (h_low , w_low ) left-top      slot 1 = (h_low , w_high) right-top
 *   slot 2 = (h_high, w_high) right-bottom  slot 3 = (h_high, w_low ) left-bottom
 * The reference visits the corners in the order LT, RT, LB, RB, i.e. slots
 * 0, 1, 3, 2; floating-point sums below keep that order.
 */

/* slot -> (dh, dw) */
static const int FN(k_dh)[4] = {0, 0, 1, 1};
static const int FN(k_dw)[4] = {0, 1, 1, 0};
/* visiting order of the reference: LT, RT, LB, RB */
static const int FN(k_visit)[4] = {0, 1, 3, 2};

/* Pixel coordinate of a normalised location (ms.cuh:133-135, wms.cuh:286-287):
 * float product, then "- 0.5" with a double literal, rounded back to REAL. */
static inline REAL FN(to_pixel)(REAL loc, int size) {
#ifdef DFA3D_ORACLE_FLOAT_GEOMETRY
  /* the float kernels' pixel coordinate (locations that are float values held in doubles), so that the
   * double sums of this instantiation are the exact sums of the terms the float path adds up */
  const float prod = (float)loc * size;
  const float imf = (float)(prod - 0.5);
  return imf;
#else
  const REAL im = loc * size - 0.5;
  return im;
#endif
}

/* floor as the reference takes it: floorf() on every scalar type, so a double
 * coordinate is first rounded to float (ms.cuh:30-32, wms.cuh:30-31). */
static inline int FN(floor_index)(REAL x) { return (int)floorf((float)x); }

/* ------------------------------------------------------------------------- *
 * Stage 1 forward: multi-scale depth-score sampling.
 * Restates ms.cuh:94-148 (loop over units and points, skip predicate :137) and
 * ms.cuh:24-93 (the four corner scores, per-bin zero padding, slot order).
 *   dist      (B,S,M,D)      shapes3 (L,3) = (H,W,Dd)     lsi (L)
 *   loc3      (B,Q,M,L,P,3)  score   (B,Q,M,L,P,4)  fully written
 * ------------------------------------------------------------------------- */
void FN(dfa3d_oracle_depth_score_forward)(
    const REAL *dist, const int64_t *shapes3, const int64_t *lsi, const REAL *loc3,
    int B, int S, int M, int D, int L, int Q, int P, REAL *score) {
  const int64_t units = (int64_t)B * Q * M;
  const int pix_stride = M * D;
#pragma omp parallel for schedule(static)
  for (int64_t u = 0; u < units; ++u) {
    const int m = (int)(u % M);
    const int b = (int)(u / M / Q);
    const REAL *dist_b = dist + (int64_t)b * S * pix_stride;
    const REAL *loc = loc3 + u * L * P * 3;
    REAL *out = score + u * L * P * 4;
    for (int l = 0; l < L; ++l) {
      const int H = (int)shapes3[l * 3], W = (int)shapes3[l * 3 + 1], Dd = (int)shapes3[l * 3 + 2];
      const REAL *lvl = dist_b + (int64_t)lsi[l] * pix_stride;
      for (int p = 0; p < P; ++p, loc += 3, out += 4) {
        out[0] = out[1] = out[2] = out[3] = 0;
        const REAL h_im = FN(to_pixel)(loc[1], H);
        const REAL w_im = FN(to_pixel)(loc[0], W);
        const REAL d_im = FN(to_pixel)(loc[2], Dd);
        if (!(h_im > -1 && w_im > -1 && d_im > -1 && h_im < H && w_im < W && d_im < Dd)) continue;
        const int h0 = FN(floor_index)(h_im), w0 = FN(floor_index)(w_im), d0 = FN(floor_index)(d_im);
        const REAL ld = d_im - d0, hd = 1 - ld;
        for (int k = 0; k < 4; ++k) {
          const int hc = h0 + FN(k_dh)[k], wc = w0 + FN(k_dw)[k];
          REAL lo = 0, hi = 0;
          if (hc >= 0 && hc <= H - 1 && wc >= 0 && wc <= W - 1) {
            const REAL *row = lvl + ((int64_t)hc * W + wc) * pix_stride + m * D;
            if (d0 >= 0) lo = row[d0];
            if (d0 + 1 <= Dd - 1) hi = row[d0 + 1];
          }
          out[k] += lo * hd + hi * ld;
        }
      }
    }
  }
}

/* ------------------------------------------------------------------------- *
 * Stage 1 backward.  Restates ms.cuh:242-327 (one worker per corner slot, the
 * four partial z-gradients summed in slot order 0..3 and STORED, x and y
 * gradients identically zero :238-239) and ms.cuh:150-241 (two scatter-adds
 * per in-range corner, z partial = Dd * g * (hi - lo)).
 *   grad_score (B,Q,M,L,P,4)
 *   grad_dist  (B,S,M,D)     accumulated into (caller zero-fills)
 *   grad_loc3  (B,Q,M,L,P,3) overwritten
 * Parallel over the batch index only: scatter targets never cross batches.
 * ------------------------------------------------------------------------- */
void FN(dfa3d_oracle_depth_score_backward)(
    const REAL *dist, const int64_t *shapes3, const int64_t *lsi, const REAL *loc3,
    const REAL *grad_score, int B, int S, int M, int D, int L, int Q, int P,
    REAL *grad_dist, REAL *grad_loc3) {
  const int pix_stride = M * D;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    const REAL *dist_b = dist + (int64_t)b * S * pix_stride;
    REAL *gdist_b = grad_dist + (int64_t)b * S * pix_stride;
    for (int64_t u = (int64_t)b * Q * M; u < (int64_t)(b + 1) * Q * M; ++u) {
      const int m = (int)(u % M);
      const REAL *loc = loc3 + u * L * P * 3;
      const REAL *gs = grad_score + u * L * P * 4;
      REAL *gl = grad_loc3 + u * L * P * 3;
      for (int l = 0; l < L; ++l) {
        const int H = (int)shapes3[l * 3], W = (int)shapes3[l * 3 + 1], Dd = (int)shapes3[l * 3 + 2];
        const int64_t lvl = (int64_t)lsi[l] * pix_stride;
        for (int p = 0; p < P; ++p, loc += 3, gs += 4, gl += 3) {
          const REAL h_im = FN(to_pixel)(loc[1], H);
          const REAL w_im = FN(to_pixel)(loc[0], W);
          const REAL d_im = FN(to_pixel)(loc[2], Dd);
          REAL part[4] = {0, 0, 0, 0};
          if (h_im > -1 && w_im > -1 && d_im > -1 && h_im < H && w_im < W && d_im < Dd) {
            const int h0 = FN(floor_index)(h_im), w0 = FN(floor_index)(w_im), d0 = FN(floor_index)(d_im);
            const REAL ld = d_im - d0, hd = 1 - ld;
            for (int k = 0; k < 4; ++k) {
              const int hc = h0 + FN(k_dh)[k], wc = w0 + FN(k_dw)[k];
              const REAL g = gs[k];
              REAL lo = 0, hi = 0;
              if (hc >= 0 && hc <= H - 1 && wc >= 0 && wc <= W - 1) {
                const int64_t row = lvl + ((int64_t)hc * W + wc) * pix_stride + m * D;
                if (d0 >= 0) {
                  lo = dist_b[row + d0];
                  gdist_b[row + d0] += hd * g;
                }
                if (d0 + 1 <= Dd - 1) {
                  hi = dist_b[row + d0 + 1];
                  gdist_b[row + d0 + 1] += ld * g;
                }
              }
              REAL dw = 0;
              dw += g * (hi - lo);
              part[k] = Dd * dw;
            }
          }
          REAL gz = part[0];
          for (int k = 1; k < 4; ++k) gz += part[k];
          gl[0] = 0;
          gl[1] = 0;
          gl[2] = gz;
        }
      }
    }
  }
}

/* ------------------------------------------------------------------------- *
 * Stage 2 forward: depth-weighted multi-scale deformable attention.
 * Restates wms.cuh:240-303 (one accumulator per (b,q,m,c), points visited l
 * then p, skip predicate :289) and wms.cuh:24-80 (corner weights
 * bilinear*score, out-of-map corners contribute neither value nor score).
 *   value  (B,S,M,C)   shapes (L,shape_stride) with (H,W) first   lsi (L)
 *   loc    (B,Q,M,L,P,loc_stride) with (x,y) first
 *   attn   (B,Q,M,L,P)   score (B,Q,M,L,P,4)   out (B,Q,M*C) fully written
 * ------------------------------------------------------------------------- */
void FN(dfa3d_oracle_wms_forward)(
    const REAL *value, const int64_t *shapes, int shape_stride, const int64_t *lsi,
    const REAL *loc, int loc_stride, const REAL *attn, const REAL *score,
    int B, int S, int M, int C, int L, int Q, int P, REAL *out) {
  const int64_t units = (int64_t)B * Q * M;
  const int pix_stride = M * C;
#pragma omp parallel for schedule(static)
  for (int64_t u = 0; u < units; ++u) {
    const int m = (int)(u % M);
    const int b = (int)(u / M / Q);
    const REAL *value_b = value + (int64_t)b * S * pix_stride;
    for (int c = 0; c < C; ++c) {
      const REAL *lp = loc + u * L * P * loc_stride;
      const REAL *aw = attn + u * L * P;
      const REAL *sc = score + u * L * P * 4;
      REAL col = 0;
      for (int l = 0; l < L; ++l) {
        const int H = (int)shapes[l * shape_stride], W = (int)shapes[l * shape_stride + 1];
        const REAL *lvl = value_b + (int64_t)lsi[l] * pix_stride + m * C + c;
        for (int p = 0; p < P; ++p, lp += loc_stride, aw += 1, sc += 4) {
          const REAL h_im = FN(to_pixel)(lp[1], H);
          const REAL w_im = FN(to_pixel)(lp[0], W);
          if (!(h_im > -1 && w_im > -1 && h_im < H && w_im < W)) continue;
          const int h0 = FN(floor_index)(h_im), w0 = FN(floor_index)(w_im);
          const REAL lh = h_im - h0, lw = w_im - w0, hh = 1 - lh, hw = 1 - lw;
          const REAL bil[4] = {hh * hw, hh * lw, lh * lw, lh * hw};
          REAL val = 0;
          for (int i = 0; i < 4; ++i) {
            const int k = FN(k_visit)[i];
            const int hc = h0 + FN(k_dh)[k], wc = w0 + FN(k_dw)[k];
            REAL v = 0, s = 0;
            if (hc >= 0 && hc <= H - 1 && wc >= 0 && wc <= W - 1) {
              s = sc[k];
              v = lvl[((int64_t)hc * W + wc) * pix_stride];
            }
            const REAL wk = bil[k] * s;
            val = (i == 0) ? wk * v : val + wk * v;
          }
          col += val * aw[0];
        }
      }
      out[u * C + c] = col;
    }
  }
}

/* ------------------------------------------------------------------------- *
 * Stage 2 backward.  Restates wms.cuh:305-419 (one worker per channel, seven
 * per-channel partials per point, summed over channels 0..C-1 in order by one
 * worker and STORED :378-407) and wms.cuh:82-159 (scatter-add into grad_value,
 * per-channel partials of grad x/y, grad attention and grad score).
 *   grad_out   (B,Q,M*C)
 *   grad_value (B,S,M,C) accumulated into (caller zero-fills)
 *   grad_loc   (B,Q,M,L,P,gl_stride): elements 0,1 overwritten, others untouched
 *   grad_attn  (B,Q,M,L,P) overwritten    grad_score (B,Q,M,L,P,4) overwritten
 * ------------------------------------------------------------------------- */
void FN(dfa3d_oracle_wms_backward)(
    const REAL *value, const int64_t *shapes, int shape_stride, const int64_t *lsi,
    const REAL *loc, int loc_stride, const REAL *attn, const REAL *score,
    const REAL *grad_out, int B, int S, int M, int C, int L, int Q, int P,
    REAL *grad_value, REAL *grad_loc, int gl_stride, REAL *grad_attn, REAL *grad_score) {
  const int pix_stride = M * C;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    const REAL *value_b = value + (int64_t)b * S * pix_stride;
    REAL *gvalue_b = grad_value + (int64_t)b * S * pix_stride;
    for (int64_t u = (int64_t)b * Q * M; u < (int64_t)(b + 1) * Q * M; ++u) {
      const int m = (int)(u % M);
      const REAL *go = grad_out + u * C;
      for (int l = 0; l < L; ++l) {
        const int H = (int)shapes[l * shape_stride], W = (int)shapes[l * shape_stride + 1];
        const int64_t lvl = (int64_t)lsi[l] * pix_stride + m * C;
        for (int p = 0; p < P; ++p) {
          const int64_t pt = (u * L + l) * P + p;
          const REAL *lp = loc + pt * loc_stride;
          const REAL a = attn[pt];
          const REAL *sc = score + pt * 4;
          REAL s_w = 0, s_h = 0, s_a = 0, s_sc[4] = {0, 0, 0, 0};
          const REAL h_im = FN(to_pixel)(lp[1], H);
          const REAL w_im = FN(to_pixel)(lp[0], W);
          if (h_im > -1 && w_im > -1 && h_im < H && w_im < W) {
            const int h0 = FN(floor_index)(h_im), w0 = FN(floor_index)(w_im);
            const REAL lh = h_im - h0, lw = w_im - w0, hh = 1 - lh, hw = 1 - lw;
            const REAL bil[4] = {hh * hw, hh * lw, lh * lw, lh * hw};
            /* d(bilinear_k)/dh and /dw up to sign, wms.cuh:116-117,127-128,138-139,149-150 */
            const REAL dh_mag[4] = {hw, lw, lw, hw};
            const REAL dw_mag[4] = {hh, hh, lh, lh};
            const int dh_sign[4] = {-1, -1, +1, +1};
            const int dw_sign[4] = {-1, +1, +1, -1};
            /* the two bilinear factors of each slot in the order the reference multiplies them */
            const REAL f1[4] = {hh, hh, lh, lh};
            const REAL f2[4] = {hw, lw, lw, hw};
            for (int c = 0; c < C; ++c) {
              const REAL top = go[c];
              const REAL tga = top * a;
              REAL gh = 0, gw = 0, val = 0;
              REAL gsc[4] = {0, 0, 0, 0};
              for (int i = 0; i < 4; ++i) {
                const int k = FN(k_visit)[i];
                const int hc = h0 + FN(k_dh)[k], wc = w0 + FN(k_dw)[k];
                const REAL wk = bil[k] * sc[k];
                REAL v = 0;
                if (hc >= 0 && hc <= H - 1 && wc >= 0 && wc <= W - 1) {
                  const int64_t idx = lvl + ((int64_t)hc * W + wc) * pix_stride + c;
                  v = value_b[idx];
                  const REAL s = sc[k];
                  if (dh_sign[k] < 0) gh -= s * dh_mag[k] * v; else gh += s * dh_mag[k] * v;
                  if (dw_sign[k] < 0) gw -= s * dw_mag[k] * v; else gw += s * dw_mag[k] * v;
                  gvalue_b[idx] += wk * tga;
                  gsc[k] += v * f1[k] * f2[k] * tga;
                }
                val = (i == 0) ? wk * v : val + wk * v;
              }
              const REAL pa = top * val;
              const REAL pw = W * gw * tga;
              const REAL ph = H * gh * tga;
              if (c == 0) {
                s_a = pa; s_w = pw; s_h = ph;
                for (int k = 0; k < 4; ++k) s_sc[k] = gsc[k];
              } else {
                s_a += pa; s_w += pw; s_h += ph;
                for (int k = 0; k < 4; ++k) s_sc[k] += gsc[k];
              }
            }
          }
          grad_loc[pt * gl_stride] = s_w;
          grad_loc[pt * gl_stride + 1] = s_h;
          grad_attn[pt] = s_a;
          for (int k = 0; k < 4; ++k) grad_score[pt * 4 + k] = s_sc[k];
        }
      }
    }
  }
}
