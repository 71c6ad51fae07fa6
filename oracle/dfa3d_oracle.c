/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the DFA3D operator (depth-score
 * sampling and depth-weighted multi-scale deformable attention, forward and
 * backward) used as the checker for the HIP kernels and as the timed CPU
 * baseline.  Nothing in the shipped library links or calls this file.
 *
 * Built by oracle/Makefile into oracle/libdfa3d_oracle.so with
 *   gcc -O2 -ffp-contract=off -fopenmp
 * (-ffp-contract=off keeps every multiply and add separately rounded, so the
 * fp32 pixel coordinates and hence every floor() and skip decision are the ones
 * the reference's expressions produce).
 *
 * The arithmetic lives in dfa3d_oracle_impl.h, instantiated for float and double
 * because the reference dispatches exactly those two types
 * (DFA3D/dfa3D/ops/csrc/cuda/wms_deform_attn_cuda.cu:267,
 *  DFA3D/dfa3D/ops/csrc/cuda/ms_depth_score_sample_cuda.cu:94).
 *
 * Parity status of each routine (what pins it is in tests/test_oracle_*.py):
 *   depth_score_forward  pinned: 5-D grid_sample identity (with wms_forward),
 *                        closed forms, brute-force loops
 *   wms_forward          pinned: 2-D grid_sample identity when score == 1,
 *                        5-D grid_sample identity composed with stage 1
 *   wms_backward         pinned: autograd through the grid_sample forms, finite differences
 *   depth_score_backward pinned: autograd through the grid_sample forms, finite differences
 * The reference holds no golden vectors for this path (its only test asserts
 * "not NaN"), so none are checked here.
 */
#include <math.h>
#include <stdint.h>
#include <omp.h>

#define REAL float
#define FN(x) x##_f32
#include "dfa3d_oracle_impl.h"
#undef REAL
#undef FN

#define REAL double
#define FN(x) x##_f64
#include "dfa3d_oracle_impl.h"
#undef REAL
#undef FN

/* Double arithmetic on the float path's geometry: every sum is (to double precision) the exact sum of the
 * terms the float instantiation rounds and adds, so |float result - this| is summation and rounding error
 * alone.  Not a restatement of anything the reference dispatches; same code as the two above. */
#define REAL double
#define FN(x) x##_f64g32
#define DFA3D_ORACLE_FLOAT_GEOMETRY
#include "dfa3d_oracle_impl.h"
#undef DFA3D_ORACLE_FLOAT_GEOMETRY
#undef REAL
#undef FN

/* Worker threads used by the loops above; returns the previous setting. */
int dfa3d_oracle_set_threads(int n) {
  int prev = omp_get_max_threads();
  if (n > 0) omp_set_num_threads(n);
  return prev;
}
int dfa3d_oracle_get_threads(void) { return omp_get_max_threads(); }
