// Host-side argument blocks and tiling choice shared by the launchers and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dfa3d {

// How the 64 lanes of a wavefront cover value rows in phase B: LPR lanes of VEC channels per
// row, 64/LPR rows per load instruction.  Channels beyond VEC*LPR are covered by extra passes.
struct RowTiling { int vec, lpr; };

#define DFA3D_ROW_TILINGS(X) \
  X(1, 4) X(1, 16) X(1, 32) X(1, 64) X(2, 8) X(2, 16) X(2, 32) X(4, 8) X(4, 16) X(4, 32) X(4, 64)

inline bool tiling_exists(int vec, int lpr) {
#define DFA3D_HAS(V, R) if (vec == V && lpr == R) return true;
  DFA3D_ROW_TILINGS(DFA3D_HAS)
#undef DFA3D_HAS
  return false;
}

// vec_hint > 0 forces that vector width when it fits the channel count.
inline RowTiling pick_row_tiling(int C, int elem_size, int vec_hint, bool atomics = false) {
  // Gathers: widest vectors first, 16 bytes per lane (fp32) measured fastest.  Rows added with device-memory atomics
  // (one instruction per channel of a lane, each touching every row of the wavefront again): narrowest first, the
  // memory side retires cache-line requests, not bytes (base shape: 11.6 / 17.5 / 29.8 ms for 1 / 2 / 4 channels per
  // lane in float, 15.9 / 26.8 / 49.6 ms in double).
  const int order_wide[3] = {4, 2, 1}, order_f64[3] = {2, 4, 1}, order_atomics[3] = {1, 2, 4};
  const int *order = atomics ? order_atomics : elem_size <= 4 ? order_wide : order_f64;
  for (int i = -1; i < 3; ++i) {
    const int vec = i < 0 ? vec_hint : order[i];
    if (vec != 1 && vec != 2 && vec != 4) continue;
    if (C % vec) continue;
    const int lpr = C / vec;
    if ((lpr & (lpr - 1)) == 0 && tiling_exists(vec, lpr)) return RowTiling{vec, lpr};
  }
  return RowTiling{1, C <= 4 ? 4 : C <= 16 ? 16 : 64};
}

struct FwdArgs {
  const void *value, *dist;          // dist == nullptr: stage 2 alone, scores read from score_in
  const int64_t *shapes; int shape_stride;
  const int64_t *level_start;
  const void *loc; int loc_stride;
  const void *attn, *score_in;
  void *out, *score_out;             // score_out may be nullptr
  void *weight_update;               // (B,Q,M) sum over a unit's points of attn * mean corner score, or nullptr
  int dist_heads;                    // heads stored in dist: M, or 1 for one distribution shared by all heads
  const void *packed_dist;           // dist_heads == 1 only: the distribution as dfa3d_pack_dist lays it out, or nullptr
  int B, S, M, C, D, L, Q, P;
  int iters;                         // groups of units each wavefront walks through
  int vec_hint;
};

struct DepthScoreArgs {
  const void *dist; const int64_t *shapes3, *level_start; const void *loc3;
  void *score;
  int B, S, M, D, L, Q, P;
};

struct BwdArgs {
  const void *value, *dist;          // dist == nullptr: stage 2 alone
  const int64_t *shapes; int shape_stride;
  const int64_t *level_start;
  const void *loc; int loc_stride;
  const void *attn, *score_in, *grad_out, *grad_score_in;
  void *grad_value, *grad_dist, *grad_loc; int grad_loc_stride;
  void *grad_attn, *grad_score_out;
  const void *grad_weight_update;    // gradient arriving at the forward's weight_update output, or nullptr
  int dist_heads;                    // as in FwdArgs; grad_dist has the same head count
  int grad_bf16;                     // grad_value / grad_dist are bfloat16 (binned fused backward on bfloat16 storage only)
  int clear_grads;                   // grad_value / grad_dist hold anything on entry (fused backward only): clear what is added to
  int B, S, M, C, D, L, Q, P;
  int iters;
  int vec_hint;
#ifdef DFA3D_EXPERIMENT
  int diag;                          // development builds only: parts of the kernels cut out
  int stage;                         // development builds only: 1 binning kernels only, 2 tile kernel only
#endif
  int tile_hint;                     // binned path: tile edge as ty * 100 + tx (0 = automatic)
  int block_hint;                    // binned path: threads per tile workgroup (0 = 512)
  int chunk_hint;                    // binned path: points of a bin per work item (0 = 4096)
  int pass_hint;                     // binned path: points per pass, 64, 128 or 256 (0 = automatic)
  void *event_binned;                // hipEvent_t recorded between the binning kernels and the tile kernel, or nullptr
};

struct DepthScoreBwdArgs {
  const void *dist; const int64_t *shapes3, *level_start; const void *loc3, *grad_score;
  void *grad_dist, *grad_loc3;
  int B, S, M, D, L, Q, P;
};

hipError_t launch_forward(const FwdArgs &a, int dtype, hipStream_t stream);
hipError_t launch_pack_dist(const void *dist, const int64_t *shapes3, const int64_t *level_start, void *packed, int B,
                            int S, int D, int L, int dtype, hipStream_t stream);
hipError_t launch_depth_score(const DepthScoreArgs &a, int dtype, hipStream_t stream);
hipError_t launch_backward(const BwdArgs &a, int dtype, hipStream_t stream);
hipError_t launch_depth_score_backward(const DepthScoreBwdArgs &a, int dtype, hipStream_t stream);
// Binned (LDS-accumulating) backward kernels; hipErrorNotSupported = use the direct launcher instead.
// kind 0: both stages, 1: stage 2 alone, 2: stage 1 alone.
size_t binned_backward_workspace_bytes(const BwdArgs &a, int kind, int dtype);
hipError_t launch_backward_binned(const BwdArgs &a, int dtype, void *workspace, size_t workspace_bytes,
                                  hipStream_t stream);
// Zero fill by a kernel (no memset node: callers may capture the stream in a graph); bytes a multiple of 4.
hipError_t launch_zero_fill(void *dst, size_t bytes, hipStream_t stream);
size_t binned_depth_score_backward_workspace_bytes(const DepthScoreBwdArgs &d, int dtype, int tile_hint);
hipError_t launch_depth_score_backward_binned(const DepthScoreBwdArgs &d, int dtype, void *workspace,
                                              size_t workspace_bytes, int tile_hint, int chunk_hint,
                                              void *event_binned, hipStream_t stream);

#ifdef DFA3D_EXPERIMENT
size_t tile_timer_offset();
#endif

// Camera re-batching (dfa3d_rebatch.hip); strides in elements.
hipError_t launch_rebatch_gather(const void *src, long long cam_stride, long long batch_stride, const int *index,
                                 const void *scale, void *dst, int bs, int cams, int max_len, int Nq, int E,
                                 int dtype, hipStream_t stream);
hipError_t launch_rebatch_combine(const void *src, const int *pos, const void *scale, void *dst, int bs, int cams,
                                  int max_len, int Nq, int E, int dtype, hipStream_t stream);

}  // namespace dfa3d
