/*
 * libdfa3d_hip - DFA3D (3D deformable attention) operator for AMD MI355X (gfx950).
 *
 * C ABI of the shared library.  Every pointer except `stream` is a DEVICE pointer
 * into memory the caller owns; the library allocates nothing, keeps no state
 * besides a thread-local error string and per-device launch attributes it has looked up once,
 * launches on `stream` (a hipStream_t, NULL = the default stream) and returns without
 * synchronising.  Return value: 0 on
 * success, a negative DFA3D_E* code for a rejected argument, a positive
 * hipError_t for a failed launch; dfa3d_last_error() describes the last failure
 * of the calling thread.
 *
 * Tensor layouts (all contiguous, row-major), with
 *   B batch, S = sum_l H_l*W_l keys, M heads, C channels per head, D depth bins,
 *   L levels, Q queries, P points per level:
 *     value        (B,S,M,C)            dist        (B,S,M,D)
 *     shapes       (L,shape_stride) int64, row = (H, W[, Dd]); shape_stride is 2 or 3
 *     level_start  (L) int64, first key of each level
 *     loc          (B,Q,M,L,P,loc_stride), (x, y[, z]) normalised to [0,1]; loc_stride 2 or 3
 *     attn         (B,Q,M,L,P)          score       (B,Q,M,L,P,4)  slots LT,RT,RB,LB
 *     out          (B,Q,M*C)
 *
 * dtype selects the element types:
 *     DFA3D_F32   every floating tensor float
 *     DFA3D_F64   every floating tensor double
 *     DFA3D_BF16  value, dist, out, score are bfloat16; loc, attn and EVERY gradient
 *                 buffer are float (accumulation is float throughout)
 *     DFA3D_BF16G dfa3d_fused_backward / dfa3d_fused_backward_static only: as DFA3D_BF16, and grad_value and
 *                 grad_dist are bfloat16 as well (what an autograd caller has to return for bfloat16 inputs):
 *                 sums are formed in float in LDS and rounded once when a tile is written; the rows that
 *                 several tiles share are added with the hardware's packed bfloat16 atomic, which rounds the
 *                 stored sum at each of the few adds.  Offered on the binned kernels only
 *                 (dfa3d_fused_backward_workspace_bytes(..., DFA3D_BF16G, ...) > 0: C and D multiples of 4)
 *
 * The four *_forward / *_backward pairs replace the reference's four native entry
 * points one for one; the two dfa3d_fused_* calls run both stages in one kernel.
 */
#ifndef DFA3D_H
#define DFA3D_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DFA3D_F32 0
#define DFA3D_F64 1
#define DFA3D_BF16 2
#define DFA3D_BF16G 3

#define DFA3D_MAX_LEVELS 16

/* Launch options of ONE call.  NULL, or a zero-filled structure, means the defaults.  They choose how the
 * work is laid out on the machine (and, `clear`, who zeroes two output buffers) and never what is computed:
 * results agree up to floating-point summation order of grad_value / grad_dist, whatever the values. */
typedef struct dfa3d_launch_options {
  int iters;    /* groups of units each wavefront walks through; 0 = 1, at most 64 */
  int vec;      /* channels per lane in the row gathers: 0 = automatic, 1, 2 or 4 (8: tile kernels only) */
  int direct;   /* non-zero: a backward ignores its workspace and adds straight into device memory */
  int tile;     /* binned backward: tile edge in pixels as ty*100+tx, 0 = automatic */
  int block;    /* binned backward: threads per tile workgroup, 256 or 0/512 */
  int pass;     /* binned backward: points a tile workgroup takes per pass, 64, 128 or 256; 0 = automatic */
  int chunk;    /* binned backward: points of one tile handled by one work item, 0 = 4096 */
  int clear;    /* dfa3d_fused_backward, dfa3d_fused_backward_static and dfa3d_wms_deform_attn_backward only (0
                 * elsewhere): non-zero = grad_value (and grad_dist) may hold anything on entry, the call clears what
                 * its kernels add to instead of storing (a quarter of the buffers with the tile kernel, all of
                 * them otherwise); 0 = they are zero on entry, as the reference's caller makes them */
  void *event_binned;   /* a hipEvent_t, or NULL: a binned backward records it on `stream` between its binning
                         * kernels and its tile kernel, so that a profiler can time the two parts of the call */
} dfa3d_launch_options;

#define DFA3D_EINVAL (-1)   /* null pointer, non-positive dimension, bad stride or dtype */
#define DFA3D_ERANGE (-2)   /* a dimension exceeds what the kernels index (see dfa3d_last_error) */

/* Stage 1 forward: multi-scale depth-score sampling.  Writes every element of `score`.
 * Replaces ms_depth_score_sample_forward
 * (DFA3D/dfa3D/ops/csrc/pybind.cpp:55-59 ->
 *  DFA3D/dfa3D/ops/csrc/cuda/ms_depth_score_sample_cuda.cu:49-111). */
int dfa3d_ms_depth_score_sample_forward(
    const void *dist, const int64_t *shapes3, const int64_t *level_start, const void *loc3,
    void *score,
    int B, int S, int M, int D, int L, int Q, int P, int dtype, const dfa3d_launch_options *opts, void *stream);

/* Stage 1 backward.  `grad_dist` is ACCUMULATED into (caller zero-fills); every element of
 * `grad_loc3` is overwritten, its x and y components with 0.  `workspace` as for
 * dfa3d_fused_backward (size from dfa3d_ms_depth_score_sample_backward_workspace_bytes; NULL =
 * every update is a device-memory atomic).
 * Replaces ms_depth_score_sample_backward
 * (pybind.cpp:60-66 -> ms_depth_score_sample_cuda.cu:137-202). */
int dfa3d_ms_depth_score_sample_backward(
    const void *dist, const int64_t *shapes3, const int64_t *level_start, const void *loc3,
    const void *grad_score,
    void *grad_dist, void *grad_loc3,
    void *workspace, size_t workspace_bytes,
    int B, int S, int M, int D, int L, int Q, int P, int dtype, const dfa3d_launch_options *opts, void *stream);
size_t dfa3d_ms_depth_score_sample_backward_workspace_bytes(int B, int S, int M, int D, int L, int Q, int P,
                                                            int dtype, const dfa3d_launch_options *opts);

/* Stage 2 forward: depth-weighted multi-scale deformable attention.  Writes every element of
 * `out`.  `score` == NULL stands for scores that are all 1: plain multi-scale deformable attention,
 * mmcv's ms_deform_attn_forward as BEVFormer's other attention layers call it
 * (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/multi_scale_deformable_attn_function.py:47-53).
 * Replaces wms_deform_attn_forward
 * (pybind.cpp:43-47 -> DFA3D/dfa3D/ops/csrc/cuda/wms_deform_attn_cuda.cu:213-288). */
int dfa3d_wms_deform_attn_forward(
    const void *value, const int64_t *shapes, int shape_stride, const int64_t *level_start,
    const void *loc, int loc_stride, const void *attn, const void *score,
    void *out,
    int B, int S, int M, int C, int L, int Q, int P, int dtype, const dfa3d_launch_options *opts, void *stream);

/* Stage 2 backward.  `grad_value` must be zero on entry (or options.clear is set) and holds the gradient on return;
 * `grad_loc` (B,Q,M,L,P,grad_loc_stride) gets its first two components overwritten, `grad_attn` and
 * `grad_score` are overwritten (`score` == NULL: scores all 1, `grad_score` may be NULL and is then not
 * written).  `workspace` as for dfa3d_fused_backward (size from
 * dfa3d_wms_deform_attn_backward_workspace_bytes; NULL = device-memory atomics).
 * Replaces wms_deform_attn_backward
 * (pybind.cpp:48-54 -> wms_deform_attn_cuda.cu:291-370). */
int dfa3d_wms_deform_attn_backward(
    const void *value, const int64_t *shapes, int shape_stride, const int64_t *level_start,
    const void *loc, int loc_stride, const void *attn, const void *score, const void *grad_out,
    void *grad_value, void *grad_loc, int grad_loc_stride, void *grad_attn, void *grad_score,
    void *workspace, size_t workspace_bytes,
    int B, int S, int M, int C, int L, int Q, int P, int dtype, const dfa3d_launch_options *opts, void *stream);
size_t dfa3d_wms_deform_attn_backward_workspace_bytes(int B, int S, int M, int C, int L, int Q, int P, int dtype,
                                                      const dfa3d_launch_options *opts);

/* Both stages in one kernel: what the reference's one-stage autograd Function does with two
 * native calls and two slice copies
 * (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/multi_scale_3ddeformable_attn_function.py:279-303).
 * Writes every element of `out` and, when they are not NULL, of `score` (B,Q,M,L,P,4) and of
 * `weight_update` (B,Q,M; float for DFA3D_F32 / DFA3D_BF16, double for DFA3D_F64).
 *
 * `dist_heads` is M for a distribution per head, dist (B,S,M,D), or 1 for one distribution shared by
 * all heads, dist (B,S,1,D): what the reference's caller builds with an 8-fold repeat
 * (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:496-497).
 * weight_update[b,q,m] = sum over (l,p) of attn * mean of the four corner scores: the reduction that
 * caller applies to the score tensor right after the call (spatial_cross_attention.py:579).
 *
 * `packed_dist` (may be NULL; dist_heads = 1 only) is the same distribution as dfa3d_pack_dist lays it out: the
 * eight depth taps of a sampling point then come from one cache line instead of four, and the distribution no
 * longer competes with the value rows for the L2.  Results are identical. */
int dfa3d_fused_forward(
    const void *value, const void *dist, const int64_t *shapes3, const int64_t *level_start,
    const void *loc3, const void *attn,
    void *out, void *score, void *weight_update, const void *packed_dist,
    int B, int S, int M, int C, int D, int L, int Q, int P, int dist_heads, int dtype,
    const dfa3d_launch_options *opts, void *stream);

/* Packs a distribution shared by all heads, dist (B,S,1,D), for the forward: for every level, every base pixel
 * (h0, w0) with -1 <= h0 < H, -1 <= w0 < W and every bin d, the values of the four pixels (h0, w0), (h0, w0+1),
 * (h0+1, w0+1), (h0+1, w0) side by side (zero outside the map), i.e. 4 (H+1)(W+1) D elements per level and batch
 * element.  No counterpart in the reference, whose caller repeats the distribution per head instead
 * (spatial_cross_attention.py:496-497).  A caller that runs several attention layers on one distribution
 * (DFA3D-BEVFormer's six encoder layers do) packs once.  `packed` holds at least dfa3d_packed_dist_bytes(...)
 * bytes (an upper bound from S and L, since the level shapes live on the device; 0 = not offered: D < 2,
 * DFA3D_F64, or a batch element of the table at or above 2^30 bytes); every byte the forward reads is written. */
size_t dfa3d_packed_dist_bytes(int B, int S, int D, int L, int dtype);
int dfa3d_pack_dist(const void *dist, const int64_t *shapes3, const int64_t *level_start, void *packed,
                    size_t packed_bytes, int B, int S, int D, int L, int dtype, void *stream);

/* Backward of dfa3d_fused_forward (…_function.py:306-352: two native calls, six zero fills and
 * a host synchronisation in the reference).  The depth scores are recomputed from `dist`, not
 * read back.  `grad_score_in` (B,Q,M,L,P,4) and `grad_weight_update` (B,Q,M; float / double as
 * above), either of which may be NULL, are incoming gradients with respect to the `score` and
 * `weight_update` outputs and are chained into grad_dist, grad_attn and the z gradient.
 * `grad_value` (B,S,M,C) and `grad_dist` (B,S,dist_heads,D) must be zero on entry, as the reference's are,
 * unless options.clear is set (then they may hold anything: the call clears what it does not overwrite),
 * and hold the gradients on return; `grad_loc3` and `grad_attn` are overwritten.
 *
 * `workspace` (may be NULL) is caller-owned scratch device memory, 256-byte aligned, of at least
 * dfa3d_fused_backward_workspace_bytes(...) bytes, whose contents need not be preserved or
 * initialised.  With it (DFA3D_F32 / DFA3D_BF16) the sampling points are first binned by image tile
 * and every tile of grad_value / grad_dist is accumulated in LDS and written once; without it every
 * update is a device-memory atomic, which is several times slower.  Results agree up to
 * floating-point summation order. */
int dfa3d_fused_backward(
    const void *value, const void *dist, const int64_t *shapes3, const int64_t *level_start,
    const void *loc3, const void *attn, const void *grad_out, const void *grad_score_in,
    const void *grad_weight_update,
    void *grad_value, void *grad_dist, void *grad_loc3, void *grad_attn,
    void *workspace, size_t workspace_bytes,
    int B, int S, int M, int C, int D, int L, int Q, int P, int dist_heads, int dtype,
    const dfa3d_launch_options *opts, void *stream);

/* Scratch bytes dfa3d_fused_backward wants for these dimensions; 0 when the binned path does not
 * apply (DFA3D_F64, rows too long for LDS tiles, more than 2^31 points, invalid dimensions).  With
 * dist_heads = 1 this includes B*S*M*D floats: grad_dist is formed per head and summed over the heads
 * by a last kernel. */
size_t dfa3d_fused_backward_workspace_bytes(int B, int S, int M, int C, int D, int L, int Q, int P, int dist_heads,
                                            int dtype, const dfa3d_launch_options *opts);

/* dfa3d_fused_backward for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * results as dfa3d_fused_backward, without the workspace: the scratch memory of the binned kernels is a static
 * array of DFA3D_STATIC_SCRATCH_BYTES inside the library's code object, which every GPU the library runs on
 * holds until the process ends.  The call allocates and frees nothing.  Dimensions whose
 * dfa3d_fused_backward_workspace_bytes exceeds that size are rejected with DFA3D_ERANGE (at the BEVFormer-small
 * shape, 1.5 M sampling points, the kernels want 29.8 MiB); dimensions the binned path does not apply to
 * (workspace size 0, e.g. DFA3D_F64) run on the direct kernels, which need no scratch.
 * Every call on one GPU uses that GPU's one array: calls that overlap in time on the same GPU (two streams, two
 * threads) race and give wrong gradients; calls on one stream, or otherwise ordered, are safe, and nothing has
 * to be cleared between them. */
#define DFA3D_STATIC_SCRATCH_BYTES (32u << 20)
int dfa3d_fused_backward_static(
    const void *value, const void *dist, const int64_t *shapes3, const int64_t *level_start,
    const void *loc3, const void *attn, const void *grad_out, const void *grad_score_in,
    const void *grad_weight_update,
    void *grad_value, void *grad_dist, void *grad_loc3, void *grad_attn,
    int B, int S, int M, int C, int D, int L, int Q, int P, int dist_heads, int dtype,
    const dfa3d_launch_options *opts, void *stream);
size_t dfa3d_static_scratch_bytes(void);

/* Camera re-batching around the operator, as DFA3D-BEVFormer's spatial cross-attention does it in python
 * loops over batch x cameras
 * (BEVFormer_DFA3D/projects/mmdet3d_plugin/bevformer/modules/spatial_cross_attention.py:716-722, 741-748).
 * `index` (cams, max_len) int32 lists the BEV queries that project into each camera, padded with -1;
 * `pos` (cams, Nq) int32 is its inverse: the position of query q in camera i's list, or -1.  Rows have E
 * contiguous elements; DFA3D_F32 or DFA3D_F64.
 *
 * gather:  dst[j,i,k,:] = scale[j,q] * src[i*cam_stride + j*batch_stride + q*E + :], q = index[i,k]; zeros for
 *          padding.  dst is (bs, cams, max_len, E); strides are in elements (cam_stride 0: one source for all
 *          cameras); scale (bs, Nq) may be NULL.  Replaces :716-722; also the backward of the combine.
 * combine: dst[j,q,:] = scale[j,q] * sum over cameras i with pos[i,q] >= 0 of src[j,i,pos[i,q],:], cameras in
 *          order, no atomics.  src is (bs, cams, max_len, E), dst (bs, Nq, E), every element written; with
 *          scale = 1 / max(number of cameras seeing q, 1) this replaces :741-748; also the backward of the gather. */
int dfa3d_rebatch_gather(const void *src, long long cam_stride, long long batch_stride, const int32_t *index,
                         const void *scale, void *dst, int bs, int cams, int max_len, int Nq, int E, int dtype,
                         void *stream);
int dfa3d_rebatch_combine(const void *src, const int32_t *pos, const void *scale, void *dst, int bs, int cams,
                          int max_len, int Nq, int E, int dtype, void *stream);

/* Message for the last non-zero return on the calling thread ("" if none). */
const char *dfa3d_last_error(void);

/* Library ABI version (bumped when a signature changes). */
int dfa3d_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* DFA3D_H */
