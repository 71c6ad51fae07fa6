// C ABI of libdfa3d_hip (declared in include/dfa3d.h): argument checks and dispatch.
// Errors are returned, never printed-and-ignored (the reference's launchers only printf a failed
// launch: DFA3D/dfa3D/ops/csrc/cuda/wms_deform_attn_cuda.cu:45-48).
#include <atomic>
#include <mutex>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/dfa3d.h"
#include "dfa3d_launch.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_result(hipError_t e, const char *what) {
  if (e == hipSuccess) return 0;
  return fail((int)e, "%s: %s", what, hipGetErrorString(e));
}

// Launch options of one call, checked.  A NULL pointer stands for the defaults.
int check_opts(const char *fn, const dfa3d_launch_options *o, dfa3d_launch_options *out, bool clear_ok = false) {
  dfa3d_launch_options r;
  memset(&r, 0, sizeof(r));
  if (o != nullptr) r = *o;
  if (r.iters < 0 || r.iters > 64) return fail(DFA3D_EINVAL, "%s: options.iters must be in [0, 64]", fn);
  if (r.iters == 0) r.iters = 1;
  if (r.vec != 0 && r.vec != 1 && r.vec != 2 && r.vec != 4 && r.vec != 8)
    return fail(DFA3D_EINVAL, "%s: options.vec must be 0 (automatic), 1, 2, 4 or 8", fn);
  const int ty = r.tile / 100, tx = r.tile % 100;
  if (r.tile != 0 && (r.tile < 0 || ty < 1 || tx < 1 || ty > 64 || tx > 64))
    return fail(DFA3D_EINVAL, "%s: options.tile must be 0 or ty*100+tx with 1 <= ty, tx <= 64", fn);
  if (r.block != 0 && r.block != 256 && r.block != 512)
    return fail(DFA3D_EINVAL, "%s: options.block must be 0, 256 or 512", fn);
  if (r.pass != 0 && r.pass != 64 && r.pass != 128 && r.pass != 256)
    return fail(DFA3D_EINVAL, "%s: options.pass must be 0, 64, 128 or 256", fn);
  if (r.chunk != 0 && (r.chunk < 64 || r.chunk > (1 << 20)))   // 64 = kMinChunk of the binned backward
    return fail(DFA3D_EINVAL, "%s: options.chunk must be 0 or in [64, 2^20]", fn);
  if (r.clear != 0 && r.clear != 1) return fail(DFA3D_EINVAL, "%s: options.clear must be 0 or 1", fn);
  if (r.clear != 0 && !clear_ok)
    return fail(DFA3D_EINVAL, "%s: options.clear is for dfa3d_fused_backward, dfa3d_fused_backward_static and "
                "dfa3d_wms_deform_attn_backward: this call's gradient buffers must be zero on entry", fn);
  *out = r;
  return 0;
}

#ifdef DFA3D_EXPERIMENT
// Development builds only: switches that cut parts out of the backward kernels to see what they cost
// (results are then incomplete).  Not part of the library's ABI.
std::atomic<int> g_diag{0};
std::atomic<int> g_stage{0};
#endif

void apply_opts(dfa3d::BwdArgs &a, const dfa3d_launch_options &o) {
  a.iters = o.iters; a.vec_hint = o.vec; a.tile_hint = o.tile; a.block_hint = o.block; a.chunk_hint = o.chunk;
  a.pass_hint = o.pass; a.event_binned = o.event_binned; a.clear_grads = o.clear;
#ifdef DFA3D_EXPERIMENT
  a.diag = g_diag.load(std::memory_order_relaxed);
  a.stage = g_stage.load(std::memory_order_relaxed);
#endif
}

// Dimension checks shared by every entry point.  `width` is the per-head row length (C or D).
int check_dims(const char *fn, int B, int S, int M, int width, int L, int Q, int P, int dtype) {
  if (dtype != DFA3D_F32 && dtype != DFA3D_F64 && dtype != DFA3D_BF16)
    return fail(DFA3D_EINVAL, "%s: unknown dtype %d%s", fn, dtype,
                dtype == DFA3D_BF16G ? " (DFA3D_BF16G is for the dfa3d_fused_backward calls only)" : "");
  if (B <= 0 || S <= 0 || M <= 0 || width <= 0 || L <= 0 || Q <= 0 || P <= 0)
    return fail(DFA3D_EINVAL, "%s: dimensions must be positive (B=%d S=%d M=%d C|D=%d L=%d Q=%d P=%d)", fn, B, S, M,
                width, L, Q, P);
  if (L > DFA3D_MAX_LEVELS) return fail(DFA3D_ERANGE, "%s: L=%d exceeds %d levels", fn, L, DFA3D_MAX_LEVELS);
  // one batch element of value / dist and of their gradients is addressed with 32-bit byte
  // offsets that must stay below 2^30 (see kMaxSliceBytes)
  const long long slice = (long long)S * M * width * (dtype == DFA3D_F64 ? 8 : 4);
  if (slice >= (1LL << 30))
    return fail(DFA3D_ERANGE, "%s: one batch element of a (B,S,M,%d) tensor takes %lld bytes, limit is 2^30", fn,
                width, slice);
  if ((long long)L * P > (1 << 20)) return fail(DFA3D_ERANGE, "%s: L*P=%lld too large", fn, (long long)L * P);
  if ((long long)B * Q * M >= (1LL << 40)) return fail(DFA3D_ERANGE, "%s: B*Q*M too large", fn);
  return 0;
}

#define REQUIRE_PTR(fn, p) \
  if ((p) == nullptr) return fail(DFA3D_EINVAL, "%s: %s is NULL", fn, #p)

}  // namespace

extern "C" {

const char *dfa3d_last_error(void) { return g_err; }
int dfa3d_abi_version(void) { return 9; }

#ifdef DFA3D_EXPERIMENT
int dfa3d_experiment_set(const char *name, int value) {
  if (name != nullptr && !strcmp(name, "diag")) { g_diag.store(value, std::memory_order_relaxed); return 0; }
  if (name != nullptr && !strcmp(name, "bwd_stage")) { g_stage.store(value, std::memory_order_relaxed); return 0; }
  return fail(DFA3D_EINVAL, "dfa3d_experiment_set: unknown switch");
}
size_t dfa3d_experiment_timer_offset(void) { return dfa3d::tile_timer_offset(); }
#endif

int dfa3d_ms_depth_score_sample_forward(const void *dist, const int64_t *shapes3, const int64_t *level_start,
                                        const void *loc3, void *score, int B, int S, int M, int D, int L, int Q, int P,
                                        int dtype, const dfa3d_launch_options *opts, void *stream) {
  const char *fn = "dfa3d_ms_depth_score_sample_forward";
  dfa3d_launch_options o;
  if (int rc = check_dims(fn, B, S, M, D, L, Q, P, dtype)) return rc;
  if (int rc = check_opts(fn, opts, &o)) return rc;
  REQUIRE_PTR(fn, dist); REQUIRE_PTR(fn, shapes3); REQUIRE_PTR(fn, level_start);
  REQUIRE_PTR(fn, loc3); REQUIRE_PTR(fn, score);
  dfa3d::DepthScoreArgs a{dist, shapes3, level_start, loc3, score, B, S, M, D, L, Q, P};
  return hip_result(dfa3d::launch_depth_score(a, dtype, (hipStream_t)stream), fn);
}

size_t dfa3d_ms_depth_score_sample_backward_workspace_bytes(int B, int S, int M, int D, int L, int Q, int P,
                                                            int dtype, const dfa3d_launch_options *opts) {
  const char *fn = "dfa3d_ms_depth_score_sample_backward_workspace_bytes";
  dfa3d_launch_options o;
  if (check_dims(fn, B, S, M, D, L, Q, P, dtype) || check_opts(fn, opts, &o)) return 0;
  if (o.direct) return 0;
  dfa3d::DepthScoreBwdArgs a{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, B, S, M, D, L, Q, P};
  return dfa3d::binned_depth_score_backward_workspace_bytes(a, dtype, o.tile);
}

int dfa3d_ms_depth_score_sample_backward(const void *dist, const int64_t *shapes3, const int64_t *level_start,
                                         const void *loc3, const void *grad_score, void *grad_dist, void *grad_loc3,
                                         void *workspace, size_t workspace_bytes,
                                         int B, int S, int M, int D, int L, int Q, int P, int dtype,
                                         const dfa3d_launch_options *opts, void *stream) {
  const char *fn = "dfa3d_ms_depth_score_sample_backward";
  dfa3d_launch_options o;
  if (int rc = check_dims(fn, B, S, M, D, L, Q, P, dtype)) return rc;
  if (int rc = check_opts(fn, opts, &o)) return rc;
  REQUIRE_PTR(fn, dist); REQUIRE_PTR(fn, shapes3); REQUIRE_PTR(fn, level_start); REQUIRE_PTR(fn, loc3);
  REQUIRE_PTR(fn, grad_score); REQUIRE_PTR(fn, grad_dist); REQUIRE_PTR(fn, grad_loc3);
  dfa3d::DepthScoreBwdArgs a{dist, shapes3, level_start, loc3, grad_score, grad_dist, grad_loc3, B, S, M, D, L, Q, P};
  if (workspace != nullptr && !o.direct) {
    const hipError_t e = dfa3d::launch_depth_score_backward_binned(a, dtype, workspace, workspace_bytes, o.tile, o.chunk,
                                                                   o.event_binned, (hipStream_t)stream);
    if (e != hipErrorNotSupported) return hip_result(e, fn);
  }
  return hip_result(dfa3d::launch_depth_score_backward(a, dtype, (hipStream_t)stream), fn);
}

int dfa3d_wms_deform_attn_forward(const void *value, const int64_t *shapes, int shape_stride,
                                  const int64_t *level_start, const void *loc, int loc_stride, const void *attn,
                                  const void *score, void *out, int B, int S, int M, int C, int L, int Q, int P,
                                  int dtype, const dfa3d_launch_options *opts, void *stream) {
  const char *fn = "dfa3d_wms_deform_attn_forward";
  dfa3d_launch_options o;
  if (int rc = check_dims(fn, B, S, M, C, L, Q, P, dtype)) return rc;
  if (int rc = check_opts(fn, opts, &o)) return rc;
  if (shape_stride < 2 || shape_stride > 3 || loc_stride < 2 || loc_stride > 3)
    return fail(DFA3D_EINVAL, "%s: shape_stride and loc_stride must be 2 or 3", fn);
  REQUIRE_PTR(fn, value); REQUIRE_PTR(fn, shapes); REQUIRE_PTR(fn, level_start); REQUIRE_PTR(fn, loc);
  REQUIRE_PTR(fn, attn); REQUIRE_PTR(fn, out);                  // score == NULL: every score is 1
  dfa3d::FwdArgs a{};
  a.value = value; a.dist = nullptr; a.shapes = shapes; a.shape_stride = shape_stride; a.level_start = level_start;
  a.loc = loc; a.loc_stride = loc_stride; a.attn = attn; a.score_in = score; a.out = out; a.score_out = nullptr;
  a.B = B; a.S = S; a.M = M; a.C = C; a.D = 1; a.L = L; a.Q = Q; a.P = P;
  a.iters = o.iters; a.vec_hint = o.vec;
  return hip_result(dfa3d::launch_forward(a, dtype, (hipStream_t)stream), fn);
}

static dfa3d::BwdArgs wms_bwd_args(const void *value, const int64_t *shapes, int shape_stride,
                                   const int64_t *level_start, const void *loc, int loc_stride, const void *attn,
                                   const void *score, const void *grad_out, void *grad_value, void *grad_loc,
                                   int grad_loc_stride, void *grad_attn, void *grad_score, int B, int S, int M, int C,
                                   int L, int Q, int P, const dfa3d_launch_options &o) {
  dfa3d::BwdArgs a{};
  a.value = value; a.dist = nullptr; a.shapes = shapes; a.shape_stride = shape_stride; a.level_start = level_start;
  a.loc = loc; a.loc_stride = loc_stride; a.attn = attn; a.score_in = score; a.grad_out = grad_out;
  a.grad_score_in = nullptr; a.grad_value = grad_value; a.grad_dist = nullptr; a.grad_loc = grad_loc;
  a.grad_loc_stride = grad_loc_stride; a.grad_attn = grad_attn; a.grad_score_out = grad_score;
  a.B = B; a.S = S; a.M = M; a.C = C; a.D = 1; a.L = L; a.Q = Q; a.P = P;
  apply_opts(a, o);
  return a;
}

size_t dfa3d_wms_deform_attn_backward_workspace_bytes(int B, int S, int M, int C, int L, int Q, int P, int dtype,
                                                      const dfa3d_launch_options *opts) {
  const char *fn = "dfa3d_wms_deform_attn_backward_workspace_bytes";
  dfa3d_launch_options o;
  if (check_dims(fn, B, S, M, C, L, Q, P, dtype) || check_opts(fn, opts, &o, true)) return 0;
  if (o.direct) return 0;
  const dfa3d::BwdArgs a = wms_bwd_args(nullptr, nullptr, 2, nullptr, nullptr, 2, nullptr, nullptr, nullptr, nullptr,
                                        nullptr, 2, nullptr, nullptr, B, S, M, C, L, Q, P, o);
  return dfa3d::binned_backward_workspace_bytes(a, 1, dtype);
}

int dfa3d_wms_deform_attn_backward(const void *value, const int64_t *shapes, int shape_stride,
                                   const int64_t *level_start, const void *loc, int loc_stride, const void *attn,
                                   const void *score, const void *grad_out, void *grad_value, void *grad_loc,
                                   int grad_loc_stride, void *grad_attn, void *grad_score,
                                   void *workspace, size_t workspace_bytes, int B, int S, int M, int C,
                                   int L, int Q, int P, int dtype, const dfa3d_launch_options *opts, void *stream) {
  const char *fn = "dfa3d_wms_deform_attn_backward";
  dfa3d_launch_options o;
  if (int rc = check_dims(fn, B, S, M, C, L, Q, P, dtype)) return rc;
  if (int rc = check_opts(fn, opts, &o, true)) return rc;
  if (shape_stride < 2 || shape_stride > 3 || loc_stride < 2 || loc_stride > 3 || grad_loc_stride < 2 ||
      grad_loc_stride > 3)
    return fail(DFA3D_EINVAL, "%s: shape_stride, loc_stride and grad_loc_stride must be 2 or 3", fn);
  REQUIRE_PTR(fn, value); REQUIRE_PTR(fn, shapes); REQUIRE_PTR(fn, level_start); REQUIRE_PTR(fn, loc);
  REQUIRE_PTR(fn, attn); REQUIRE_PTR(fn, grad_out); REQUIRE_PTR(fn, grad_value);
  REQUIRE_PTR(fn, grad_loc); REQUIRE_PTR(fn, grad_attn);
  if (score != nullptr) REQUIRE_PTR(fn, grad_score);            // score == NULL: every score is 1, no gradient for it
  const dfa3d::BwdArgs a = wms_bwd_args(value, shapes, shape_stride, level_start, loc, loc_stride, attn, score,
                                        grad_out, grad_value, grad_loc, grad_loc_stride, grad_attn, grad_score, B, S,
                                        M, C, L, Q, P, o);
  if (workspace != nullptr && !o.direct) {
    const hipError_t e = dfa3d::launch_backward_binned(a, dtype, workspace, workspace_bytes, (hipStream_t)stream);
    if (e != hipErrorNotSupported) return hip_result(e, fn);
  }
  if (a.clear_grads) {          // the direct kernels add every term into grad_value: all of it is cleared first
    if (hipError_t e = dfa3d::launch_zero_fill(grad_value, (size_t)B * S * M * C * (dtype == DFA3D_F64 ? 8 : 4),
                                               (hipStream_t)stream))
      return hip_result(e, fn);
  }
  return hip_result(dfa3d::launch_backward(a, dtype, (hipStream_t)stream), fn);
}

// cells of a packed distribution: sum over levels of (H + 1)(W + 1) <= sum of (2 H W + 2) <= 2 S + 2 L for levels that
// share no keys; the kernels check the level table they find on the device against the same bound
static long long packed_cells_bound(int S, int L) { return 2LL * S + 2LL * L; }

size_t dfa3d_packed_dist_bytes(int B, int S, int D, int L, int dtype) {
  if (B <= 0 || S <= 0 || D < 2 || L <= 0 || L > DFA3D_MAX_LEVELS || (dtype != DFA3D_F32 && dtype != DFA3D_BF16)) return 0;
  const long long slice = packed_cells_bound(S, L) * D * 4 * (dtype == DFA3D_F32 ? 4 : 2);
  if (slice >= (1LL << 30)) return 0;
  return (size_t)slice * B;
}

int dfa3d_pack_dist(const void *dist, const int64_t *shapes3, const int64_t *level_start, void *packed,
                    size_t packed_bytes, int B, int S, int D, int L, int dtype, void *stream) {
  const char *fn = "dfa3d_pack_dist";
  REQUIRE_PTR(fn, dist); REQUIRE_PTR(fn, shapes3); REQUIRE_PTR(fn, level_start); REQUIRE_PTR(fn, packed);
  const size_t need = dfa3d_packed_dist_bytes(B, S, D, L, dtype);
  if (need == 0)
    return fail(DFA3D_EINVAL, "%s: not offered for these dimensions (needs D >= 2, DFA3D_F32 or DFA3D_BF16, and a batch "
                "element of the packed table below 2^30 bytes)", fn);
  if (packed_bytes < need) return fail(DFA3D_EINVAL, "%s: packed holds %zu bytes, %zu are needed", fn, packed_bytes, need);
  return hip_result(dfa3d::launch_pack_dist(dist, shapes3, level_start, packed, B, S, D, L, dtype, (hipStream_t)stream), fn);
}

int dfa3d_fused_forward(const void *value, const void *dist, const int64_t *shapes3, const int64_t *level_start,
                        const void *loc3, const void *attn, void *out, void *score, void *weight_update,
                        const void *packed_dist, int B, int S,
                        int M, int C, int D, int L, int Q, int P, int dist_heads, int dtype,
                        const dfa3d_launch_options *opts, void *stream) {
  const char *fn = "dfa3d_fused_forward";
  dfa3d_launch_options o;
  if (int rc = check_dims(fn, B, S, M, C, L, Q, P, dtype)) return rc;
  if (int rc = check_dims(fn, B, S, M, D, L, Q, P, dtype)) return rc;
  if (int rc = check_opts(fn, opts, &o)) return rc;
  if (dist_heads != M && dist_heads != 1) return fail(DFA3D_EINVAL, "%s: dist_heads must be M or 1", fn);
  if (packed_dist != nullptr && (dist_heads != 1 || dfa3d_packed_dist_bytes(B, S, D, L, dtype) == 0))
    return fail(DFA3D_EINVAL, "%s: packed_dist goes with dist_heads = 1 and dimensions dfa3d_packed_dist_bytes accepts", fn);
  REQUIRE_PTR(fn, value); REQUIRE_PTR(fn, dist); REQUIRE_PTR(fn, shapes3); REQUIRE_PTR(fn, level_start);
  REQUIRE_PTR(fn, loc3); REQUIRE_PTR(fn, attn); REQUIRE_PTR(fn, out);
  dfa3d::FwdArgs a{};
  a.value = value; a.dist = dist; a.shapes = shapes3; a.shape_stride = 3; a.level_start = level_start;
  a.loc = loc3; a.loc_stride = 3; a.attn = attn; a.score_in = nullptr; a.out = out; a.score_out = score;
  a.weight_update = weight_update; a.dist_heads = dist_heads; a.packed_dist = packed_dist;
  a.B = B; a.S = S; a.M = M; a.C = C; a.D = D; a.L = L; a.Q = Q; a.P = P;
  a.iters = o.iters; a.vec_hint = o.vec;
  return hip_result(dfa3d::launch_forward(a, dtype, (hipStream_t)stream), fn);
}

static dfa3d::BwdArgs fused_bwd_args(const void *value, const void *dist, const int64_t *shapes3,
                                     const int64_t *level_start, const void *loc3, const void *attn,
                                     const void *grad_out, const void *grad_score_in, const void *grad_weight_update,
                                     void *grad_value, void *grad_dist, void *grad_loc3, void *grad_attn, int B, int S,
                                     int M, int C, int D, int L, int Q, int P, int dist_heads,
                                     const dfa3d_launch_options &o) {
  dfa3d::BwdArgs a{};
  a.value = value; a.dist = dist; a.shapes = shapes3; a.shape_stride = 3; a.level_start = level_start;
  a.loc = loc3; a.loc_stride = 3; a.attn = attn; a.score_in = nullptr; a.grad_out = grad_out;
  a.grad_score_in = grad_score_in; a.grad_value = grad_value; a.grad_dist = grad_dist; a.grad_loc = grad_loc3;
  a.grad_loc_stride = 3; a.grad_attn = grad_attn; a.grad_score_out = nullptr;
  a.grad_weight_update = grad_weight_update; a.dist_heads = dist_heads;
  a.B = B; a.S = S; a.M = M; a.C = C; a.D = D; a.L = L; a.Q = Q; a.P = P;
  apply_opts(a, o);
  return a;
}

// The fused backward on the direct kernels, which add every term straight into grad_value / grad_dist: with
// options.clear the whole of both buffers is cleared first (float or double gradients here).
static int direct_fused_backward(const char *fn, const dfa3d::BwdArgs &a, int dtype, int dist_heads, hipStream_t stream) {
  if (a.clear_grads) {
    const size_t elem = dtype == DFA3D_F64 ? 8 : 4;
    if (hipError_t e = dfa3d::launch_zero_fill(a.grad_value, (size_t)a.B * a.S * a.M * a.C * elem, stream))
      return hip_result(e, fn);
    if (hipError_t e = dfa3d::launch_zero_fill(a.grad_dist, (size_t)a.B * a.S * dist_heads * a.D * elem, stream))
      return hip_result(e, fn);
  }
  return hip_result(dfa3d::launch_backward(a, dtype, stream), fn);
}

size_t dfa3d_fused_backward_workspace_bytes(int B, int S, int M, int C, int D, int L, int Q, int P, int dist_heads,
                                            int dtype, const dfa3d_launch_options *opts) {
  const char *fn = "dfa3d_fused_backward_workspace_bytes";
  dfa3d_launch_options o;
  const bool g16 = dtype == DFA3D_BF16G;
  if (g16) dtype = DFA3D_BF16;
  if (check_dims(fn, B, S, M, C, L, Q, P, dtype) || check_dims(fn, B, S, M, D, L, Q, P, dtype) ||
      check_opts(fn, opts, &o, true))
    return 0;
  if (o.direct) return 0;
  dfa3d::BwdArgs a = fused_bwd_args(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                                    nullptr, nullptr, nullptr, nullptr, nullptr, B, S, M, C, D, L, Q, P,
                                    dist_heads == 1 ? 1 : M, o);
  a.grad_bf16 = g16;
  return dfa3d::binned_backward_workspace_bytes(a, 0, dtype);
}

int dfa3d_fused_backward(const void *value, const void *dist, const int64_t *shapes3, const int64_t *level_start,
                         const void *loc3, const void *attn, const void *grad_out, const void *grad_score_in,
                         const void *grad_weight_update, void *grad_value, void *grad_dist, void *grad_loc3,
                         void *grad_attn, void *workspace, size_t workspace_bytes, int B, int S, int M,
                         int C, int D, int L, int Q, int P, int dist_heads, int dtype,
                         const dfa3d_launch_options *opts, void *stream) {
  const char *fn = "dfa3d_fused_backward";
  dfa3d_launch_options o;
  const bool g16 = dtype == DFA3D_BF16G;
  if (g16) dtype = DFA3D_BF16;
  if (int rc = check_dims(fn, B, S, M, C, L, Q, P, dtype)) return rc;
  if (int rc = check_dims(fn, B, S, M, D, L, Q, P, dtype)) return rc;
  if (int rc = check_opts(fn, opts, &o, true)) return rc;
  if (dist_heads != M && dist_heads != 1) return fail(DFA3D_EINVAL, "%s: dist_heads must be M or 1", fn);
  REQUIRE_PTR(fn, value); REQUIRE_PTR(fn, dist); REQUIRE_PTR(fn, shapes3); REQUIRE_PTR(fn, level_start);
  REQUIRE_PTR(fn, loc3); REQUIRE_PTR(fn, attn); REQUIRE_PTR(fn, grad_out); REQUIRE_PTR(fn, grad_value);
  REQUIRE_PTR(fn, grad_dist); REQUIRE_PTR(fn, grad_loc3); REQUIRE_PTR(fn, grad_attn);
  dfa3d::BwdArgs a = fused_bwd_args(value, dist, shapes3, level_start, loc3, attn, grad_out, grad_score_in,
                                    grad_weight_update, grad_value, grad_dist, grad_loc3, grad_attn, B, S, M, C,
                                    D, L, Q, P, dist_heads, o);
  a.grad_bf16 = g16;
  if (workspace != nullptr && !o.direct) {
    const hipError_t e = dfa3d::launch_backward_binned(a, dtype, workspace, workspace_bytes, (hipStream_t)stream);
    if (e != hipErrorNotSupported) return hip_result(e, fn);
  }
  if (g16) return fail(DFA3D_EINVAL, "%s: DFA3D_BF16G (bfloat16 gradients) runs on the binned kernels only: pass a "
                       "workspace of dfa3d_fused_backward_workspace_bytes(..., DFA3D_BF16G, ...) bytes (0 = not offered "
                       "for these dimensions: use DFA3D_BF16 with float gradients)", fn);
  return direct_fused_backward(fn, a, dtype, dist_heads, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------
// dfa3d_fused_backward_static: the binned backward on a scratch buffer that is part of the library's
// code object instead of memory the caller allocates.  Each GPU holds its own copy of the array at its
// own address; host code must not use the array's name as a pointer (it is a host-side stand-in), so the
// device address is asked for once per device and kept.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[DFA3D_STATIC_SCRATCH_BYTES];

static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[kMaxDevices];          // device address of `scratch` on each GPU, nullptr = not asked yet

// Device address of this GPU's copy of `scratch` (the current device's), looked up on first use.
static int static_scratch(const char *fn, void **out) {
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev)) return hip_result(e, fn);
  if (dev < 0 || dev >= kMaxDevices) return fail(DFA3D_ERANGE, "%s: device ordinal %d not supported", fn, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) return hip_result(e, fn);
    if (p == nullptr || ((uintptr_t)p & 255) != 0) return fail(DFA3D_EINVAL, "%s: bad address for the static scratch", fn);
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

size_t dfa3d_static_scratch_bytes(void) { return DFA3D_STATIC_SCRATCH_BYTES; }

int dfa3d_fused_backward_static(const void *value, const void *dist, const int64_t *shapes3,
                                const int64_t *level_start, const void *loc3, const void *attn,
                                const void *grad_out, const void *grad_score_in, const void *grad_weight_update,
                                void *grad_value, void *grad_dist, void *grad_loc3, void *grad_attn, int B, int S,
                                int M, int C, int D, int L, int Q, int P, int dist_heads, int dtype,
                                const dfa3d_launch_options *opts, void *stream) {
  const char *fn = "dfa3d_fused_backward_static";
  dfa3d_launch_options o;
  const bool g16 = dtype == DFA3D_BF16G;
  if (g16) dtype = DFA3D_BF16;
  if (int rc = check_dims(fn, B, S, M, C, L, Q, P, dtype)) return rc;
  if (int rc = check_dims(fn, B, S, M, D, L, Q, P, dtype)) return rc;
  if (int rc = check_opts(fn, opts, &o, true)) return rc;
  if (dist_heads != M && dist_heads != 1) return fail(DFA3D_EINVAL, "%s: dist_heads must be M or 1", fn);
  REQUIRE_PTR(fn, value); REQUIRE_PTR(fn, dist); REQUIRE_PTR(fn, shapes3); REQUIRE_PTR(fn, level_start);
  REQUIRE_PTR(fn, loc3); REQUIRE_PTR(fn, attn); REQUIRE_PTR(fn, grad_out); REQUIRE_PTR(fn, grad_value);
  REQUIRE_PTR(fn, grad_dist); REQUIRE_PTR(fn, grad_loc3); REQUIRE_PTR(fn, grad_attn);
  dfa3d::BwdArgs a = fused_bwd_args(value, dist, shapes3, level_start, loc3, attn, grad_out, grad_score_in,
                                    grad_weight_update, grad_value, grad_dist, grad_loc3, grad_attn, B, S, M, C,
                                    D, L, Q, P, dist_heads, o);
  a.grad_bf16 = g16;
  const size_t need = o.direct ? 0 : dfa3d::binned_backward_workspace_bytes(a, 0, dtype);
  if (need > DFA3D_STATIC_SCRATCH_BYTES)
    return fail(DFA3D_ERANGE, "%s: these dimensions need %zu bytes of scratch, the static buffer holds %zu; use "
                "dfa3d_fused_backward with a workspace", fn, need, (size_t)DFA3D_STATIC_SCRATCH_BYTES);
  if (need > 0) {
    void *ws = nullptr;
    if (int rc = static_scratch(fn, &ws)) return rc;
    const hipError_t e = dfa3d::launch_backward_binned(a, dtype, ws, DFA3D_STATIC_SCRATCH_BYTES, (hipStream_t)stream);
    if (e != hipErrorNotSupported) return hip_result(e, fn);
  }
  if (g16) return fail(DFA3D_EINVAL, "%s: DFA3D_BF16G is not offered for these dimensions", fn);
  return direct_fused_backward(fn, a, dtype, dist_heads, (hipStream_t)stream);   // no scratch needed at all
}

static int check_rebatch(const char *fn, int bs, int cams, int max_len, int Nq, int E, int dtype) {
  if (dtype != DFA3D_F32 && dtype != DFA3D_F64) return fail(DFA3D_EINVAL, "%s: dtype must be DFA3D_F32 or DFA3D_F64", fn);
  if (bs <= 0 || cams <= 0 || max_len <= 0 || Nq <= 0 || E <= 0)
    return fail(DFA3D_EINVAL, "%s: dimensions must be positive (bs=%d cams=%d max_len=%d Nq=%d E=%d)", fn, bs, cams,
                max_len, Nq, E);
  return 0;
}

int dfa3d_rebatch_gather(const void *src, long long cam_stride, long long batch_stride, const int32_t *index,
                         const void *scale, void *dst, int bs, int cams, int max_len, int Nq, int E, int dtype,
                         void *stream) {
  const char *fn = "dfa3d_rebatch_gather";
  if (int rc = check_rebatch(fn, bs, cams, max_len, Nq, E, dtype)) return rc;
  if (cam_stride < 0 || batch_stride < 0) return fail(DFA3D_EINVAL, "%s: strides must not be negative", fn);
  REQUIRE_PTR(fn, src); REQUIRE_PTR(fn, index); REQUIRE_PTR(fn, dst);
  return hip_result(dfa3d::launch_rebatch_gather(src, cam_stride, batch_stride, index, scale, dst, bs, cams, max_len,
                                                 Nq, E, dtype, (hipStream_t)stream), fn);
}

int dfa3d_rebatch_combine(const void *src, const int32_t *pos, const void *scale, void *dst, int bs, int cams,
                          int max_len, int Nq, int E, int dtype, void *stream) {
  const char *fn = "dfa3d_rebatch_combine";
  if (int rc = check_rebatch(fn, bs, cams, max_len, Nq, E, dtype)) return rc;
  REQUIRE_PTR(fn, src); REQUIRE_PTR(fn, pos); REQUIRE_PTR(fn, dst);
  return hip_result(dfa3d::launch_rebatch_combine(src, pos, scale, dst, bs, cams, max_len, Nq, E, dtype,
                                                  (hipStream_t)stream), fn);
}

}  // extern "C"
