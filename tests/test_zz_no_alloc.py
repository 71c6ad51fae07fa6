"""dfa3d_fused_backward_static (the backward on the library's own static scratch buffer, for callers that cannot
allocate device memory) against dfa3d_fused_backward with a caller-provided workspace and against the CPU checker,
through the C ABI."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _operands(w, dev):
    from dfa3D.workloads import make_inputs
    inp = make_inputs(w, device=dev)
    return (inp["value"], inp["value_dpt_dist"], inp["spatial_shapes"], inp["level_start_index"],
            inp["sampling_locations"], inp["attention_weights"], inp["grad_output"])


def _backward(entry, ops, workspace):
    """One call of `entry` ("dfa3d_fused_backward" with a workspace tensor, "dfa3d_fused_backward_static" without)."""
    from dfa3D import _lib
    L = _lib.lib()
    value, dist, shapes, lsi, loc, attn, go = ops
    B, S, M, C = value.shape
    D = dist.shape[3]
    _, Q, _, Lv, P, _ = loc.shape
    gv, gd = torch.zeros_like(value), torch.zeros_like(dist)
    gl, ga = torch.full_like(loc, float("nan")), torch.full_like(attn, float("nan"))
    head = [_lib.ptr(t) for t in (value, dist, shapes, lsi, loc, attn, go)] + [None, None] + \
           [_lib.ptr(t) for t in (gv, gd, gl, ga)]
    tail = [B, S, M, C, D, Lv, Q, P, M, _lib.DFA3D_F32, None, _lib.stream_of(value)]
    if workspace is not None:
        rc = L.dfa3d_fused_backward(*head, _lib.ptr(workspace), workspace.numel(), *tail)
    else:
        rc = L.dfa3d_fused_backward_static(*head, *tail)
    _lib.check(rc, entry)
    torch.cuda.synchronize()
    return gv, gd, gl, ga


def test_static_scratch_backward_matches_workspace_backward(oracle):
    from dfa3D import _lib
    from dfa3D.workloads import WORKLOADS, scaled
    assert torch.cuda.is_available(), "needs the MI355X"
    dev = torch.device("cuda:0")
    L = _lib.lib()
    cap = L.dfa3d_static_scratch_bytes()
    assert cap == 32 << 20
    # two calls in a row on the one static buffer, the second with a smaller input: the BEVFormer-small workload
    # (1.5 M points, 29.8 MiB of scratch) and then a sixth of it with other locations
    for w in (WORKLOADS["small"], scaled(WORKLOADS["small"], B=2, Q=1900)):
        ops = _operands(w, dev)
        value, dist, _, _, loc, _, _ = ops
        B, S, M, C = value.shape
        need = L.dfa3d_fused_backward_workspace_bytes(B, S, M, C, dist.shape[3], loc.shape[3], loc.shape[1], loc.shape[4],
                                                      M, _lib.DFA3D_F32, None)
        assert 0 < need <= cap, (need, cap)
        print("static scratch case", w.name, "needs", need, flush=True)
        want = _backward("dfa3d_fused_backward", ops, torch.empty(need, dtype=torch.uint8, device=dev))
        got = _backward("dfa3d_fused_backward_static", ops, None)
        cpu = [t.cpu() for t in ops]
        _, score = oracle.dfa3d_forward(*cpu[:6])
        checker = oracle.dfa3d_backward(*cpu[:6], score, cpu[6])
        for name, g, x, c in zip(("grad_value", "grad_dist", "grad_loc", "grad_attn"), got, want, checker):
            assert torch.isfinite(g).all(), name
            # same kernels on the same bins: only the order of the atomic adds on tile rims differs
            torch.testing.assert_close(g, x, rtol=1e-4, atol=1e-4, msg=lambda m, n=name: f"{n}: {m}")
            # and the float32 backward gate against the CPU checker
            torch.testing.assert_close(g.cpu(), c, rtol=1e-4, atol=1e-4, msg=lambda m, n=name: f"{n} vs checker: {m}")


def test_static_scratch_backward_rejects_what_does_not_fit():
    from dfa3D import _lib
    L = _lib.lib()
    one, null = ctypes.c_void_p(256), ctypes.c_void_p(0)        # never dereferenced: the size check comes first
    # BEVFormer-base: 301 MiB of scratch wanted
    rc = L.dfa3d_fused_backward_static(*([one] * 7), None, None, *([one] * 4), 6, 30825, 8, 32, 64, 4, 10000, 8, 8, 0,
                                       None, null)
    assert rc == -2 and b"static buffer holds" in L.dfa3d_last_error()
    rc = L.dfa3d_fused_backward_static(null, *([one] * 6), None, None, *([one] * 4), 1, 100, 8, 32, 16, 2, 5, 4, 8, 0,
                                       None, null)
    assert rc == -1 and b"NULL" in L.dfa3d_last_error()
