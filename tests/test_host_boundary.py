"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol the
header declares, argument validation rejects bad calls before anything is launched, and the
python surface mirrors the reference's names, signatures and error behaviour.  No GPU compute."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dfa3d.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dfa3d_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from dfa3D import _lib
    handle = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 9, names
    for n in names:
        assert hasattr(handle, n), f"{n} declared in include/dfa3d.h but not exported"
    for n in _lib.SIGNATURES:
        assert n in names, f"{n} bound in python but not declared in the header"
    assert _lib.lib().dfa3d_abi_version() == _lib.ABI_VERSION


def test_c_abi_rejects_bad_arguments_without_launching():
    from dfa3D import _lib
    L = _lib.lib()
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(256)          # never dereferenced: validation fails first
    # non-positive dimension
    rc = L.dfa3d_fused_forward(one, one, one, one, one, one, one, one, null, null, 0, 10, 8, 32, 16, 2, 5, 4, 8, 0, None, null)
    assert rc == -1 and b"positive" in L.dfa3d_last_error()
    # unknown dtype
    rc = L.dfa3d_fused_forward(one, one, one, one, one, one, one, one, null, null, 1, 10, 8, 32, 16, 2, 5, 4, 8, 7, None, null)
    assert rc == -1 and b"dtype" in L.dfa3d_last_error()
    # too many levels
    rc = L.dfa3d_fused_forward(one, one, one, one, one, one, one, one, null, null, 1, 10, 8, 32, 16, 17, 5, 4, 8, 0, None, null)
    assert rc == -2 and b"levels" in L.dfa3d_last_error()
    # a batch element beyond 2^30 bytes
    rc = L.dfa3d_fused_forward(one, one, one, one, one, one, one, one, null, null, 1, 1 << 20, 8, 64, 16, 2, 5, 4, 8, 0, None, null)
    assert rc == -2 and b"2^30" in L.dfa3d_last_error()
    # NULL operand
    rc = L.dfa3d_fused_forward(null, one, one, one, one, one, one, one, null, null, 1, 10, 8, 32, 16, 2, 5, 4, 8, 0, None, null)
    assert rc == -1 and b"NULL" in L.dfa3d_last_error()
    # a distribution for 3 of the 8 heads
    rc = L.dfa3d_fused_forward(one, one, one, one, one, one, one, one, null, null, 1, 10, 8, 32, 16, 2, 5, 4, 3, 0, None, null)
    assert rc == -1 and b"dist_heads" in L.dfa3d_last_error()
    rc = L.dfa3d_wms_deform_attn_forward(one, one, 4, one, one, 2, one, one, one, 1, 10, 8, 32, 2, 5, 4, 0, None, null)
    assert rc == -1 and b"stride" in L.dfa3d_last_error()
    rc = L.dfa3d_ms_depth_score_sample_backward(one, one, one, one, one, null, one, null, 0, 1, 10, 8, 16, 2, 5, 4, 0, None,
                                                null)
    assert rc == -1 and b"grad_dist" in L.dfa3d_last_error()
    # camera re-batching: dtype, dimensions, pointers
    rc = L.dfa3d_rebatch_gather(one, 0, 16, one, null, one, 1, 6, 8, 16, 4, 2, null)
    assert rc == -1 and b"dtype" in L.dfa3d_last_error()          # bf16 is not offered
    rc = L.dfa3d_rebatch_gather(one, 0, 16, one, null, one, 1, 6, 0, 16, 4, 0, null)
    assert rc == -1 and b"positive" in L.dfa3d_last_error()
    rc = L.dfa3d_rebatch_gather(one, -1, 16, one, null, one, 1, 6, 8, 16, 4, 0, null)
    assert rc == -1 and b"strides" in L.dfa3d_last_error()
    rc = L.dfa3d_rebatch_combine(one, null, null, one, 1, 6, 8, 16, 4, 0, null)
    assert rc == -1 and b"pos is NULL" in L.dfa3d_last_error()
    dims = (6, 30825, 8, 32, 64, 4, 10000, 8)
    assert L.dfa3d_fused_backward_workspace_bytes(*dims, 1, 0, None) > \
        L.dfa3d_fused_backward_workspace_bytes(*dims, 8, 0, None) > 0
    assert L.dfa3d_fused_backward_workspace_bytes(*dims, 8, 1, None) == 0    # fp64: direct kernels
    # packed head-shared distribution: a bound from S and L (the level shapes live on the device); not for one bin / fp64
    assert L.dfa3d_packed_dist_bytes(6, 30825, 64, 4, 0) == 6 * (2 * 30825 + 8) * 64 * 16
    assert L.dfa3d_packed_dist_bytes(6, 30825, 64, 4, 2) == 6 * (2 * 30825 + 8) * 64 * 8
    assert L.dfa3d_packed_dist_bytes(6, 30825, 1, 4, 0) == 0 and L.dfa3d_packed_dist_bytes(6, 30825, 64, 4, 1) == 0
    rc = L.dfa3d_pack_dist(one, one, one, one, 16, 6, 30825, 64, 4, 0, null)
    assert rc == -1 and b"are needed" in L.dfa3d_last_error()
    rc = L.dfa3d_fused_forward(one, one, one, one, one, one, one, one, null, one, 1, 10, 8, 32, 16, 2, 5, 4, 8, 0, None, null)
    assert rc == -1 and b"packed_dist" in L.dfa3d_last_error()           # a packed table with a distribution per head
    # bfloat16 gradient buffers (DFA3D_BF16G = 3): fused backward only, C and D multiples of 4
    assert L.dfa3d_fused_backward_workspace_bytes(*dims, 8, 3, None) == L.dfa3d_fused_backward_workspace_bytes(*dims, 8, 2, None)
    assert L.dfa3d_fused_backward_workspace_bytes(6, 30825, 8, 32, 63, 4, 10000, 8, 8, 3, None) == 0
    rc = L.dfa3d_fused_forward(one, one, one, one, one, one, one, one, null, null, 1, 10, 8, 32, 16, 2, 5, 4, 8, 3, None, null)
    assert rc == -1 and b"DFA3D_BF16G" in L.dfa3d_last_error()


def test_launch_options_are_per_call_and_checked():
    """Launch options travel with each call (no process-wide state): bad values are rejected before anything
    is launched, `direct` asks for no workspace, and the python context manager restores what it found."""
    from dfa3D import _lib
    L = _lib.lib()
    null, one = ctypes.c_void_p(0), ctypes.c_void_p(256)
    dims = (1, 10, 8, 32, 16, 2, 5, 4)

    def fwd(**fields):
        o = _lib.LaunchOptions(**fields)
        # value is NULL: a call that passes the option checks stops at the operand check
        return L.dfa3d_fused_forward(null, one, one, one, one, one, one, one, null, null, *dims, 8, 0, ctypes.pointer(o), null)

    for bad in (dict(iters=-1), dict(iters=65), dict(vec=3), dict(tile=7), dict(tile=6500), dict(block=128),
                dict(pass_=32), dict(chunk=8), dict(clear=2), dict(clear=1)):   # clear: the fused backward calls only
        assert fwd(**bad) == -1 and b"options." in L.dfa3d_last_error(), bad
    assert fwd(iters=2, vec=4, tile=808, block=256, pass_=128, chunk=1024) == -1 and b"NULL" in L.dfa3d_last_error()
    big = (6, 30825, 8, 32, 64, 4, 10000, 8)
    assert L.dfa3d_fused_backward_workspace_bytes(*big, 8, 0, ctypes.pointer(_lib.LaunchOptions(direct=1))) == 0
    assert L.dfa3d_fused_backward_workspace_bytes(*big, 8, 0, ctypes.pointer(_lib.LaunchOptions(vec=3))) == 0
    assert L.dfa3d_fused_backward_workspace_bytes(*big, 8, 0, ctypes.pointer(_lib.LaunchOptions(clear=1))) == \
        L.dfa3d_fused_backward_workspace_bytes(*big, 8, 0, None)
    assert L.dfa3d_fused_backward_workspace_bytes(*big, 8, 0, ctypes.pointer(_lib.LaunchOptions(tile=404))) > \
        L.dfa3d_fused_backward_workspace_bytes(*big, 8, 0, None)            # more, smaller tiles: more counters
    assert not hasattr(L, "dfa3d_set_tunable") and not hasattr(L, "dfa3d_stream_copy")

    assert _lib.options() is None
    with _lib.launch_options(tile=404, **{"pass": 128}):
        with _lib.launch_options(direct=1):
            o = _lib.options().contents
            assert (o.tile, o.pass_, o.direct) == (404, 128, 1)
        o = _lib.options().contents
        assert (o.tile, o.pass_, o.direct) == (404, 128, 0)
    assert _lib.options() is None
    with pytest.raises(TypeError):
        with _lib.launch_options(nope=1):
            pass


def test_reference_import_paths_and_names():
    from dfa3D import ext_loader
    from dfa3D.ops import MultiScaleDepthScoreSampleFunction, WeightedMultiScaleDeformableAttnFunction  # noqa: F401
    from dfa3D.ops.multi_scale_3D_deform_attn import (MultiScale3DDeformableAttnFunction,  # noqa: F401
                                                      MultiScale3DDeformableAttnFunction_fp16,
                                                      MultiScale3DDeformableAttnFunction_fp32,
                                                      MultiScaleDepthScoreSampleFunction_fp16,
                                                      MultiScaleDepthScoreSampleFunction_fp32,
                                                      WeightedMultiScaleDeformableAttnFunction_fp16,
                                                      WeightedMultiScaleDeformableAttnFunction_fp32)
    ext = ext_loader.load_ext("_ext", ["wms_deform_attn_backward", "wms_deform_attn_forward",
                                       "ms_depth_score_sample_forward", "ms_depth_score_sample_backward"])
    # keyword names of the reference's pybind11 module (pybind.cpp:42-67)
    expect = {
        "wms_deform_attn_forward": ["value", "value_spatial_shapes", "value_level_start_index", "sampling_locations",
                                    "attention_weights", "depth_scores", "im2col_step"],
        "wms_deform_attn_backward": ["value", "value_spatial_shapes", "value_level_start_index", "sampling_locations",
                                     "attention_weights", "depth_scores", "grad_output", "grad_value",
                                     "grad_sampling_loc", "grad_attn_weight", "grad_depth_score", "im2col_step"],
        "ms_depth_score_sample_forward": ["value", "value_spatial_shapes", "value_level_start_index",
                                          "sampling_locations", "im2col_step"],
        "ms_depth_score_sample_backward": ["value", "value_spatial_shapes", "value_level_start_index",
                                           "sampling_locations", "grad_output", "grad_value", "grad_sampling_loc",
                                           "im2col_step"],
    }
    for name, params in expect.items():
        assert list(inspect.signature(getattr(ext, name)).parameters) == params, name
    assert issubclass(MultiScale3DDeformableAttnFunction_fp32, MultiScale3DDeformableAttnFunction)
    fwd = inspect.signature(MultiScale3DDeformableAttnFunction.forward)
    assert list(fwd.parameters) == ["ctx", "value", "value_dpt_dist", "value_spatial_shapes",
                                    "value_level_start_index", "sampling_locations", "attention_weights", "im2col_step"]


def _cpu_operands():
    B, S, M, C, D, L, Q, P = 2, 6, 2, 4, 3, 1, 3, 2
    return dict(
        value=torch.randn(B, S, M, C), dist=torch.rand(B, S, M, D), shapes3=torch.tensor([[2, 3, D]]),
        lsi=torch.tensor([0]), loc=torch.rand(B, Q, M, L, P, 3), attn=torch.rand(B, Q, M, L, P))


def test_errors_mirror_the_reference_launchers():
    """Contiguity / device / im2col_step checks (wms_deform_attn_cuda.cu:220-253) raise RuntimeError."""
    from dfa3D import _ext
    t = _cpu_operands()
    with pytest.raises(RuntimeError, match="value tensor has to be contiguous"):
        _ext.dfa3d_fused_forward(t["value"].transpose(1, 2), t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"], 64)
    with pytest.raises(RuntimeError, match="sampling_loc tensor has to be contiguous"):
        _ext.ms_depth_score_sample_forward(t["dist"], t["shapes3"], t["lsi"], t["loc"].transpose(1, 2), 64)
    # CPU tensors: there is no CPU implementation behind the product surface
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _ext.dfa3d_fused_forward(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"], 64)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _ext.wms_deform_attn_forward(t["value"], t["shapes3"], t["lsi"], t["loc"], t["attn"],
                                     torch.zeros(2, 3, 2, 1, 2, 4), 64)


def test_one_stage_function_refuses_cpu_tensors():
    from dfa3D.functional import MultiScale3DDeformableAttnFunction
    t = _cpu_operands()
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        MultiScale3DDeformableAttnFunction.apply(t["value"], t["dist"], t["shapes3"], t["lsi"], t["loc"], t["attn"], 64)


def test_im2col_step_rule():
    from dfa3D._ext import _step
    assert _step(6, 64) == 6 and _step(6, 3) == 3 and _step(6, 6) == 6
    with pytest.raises(RuntimeError, match="must divide"):
        _step(6, 4)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from dfa3D import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libdfa3d_hip.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.lib()


def test_workload_byte_model_matches_published_table():
    """Algorithmic bytes of the benchmark configurations against hand-computed MB figures."""
    from dfa3D.workloads import WORKLOADS
    w = WORKLOADS["base"]
    assert w.S == 30825 and w.points == 15_360_000 and w.level_start_index() == [0, 23200, 29000, 30450]
    assert round(w.forward_bytes() / 1e6, 1) == 1121.1 and round(w.backward_bytes() / 1e6, 1) == 1935.1
    assert round(w.forward_bytes(2, 2) / 1e6, 1) == 683.4 and round(w.backward_bytes(2, 2) / 1e6, 1) == 1213.3
    assert round(WORKLOADS["small"].forward_bytes() / 1e6, 1) == 90.7
    assert round(WORKLOADS["dense"].forward_bytes() / 1e6, 1) == 3158.8
    assert round(WORKLOADS["dense"].backward_bytes() / 1e6, 1) == 5088.8
    assert WORKLOADS["unit"].points == 12800


def test_launch_options_follow_a_function_into_its_backward():
    """Launch options are per thread, and PyTorch runs the backward of a Function from another thread than the one
    that called forward (the autograd engine's device thread for GPU tensors; here: a thread of the test's own).
    Every Function records the options its forward ran under and puts them in force again around its backward."""
    import threading
    import torch
    from dfa3D import _lib, functional
    from torch.autograd.function import Function, once_differentiable

    seen = {}

    class Probe(Function):
        @staticmethod
        def forward(ctx, x):
            ctx.launch_fields = _lib.current_fields()
            return x * 2

        @staticmethod
        @once_differentiable
        @functional._with_forward_options
        def backward(ctx, g):
            seen["fields"] = _lib.current_fields()
            seen["options"] = _lib.options()
            return g * 2

    x = torch.ones(3, requires_grad=True)
    with _lib.launch_options(tile=404, **{"pass": 128}):
        y = Probe.apply(x).sum()
    assert _lib.options() is None                                  # the block is over on this thread
    t = threading.Thread(target=y.backward)
    t.start()
    t.join()
    assert seen["fields"] == {"tile": 404, "pass_": 128}
    assert seen["options"] is not None and seen["options"].contents.tile == 404 and seen["options"].contents.pass_ == 128
    assert _lib.options() is None
    # every Function of the package is wired that way
    for name in functional.__all__:
        cls = getattr(functional, name)
        base = cls.__mro__[1] if name.endswith(("_fp16", "_fp32")) else cls
        assert hasattr(base.backward.__wrapped__, "__wrapped__"), name     # once_differentiable(_with_forward_options(backward))
