"""The C ABI library loads without a GPU, exports every symbol include/sspmm.h declares, and
rejects bad arguments before touching the device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "sspmm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:sspmm|svc)_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(built_library):
    from sspmm_amd import _lib
    L = ctypes.CDLL(built_library)
    names = _declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(L, n), "library does not export %s" % n
        assert n in _lib.SIGNATURES, "ctypes binding misses %s" % n
    assert sorted(_lib.SIGNATURES) == names


def test_argument_errors_without_device_work(built_library):
    from sspmm_amd import _lib
    L = _lib.lib()
    assert L.sspmm_version() >= 1
    one = 1  # any non-null pointer value; rejected calls never dereference it
    # unsupported vector length (the reference prints and carries on: sspmm.cu:582-583)
    assert L.sspmm_f16_f32(4, 4, 64, 64, None, one, one, one, one, one, None) == 1
    assert L.sspmm_f16_f16(4, 2, 64, 64, None, one, one, one, one, one, None) == 1
    # negative sizes, null outputs
    assert L.sspmm_f16_f32(-1, 8, 64, 64, None, one, one, one, one, one, None) == 1
    assert L.sspmm_f16_f32(4, 8, 64, 64, None, None, one, one, one, one, None) == 1
    assert L.sspmm_f16_f32(4, 8, 64, 64, None, one, one, one, one, None, None) == 1
    assert L.sspmm_f16_f32(4, 8, 1 << 20, 1 << 12, None, one, one, one, one, one, None) == 1  # K*N >= 2^31
    # nothing to do is success
    assert L.sspmm_f16_f32(0, 8, 64, 64, None, None, None, None, None, None, None) == 0
    assert L.sspmm_f16_f16(4, 16, 0, 64, None, one, one, one, one, one, None) == 0
    assert L.sspmm_batched_f16_f16(0, 4, 8, 64, 64, None, one, one, one, 0, one, 0, one, 0, None) == 0
    assert L.sspmm_batched_f16_f16(2, 4, 8, 64, 64, None, one, one, one, 0, one, 0, one, 5, None) == 1  # C overlaps
    assert L.sspmm_sorted_row_swizzle(-3, one, one, None) == 1
    assert L.sspmm_sorted_row_swizzle(0, None, None, None) == 0
    assert L.svc_count(8, 8, 8, one, one, 4, 7, one, one, None) == 1  # unknown order
    assert L.svc_count(8, 8, 0, one, one, 4, 0, one, one, None) == 1  # V < 1
    assert L.svc_count(8, 8, 8, one, one, 4, 0, one, None, None) == 1  # no workspace
    assert L.svc_fill(8, 8, 8, one, one, one, 4, 0, one, one, one, None, None) == 1  # values in, no values out
    # plans: unsupported V, no place to put the handle, no pattern
    import ctypes as C
    handle = C.c_void_p()
    assert L.sspmm_plan_create(4, 4, 64, one, 64, 1, 0, None, C.byref(handle)) == 1
    assert L.sspmm_plan_create(4, 8, 64, one, 64, 1, 0, None, None) == 1
    assert L.sspmm_plan_create(4, 8, 64, None, 64, 1, 0, None, C.byref(handle)) == 1
    assert L.sspmm_plan_destroy(None) == 0
    assert L.sspmm_plan_info(None, None) == 1
    assert L.sspmm_plan_batched_f16_f32(None, 1, 64, one, one, one, 0, one, 0, one, 0, None) == 1
    # the linear-layer and attention entry points reject what they do not cover before touching the device
    assert L.sspmm_linear_f16(4, 8, 64, 64, one, one, one, one, None, 7, one, None) == 1       # unknown activation
    assert L.sspmm_linear_f16(4, 4, 64, 64, one, one, one, one, None, 0, one, None) == 1       # unsupported V
    assert L.sspmm_linear_f16(0, 8, 64, 64, None, None, None, None, None, 1, None, None) == 0  # nothing to do
    assert L.sspmm_attention_fm_f16(1, 1, 64, 32, 16, 16, 16, 64, 16, 64, 0.125, None) == 1    # head size
    assert L.sspmm_attention_fm_f16(1, 1, 96, 64, 16, 16, 16, 96, 16, 96, 0.125, None) == 1    # sequence not a multiple of 64
    assert L.sspmm_attention_fm_f16(0, 1, 64, 64, None, None, None, 0, None, 0, 0.125, None) == 0
    for bad_scale in (0.0, -0.125, float("nan"), float("inf")):
        assert L.sspmm_attention_fm_f16(1, 1, 64, 64, 16, 16, 16, 64, 16, 64, bad_scale, None) == 1
    # the one-launch sparse attention block: heads of 32, 64 or 128 features, V of 8 or 16, a positive finite scale, aligned operands
    sa = lambda V=8, F=64, q=16, stride=512, scale=0.125: L.sspmm_sparse_attention_f16(  # noqa: E731
        1, 1, V, F, 8, None, 16, 16, q, stride, 16, 512, 16, 512, scale, 16, 512, None)
    assert sa(V=4) == 1 and sa(F=48) == 1 and sa(F=256) == 1 and sa(q=8) == 1 and sa(stride=4) == 1
    for bad_scale in (0.0, -0.125, float("nan"), float("inf")):
        assert sa(scale=bad_scale) == 1
    assert L.sspmm_sparse_attention_f16(0, 4, 8, 64, 8, None, None, None, None, 0, None, 0, None, 0, 0.125, None, 0, None) == 0
    # ... and its form for heads that lie side by side: no heads, a row pitch below the head's width, a pitch that is not a
    # multiple of 8, a negative stride
    sh = lambda heads=2, ld=384, head=64, stride=128: L.sspmm_sparse_attention_heads_f16(  # noqa: E731
        1, heads, 1, 8, 64, 8, None, 16, 16, 16, stride, head, ld, 16, stride, head, ld, 16, stride, head, ld, 0.125, 16, stride, head, ld, None)
    assert sh(heads=0) == 1 and sh(ld=32) == 1 and sh(ld=388) == 1 and sh(stride=-128) == 1 and sh(ld=1 << 23) == 1
    assert L.svc_workspace_bytes(16, 100, 8) >= 100 * 8
    assert b"invalid" in L.sspmm_error_string(1)
    assert L.sspmm_error_string(0) == b"success"


def test_python_operator_rejects_bad_arguments(built_library):
    import torch
    import sspmm_amd
    t = torch.zeros(4, dtype=torch.int32)
    h = torch.zeros(4, dtype=torch.float16)
    with pytest.raises(ValueError):
        sspmm_amd.spmm(None, t, t, h, h.reshape(2, 2), 4)
    with pytest.raises(TypeError):
        sspmm_amd.spmm(None, t.long(), t, h, h.reshape(2, 2), 8)
    with pytest.raises(ValueError):  # CPU tensors: there is no CPU path
        sspmm_amd.spmm(None, t, t, h, h.reshape(2, 2), 8)
