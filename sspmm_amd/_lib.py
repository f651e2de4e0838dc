"""ctypes binding of libsspmm_amd.so (the C ABI declared in include/sspmm.h)."""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsspmm_amd.so")
_lib = None

_i32p = ctypes.c_void_p  # device pointers travel as integers
_vp = ctypes.c_void_p
_int = ctypes.c_int
_i64 = ctypes.c_int64

# name -> (restype, argtypes); must list every symbol include/sspmm.h declares.
SIGNATURES = {
    "sspmm_version": (_int, []),
    "sspmm_error_string": (ctypes.c_char_p, [_int]),
    "sspmm_select_kernel": (_int, [_int]),
    "sspmm_last_kernel": (_int, []),
    "sspmm_f16_f32": (_int, [_int] * 4 + [_vp] * 7),
    "sspmm_f16_f16": (_int, [_int] * 4 + [_vp] * 7),
    "sspmm_batched_f16_f16": (_int, [_int] * 5 + [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "sspmm_batched_f16_f32": (_int, [_int] * 5 + [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "sspmm_noalloc_f16_f32": (_int, [_int] * 4 + [_vp] * 6),
    "sspmm_sorted_row_swizzle": (_int, [_int, _vp, _vp, _vp]),
    "sspmm_sorted_row_swizzle_workspace_bytes": (ctypes.c_size_t, [_int]),
    "sspmm_sorted_row_swizzle_ws": (_int, [_int, _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    "sspmm_plan_create": (_int, [_int, _int, _int, _vp, _int, _int, _int, _vp, ctypes.POINTER(ctypes.c_void_p)]),
    "sspmm_plan_destroy": (_int, [_vp]),
    "sspmm_plan_info": (_int, [_vp, ctypes.POINTER(ctypes.c_int64)]),
    "sspmm_plan_batched_f16_f32": (_int, [_vp, _int, _int, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "sspmm_plan_batched_f16_f16": (_int, [_vp, _int, _int, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "sspmm_sddmm_f16": (_int, [_int] * 4 + [_vp] * 7),
    "sspmm_sddmm_batched_f16": (_int, [_int] * 5 + [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "sspmm_softmax_f16": (_int, [_int, _int, _vp, _vp, _vp, ctypes.c_float, _vp, _vp]),
    "sspmm_softmax_batched_f16": (_int, [_int, _int, _int, _vp, _vp, _vp, ctypes.c_float, _vp, _i64, _vp]),
    "sspmm_sparse_attention_f16": (_int, [_int, _int, _int, _int, _int, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64,
                                          ctypes.c_float, _vp, _i64, _vp]),
    "sspmm_sparse_attention_heads_f16": (_int, [_int, _int, _int, _int, _int, _int, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                                _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, ctypes.c_float, _vp, _i64, _i64, _i64, _vp]),
    "svc_workspace_bytes": (ctypes.c_size_t, [_int, _i64, _int]),
    "svc_count": (_int, [_int, _int, _int, _vp, _vp, _i64, _int, _vp, _vp, _vp]),
    "svc_fill": (_int, [_int, _int, _int, _vp, _vp, _vp, _i64, _int, _vp, _vp, _vp, _vp, _vp]),
    "svc_batched_workspace_bytes": (ctypes.c_size_t, [_int, _int, _i64, _int]),
    "svc_count_batched": (_int, [_int, _int, _vp, _int, _int, _int, _vp, _vp, _i64, _int, _vp, _vp, _vp, _vp]),
    "svc_fill_batched": (_int, [_int, _int, _vp, _int, _int, _int, _vp, _vp, _vp, _i64, _int, _vp, _vp, _vp, _vp, _vp]),
    "sspmm_add_layernorm_f16": (_int, [_int, _int, _vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp]),
    "sspmm_linear_f16": (_int, [_int, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _int, _vp, _vp]),
    "sspmm_attention_fm_f16": (_int, [_int, _int, _int, _int, _vp, _vp, _vp, ctypes.c_int64, _vp, ctypes.c_int64, ctypes.c_float, _vp]),
    "svc_coo_workspace_bytes": (ctypes.c_size_t, [_i64]),
    "svc_coo_to_csr": (_int, [_int, _int, _i64, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    "svc_reorder_workspace_bytes": (ctypes.c_size_t, [_int]),
    "svc_reorder_minhash": (_int, [_int, _vp, _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    "svc_permute_csr": (_int, [_int] + [_vp] * 8 + [ctypes.c_size_t, _vp]),
}


def library_path():
    return _LIB_PATH


def build_library(force=True):
    """Compile the HIP sources for gfx950 with hipcc (cross-compiles without a GPU)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j8"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return _LIB_PATH


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                "libsspmm_amd.so is not built (%s missing); run `python -c 'import __graft_entry__ as g; "
                "g.build()'` or `make -C sspmm_amd/csrc`.  sspmm_amd has no CPU fallback." % _LIB_PATH)
        L = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(code, what):
    if code != 0:
        msg = lib().sspmm_error_string(code)
        raise RuntimeError("%s failed with code %d: %s" % (what, code, msg.decode() if msg else "?"))
