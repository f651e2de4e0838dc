"""ctypes/numpy front end of the C oracle plus the pure-Python RowMerge restatement.

TEST INFRASTRUCTURE ONLY (see sspmm_oracle.c for what each function follows and
what pins it).  Nothing in sspmm_amd/ imports this module.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile liboracle.so with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i32p = ctypes.POINTER(ctypes.c_int32)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        f32p = ctypes.POINTER(ctypes.c_float)
        L.oracle_pyset_order.restype = ctypes.c_int64
        L.oracle_pyset_order.argtypes = [i32p, ctypes.c_int64, i32p]
        L.oracle_svc.restype = ctypes.c_int64
        L.oracle_svc.argtypes = [ctypes.c_int32] * 3 + [i32p, i32p, u16p, ctypes.c_int32, i32p, i32p, u16p]
        L.oracle_spmm_f32.restype = None
        L.oracle_spmm_f32.argtypes = [ctypes.c_int32] * 4 + [i32p, i32p, u16p, u16p, f32p, ctypes.c_int32]
        L.oracle_spmm_f16.restype = None
        L.oracle_spmm_f16.argtypes = [ctypes.c_int32] * 4 + [i32p, i32p, u16p, u16p, u16p, ctypes.c_int32]
        L.oracle_sorted_row_swizzle.restype = None
        L.oracle_sorted_row_swizzle.argtypes = [ctypes.c_int32, i32p, i32p]
        L.oracle_sddmm_f16.restype = None
        L.oracle_sddmm_f16.argtypes = [ctypes.c_int32] * 3 + [i32p, i32p, u16p, u16p, u16p]
        L.oracle_softmax_f16.restype = None
        L.oracle_softmax_f16.argtypes = [ctypes.c_int32] * 2 + [i32p, u16p, ctypes.c_float, u16p]
        L.oracle_minhash_order.restype = None
        L.oracle_minhash_order.argtypes = [ctypes.c_int32, i32p, i32p, i32p, ctypes.POINTER(ctypes.c_uint64)]
        L.oracle_permute_csr.restype = None
        L.oracle_permute_csr.argtypes = [ctypes.c_int32, i32p, i32p, i32p, u16p, i32p, i32p, u16p]
        L.oracle_h2f.restype = ctypes.c_float
        L.oracle_h2f.argtypes = [ctypes.c_uint16]
        L.oracle_f2h.restype = ctypes.c_uint16
        L.oracle_f2h.argtypes = [ctypes.c_float]
        _lib = L
    return _lib


def _p(a, ct):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ct))


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _u16(a):
    """fp16 array -> its bit pattern as uint16 (no copy when already contiguous)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return a.view(np.uint16)
    return np.ascontiguousarray(a, dtype=np.uint16)


def pyset_order(keys):
    """C model of list(set(keys)) for non-negative ints."""
    keys = _i32(keys)
    out = np.empty(max(len(keys), 1), dtype=np.int32)
    n = lib().oracle_pyset_order(_p(keys, ctypes.c_int32), len(keys), _p(out, ctypes.c_int32))
    return out[:n].copy()


def svc(M, K, V, row_ptr, col_ind, csr_val=None, order="cpython"):
    """RowMerge.  Returns (vec_row_ptr[int32 m_vec+1], vec_col[int32 nvec], vec_val[fp16 nvec*V] or None)."""
    row_ptr, col_ind = _i32(row_ptr), _i32(col_ind)
    nnz = int(row_ptr[M]) if M > 0 else 0
    m_vec = (M + V - 1) // V
    vrp = np.zeros(m_vec + 1, dtype=np.int32)
    vcol = np.empty(max(nnz, 1), dtype=np.int32)
    vval = None
    cv = None
    if csr_val is not None:
        cv = _u16(csr_val)
        vval = np.empty(max(nnz, 1) * V, dtype=np.uint16)
    nvec = lib().oracle_svc(M, K, V, _p(row_ptr, ctypes.c_int32), _p(col_ind, ctypes.c_int32),
                            _p(cv, ctypes.c_uint16), {"cpython": 0, "sorted": 1}[order],
                            _p(vrp, ctypes.c_int32), _p(vcol, ctypes.c_int32), _p(vval, ctypes.c_uint16))
    if nvec < 0:
        raise ValueError("oracle_svc: bad arguments")
    return vrp, vcol[:nvec].copy(), (None if vval is None else vval[:nvec * V].copy().view(np.float16))


def spmm(m_vec, V, N, K, row_offsets, col_idx, values, B, out_dtype=np.float32, threads=1):
    """Host SpMM check loop of the reference harness; values/B are fp16 arrays."""
    row_offsets, col_idx = _i32(row_offsets), _i32(col_idx)
    vals, Bb = _u16(values), _u16(B)
    M = m_vec * V
    if out_dtype == np.float32:
        C = np.empty((M, N), dtype=np.float32)
        lib().oracle_spmm_f32(m_vec, V, N, K, _p(row_offsets, ctypes.c_int32), _p(col_idx, ctypes.c_int32),
                              _p(vals, ctypes.c_uint16), _p(Bb, ctypes.c_uint16), _p(C, ctypes.c_float), threads)
        return C
    C = np.empty((M, N), dtype=np.uint16)
    lib().oracle_spmm_f16(m_vec, V, N, K, _p(row_offsets, ctypes.c_int32), _p(col_idx, ctypes.c_int32),
                          _p(vals, ctypes.c_uint16), _p(Bb, ctypes.c_uint16), _p(C, ctypes.c_uint16), threads)
    return C.view(np.float16)


def sddmm(m_vec, V, row_offsets, col_idx, lhs, rhs):
    """Sampled dense-dense product at the vector pattern: lhs [m_vec*V, F], rhs [n, F] fp16 -> fp16 [nvec*V]."""
    row_offsets, col_idx = _i32(row_offsets), _i32(col_idx)
    F = lhs.shape[1]
    a, b = _u16(lhs), _u16(rhs)
    out = np.empty(max(col_idx.size * V, 1), dtype=np.uint16)
    lib().oracle_sddmm_f16(m_vec, V, F, _p(row_offsets, ctypes.c_int32), _p(col_idx, ctypes.c_int32),
                           _p(a, ctypes.c_uint16), _p(b, ctypes.c_uint16), _p(out, ctypes.c_uint16))
    return out[:col_idx.size * V].copy().view(np.float16)


def softmax(m_vec, V, row_offsets, values, scaler):
    """Row softmax over the stored entries of a vector-sparse matrix: fp16 [nvec*V] -> fp16 [nvec*V]."""
    row_offsets = _i32(row_offsets)
    vals = _u16(values)
    out = np.zeros(max(vals.size, 1), dtype=np.uint16)
    lib().oracle_softmax_f16(m_vec, V, _p(row_offsets, ctypes.c_int32), _p(vals, ctypes.c_uint16),
                             ctypes.c_float(scaler), _p(out, ctypes.c_uint16))
    return out[:vals.size].copy().view(np.float16)


def sorted_row_swizzle(row_offsets):
    row_offsets = _i32(row_offsets)
    rows = len(row_offsets) - 1
    out = np.empty(max(rows, 1), dtype=np.int32)
    lib().oracle_sorted_row_swizzle(rows, _p(row_offsets, ctypes.c_int32), _p(out, ctypes.c_int32))
    return out[:rows].copy()


def minhash_order(M, row_ptr, col_ind, return_keys=False):
    """Row order of the reordering step: stable argsort of the rows' two-min-hash keys."""
    row_ptr, col_ind = _i32(row_ptr), _i32(col_ind)
    perm = np.empty(max(M, 1), dtype=np.int32)
    keys = np.empty(max(M, 1), dtype=np.uint64)
    lib().oracle_minhash_order(M, _p(row_ptr, ctypes.c_int32), _p(col_ind, ctypes.c_int32), _p(perm, ctypes.c_int32),
                               _p(keys, ctypes.c_uint64))
    return (perm[:M].copy(), keys[:M].copy()) if return_keys else perm[:M].copy()


def permute_csr(M, perm, row_ptr, col_ind, val=None):
    """CSR arrays with row i taken from source row perm[i]."""
    perm, row_ptr, col_ind = _i32(perm), _i32(row_ptr), _i32(col_ind)
    nnz = int(row_ptr[M]) if M else 0
    out_ptr = np.zeros(M + 1, dtype=np.int32)
    out_col = np.empty(max(nnz, 1), dtype=np.int32)
    v = None if val is None else _u16(val)
    out_val = None if val is None else np.empty(max(nnz, 1), dtype=np.uint16)
    lib().oracle_permute_csr(M, _p(perm, ctypes.c_int32), _p(row_ptr, ctypes.c_int32), _p(col_ind, ctypes.c_int32),
                             None if v is None else _p(v, ctypes.c_uint16), _p(out_ptr, ctypes.c_int32),
                             _p(out_col, ctypes.c_int32), None if v is None else _p(out_val, ctypes.c_uint16))
    return out_ptr, out_col[:nnz].copy(), None if val is None else out_val[:nnz].copy().view(np.float16)


def rowmerge_python(M, V, col_lists):
    """Pure-Python RowMerge, the reference's own algorithm on the language runtime's set.

    Follows CVSE.__init__ (RowMerge/sparse_matrix_format.py:100-123): per vector-row,
    fold `list(set(acc + row))` over its V member rows (rows >= M skipped), then the
    running total becomes the next row pointer.  This is the timed "Python RowMerge"
    CPU baseline and the ground truth for column order.
    """
    m_vec = math.ceil(M / V)
    ptr = [0]
    flat = []
    total = 0
    for i in range(m_vec):
        acc = []
        for j in range(V):
            if V * i + j < M:
                acc = list(set(acc + col_lists[V * i + j]))
        total += len(acc)
        ptr.append(total)
        flat.extend(acc)
    return ptr, flat


def coo_to_csr(M, K, rows, cols):
    """The pattern of `coo.tocsr()` as the reference's SuiteSparse path uses it (RowMerge/suit_sparse_matrix.py:
    109-111): scipy's conversion sorts each row's columns and merges repeated (row, column) pairs; entries
    outside the matrix are dropped.  Pinned by scipy's own tocsr() and by the reference-written `_csr.mtx` files
    (tests/test_suitesparse.py)."""
    rows = np.asarray(rows, dtype=np.int64)
    cols = np.asarray(cols, dtype=np.int64)
    ok = (rows >= 0) & (rows < M) & (cols >= 0) & (cols < K)
    keys = np.unique(rows[ok] * (1 << 32) + cols[ok])
    row_ptr = np.searchsorted(keys >> 32, np.arange(M + 1), side="left").astype(np.int32)
    return row_ptr, (keys & 0xffffffff).astype(np.int32)


def csr_col_lists(M, row_ptr, col_ind):
    """colInd_list_array of the reference (sparse_matrix_format.py:41-53): per-row python lists."""
    ci = [int(c) for c in col_ind]
    return [ci[int(row_ptr[i]):int(row_ptr[i + 1])] for i in range(M)]


def densify(m_vec, V, K, row_offsets, col_idx, values):
    """csr2dense of the reference (end2end/sspmm_e2e/verify/static_mask.py:29-45), fp16 [m_vec*V, K]."""
    A = np.zeros((m_vec * V, K), dtype=np.float16)
    values = np.asarray(values).reshape(-1, V)
    for i in range(m_vec):
        for j in range(int(row_offsets[i]), int(row_offsets[i + 1])):
            A[i * V:(i + 1) * V, int(col_idx[j])] = values[j]
    return A
