"""Row reordering ahead of the SVC, on the GPU.

The reference runs a reordering pass before RowMerge to write its `dataset-v8` / `dataset-v16`
folders (`python row_merge_reorder.py`, reference README.md:36; the harness reads those folders
when its `reorder` argument is 1, reference SSpMM/sspmm_test.cpp:313-320).  The reorder module
itself is not among the reference's sources, so the method is this library's own: rows are
sorted by a key of two min-hashes of their column sets, which puts rows that name the same
columns into the same group of V rows, so the merged group has fewer, fuller vectors.

    perm = minhash_order(row_ptr, col_ind, M)            # row i of the new matrix = old row perm[i]
    rp, ci, val = permute_csr(row_ptr, col_ind, csr_val, perm)
    r = svc(rp, ci, val, M, K, V)                         # or svc_reordered(...) for all three steps

The SpMM of the reordered matrix yields the rows of C in the new order: C_new[i] = C_old[perm[i]].
"""
import collections

import torch

from . import _lib
from .svc import svc

ReorderedSvc = collections.namedtuple("ReorderedSvc", ["svc", "perm", "row_ptr", "col_ind", "csr_val"])


def _check_csr(row_ptr, col_ind, M):
    if row_ptr.dtype != torch.int32 or col_ind.dtype != torch.int32:
        raise TypeError("row_ptr and col_ind must be int32")
    if not (row_ptr.is_cuda and col_ind.is_cuda):
        raise ValueError("row_ptr and col_ind must live on the GPU")
    if row_ptr.numel() != M + 1:
        raise ValueError("row_ptr must have M + 1 entries")


def _workspace(L, M, dev):
    nbytes = L.svc_reorder_workspace_bytes(M)
    if nbytes == 0:
        raise RuntimeError("svc_reorder_workspace_bytes failed (no usable GPU?)")
    return torch.empty(nbytes, dtype=torch.uint8, device=dev), nbytes


def minhash_order(row_ptr, col_ind, M):
    """int32 GPU tensor perm[M]: the rows in the order of their min-hash keys (ties in source order)."""
    _check_csr(row_ptr, col_ind, M)
    L = _lib.lib()
    dev = row_ptr.device
    perm = torch.empty(M, dtype=torch.int32, device=dev)
    if M == 0:
        return perm
    with torch.cuda.device(dev):
        ws, nbytes = _workspace(L, M, dev)
        _lib.check(L.svc_reorder_minhash(M, row_ptr.data_ptr(), col_ind.data_ptr(), perm.data_ptr(), ws.data_ptr(),
                                         nbytes, torch.cuda.current_stream().cuda_stream), "svc_reorder_minhash")
    return perm


def permute_csr(row_ptr, col_ind, csr_val, perm):
    """The CSR arrays with row i taken from source row perm[i]; csr_val may be None."""
    M = perm.numel()
    _check_csr(row_ptr, col_ind, M)
    if perm.dtype != torch.int32 or not perm.is_cuda:
        raise TypeError("perm must be an int32 GPU tensor")
    if csr_val is not None and csr_val.dtype != torch.float16:
        raise TypeError("csr_val must be float16")
    L = _lib.lib()
    dev = row_ptr.device
    out_ptr = torch.empty(M + 1, dtype=torch.int32, device=dev)
    out_col = torch.empty_like(col_ind)
    out_val = None if csr_val is None else torch.empty_like(csr_val)
    with torch.cuda.device(dev):
        ws, nbytes = _workspace(L, M, dev)
        _lib.check(L.svc_permute_csr(M, perm.data_ptr(), row_ptr.data_ptr(), col_ind.data_ptr(),
                                     0 if csr_val is None else csr_val.data_ptr(), out_ptr.data_ptr(),
                                     out_col.data_ptr(), 0 if out_val is None else out_val.data_ptr(), ws.data_ptr(),
                                     nbytes, torch.cuda.current_stream().cuda_stream), "svc_permute_csr")
    return out_ptr, out_col, out_val


def svc_reordered(row_ptr, col_ind, csr_val, M, K, V, order="cpython"):
    """Reorder the rows, then merge every V of them: ReorderedSvc(svc result, perm, reordered CSR arrays)."""
    perm = minhash_order(row_ptr, col_ind, M)
    rp, ci, val = permute_csr(row_ptr, col_ind, csr_val, perm)
    return ReorderedSvc(svc(rp, ci, val, M, K, V, order=order), perm, rp, ci, val)
