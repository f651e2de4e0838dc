"""Sparse Vector Compression (RowMerge) on the GPU: CSR -> CVSE.

Host-side mirror of the reference's `CVSE(ROW, COL, NNZ, colInd_list_array, vec_len)`
(reference RowMerge/sparse_matrix_format.py:94-123) over device tensors; the merge runs in the
HIP kernels behind svc_count / svc_fill of the C ABI.
"""
import collections

import torch

from . import _lib

SvcResult = collections.namedtuple("SvcResult", ["vec_row_ptr", "vec_col", "vec_val", "num_vec"])

_ORDERS = {"cpython": 0, "sorted": 1}


def svc(row_ptr, col_ind, csr_val, M, K, V, order="cpython", exact_size=True):
    """Merge every V consecutive rows of a CSR matrix into column vectors.

    row_ptr[M+1], col_ind[nnz]: int32 GPU tensors; csr_val: fp16 GPU tensor or None.
    order="cpython" gives exactly the column order the reference's RowMerge writes;
    order="sorted" gives ascending columns.
    Returns SvcResult(vec_row_ptr[int32 m_vec+1], vec_col[int32 nvec], vec_val[fp16 nvec*V] or None, nvec).

    exact_size=True reads nvec back from the device between the two phases (the call's one synchronisation) and
    returns arrays of exactly nvec vectors.  exact_size=False sizes them for the bound nvec <= nnz instead: the call
    then never waits for the device (both phases are queued on the current stream), num_vec is None, the vectors
    are the first vec_row_ptr[-1] entries of vec_col / vec_val and what lies behind them is unspecified.  The SpMM
    operators take such arrays as they are: they read the extent from vec_row_ptr on the device.
    """
    if order not in _ORDERS:
        raise ValueError("order must be 'cpython' or 'sorted'")
    if row_ptr.dtype != torch.int32 or col_ind.dtype != torch.int32:
        raise TypeError("row_ptr and col_ind must be int32")
    if csr_val is not None and csr_val.dtype != torch.float16:
        raise TypeError("csr_val must be float16")
    if not (row_ptr.is_cuda and col_ind.is_cuda):
        raise ValueError("row_ptr and col_ind must live on the GPU")
    if row_ptr.numel() != M + 1:
        raise ValueError("row_ptr must have M + 1 entries")
    L = _lib.lib()
    dev = row_ptr.device
    nnz = col_ind.numel()
    m_vec = (M + V - 1) // V
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream().cuda_stream
        ws = torch.empty(L.svc_workspace_bytes(M, nnz, V), dtype=torch.uint8, device=dev)
        vec_row_ptr = torch.zeros(m_vec + 1, dtype=torch.int32, device=dev)
        if M == 0:
            return SvcResult(vec_row_ptr, torch.empty(0, dtype=torch.int32, device=dev),
                             None if csr_val is None else torch.empty(0, dtype=torch.float16, device=dev), 0)
        _lib.check(L.svc_count(M, K, V, row_ptr.data_ptr(), col_ind.data_ptr(), nnz, _ORDERS[order],
                               vec_row_ptr.data_ptr(), ws.data_ptr(), stream), "svc_count")
        nvec = int(vec_row_ptr[-1].item()) if exact_size else None  # the one host read-back: sizes the outputs
        cap = nvec if exact_size else nnz
        vec_col = torch.empty(cap, dtype=torch.int32, device=dev)
        vec_val = None if csr_val is None else torch.empty(cap * V, dtype=torch.float16, device=dev)
        _lib.check(L.svc_fill(M, K, V, row_ptr.data_ptr(), col_ind.data_ptr(),
                              0 if csr_val is None else csr_val.data_ptr(), nnz, _ORDERS[order],
                              vec_row_ptr.data_ptr(), ws.data_ptr(), vec_col.data_ptr(),
                              0 if vec_val is None else vec_val.data_ptr(), stream), "svc_fill")
    return SvcResult(vec_row_ptr, vec_col, vec_val, nvec)
