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


class SvcBatch:
    """The SVC of a stack of matrices (svc_batched): device arrays over the whole stack and views per matrix.

    vec_row_ptr[groups + 1] runs over all groups of all matrices; vec_col / vec_val hold the matrices' vectors one
    after the other and are sized for the bound nvec <= nnz (what lies behind vec_row_ptr[-1] vectors is
    unspecified).  `matrix(i)` returns matrix i's SvcResult as device views (its row pointer rebased to zero);
    `to_host()` brings everything over in one go and returns one (vec_row_ptr, vec_col, vec_val) numpy triple per
    matrix."""

    def __init__(self, V, rows, cols, groups_of, vec_row_ptr, vec_col, vec_val):
        self.V, self.rows, self.cols = V, rows, cols
        self._groups = groups_of            # host: first group of every matrix, [count + 1]
        self.vec_row_ptr, self.vec_col, self.vec_val = vec_row_ptr, vec_col, vec_val

    def __len__(self):
        return len(self.rows)

    def matrix(self, i):
        g0, g1 = int(self._groups[i]), int(self._groups[i + 1])
        ptr = self.vec_row_ptr[g0:g1 + 1]
        lo, hi = (int(x) for x in ptr[[0, -1]].tolist())   # (one read-back: the views need their extent)
        return SvcResult(ptr - ptr[0], self.vec_col[lo:hi], None if self.vec_val is None else self.vec_val[lo * self.V:hi * self.V],
                         hi - lo)

    def to_host(self):
        ptr = self.vec_row_ptr.cpu().numpy()
        n = int(ptr[-1])
        col = self.vec_col[:n].cpu().numpy()
        val = None if self.vec_val is None else self.vec_val[:n * self.V].cpu().numpy()
        out = []
        for i in range(len(self.rows)):
            p = ptr[self._groups[i]:self._groups[i + 1] + 1]
            lo, hi = int(p[0]), int(p[-1])
            out.append((p - p[0], col[lo:hi], None if val is None else val[lo * self.V:hi * self.V]))
        return out


def stack_csr(mats):
    """Stacks CSR matrices along the rows on the host.  mats: sequence of (M, K, row_ptr, col_ind, values or None)
    numpy arrays.  Returns (mat_rows[count + 1], K_max, row_ptr[M_total + 1], col_ind[nnz], values or None), int32 /
    fp16, the row pointer holding entry offsets into the stacked col_ind."""
    import numpy as np
    rows = np.zeros(len(mats) + 1, np.int64)
    ptrs, cols, vals, base = [np.zeros(1, np.int64)], [], [], 0
    with_values = len(mats) > 0 and all(m[4] is not None for m in mats)
    for i, (M, K, rp, ci, cv) in enumerate(mats):
        rp = np.asarray(rp, dtype=np.int64)
        if rp.size != M + 1 or rp[0] != 0 or rp[-1] != np.asarray(ci).size:
            raise ValueError("matrix %d: row_ptr does not describe col_ind" % i)
        rows[i + 1] = rows[i] + M
        ptrs.append(rp[1:] + base)
        cols.append(np.asarray(ci, dtype=np.int32))
        if with_values:
            vals.append(np.asarray(cv, dtype=np.float16))
        base += int(rp[-1])
    if base >= 1 << 28 or rows[-1] >= 1 << 31:
        raise ValueError("the stack is too large for one call: split it")
    cat = lambda parts, dt: np.concatenate(parts).astype(dt) if parts else np.zeros(0, dt)  # noqa: E731
    return (rows.astype(np.int32), max([m[1] for m in mats] + [0]), np.concatenate(ptrs).astype(np.int32),
            cat(cols, np.int32), cat(vals, np.float16) if with_values else None)


def svc_batched(mat_rows, K_max, row_ptr, col_ind, csr_val, V, order="cpython", cols=None):
    """The SVC of a stack of matrices in one chain of launches (svc_count_batched / svc_fill_batched of the C ABI).

    mat_rows: host int array [count + 1], first row of every matrix in the stack (as stack_csr returns it);
    row_ptr[M_total + 1], col_ind[nnz]: int32 GPU tensors of the stacked CSR; csr_val: fp16 GPU tensor or None.
    Nothing is read back: both phases are queued on the current stream.  Returns an SvcBatch."""
    import numpy as np
    if order not in _ORDERS:
        raise ValueError("order must be 'cpython' or 'sorted'")
    if row_ptr.dtype != torch.int32 or col_ind.dtype != torch.int32:
        raise TypeError("row_ptr and col_ind must be int32")
    if csr_val is not None and csr_val.dtype != torch.float16:
        raise TypeError("csr_val must be float16")
    if not (row_ptr.is_cuda and col_ind.is_cuda):
        raise ValueError("row_ptr and col_ind must live on the GPU")
    mat_rows = np.asarray(mat_rows, dtype=np.int64)
    count, M_total = mat_rows.size - 1, int(mat_rows[-1])
    if count < 0 or row_ptr.numel() != M_total + 1 or np.any(np.diff(mat_rows) < 0):
        raise ValueError("mat_rows must be non-decreasing with mat_rows[-1] + 1 == len(row_ptr)")
    per = (np.diff(mat_rows) + V - 1) // V
    groups_of = np.concatenate([[0], np.cumsum(per)]).astype(np.int64)
    groups = int(groups_of[-1])
    L = _lib.lib()
    dev = row_ptr.device
    nnz = col_ind.numel()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream().cuda_stream
        d_rows = torch.from_numpy(mat_rows.astype(np.int32)).to(dev)
        d_groups = torch.empty(count + 1, dtype=torch.int32, device=dev)
        ws = torch.empty(L.svc_batched_workspace_bytes(count, M_total, nnz, V), dtype=torch.uint8, device=dev)
        vec_row_ptr = torch.zeros(groups + 1, dtype=torch.int32, device=dev)
        vec_col = torch.empty(nnz, dtype=torch.int32, device=dev)
        vec_val = None if csr_val is None else torch.empty(nnz * V, dtype=torch.float16, device=dev)
        if groups > 0:
            _lib.check(L.svc_count_batched(count, groups, d_rows.data_ptr(), M_total, K_max, V, row_ptr.data_ptr(),
                                           col_ind.data_ptr(), nnz, _ORDERS[order], d_groups.data_ptr(),
                                           vec_row_ptr.data_ptr(), ws.data_ptr(), stream), "svc_count_batched")
            _lib.check(L.svc_fill_batched(count, groups, d_rows.data_ptr(), M_total, K_max, V, row_ptr.data_ptr(),
                                          col_ind.data_ptr(), 0 if csr_val is None else csr_val.data_ptr(), nnz,
                                          _ORDERS[order], vec_row_ptr.data_ptr(), ws.data_ptr(), vec_col.data_ptr(),
                                          0 if vec_val is None else vec_val.data_ptr(), stream), "svc_fill_batched")
    return SvcBatch(V, np.diff(mat_rows), cols, groups_of, vec_row_ptr, vec_col, vec_val)
