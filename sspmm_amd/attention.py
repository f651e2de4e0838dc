"""Python operator surface of the steps either side of `bspmm` in the reference's sparse
attention block, mirroring its torch extensions `sptrans.sddmm` and `sptrans.softmax`
(reference end2end/sspmm_e2e/src/cuda/sddmm.cpp:11-46, softmax.cpp:11-43): same names, same
argument order, same shape inference (sddmm_kernel.cu:1169-1186 and 1236-1258,
softmax_kernel.cu:208-216 and 256-266), and the block that chains them
(end2end/sspmm_e2e/spattention.py:167-179).
"""
import torch

from . import _lib
from .spmm import _check_inputs, _ptr, _stream, bspmm


def _check_pattern(row_indices, row_offsets, column_indices, vec_length):
    if vec_length not in (8, 16):
        raise ValueError("vec_length must be 8 or 16, got %r" % (vec_length,))
    for name, t in (("row_offsets", row_offsets), ("column_indices", column_indices), ("row_indices", row_indices)):
        if t is None:
            continue
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
            raise TypeError("%s must be a contiguous int32 GPU tensor" % name)


def _check_half(name, t):
    if t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous():
        raise TypeError("%s must be a contiguous float16 GPU tensor" % name)


def bsddmm(row_indices, row_offsets, column_indices, lhs_matrix, rhs_matrix, vec_length):
    """out[b, j*V + v] = lhs[b, i*V + v, :] . rhs[b, col_j, :]: lhs [batch, M, F], rhs [batch, n, F] ->
    fp16 [batch, nvec*V] (reference batched_sddmm_cuda)."""
    _check_pattern(row_indices, row_offsets, column_indices, vec_length)
    _check_half("lhs_matrix", lhs_matrix)
    _check_half("rhs_matrix", rhs_matrix)
    m, k, n = lhs_matrix.size(-2), lhs_matrix.size(-1), rhs_matrix.size(-2)
    if rhs_matrix.size(-1) != k:
        raise ValueError("lhs_matrix and rhs_matrix must have the same feature length")
    batch = lhs_matrix.numel() // (m * k) if m * k > 0 else 1
    m_vec = row_offsets.numel() - 1
    if m != m_vec * vec_length:
        raise ValueError("lhs_matrix must have m_vec * vec_length = %d rows, got %d" % (m_vec * vec_length, m))
    nvec = column_indices.numel()
    out = torch.empty((batch, nvec * vec_length), dtype=torch.float16, device=lhs_matrix.device)
    with torch.cuda.device(lhs_matrix.device):
        rc = _lib.lib().sspmm_sddmm_batched_f16(batch, m_vec, vec_length, k, n, _ptr(row_indices), _ptr(row_offsets),
                                                _ptr(column_indices), _ptr(lhs_matrix), m * k, _ptr(rhs_matrix), n * k,
                                                _ptr(out), nvec * vec_length, _stream())
    _lib.check(rc, "sspmm_sddmm")
    return out


def sddmm(row_indices, row_offsets, column_indices, lhs_matrix, rhs_matrix, vec_length):
    """lhs [M, F], rhs [n, F] -> fp16 [nvec*V] (reference sddmm_cuda)."""
    if lhs_matrix.dim() != 2 or rhs_matrix.dim() != 2:
        raise ValueError("lhs_matrix and rhs_matrix must be 2-D")
    return bsddmm(row_indices, row_offsets, column_indices, lhs_matrix, rhs_matrix, vec_length).view(-1)


def bcsr_softmax(row_indices, row_offsets, values, scaler, vec_length, batch_size):
    """Row softmax over the stored entries, values [batch, nvec*V] -> fp16 of the same shape
    (reference batched_csr_softmax_cuda)."""
    _check_pattern(row_indices, row_offsets, None, vec_length)
    _check_half("values", values)
    m_vec = row_offsets.numel() - 1
    stride = values.numel() // batch_size if batch_size > 0 else 0
    out = torch.empty_like(values)
    with torch.cuda.device(values.device):
        rc = _lib.lib().sspmm_softmax_batched_f16(batch_size, m_vec, vec_length, _ptr(row_indices), _ptr(row_offsets),
                                                  _ptr(values), float(scaler), _ptr(out), stride, _stream())
    _lib.check(rc, "sspmm_softmax")
    return out


def csr_softmax(row_indices, row_offsets, values, scaler, vec_length):
    """values [nvec*V] -> fp16 [nvec*V] (reference csr_softmax_cuda)."""
    return bcsr_softmax(row_indices, row_offsets, values, scaler, vec_length, 1)


def sparse_attention(row_indices, row_offsets, column_indices, q, k, v, scaling, vec_length):
    """softmax(mask(q k^T) * scaling) v on a vector-sparse mask shared by the batch:
    q [batch, tgt, d], k [batch, src, d], v [batch, src, d_v] -> fp16 [batch, tgt, d_v]; the three
    steps of the reference's block (spattention.py:167-179)."""
    w = bsddmm(row_indices, row_offsets, column_indices, q, k, vec_length)
    w = bcsr_softmax(row_indices, row_offsets, w, scaling, vec_length, w.size(0))
    _check_inputs(row_indices, row_offsets, column_indices, w, v, vec_length)
    return bspmm(row_indices, row_offsets, column_indices, w, v, vec_length)
