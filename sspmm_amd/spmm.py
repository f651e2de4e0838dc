"""Python operator surface of the SpMM, mirroring the reference's torch extension
`sptrans.spmm` (reference end2end/sspmm_e2e/src/cuda/spmm.cpp:11-46): same names, same
argument order, same shape inference (reference end2end/sspmm_e2e/src/cuda/spmm_kernel.cu:
468-475 and 524-538).  Tensors are torch-ROCm device tensors; torch only provides the device
memory and the stream, the arithmetic happens in the HIP kernels behind the C ABI.
"""
import torch

from . import _lib


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _check_inputs(row_indices, row_offsets, column_indices, values, rhs_matrix, vec_length):
    if vec_length not in (8, 16):
        raise ValueError("vec_length must be 8 or 16, got %r" % (vec_length,))
    for name, t, dt in (("row_offsets", row_offsets, torch.int32), ("column_indices", column_indices, torch.int32),
                        ("values", values, torch.float16), ("rhs_matrix", rhs_matrix, torch.float16)):
        if t.dtype != dt:
            raise TypeError("%s must be %s, got %s" % (name, dt, t.dtype))
        if not t.is_cuda:
            raise ValueError("%s must live on the GPU" % name)
        if not t.is_contiguous():
            raise ValueError("%s must be contiguous" % name)
    if row_indices is not None:
        if row_indices.dtype != torch.int32 or not row_indices.is_cuda or not row_indices.is_contiguous():
            raise TypeError("row_indices must be a contiguous int32 GPU tensor")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _check_plan(plan, m_vec, vec_length, K):
    if (plan.m_vec, plan.vec_length, plan.K) != (m_vec, vec_length, K):
        raise ValueError("the plan was made for m_vec=%d, V=%d, K=%d, the product has m_vec=%d, V=%d, K=%d"
                         % (plan.m_vec, plan.vec_length, plan.K, m_vec, vec_length, K))


def spmm(row_indices, row_offsets, column_indices, values, rhs_matrix, vec_length, out_dtype=torch.float16, plan=None):
    """C[m_vec*V, N] = A_cvse @ rhs_matrix[K, N].

    Same call as the reference's `spmm(row_indices, row_offsets, column_indices, values,
    rhs_matrix, vec_length)`; returns a new fp16 tensor like the reference, or fp32 when
    out_dtype=torch.float32 (the reference's C++ `float*` overload, SSpMM/include/sspmm.cuh:31-37).
    With `plan` (a sspmm_amd.Plan of this pattern) the plan's schedule replaces row_indices.
    """
    _check_inputs(row_indices, row_offsets, column_indices, values, rhs_matrix, vec_length)
    if rhs_matrix.dim() != 2:
        raise ValueError("rhs_matrix must be [K, N]")
    m_vec = row_offsets.size(-1) - 1
    K, N = rhs_matrix.size(0), rhs_matrix.size(1)
    out = torch.empty((m_vec * vec_length, N), dtype=out_dtype, device=rhs_matrix.device)
    if plan is not None:
        _check_plan(plan, m_vec, vec_length, K)
        fn = {torch.float16: _lib.lib().sspmm_plan_batched_f16_f16,
              torch.float32: _lib.lib().sspmm_plan_batched_f16_f32}[out_dtype]
        with torch.cuda.device(rhs_matrix.device):
            rc = fn(plan.handle, 1, N, _ptr(row_offsets), _ptr(column_indices), _ptr(values), 0, _ptr(rhs_matrix), 0,
                    _ptr(out), 0, _stream())
        _lib.check(rc, "sspmm_plan")
        return out
    fn = {torch.float16: _lib.lib().sspmm_f16_f16, torch.float32: _lib.lib().sspmm_f16_f32}[out_dtype]
    with torch.cuda.device(rhs_matrix.device):
        rc = fn(m_vec, vec_length, N, K, _ptr(row_indices), _ptr(row_offsets), _ptr(column_indices), _ptr(values),
                _ptr(rhs_matrix), _ptr(out), _stream())
    _lib.check(rc, "sspmm")
    return out


ACTIVATIONS = {None: 0, "none": 0, "gelu": 1}


def linear(row_offsets, column_indices, values, rhs_matrix, vec_length, bias=None, activation=None):
    """act(A_cvse @ rhs_matrix + bias[:, None]) as one launch, fp16 out (sspmm_linear_f16 of the C ABI): what the
    reference's model code computes with nn.Linear and the activation behind it (reference
    end2end/sspmm_e2e/end_to_end.py:55-56, 70-73), bias and activation applied to the fp32 sums.
    bias: fp16 [m_vec * V] or None; activation: None / "none" / "gelu" (the erf form, torch's default)."""
    _check_inputs(None, row_offsets, column_indices, values, rhs_matrix, vec_length)
    if activation not in ACTIVATIONS:
        raise ValueError("activation must be one of %r" % (sorted(k for k in ACTIVATIONS if k),))
    if rhs_matrix.dim() != 2:
        raise ValueError("rhs_matrix must be [K, N]")
    m_vec = row_offsets.size(-1) - 1
    K, N = rhs_matrix.size(0), rhs_matrix.size(1)
    if bias is not None and (bias.dtype != torch.float16 or not bias.is_cuda or not bias.is_contiguous() or
                             bias.numel() != m_vec * vec_length):
        raise ValueError("bias must be a contiguous fp16 GPU tensor of m_vec * vec_length = %d elements" % (m_vec * vec_length))
    out = torch.empty((m_vec * vec_length, N), dtype=torch.float16, device=rhs_matrix.device)
    with torch.cuda.device(rhs_matrix.device):
        rc = _lib.lib().sspmm_linear_f16(m_vec, vec_length, N, K, _ptr(row_offsets), _ptr(column_indices), _ptr(values),
                                         _ptr(rhs_matrix), _ptr(bias), ACTIVATIONS[activation], _ptr(out), _stream())
    _lib.check(rc, "sspmm_linear_f16")
    return out


def bspmm(row_indices, row_offsets, column_indices, values, rhs_matrix, vec_length, out_dtype=torch.float16, plan=None):
    """Batched SpMM with one pattern for the whole batch: values [batch, nvec*V],
    rhs_matrix [batch, K, N] -> [batch, m_vec*V, N] (reference batched_spmm_cuda,
    end2end/sspmm_e2e/src/cuda/spmm_kernel.cu:516-586)."""
    _check_inputs(row_indices, row_offsets, column_indices, values, rhs_matrix, vec_length)
    m_vec = row_offsets.size(-1) - 1
    K, N = rhs_matrix.size(-2), rhs_matrix.size(-1)
    batch = rhs_matrix.numel() // (K * N) if K * N > 0 else (rhs_matrix.size(0) if rhs_matrix.dim() > 2 else 1)
    nvec = column_indices.numel()
    if values.numel() != batch * nvec * vec_length:
        raise ValueError("values must hold batch * nvec * vec_length = %d elements, got %d"
                         % (batch * nvec * vec_length, values.numel()))
    M = m_vec * vec_length
    out = torch.empty((batch, M, N), dtype=out_dtype, device=rhs_matrix.device)
    if plan is not None:
        _check_plan(plan, m_vec, vec_length, K)
        fn = {torch.float16: _lib.lib().sspmm_plan_batched_f16_f16,
              torch.float32: _lib.lib().sspmm_plan_batched_f16_f32}[out_dtype]
        with torch.cuda.device(rhs_matrix.device):
            rc = fn(plan.handle, batch, N, _ptr(row_offsets), _ptr(column_indices), _ptr(values), nvec * vec_length,
                    _ptr(rhs_matrix), K * N, _ptr(out), M * N, _stream())
        _lib.check(rc, "sspmm_plan_batched")
        return out
    fn = {torch.float16: _lib.lib().sspmm_batched_f16_f16,
          torch.float32: _lib.lib().sspmm_batched_f16_f32}[out_dtype]
    with torch.cuda.device(rhs_matrix.device):
        rc = fn(batch, m_vec, vec_length, N, K, _ptr(row_indices), _ptr(row_offsets), _ptr(column_indices),
                _ptr(values), nvec * vec_length, _ptr(rhs_matrix), K * N, _ptr(out), M * N, _stream())
    _lib.check(rc, "sspmm_batched")
    return out


SWIZZLE_SORT_FROM = 4096  # vector-rows; measured crossover of the two entry points on an MI355X (13 against 17 us at 2048, 48 against 26 at 8192)


def sorted_row_swizzle(row_offsets):
    """Vector-rows ordered by descending length (reference SortedRowSwizzle,
    SSpMM/include/bm_test_utils.h:210-225), computed on the GPU."""
    if row_offsets.dtype != torch.int32 or not row_offsets.is_cuda:
        raise TypeError("row_offsets must be an int32 GPU tensor")
    m_vec = row_offsets.numel() - 1
    out = torch.empty(max(m_vec, 0), dtype=torch.int32, device=row_offsets.device)
    L = _lib.lib()
    with torch.cuda.device(row_offsets.device):
        if m_vec > SWIZZLE_SORT_FROM:
            # every pair of rows compared in one launch grows with the square of m_vec: a radix sort from here on
            ws = torch.empty(L.sspmm_sorted_row_swizzle_workspace_bytes(m_vec), dtype=torch.uint8, device=row_offsets.device)
            rc = L.sspmm_sorted_row_swizzle_ws(m_vec, _ptr(row_offsets), _ptr(out), _ptr(ws), ws.numel(), _stream())
        else:
            rc = L.sspmm_sorted_row_swizzle(m_vec, _ptr(row_offsets), _ptr(out), _stream())
    _lib.check(rc, "sspmm_sorted_row_swizzle")
    return out
