"""Plans: what the library works out about a sparsity pattern before its first product.

The reference's handle on uneven vector-rows is the permutation `row_indices` (SortedRowSwizzle,
reference SSpMM/include/bm_test_utils.h:210-225, consumed at end2end/sspmm_e2e/src/cuda/
spmm_kernel.cu:48).  A Plan takes its place for callers that keep a pattern: it is built once from
`row_offsets` on the GPU (sspmm_plan_create of the C ABI), and `spmm(..., plan=plan)` /
`bspmm(..., plan=plan)` then cut overlong vector-rows into panels of equal work.
"""
import collections
import ctypes

import torch

from . import _lib

PlanInfo = collections.namedtuple(
    "PlanInfo", ["num_vec", "longest_row_steps", "total_steps", "panel_steps", "cut_rows", "panels", "items", "device_bytes"])


class Plan:
    """plan = Plan(row_offsets, vec_length, K, max_N, max_batch=1)

    row_offsets: int32 GPU tensor [m_vec + 1].  max_N / max_batch: the widest right-hand side and the largest
    batch the plan will see.  One plan serves one product at a time (one plan per stream)."""

    def __init__(self, row_offsets, vec_length, K, max_N, max_batch=1, panel_steps=0):
        if row_offsets.dtype != torch.int32 or not row_offsets.is_cuda or not row_offsets.is_contiguous():
            raise TypeError("row_offsets must be a contiguous int32 GPU tensor")
        self._handle = ctypes.c_void_p()
        self._lib = _lib.lib()
        self.device = row_offsets.device
        self.m_vec = row_offsets.numel() - 1
        self.vec_length, self.K, self.max_N, self.max_batch = vec_length, K, max_N, max_batch
        with torch.cuda.device(self.device):
            rc = self._lib.sspmm_plan_create(self.m_vec, vec_length, K, row_offsets.data_ptr(), max_N, max_batch,
                                             panel_steps, torch.cuda.current_stream().cuda_stream,
                                             ctypes.byref(self._handle))
        _lib.check(rc, "sspmm_plan_create")

    @property
    def handle(self):
        if not self._handle:
            raise RuntimeError("the plan has been destroyed")
        return self._handle

    def info(self):
        buf = (ctypes.c_int64 * 8)()
        _lib.check(self._lib.sspmm_plan_info(self.handle, buf), "sspmm_plan_info")
        return PlanInfo(*[int(x) for x in buf])

    def destroy(self):
        if self._handle:
            self._lib.sspmm_plan_destroy(self._handle)
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:  # interpreter shutdown
            pass
