"""MI355X (gfx950) implementation of the SSpMM hot path: Sparse Vector Compression (RowMerge)
and the vector-sparse SpMM, behind the reference's operator surface.

    from sspmm_amd import spmm, bspmm, svc
    C = spmm(row_indices, row_offsets, column_indices, values, rhs_matrix, vec_length)

All compute runs in hand-written HIP kernels reached through the C ABI of libsspmm_amd.so
(include/sspmm.h); there is no CPU or PyTorch fallback: without the built library every
operator raises.
"""
from .spmm import spmm, bspmm, sorted_row_swizzle  # noqa: F401
from .plan import Plan, PlanInfo  # noqa: F401
from .svc import svc, svc_batched, stack_csr, SvcBatch, SvcResult  # noqa: F401
from .attention import sddmm, bsddmm, csr_softmax, bcsr_softmax, sparse_attention, fused_sparse_attention, sparse_attention_packed  # noqa: F401
from .reorder import minhash_order, permute_csr, svc_reordered  # noqa: F401
from .layers import SparseLinear, SparseEncoderLayer  # noqa: F401
from .formats import Cvse, read_smtx, write_smtx, read_cvse, write_cvse, cvse_text  # noqa: F401
from ._lib import build_library, library_path  # noqa: F401
