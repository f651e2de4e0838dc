"""Model-side callers of the SpMM: a linear layer whose weight is vector-sparse, and the
transformer encoder layer of the BERT-base shaped benchmark configuration built from six of
them.

The reference reaches its kernels from torch modules the same way (the sparse attention block
calls `bspmm(row_indices, row_offsets, column_indices, values, v, vec_length)`, reference
end2end/sspmm_e2e/spattention.py:179; the weight-sparse layers of its evaluation are the SpMM
harness shapes, reference SSpMM/sspmm_test.cpp:141,189).  Activations are kept feature-major
([features, tokens]) so that every weight-sparse product is C[out, tokens] = W[out, in] @
X[in, tokens], the SpMM's native orientation, and no transposes sit between the layers.

Inference only: the operators have no backward pass.  Everything that is not an SpMM (attention
scores, softmax, LayerNorm, GELU, bias) runs in torch-ROCm; the products with the sparse
weights run in the HIP kernels behind the C ABI.
"""
import math

import numpy as np
import torch

from .spmm import spmm
from .svc import svc


class SparseLinear(torch.nn.Module):
    """y[out, tokens] = W @ x[in, tokens] (+ bias[:, None]) with W in the vector-sparse format.

    Build one with `from_dense` (a dense weight whose zero pattern is already vector-structured
    or not: RowMerge on the GPU packs whatever is there) or `from_cvse` (arrays as the SpMM
    takes them)."""

    def __init__(self, in_features, out_features, vec_length, row_offsets, column_indices, values, bias=None,
                 out_dtype=torch.float16):
        super().__init__()
        if out_features % vec_length:
            raise ValueError("out_features must be a multiple of vec_length")
        self.in_features, self.out_features, self.vec_length = in_features, out_features, vec_length
        self.out_dtype = out_dtype
        self.register_buffer("row_offsets", row_offsets)
        self.register_buffer("column_indices", column_indices)
        self.register_buffer("values", values)
        self.register_buffer("bias", bias)

    @classmethod
    def from_cvse(cls, in_features, vec_length, row_offsets, column_indices, values, bias=None, **kw):
        m_vec = row_offsets.numel() - 1
        return cls(in_features, m_vec * vec_length, vec_length, row_offsets, column_indices, values, bias, **kw)

    @classmethod
    def from_dense(cls, weight, vec_length, bias=None, order="sorted", **kw):
        """weight: [out, in] fp16 GPU tensor; its non-zeros are merged V rows at a time (SVC on the GPU)."""
        if weight.dtype != torch.float16 or not weight.is_cuda:
            raise TypeError("weight must be a float16 GPU tensor")
        out_features, in_features = weight.shape
        mask = weight != 0
        row_ptr = torch.zeros(out_features + 1, dtype=torch.int32, device=weight.device)
        row_ptr[1:] = mask.sum(dim=1).cumsum(0).to(torch.int32)
        col_ind = mask.nonzero()[:, 1].to(torch.int32).contiguous()
        r = svc(row_ptr, col_ind, weight[mask].contiguous(), out_features, in_features, vec_length, order=order)
        return cls(in_features, out_features, vec_length, r.vec_row_ptr, r.vec_col, r.vec_val, bias, **kw)

    def forward(self, x):
        if x.dim() != 2 or x.size(0) != self.in_features:
            raise ValueError("x must be [in_features, tokens] = [%d, *], got %s" % (self.in_features, tuple(x.shape)))
        y = spmm(None, self.row_offsets, self.column_indices, self.values, x.contiguous(), self.vec_length,
                 out_dtype=self.out_dtype)
        if self.bias is not None:
            y = y + self.bias[:, None].to(y.dtype)
        return y

    def dense_weight(self):
        """The weight as a dense [out, in] fp16 tensor (for checks)."""
        V = self.vec_length
        off = self.row_offsets.cpu().numpy()
        cols = self.column_indices.cpu().numpy()
        vals = self.values.cpu().numpy().reshape(-1, V)
        W = np.zeros((self.out_features, self.in_features), np.float16)
        for i in range(off.size - 1):
            W[i * V:(i + 1) * V, cols[off[i]:off[i + 1]]] = vals[off[i]:off[i + 1]].T
        return torch.from_numpy(W).to(self.values.device)


class SparseEncoderLayer(torch.nn.Module):
    """Post-LayerNorm transformer encoder layer with vector-sparse Q, K, V, output and FFN weights
    and dense attention, on feature-major activations x[hidden, batch * seq]."""

    def __init__(self, hidden, heads, ffn, q, k, v, o, ffn1, ffn2):
        super().__init__()
        self.hidden, self.heads, self.ffn = hidden, heads, ffn
        self.q, self.k, self.v, self.o, self.ffn1, self.ffn2 = q, k, v, o, ffn1, ffn2
        self.ln1 = torch.nn.LayerNorm(hidden)
        self.ln2 = torch.nn.LayerNorm(hidden)

    def _attention(self, q, k, v, batch, seq):
        h, d = self.heads, self.hidden // self.heads
        # [hidden, batch*seq] -> [batch, heads, seq, d]
        def split(t):
            return t.view(h, d, batch, seq).permute(2, 0, 3, 1)
        ctx = torch.nn.functional.scaled_dot_product_attention(split(q), split(k), split(v), scale=1.0 / math.sqrt(d))
        return ctx.permute(1, 3, 0, 2).reshape(self.hidden, batch * seq)

    def forward(self, x, batch, seq, linear=None):
        """x: [hidden, batch*seq] fp16.  `linear(name, layer, x)` may replace how a projection is
        evaluated (the benchmark passes a dense matmul there to time the same layer without sparsity)."""
        f = linear or (lambda name, layer, t: layer(t))
        q, k, v = f("q", self.q, x), f("k", self.k, x), f("v", self.v, x)
        a = f("o", self.o, self._attention(q, k, v, batch, seq))
        x = self.ln1((x + a).t()).t().contiguous()
        y = f("ffn2", self.ffn2, torch.nn.functional.gelu(f("ffn1", self.ffn1, x)))
        return self.ln2((x + y).t()).t().contiguous()
