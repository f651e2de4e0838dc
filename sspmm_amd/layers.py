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

from .spmm import linear as linear_op, spmm
from .svc import svc


class SparseLinear(torch.nn.Module):
    """y[out, tokens] = W @ x[in, tokens] (+ bias[:, None]) with W in the vector-sparse format.

    Build one with `from_dense` (a dense weight whose zero pattern is already vector-structured
    or not: RowMerge on the GPU packs whatever is there) or `from_cvse` (arrays as the SpMM
    takes them)."""

    def __init__(self, in_features, out_features, vec_length, row_offsets, column_indices, values, bias=None,
                 out_dtype=torch.float16, activation=None):
        super().__init__()
        self.activation = activation  # None or "gelu": applied to W @ x + bias
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
    def concat(cls, layers):
        """One layer whose output is the outputs of `layers` stacked along the feature axis: their patterns
        concatenated along M.  Three projections of the same input (query, key, value) become one SpMM that reads
        the input once."""
        first = layers[0]
        if any(l.in_features != first.in_features or l.vec_length != first.vec_length or l.out_dtype != first.out_dtype
               for l in layers):
            raise ValueError("the layers must share in_features, vec_length and output type")
        offsets, base = [first.row_offsets[:1]], 0
        for l in layers:
            offsets.append(l.row_offsets[1:] + base)
            base += int(l.column_indices.numel())
        biases = [l.bias for l in layers]
        bias = None
        if any(b is not None for b in biases):
            bias = torch.cat([b if b is not None else torch.zeros(l.out_features, dtype=torch.float16, device=first.values.device)
                              for b, l in zip(biases, layers)])
        return cls(first.in_features, sum(l.out_features for l in layers), first.vec_length,
                   torch.cat(offsets).to(torch.int32).contiguous(), torch.cat([l.column_indices for l in layers]).contiguous(),
                   torch.cat([l.values for l in layers]).contiguous(), bias, out_dtype=first.out_dtype)

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

    def rows(self, first, last):
        """The layer of output features first .. last-1 (multiples of vec_length) as a layer of its own whose arrays
        are views of this one's: nothing is copied, and the view is not registered anywhere."""
        V = self.vec_length
        if first % V or last % V or not 0 <= first <= last <= self.out_features:
            raise ValueError("row range must be multiples of vec_length inside [0, out_features]")
        off = self.row_offsets[first // V:last // V + 1]
        lo, hi = int(off[0]), int(off[-1])
        return SparseLinear(self.in_features, last - first, V, (off - lo).to(torch.int32), self.column_indices[lo:hi],
                            self.values[lo * V:hi * V], None if self.bias is None else self.bias[first:last],
                            out_dtype=self.out_dtype, activation=self.activation)

    def _apply(self, fn, *args, **kw):
        # a plan lives on the device it was built on and describes the row offsets it was built from: when the
        # buffers are moved or converted it is dropped, and make_plan has to be called again
        self.plan = None
        return super()._apply(fn, *args, **kw)

    def make_plan(self, max_tokens):
        """Builds the pattern's plan (sspmm_amd.Plan) for inputs of up to max_tokens columns; later calls of the
        layer use it.  Worth it for weights whose merged rows are uneven (unstructured pruning through RowMerge)."""
        from .plan import Plan
        self.plan = Plan(self.row_offsets, self.vec_length, self.in_features, max_N=max_tokens)
        return self.plan

    def forward(self, x, activation="layer"):
        """activation: "layer" applies the layer's own (self.activation); None or "gelu" override it for this call."""
        act = self.activation if activation == "layer" else activation
        if x.dim() != 2 or x.size(0) != self.in_features:
            raise ValueError("x must be [in_features, tokens] = [%d, *], got %s" % (self.in_features, tuple(x.shape)))
        plan = getattr(self, "plan", None)
        if plan is not None and x.size(1) > plan.max_N:
            plan = None
        fuse = plan is None and self.out_dtype == torch.float16 and (self.bias is None or self.bias.dtype == torch.float16)
        if fuse and (self.bias is not None or act is not None):
            # bias and activation in the product's epilogue: one launch, the output written once
            return linear_op(self.row_offsets, self.column_indices, self.values, x.contiguous(), self.vec_length,
                             bias=self.bias, activation=act)
        y = spmm(None, self.row_offsets, self.column_indices, self.values, x.contiguous(), self.vec_length,
                 out_dtype=self.out_dtype, plan=plan)
        if self.bias is not None:
            y = y + self.bias[:, None].to(y.dtype)
        if act == "gelu":
            y = torch.nn.functional.gelu(y)
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


def add_layernorm(x, a, ln):
    """LayerNorm over the features of the feature-major sum x + a ([features, tokens] fp16; a may be None) with the
    weights of `ln` (a torch.nn.LayerNorm over `features`).  One HIP kernel (sspmm_add_layernorm_f16 of the C ABI)
    where its shape limits hold, torch on transposed copies otherwise."""
    from . import _lib
    H, T = x.shape
    ok = (x.dtype == torch.float16 and x.is_cuda and x.is_contiguous() and T % 4 == 0 and H <= 4096 and
          (a is None or (a.dtype == torch.float16 and a.is_contiguous() and a.shape == x.shape)) and
          ln.weight is not None and ln.weight.dtype == torch.float16 and tuple(ln.normalized_shape) == (H,))
    if not ok:
        s = x if a is None else x + a
        return ln(s.t()).t().contiguous()
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = _lib.lib().sspmm_add_layernorm_f16(H, T, x.data_ptr(), 0 if a is None else a.data_ptr(), ln.weight.data_ptr(),
                                                0 if ln.bias is None else ln.bias.data_ptr(), float(ln.eps), out.data_ptr(),
                                                torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "sspmm_add_layernorm_f16")
    return out


def attention_fm(qkv, hidden, heads, batch, seq, scale=None):
    """softmax(Q^T K * scale) V per (batch element, head) on the fused feature-major projections qkv
    [3 * hidden, batch * seq] fp16 (rows 0 .. hidden-1 the queries, then keys, then values; token b * seq + s in
    column b * seq + s); returns the context [hidden, batch * seq], or None where the kernel's shape limits do not
    hold (the caller then takes another route)."""
    from . import _lib
    d = hidden // heads
    T = batch * seq
    if not (qkv.dtype == torch.float16 and qkv.is_cuda and qkv.is_contiguous() and tuple(qkv.shape) == (3 * hidden, T) and
            d == 64 and hidden == heads * d and seq % 64 == 0 and 64 <= seq <= 16384 and T % 8 == 0):
        return None
    out = torch.empty(hidden, T, dtype=torch.float16, device=qkv.device)
    esz = qkv.element_size()
    with torch.cuda.device(qkv.device):
        rc = _lib.lib().sspmm_attention_fm_f16(batch, heads, seq, d, qkv.data_ptr(), qkv.data_ptr() + hidden * T * esz,
                                               qkv.data_ptr() + 2 * hidden * T * esz, T, out.data_ptr(), T,
                                               float(1.0 / math.sqrt(d) if scale is None else scale),
                                               torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "sspmm_attention_fm_f16")
    return out


class SparseEncoderLayer(torch.nn.Module):
    """Post-LayerNorm transformer encoder layer with vector-sparse Q, K, V, output and FFN weights
    and dense attention, on feature-major activations x[hidden, batch * seq]."""

    def __init__(self, hidden, heads, ffn, q, k, v, o, ffn1, ffn2):
        super().__init__()
        self.hidden, self.heads, self.ffn = hidden, heads, ffn
        self.o, self.ffn1, self.ffn2 = o, ffn1, ffn2
        # query, key and value projections as one SpMM over the three patterns stacked along M.  The fused layer is
        # the only copy the module keeps (q, k and v below are views of its arrays), so the weights are held once and
        # state_dict names them once.
        self.qkv = SparseLinear.concat([q, k, v])
        self._qkv_rows = (0, q.out_features, q.out_features + k.out_features,
                          q.out_features + k.out_features + v.out_features)
        self.ln1 = torch.nn.LayerNorm(hidden)
        self.ln2 = torch.nn.LayerNorm(hidden)

    q = property(lambda self: self.qkv.rows(self._qkv_rows[0], self._qkv_rows[1]))
    k = property(lambda self: self.qkv.rows(self._qkv_rows[1], self._qkv_rows[2]))
    v = property(lambda self: self.qkv.rows(self._qkv_rows[2], self._qkv_rows[3]))

    @property
    def ffn1_gelu(self):
        """The first feed-forward product with its GELU in the product's epilogue: ffn1 itself, called with the
        activation (no second module, no second copy of the arrays)."""
        ffn1 = self.ffn1

        class _WithGelu:
            in_features, out_features = ffn1.in_features, ffn1.out_features
            dense_weight = staticmethod(ffn1.dense_weight)

            def __call__(self, x):
                return ffn1(x, activation="gelu")

        return _WithGelu()

    def _attention(self, qkv, batch, seq):
        """qkv: [3 * hidden, batch*seq] feature-major; returns the context [hidden, batch*seq].  One HIP kernel that
        reads and writes the feature-major layout (sspmm_attention_fm_f16 of the C ABI) where its shape limits hold
        (head size 64, seq a multiple of 64).  Otherwise torch's attention between two relayout copies:
        one brings the three projections into the [batch, heads, seq, head size] layout it wants contiguous (on
        strided views of the feature-major activations it runs ten times slower), one brings the context back."""
        h, d = self.heads, self.hidden // self.heads
        ctx = attention_fm(qkv, self.hidden, h, batch, seq)
        if ctx is not None:
            return ctx
        c = qkv.view(3, h, d, batch, seq).permute(0, 3, 1, 4, 2).contiguous()
        ctx = torch.nn.functional.scaled_dot_product_attention(c[0], c[1], c[2], scale=1.0 / math.sqrt(d))
        return ctx.permute(1, 3, 0, 2).reshape(self.hidden, batch * seq)

    def forward(self, x, batch, seq, linear=None):
        """x: [hidden, batch*seq] fp16.  `linear(name, layer, x)` may replace how a projection ("qkv", "o",
        "ffn1_gelu", "ffn2"; "ffn1_gelu" is the first feed-forward product with the GELU behind it) is evaluated
        (the benchmark passes a dense matmul there to time the same layer without sparsity)."""
        f = linear or (lambda name, layer, t: layer(t))
        a = f("o", self.o, self._attention(f("qkv", self.qkv, x), batch, seq))
        x = add_layernorm(x, a, self.ln1)
        y = f("ffn2", self.ffn2, f("ffn1_gelu", self.ffn1_gelu, x))
        return add_layernorm(x, y, self.ln2)
