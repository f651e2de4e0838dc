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


FUSED_HEAD_WIDTHS = (32, 64, 128)


def fused_sparse_attention(row_indices, row_offsets, column_indices, q, k, v, scaling, vec_length):
    """The block's three steps in one launch (heads of 32, 64 or 128 features): scores and probabilities never leave the
    chip.  Same arguments and result shape as `sparse_attention`; differs from the three-step chain by fp16 rounding
    of intermediate values only (the chain rounds the scores and the normalised probabilities to fp16, this rounds
    the probabilities before the division by their sum)."""
    _check_pattern(row_indices, row_offsets, column_indices, vec_length)
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_half(name, t)
    m, d, n = q.size(-2), q.size(-1), k.size(-2)
    if d not in FUSED_HEAD_WIDTHS or k.size(-1) != d or v.size(-1) != d:
        raise ValueError("fused_sparse_attention takes heads of 32, 64 or 128 features, the same for q, k and v")
    if v.size(-2) != n:
        raise ValueError("k and v must have the same number of rows")
    m_vec = row_offsets.numel() - 1
    if m != m_vec * vec_length:
        raise ValueError("q must have m_vec * vec_length = %d rows, got %d" % (m_vec * vec_length, m))
    batch = q.numel() // (m * d) if m > 0 else 1
    if k.numel() != batch * n * d or v.numel() != batch * n * d:
        raise ValueError("q, k and v must have the same batch size")
    out = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    with torch.cuda.device(q.device):
        rc = _lib.lib().sspmm_sparse_attention_f16(batch, m_vec, vec_length, d, n, _ptr(row_indices), _ptr(row_offsets),
                                                   _ptr(column_indices), _ptr(q), m * d, _ptr(k), n * d, _ptr(v), n * d,
                                                   float(scaling), _ptr(out), m * d, _stream())
    _lib.check(rc, "sspmm_sparse_attention")
    return out


def packed_attention_fits(seq, bsz, three_e):
    """Whether `sparse_attention_packed` takes a projection of this shape: the rows of one (batch element, head) pair,
    which lie `bsz * three_e` elements apart, must span less than 2 GiB (one 32-bit buffer descriptor)."""
    return (seq - 1) * bsz * three_e * 2 < (1 << 31) - 256 and bsz * three_e < (1 << 23) and seq < (1 << 24)


def sparse_attention_packed(row_indices, row_offsets, column_indices, qkv, num_heads, scaling, vec_length):
    """Multi-head attention on a vector-sparse mask straight from a fused projection: qkv [seq, batch, 3 * embed] (q,
    k and v side by side in the last dimension, heads of 32, 64 or 128 features side by side in each) -> [seq, batch, embed],
    in one launch and without the copies into [batch * heads, seq, 64] and back that the reference's module makes
    around its three operators (spattention.py:151-157 and 181-184)."""
    _check_pattern(row_indices, row_offsets, column_indices, vec_length)
    _check_half("qkv", qkv)
    if qkv.dim() != 3 or qkv.size(-1) % (3 * num_heads) or qkv.size(-1) // (3 * num_heads) not in FUSED_HEAD_WIDTHS:
        raise ValueError("qkv must be [seq, batch, 3 * num_heads * d] with d = 32, 64 or 128")
    seq, bsz, three_e = qkv.shape
    e = three_e // 3
    d = e // num_heads
    m_vec = row_offsets.numel() - 1
    if seq != m_vec * vec_length:
        raise ValueError("qkv must have m_vec * vec_length = %d rows, got %d" % (m_vec * vec_length, seq))
    out = torch.empty((seq, bsz, e), dtype=torch.float16, device=qkv.device)
    base, ld = qkv.data_ptr(), bsz * three_e
    with torch.cuda.device(qkv.device):
        rc = _lib.lib().sspmm_sparse_attention_heads_f16(
            bsz, num_heads, m_vec, vec_length, d, seq, _ptr(row_indices), _ptr(row_offsets), _ptr(column_indices),
            base, three_e, d, ld, base + 2 * e, three_e, d, ld, base + 4 * e, three_e, d, ld, float(scaling),
            _ptr(out), e, d, bsz * e, _stream())
    _lib.check(rc, "sspmm_sparse_attention_heads")
    return out


def sparse_attention(row_indices, row_offsets, column_indices, q, k, v, scaling, vec_length, fused=None):
    """softmax(mask(q k^T) * scaling) v on a vector-sparse mask shared by the batch:
    q [batch, tgt, d], k [batch, src, d], v [batch, src, d_v] -> fp16 [batch, tgt, d_v]; the three
    steps of the reference's block (spattention.py:167-179).  fused: None = one launch where the shapes allow it
    (d = d_v = 32, 64 or 128), False = always the three operators, True = one launch or an error."""
    if fused is None:
        fused = q.size(-1) in FUSED_HEAD_WIDTHS and v.size(-1) == q.size(-1) and row_offsets.numel() > 1 and q.numel() > 0
    if fused:
        return fused_sparse_attention(row_indices, row_offsets, column_indices, q, k, v, scaling, vec_length)
    w = bsddmm(row_indices, row_offsets, column_indices, q, k, vec_length)
    w = bcsr_softmax(row_indices, row_offsets, w, scaling, vec_length, w.size(0))
    _check_inputs(row_indices, row_offsets, column_indices, w, v, vec_length)
    return bspmm(row_indices, row_offsets, column_indices, w, v, vec_length)


def static_random_mask(m_vec, n, sparsity, seed=0):
    """A vector-sparse attention mask as the reference's end-to-end model draws it (verify/static_mask.py:7-27:
    scipy.sparse.random of m_vec x n with density 1 - sparsity, i.e. round(density * m_vec * n) positions drawn uniformly
    without replacement, CSR with ascending columns; row_indices = vector-rows by ascending length).  Seeded numpy
    in place of scipy's global state.  Returns (column_indices, row_offsets, row_indices) as int32 numpy arrays."""
    import numpy as np
    rng = np.random.default_rng(seed)
    k = int(round((1.0 - sparsity) * m_vec * n))
    flat = np.sort(rng.choice(m_vec * n, size=k, replace=False))
    rows, cols = flat // n, flat % n
    row_offsets = np.concatenate([[0], np.cumsum(np.bincount(rows, minlength=m_vec))]).astype(np.int32)
    row_indices = np.argsort(np.diff(row_offsets), kind="stable").astype(np.int32)
    return cols.astype(np.int32), row_offsets, row_indices


class SparseAttentionBlock(torch.nn.Module):
    """One block of the reference's end-to-end model (SparseTransformerBlock, end2end/sspmm_e2e/end_to_end.py:45-78):
    LayerNorm -> multi-head attention on a static vector-sparse mask (bsddmm -> bcsr_softmax -> bspmm,
    spattention.py:151-186) -> + x -> LayerNorm -> linear1 -> linear2 -> + x, on [seq, batch, embed] activations.
    The block's arithmetic follows the reference as written, including the second residual adding the block's input
    and the two linear layers without an activation between them."""

    def __init__(self, embed_dim, mlp_dim, num_heads, column_indices, row_offsets, row_indices, vec_length=8):
        super().__init__()
        if embed_dim % num_heads:
            raise ValueError("embed_dim must be a multiple of num_heads")
        self.embed_dim, self.num_heads, self.vec_length = embed_dim, num_heads, vec_length
        self.in_proj = torch.nn.Linear(embed_dim, 3 * embed_dim)
        self.out_proj = torch.nn.Linear(embed_dim, embed_dim)
        self.layer_norm1 = torch.nn.LayerNorm(embed_dim)
        self.layer_norm2 = torch.nn.LayerNorm(embed_dim)
        self.linear1 = torch.nn.Linear(embed_dim, mlp_dim)
        self.linear2 = torch.nn.Linear(mlp_dim, embed_dim)
        self.register_buffer("column_indices", column_indices)
        self.register_buffer("row_offsets", row_offsets)
        self.register_buffer("row_indices", row_indices)

    def attention(self, x, dense_mask=None):
        """x [seq, batch, embed] -> [seq, batch, embed].  With dense_mask (bool [seq, seq]) the three sparse steps
        are replaced by dense masked attention in fp32 (for checks)."""
        seq, bsz, E = x.shape
        h, d = self.num_heads, E // self.num_heads
        scaling = float(d) ** -0.5
        qkv = self.in_proj(x)
        if dense_mask is None and d in FUSED_HEAD_WIDTHS and qkv.dtype == torch.float16 and packed_attention_fits(seq, bsz, 3 * E):
            # the heads are read where the projection left them and written where the output projection wants them
            return self.out_proj(sparse_attention_packed(self.row_indices, self.row_offsets, self.column_indices,
                                                         qkv.contiguous(), h, scaling, self.vec_length))
        q, k, v = qkv.chunk(3, dim=-1)
        # [seq, batch * heads, d] -> [batch * heads, seq, d] (spattention.py:151-157)
        q, k, v = (t.contiguous().view(seq, bsz * h, d).transpose(0, 1).contiguous() for t in (q, k, v))
        if dense_mask is None:
            out = sparse_attention(self.row_indices, self.row_offsets, self.column_indices, q, k, v, scaling, self.vec_length)
        else:
            s = (q.float() @ k.float().transpose(1, 2)) * scaling
            s = s.masked_fill(~dense_mask, float("-inf"))
            out = (torch.softmax(s, dim=-1) @ v.float()).to(x.dtype)
        out = out.transpose(0, 1).contiguous().view(seq, bsz, E)
        return self.out_proj(out)

    def forward(self, x, dense_mask=None):
        out = self.attention(self.layer_norm1(x), dense_mask) + x
        out = self.linear2(self.linear1(self.layer_norm2(out)))
        return out + x


class SparseAttentionEncoder(torch.nn.Module):
    """The reference's end-to-end model (SparseTransformerEncoder, end_to_end.py:123-153): embedding * sqrt(embed),
    sinusoidal positions, four SparseAttentionBlocks each with a mask of its own, LayerNorm, linear head."""

    def __init__(self, vocab_size, embed_dim, num_heads, sparsity, seq_len, mlp_dim, num_class, vec_length=8, layers=4, seed=0):
        super().__init__()
        import math
        self.embed_dim = embed_dim
        self.encoder = torch.nn.Embedding(vocab_size, embed_dim)
        pe = torch.zeros(seq_len, embed_dim)
        pos = torch.arange(0, seq_len, dtype=torch.float).unsqueeze(1)
        div = torch.exp(torch.arange(0, embed_dim, 2).float() * (-math.log(10000.0) / embed_dim))
        pe[:, 0::2] = torch.sin(pos * div)
        pe[:, 1::2] = torch.cos(pos * div)
        self.register_buffer("pe", pe.unsqueeze(1))
        blocks = []
        for i in range(layers):
            cols, offs, rows = static_random_mask(seq_len // vec_length, seq_len, sparsity, seed=seed + i)
            blocks.append(SparseAttentionBlock(embed_dim, mlp_dim, num_heads, torch.from_numpy(cols), torch.from_numpy(offs),
                                               torch.from_numpy(rows), vec_length))
        self.blocks = torch.nn.ModuleList(blocks)
        self.layer_norm = torch.nn.LayerNorm(embed_dim)
        self.linear = torch.nn.Linear(embed_dim, num_class)

    def forward(self, tokens, dense_masks=None):
        """tokens: int [batch, seq] -> [seq, batch, num_class]."""
        out = self.encoder(tokens) * (self.embed_dim ** 0.5)
        out = out.transpose(0, 1) + self.pe[:tokens.size(1)].to(out.dtype)
        for i, blk in enumerate(self.blocks):
            out = blk(out, None if dense_masks is None else dense_masks[i])
        return self.linear(self.layer_norm(out))
