"""GPU parity of the sampled product, the sparse softmax and the attention block that chains them
with the batched SpMM, through the C ABI, against the CPU oracle and dense torch arithmetic."""
import math

import numpy as np
import pytest
import torch

import sspmm_amd
from sspmm_amd import synth
from gpu_util import dev, max_rel_err

pytestmark = pytest.mark.gpu


def _pattern(m_rows, K, V, sparsity, seed):
    return synth.vector_sparse(m_rows * V, K, V, sparsity, seed=seed)


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("F", [8, 40, 64, 128, 200, 256])
def test_sddmm_matches_oracle(oracle, built_library, V, F):
    vs = _pattern(20, 300, V, 0.8, seed=100 + F)
    rng = np.random.default_rng(F)
    lhs = rng.standard_normal((vs.m_vec * V, F)).astype(np.float16)
    rhs = rng.standard_normal((300, F)).astype(np.float16)
    print("sddmm V=%d F=%d nvec=%d" % (V, F, vs.col_idx.size), flush=True)
    got = sspmm_amd.sddmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(lhs), dev(rhs), V)
    torch.cuda.synchronize()
    want = oracle.sddmm(vs.m_vec, V, vs.row_offsets, vs.col_idx, lhs, rhs)
    assert got.shape == (vs.col_idx.size * V,)
    assert max_rel_err(got.cpu().numpy(), want) <= 2e-3
    # exact on small integers (every product and partial sum is representable)
    lhs_i = rng.integers(-3, 4, lhs.shape).astype(np.float16)
    rhs_i = rng.integers(-3, 4, rhs.shape).astype(np.float16)
    got = sspmm_amd.sddmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(lhs_i), dev(rhs_i), V).cpu().numpy()
    assert np.array_equal(got, oracle.sddmm(vs.m_vec, V, vs.row_offsets, vs.col_idx, lhs_i, rhs_i))


@pytest.mark.parametrize("per_row", [0, 1, 15, 16, 17, 31, 32, 33, 100])
def test_sddmm_row_length_tails_and_permutation(oracle, built_library, per_row):
    V, K, F, m_vec = 8, 128, 64, 6
    rng = np.random.default_rng(per_row)
    cols = np.concatenate([rng.permutation(K)[:per_row] for _ in range(m_vec)] or [[]]).astype(np.int32)
    off = (np.arange(m_vec + 1) * per_row).astype(np.int32)
    lhs = rng.standard_normal((m_vec * V, F)).astype(np.float16)
    rhs = rng.standard_normal((K, F)).astype(np.float16)
    want = oracle.sddmm(m_vec, V, off, cols, lhs, rhs)
    perm = dev(rng.permutation(m_vec).astype(np.int32))
    for ri in (None, perm):
        got = sspmm_amd.sddmm(ri, dev(off), dev(cols) if cols.size else torch.empty(0, dtype=torch.int32, device="cuda"),
                              dev(lhs), dev(rhs), V)
        torch.cuda.synchronize()
        assert got.numel() == cols.size * V
        if cols.size:
            assert max_rel_err(got.cpu().numpy(), want) <= 2e-3


@pytest.mark.parametrize("V", [8, 16])
def test_softmax_matches_oracle_and_rows_sum_to_one(oracle, built_library, V):
    rng = np.random.default_rng(7)
    lens = np.array([0, 1, 5, 64, 65, 200, 0, 1000, 3, 256, 257, 512, 513])  # around what a wave keeps in registers
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    vals = (rng.standard_normal(off[-1] * V) * 4).astype(np.float16)
    scaler = 1.0 / math.sqrt(64)
    got = sspmm_amd.csr_softmax(None, dev(off), dev(vals), scaler, V)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    want = oracle.softmax(len(lens), V, off, vals, scaler)
    assert np.abs(got.astype(np.float64) - want.astype(np.float64)).max() <= 2e-3
    g = got.astype(np.float64).reshape(-1, V)
    for i, n in enumerate(lens):
        if n:
            assert np.all(np.abs(g[off[i]:off[i + 1]].sum(axis=0) - 1) < 1e-2)
    # a negative scaler turns the row's minimum into the reference point
    neg = sspmm_amd.csr_softmax(None, dev(off), dev(vals), -0.25, V).cpu().numpy()
    assert np.abs(neg.astype(np.float64) - oracle.softmax(len(lens), V, off, vals, -0.25).astype(np.float64)).max() <= 2e-3
    # a large common offset must not overflow: softmax is shift invariant
    big = (vals.astype(np.float32) + 30000).astype(np.float16)
    shifted = sspmm_amd.csr_softmax(None, dev(off), dev(big), 1.0, V).cpu().numpy()
    assert np.isfinite(shifted).all()


def test_batched_ops_match_looped_single_calls(oracle, built_library):
    V, K, F, batch = 8, 160, 64, 5
    vs = _pattern(16, K, V, 0.85, seed=9)
    rng = np.random.default_rng(10)
    q = rng.standard_normal((batch, vs.m_vec * V, F)).astype(np.float16)
    k = rng.standard_normal((batch, K, F)).astype(np.float16)
    off, col = dev(vs.row_offsets), dev(vs.col_idx)
    w = sspmm_amd.bsddmm(None, off, col, dev(q), dev(k), V)
    p = sspmm_amd.bcsr_softmax(None, off, w, 0.125, V, batch)
    torch.cuda.synchronize()
    assert w.shape == (batch, vs.col_idx.size * V) and p.shape == w.shape
    for b in range(batch):
        assert torch.equal(w[b], sspmm_amd.sddmm(None, off, col, dev(q[b]), dev(k[b]), V))
        assert torch.equal(p[b], sspmm_amd.csr_softmax(None, off, w[b].contiguous(), 0.125, V))


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("V", [8, 16])
def test_sparse_attention_matches_dense_masked_attention(built_library, V, fused):
    """The reference's block (sddmm -> softmax -> spmm), as three launches and as one, against torch attention
    with a -inf mask."""
    seq, d, batch = 256, 64, 6
    vs = _pattern(seq // V, seq, V, 0.8, seed=11)
    g = torch.Generator("cuda").manual_seed(12)
    q, k, v = (torch.randn(batch, seq, d, device="cuda", generator=g).half() for _ in range(3))
    out = sspmm_amd.sparse_attention(None, dev(vs.row_offsets), dev(vs.col_idx), q, k, v, 1.0 / math.sqrt(d), V, fused=fused)
    torch.cuda.synchronize()
    mask = torch.full((seq, seq), float("-inf"), device="cuda")
    for i in range(vs.m_vec):
        cols = torch.from_numpy(vs.col_idx[vs.row_offsets[i]:vs.row_offsets[i + 1]].astype(np.int64)).cuda()
        mask[i * V:(i + 1) * V, cols] = 0
    scores = q.float() @ k.float().transpose(1, 2) / math.sqrt(d) + mask
    want = torch.softmax(scores, dim=-1) @ v.float()
    assert out.shape == (batch, seq, d) and out.dtype == torch.float16
    assert max_rel_err(out.float().cpu().numpy(), want.cpu().numpy()) <= 1e-2


def _dense_attention(off, cols, V, q, k, v, scale):
    """float64 numpy: per vector-row, softmax over the stored columns, rows without any give zeros."""
    batch, m, d = q.shape
    out = np.zeros((batch, m, v.shape[-1]))
    q64, k64, v64 = (t.astype(np.float64) for t in (q, k, v))
    for i in range(len(off) - 1):
        c = cols[off[i]:off[i + 1]]
        if c.size == 0:
            continue
        s = np.einsum("bvd,bjd->bvj", q64[:, i * V:(i + 1) * V], k64[:, c]) * scale
        e = np.exp(s - s.max(axis=-1, keepdims=True))
        out[:, i * V:(i + 1) * V] = np.einsum("bvj,bjd->bvd", e / e.sum(axis=-1, keepdims=True), v64[:, c])
    return out


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("V", [8, 16])
def test_one_launch_attention_row_lengths_permutation_and_large_scores(built_library, V, d):
    """Rows of every length around the kernel's step of 32 vectors (none, one, a full step, one more, several steps
    and a tail), visited through a permutation, with scores large enough that the running maximum has to move by
    hundreds between steps; against float64 arithmetic and against the three launches."""
    n_keys, batch = 200, 3
    lens = [0, 1, 2, 31, 32, 33, 63, 64, 65, 96, 100, 200, 0, 7]
    rng = np.random.default_rng(40 + V + d)
    cols = np.concatenate([np.sort(rng.permutation(n_keys)[:n]) for n in lens]).astype(np.int32)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    m = len(lens) * V
    q = (rng.standard_normal((batch, m, d)) * 3 * (64 / d) ** 0.5).astype(np.float16)
    k = (rng.standard_normal((batch, n_keys, d)) * 3).astype(np.float16)
    v = rng.standard_normal((batch, n_keys, d)).astype(np.float16)
    perm = dev(rng.permutation(len(lens)).astype(np.int32))
    for scale in (0.125, 2.0):  # scores up to a few hundred, then a few thousand
        want = _dense_attention(off, cols, V, q, k, v, scale)
        for ri in (None, perm):
            print("attention V=%d d=%d scale=%g permuted=%s" % (V, d, scale, ri is not None), flush=True)
            got = sspmm_amd.fused_sparse_attention(ri, dev(off), dev(cols), dev(q), dev(k), dev(v), scale, V)
            torch.cuda.synchronize()
            got = got.cpu().numpy().astype(np.float64)
            assert np.isfinite(got).all()
            assert np.abs(got - want).max() <= 4e-3 * max(1.0, np.abs(want).max())
            for i, n in enumerate(lens):
                if n == 0:
                    assert not got[:, i * V:(i + 1) * V].any()
    chain = sspmm_amd.sparse_attention(None, dev(off), dev(cols), dev(q), dev(k), dev(v), 0.125, V, fused=False)
    one = sspmm_amd.sparse_attention(None, dev(off), dev(cols), dev(q), dev(k), dev(v), 0.125, V)  # picks the one launch
    assert torch.equal(one, sspmm_amd.fused_sparse_attention(None, dev(off), dev(cols), dev(q), dev(k), dev(v), 0.125, V))
    # (the chain rounds scores of magnitude up to ~100 to fp16, a step of 1/16 in the exponent's argument before the scale)
    assert (one.float() - chain.float()).abs().max().item() <= 3e-2


def test_one_launch_attention_at_full_size_by_its_properties(built_library):
    """The benchmark's block (4096 tokens, 90 % of the vectors masked out, 48 heads of 64 features): with every row of
    v the same the probabilities of a row must add up to one, so every query gets that row back; columns stored in
    another order inside the vector-rows change the sums' order only; a permutation of the vector-rows changes nothing."""
    V, seq, heads, d = 8, 4096, 48, 64
    from sspmm_amd.attention import static_random_mask
    cols, off, rows = static_random_mask(seq // V, seq, 0.9, seed=5)
    rng = np.random.default_rng(6)
    shuffled = cols.copy()
    for i in range(len(off) - 1):
        rng.shuffle(shuffled[off[i]:off[i + 1]])
    g = torch.Generator("cuda").manual_seed(7)
    q, k, v = (torch.randn(heads, seq, d, device="cuda", generator=g).half() for _ in range(3))
    const = torch.full((d,), 0.0, device="cuda").half()
    const[::2], const[1::2] = 0.75, -1.5
    v_const = const.expand(heads, seq, d).contiguous()
    d_off, d_cols, d_rows, d_shuf = dev(off), dev(cols), dev(rows), dev(shuffled)
    print("attention at full size: %d vectors per head" % cols.size, flush=True)
    out = sspmm_amd.fused_sparse_attention(None, d_off, d_cols, q, k, v_const, 0.125, V)
    assert (out.float() - const.float()).abs().max().item() <= 2e-3
    a = sspmm_amd.fused_sparse_attention(None, d_off, d_cols, q, k, v, 0.125, V)
    b = sspmm_amd.fused_sparse_attention(d_rows, d_off, d_cols, q, k, v, 0.125, V)
    c = sspmm_amd.fused_sparse_attention(None, d_off, d_shuf, q, k, v, 0.125, V)
    assert torch.equal(a, b)
    assert (a.float() - c.float()).abs().max().item() <= 2e-3
    chain = sspmm_amd.sparse_attention(None, d_off, d_cols, q, k, v, 0.125, V, fused=False)
    assert (a.float() - chain.float()).abs().max().item() <= 4e-3


@pytest.mark.parametrize("d", [40, 256])
def test_heads_of_other_widths_take_the_three_operators(built_library, d):
    """`sparse_attention` with nothing forced: heads that are not 32, 64 or 128 wide run the chain, and `fused=True` says so."""
    V, seq, batch = 8, 128, 2
    vs = _pattern(seq // V, seq, V, 0.75, seed=31)
    off, col = dev(vs.row_offsets), dev(vs.col_idx)
    g = torch.Generator("cuda").manual_seed(32)
    q, k, v = (torch.randn(batch, seq, d, device="cuda", generator=g).half() for _ in range(3))
    out = sspmm_amd.sparse_attention(None, off, col, q, k, v, d ** -0.5, V)
    want = _dense_attention(vs.row_offsets, vs.col_idx, V, *(t.cpu().numpy() for t in (q, k, v)), d ** -0.5)
    assert np.abs(out.float().cpu().numpy() - want).max() <= 1e-2
    with pytest.raises(ValueError):
        sspmm_amd.sparse_attention(None, off, col, q, k, v, d ** -0.5, V, fused=True)


@pytest.mark.parametrize("d", [32, 64, 128])
def test_one_launch_attention_of_a_single_key_returns_its_value_row(built_library, d):
    """A query that attends to one key gets that row of v back exactly (probability one, fp16 in and out)."""
    V, n_keys, m_vec = 8, 50, 5
    rng = np.random.default_rng(3 + d)
    cols = rng.integers(0, n_keys, m_vec).astype(np.int32)
    off = np.arange(m_vec + 1, dtype=np.int32)
    q, k, v = (rng.standard_normal((2, n, d)).astype(np.float16) for n in (m_vec * V, n_keys, n_keys))
    got = sspmm_amd.fused_sparse_attention(None, dev(off), dev(cols), dev(q), dev(k), dev(v), 0.125, V).cpu().numpy()
    for i in range(m_vec):
        assert np.array_equal(got[:, i * V:(i + 1) * V], np.repeat(v[:, cols[i]][:, None], V, axis=1))


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("V", [8, 16])
def test_packed_heads_give_the_bits_of_the_copied_out_heads(built_library, V, d):
    """The launch on a fused projection [seq, batch, 3 * heads * d] against the same launch on q, k and v copied out
    into [batch * heads, seq, d] as the reference's module lays them out (spattention.py:151-157, 181-184)."""
    seq, bsz, heads = 192, 3, 5
    E = heads * d
    vs = _pattern(seq // V, seq, V, 0.7, seed=21)
    off, col = dev(vs.row_offsets), dev(vs.col_idx)
    g = torch.Generator("cuda").manual_seed(22)
    qkv = torch.randn(seq, bsz, 3 * E, device="cuda", generator=g).half()
    got = sspmm_amd.sparse_attention_packed(None, off, col, qkv, heads, 0.125, V)
    torch.cuda.synchronize()
    q, k, v = (t.contiguous().view(seq, bsz * heads, d).transpose(0, 1).contiguous() for t in qkv.chunk(3, dim=-1))
    want = sspmm_amd.fused_sparse_attention(None, off, col, q, k, v, 0.125, V)
    want = want.transpose(0, 1).contiguous().view(seq, bsz, E)
    assert got.shape == (seq, bsz, E)
    assert torch.equal(got, want)
    with pytest.raises(ValueError):
        sspmm_amd.sparse_attention_packed(None, off, col, qkv, heads + 1, 0.125, V)
    from sspmm_amd.attention import packed_attention_fits
    assert packed_attention_fits(8192, 8, 3 * 512) and not packed_attention_fits(16384, 32, 3 * 1024)


def test_argument_errors(built_library):
    off = torch.zeros(3, dtype=torch.int32, device="cuda")
    col = torch.zeros(0, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        sspmm_amd.sddmm(None, off, col, torch.zeros(16, 64, device="cuda").half(), torch.zeros(8, 64, device="cuda").half(), 4)
    with pytest.raises(ValueError):
        sspmm_amd.sddmm(None, off, col, torch.zeros(16, 64, device="cuda").half(), torch.zeros(8, 32, device="cuda").half(), 8)
    with pytest.raises(TypeError):
        sspmm_amd.csr_softmax(None, off, torch.zeros(0, device="cuda"), 1.0, 8)
    with pytest.raises(ValueError):  # the one-launch block takes heads of 32, 64 or 128 features
        sspmm_amd.fused_sparse_attention(None, off, col, *(torch.zeros(1, 16, 48, device="cuda").half() for _ in range(3)), 1.0, 8)
    with pytest.raises(RuntimeError):  # scale must be positive
        sspmm_amd.fused_sparse_attention(None, off, col, *(torch.zeros(1, 16, 64, device="cuda").half() for _ in range(3)), 0.0, 8)
    with pytest.raises(RuntimeError):  # F must be a multiple of 8
        sspmm_amd.sddmm(None, off, col, torch.zeros(16, 12, device="cuda").half(), torch.zeros(8, 12, device="cuda").half(), 8)


def test_sparse_attention_encoder_matches_dense_masked_attention(built_library):
    """The end-to-end model of the reference (four blocks, each with its own static mask) against the same model
    whose attention is dense fp32 arithmetic with the mask applied as -inf (the recipe of the reference's own checks,
    verify/softmax.py:36-38, verify/spmm.py:36-41)."""
    from sspmm_amd.attention import SparseAttentionEncoder
    torch.manual_seed(3)
    seq, V = 512, 8
    model = SparseAttentionEncoder(vocab_size=257, embed_dim=128, num_heads=2, sparsity=0.9, seq_len=seq, mlp_dim=256,
                                   num_class=16, vec_length=V, layers=4, seed=11).cuda().half().eval()
    tokens = torch.randint(0, 257, (2, seq), device="cuda", generator=torch.Generator("cuda").manual_seed(4))
    masks = []
    for blk in model.blocks:
        off, col = blk.row_offsets.cpu().numpy(), blk.column_indices.cpu().numpy()
        assert off[-1] == col.size == round(0.1 * (seq // V) * seq)
        dense = np.zeros((seq, seq), bool)
        for i in range(seq // V):
            dense[i * V:(i + 1) * V, col[off[i]:off[i + 1]]] = True
        assert np.array_equal(np.sort(np.diff(off)[blk.row_indices.cpu().numpy()]), np.diff(off)[blk.row_indices.cpu().numpy()])
        masks.append(torch.from_numpy(dense).cuda())
    with torch.no_grad():
        got = model(tokens)
        want = model(tokens, dense_masks=masks)
    assert got.shape == (seq, 2, 16) and got.dtype == torch.float16
    assert torch.isfinite(got).all()
    assert max_rel_err(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 1e-2
