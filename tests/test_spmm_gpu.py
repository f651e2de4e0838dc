"""GPU parity of the SpMM through the C ABI (via the ctypes operator) against the CPU oracle."""
import numpy as np
import pytest
import torch

import sspmm_amd
from sspmm_amd import synth
from gpu_util import PARITY_TOL, TIGHT_F16, TIGHT_F32, dev, max_rel_err

pytestmark = pytest.mark.gpu

KERNELS = {"auto": 0, "gather": 2, "slab": 3, "staged": 6}


@pytest.fixture(params=sorted(KERNELS))
def kernel(request, built_library):
    """Runs the test once per SpMM kernel (the automatic choice, and each MFMA kernel forced)."""
    from sspmm_amd import _lib
    _lib.lib().sspmm_select_kernel(KERNELS[request.param])
    yield request.param
    _lib.lib().sspmm_select_kernel(0)


def run(vs, B, out_dtype, row_indices=None):
    out = sspmm_amd.spmm(row_indices, dev(vs.row_offsets), dev(vs.col_idx), dev(vs.values), dev(B), vs.V,
                         out_dtype=out_dtype)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def check(oracle, vs, B, out_dtype=torch.float32, row_indices=None):
    K, N = B.shape
    print("case M=%d K=%d N=%d V=%d nvec=%d out=%s" % (vs.M, K, N, vs.V, vs.col_idx.size, out_dtype), flush=True)
    got = run(vs, B, out_dtype, row_indices)
    want = oracle.spmm(vs.m_vec, vs.V, N, K, vs.row_offsets, vs.col_idx, vs.values, B, threads=8)
    assert got.shape == (vs.m_vec * vs.V, N)
    err = max_rel_err(got, want)
    assert err <= PARITY_TOL, err
    assert err <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16), err
    return got, want


# the benchmark configurations at their real shapes (the oracle runs each in well under a second with 8 threads)
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_cfg1_512x512_v8(oracle, kernel, out_dtype):
    vs = synth.vector_sparse(512, 512, 8, 0.9, seed=1)
    check(oracle, vs, synth.dense_rhs(512, 256, seed=11), out_dtype)


@pytest.mark.parametrize("shape", [(2048, 512), (512, 2048)])
@pytest.mark.parametrize("sparsity", [0.7, 0.9, 0.98])
def test_cfg2_ffn_v8(oracle, kernel, shape, sparsity):
    vs = synth.vector_sparse(shape[0], shape[1], 8, sparsity, seed=2, std=0.02)
    check(oracle, vs, synth.dense_rhs(shape[1], 256, seed=12))
    from sspmm_amd import _lib
    if kernel != "auto":  # the forced kernel is the one that ran (K = 2048 takes the 32-column slab)
        assert _lib.lib().sspmm_last_kernel() == (5 if kernel == "slab" and shape[1] == 2048 else KERNELS[kernel])


@pytest.mark.parametrize("shape", [(1024, 2304), (2048, 1024)])
@pytest.mark.parametrize("sparsity", [0.8, 0.95])
@pytest.mark.parametrize("N", [256, 3136])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_cfg3_conv_v16(oracle, built_library, shape, sparsity, N, out_dtype):
    """All eight (shape, sparsity, N) points of the im2col configuration."""
    vs = synth.vector_sparse(shape[0], shape[1], 16, sparsity, seed=3, std=0.05)
    check(oracle, vs, synth.dense_rhs(shape[1], N, seed=13), out_dtype)


@pytest.mark.parametrize("shape", [(2048, 512), (512, 2048)])
@pytest.mark.parametrize("sparsity", [0.7, 0.9, 0.98])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_cfg2_shapes_v16(oracle, built_library, shape, sparsity, out_dtype):
    vs = synth.vector_sparse(shape[0], shape[1], 16, sparsity, seed=2, std=0.02)
    check(oracle, vs, synth.dense_rhs(shape[1], 256, seed=12), out_dtype)


# the six weights of the BERT-base shaped encoder layer: hidden 768, FFN 3072, 8 x 512 tokens
CFG5_WEIGHTS = {"q": (768, 768, 51), "k": (768, 768, 52), "v": (768, 768, 53), "o": (768, 768, 54),
                "ffn1": (3072, 768, 55), "ffn2": (768, 3072, 56)}


@pytest.mark.parametrize("name", sorted(CFG5_WEIGHTS))
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_cfg5_encoder_weights_v16_n4096(oracle, built_library, name, out_dtype):
    """Every weight of the encoder-layer configuration at its real shape: V = 16, 90 %, N = 8 x 512 tokens."""
    out_f, in_f, seed = CFG5_WEIGHTS[name]
    vs = synth.vector_sparse(out_f, in_f, 16, 0.9, seed=seed, std=0.02)
    check(oracle, vs, synth.dense_rhs(in_f, 4096, seed=seed + 100), out_dtype)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_headline_batch_128_every_element(oracle, built_library, out_dtype):
    """The launch the benchmark times (A 2048x512, V = 8, 90 %, B 512x256, 128 batch elements that share the
    pattern, dealt to the XCDs by batch element): every element against the oracle."""
    from sspmm_amd import _lib
    V, K, N, batch = 8, 512, 256, 128
    vs = synth.vector_sparse(2048, K, V, 0.9, seed=2, std=0.02)
    g = torch.Generator(device="cuda").manual_seed(2)
    vals = (torch.randn(batch, vs.col_idx.size * V, generator=g, device="cuda") * 0.02).half()
    B = torch.randn(batch, K, N, generator=g, device="cuda").half()
    print("headline batch %d out=%s" % (batch, out_dtype), flush=True)
    out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), vals, B, V, out_dtype=out_dtype)
    torch.cuda.synchronize()
    assert _lib.lib().sspmm_last_kernel() == (3 if out_dtype == torch.float32 else 9)  # (fp16 C: 128-column slabs)
    out, vals_h, B_h = out.cpu().numpy(), vals.cpu().numpy(), B.cpu().numpy()
    tol = TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16
    for b in range(batch):
        want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals_h[b], B_h[b], threads=8)
        assert max_rel_err(out[b], want) <= tol, b


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("N", [8, 24, 64, 120, 128, 136, 200, 264])
def test_column_tails(oracle, kernel, V, N):
    """N that is not a multiple of the 128-column tile (the reference needs N % 64 == 0)."""
    vs = synth.vector_sparse(6 * V, 80, V, 0.6, seed=20 + N)
    check(oracle, vs, synth.dense_rhs(80, N, seed=N))


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("N", [8, 40, 56, 64])
def test_narrow_right_hand_sides(oracle, built_library, V, out_dtype, N):
    """N <= 64 (an attention head's features) runs the staged gather kernel: ragged rows with partial last chunks,
    rows of several chunks, empty rows, a batch."""
    from sspmm_amd import _lib
    rng = np.random.default_rng(700 + V + N)
    K, m_vec = 900, 37
    lens = rng.integers(0, 70, m_vec)
    lens[[0, 4, 20]] = [0, 333, 32]
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols,
                            (rng.standard_normal(cols.size * V) * 0.1).astype(np.float16), cols.size * V)
    B = synth.dense_rhs(K, N, seed=N)
    got, _ = check(oracle, vs, B, out_dtype)
    assert _lib.lib().sspmm_last_kernel() == 6
    assert not got[:V].any()
    vals3 = (rng.standard_normal((3, cols.size * V)) * 0.1).astype(np.float16)
    B3 = np.stack([synth.dense_rhs(K, N, seed=60 + b) for b in range(3)])
    out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals3), dev(B3), V, out_dtype=out_dtype)
    torch.cuda.synchronize()
    for b in range(3):
        want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals3[b], B3[b], threads=8)
        assert max_rel_err(out[b].cpu().numpy(), want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16)


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_narrow_right_hand_side_on_a_wide_matrix(oracle, built_library, V, out_dtype):
    """N <= 64 keeps the staged gather kernel above K = 4096 too (an attention mask over a long sequence), long and
    empty vector-rows included."""
    from sspmm_amd import _lib
    rng = np.random.default_rng(750 + V)
    K, N, m_vec = 6000, 64, 19
    lens = rng.integers(0, 90, m_vec)
    lens[[0, 3, 11]] = [4100, 0, 513]
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols,
                            (rng.standard_normal(cols.size * V) * 0.05).astype(np.float16), cols.size * V)
    got, _ = check(oracle, vs, synth.dense_rhs(K, N, seed=17), out_dtype)
    assert _lib.lib().sspmm_last_kernel() == 6
    assert not got[3 * V:4 * V].any()


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("N", [1, 3, 17, 66, 130])
def test_odd_widths_take_the_generic_kernel_and_match_the_oracle_bit_for_bit(oracle, built_library, V, N):
    """N % 8 != 0 runs the scalar kernel, which adds in the oracle's order: fp32 results are identical."""
    vs = synth.vector_sparse(5 * V, 70, V, 0.5, seed=40 + N)
    got, want = check(oracle, vs, synth.dense_rhs(70, N, seed=N))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("per_row", [0, 1, 7, 31, 32, 33, 63, 64, 65, 97])
def test_row_length_tails(oracle, kernel, V, per_row):
    """Vector-row lengths around the 32-vector step of the kernel."""
    K = 128
    rng = np.random.default_rng(per_row)
    m_vec = 5
    cols = np.concatenate([np.sort(rng.choice(K, per_row, replace=False)) for _ in range(m_vec)] or [[]]).astype(np.int32)
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, (np.arange(m_vec + 1) * per_row).astype(np.int32), cols,
                            rng.standard_normal(m_vec * per_row * V).astype(np.float16), m_vec * per_row * V)
    check(oracle, vs, synth.dense_rhs(K, 128, seed=3))


def test_ragged_rows_empty_rows_and_unsorted_columns(oracle, kernel):
    rng = np.random.default_rng(77)
    K, V, N = 300, 8, 256
    lens = np.array([0, 5, 0, 0, 200, 33, 1, 0, 64, 0])
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)  # not sorted
    vs = synth.VectorSparse(len(lens) * V, K, V, len(lens), off, cols,
                            rng.standard_normal(cols.size * V).astype(np.float16), cols.size * V)
    B = synth.dense_rhs(K, N, seed=5)
    got, want = check(oracle, vs, B)
    for i in np.flatnonzero(lens == 0):
        assert not got[i * V:(i + 1) * V].any()


def test_inf_in_unreferenced_row_of_B_does_not_leak(oracle, kernel):
    """Padding slots of a partial step must not multiply a real row of B."""
    V, K, N = 8, 64, 128
    vs = synth.vector_sparse(4 * V, K, V, 0.9, seed=9)  # 6 vectors per row, none is a full step
    B = synth.dense_rhs(K, N, seed=9)
    unused = sorted(set(range(K)) - set(vs.col_idx.tolist()))
    B[unused] = np.inf
    got = run(vs, B, torch.float32)
    assert np.isfinite(got).all()


def test_result_does_not_depend_on_row_indices(oracle, kernel):
    vs = synth.vector_sparse(40 * 8, 256, 8, 0.85, seed=31)
    B = synth.dense_rhs(256, 256, seed=32)
    base = run(vs, B, torch.float32)
    perm = np.random.default_rng(1).permutation(vs.m_vec).astype(np.int32)
    assert np.array_equal(run(vs, B, torch.float32, dev(perm)), base)
    swz = sspmm_amd.sorted_row_swizzle(dev(vs.row_offsets))
    assert np.array_equal(run(vs, B, torch.float32, swz), base)


def test_special_patterns(oracle, kernel):
    V, K, N = 16, 32, 128
    B = synth.dense_rhs(K, N, seed=6)
    # one vector: outer product, exact
    vals = np.arange(1, V + 1).astype(np.float16)
    vs = synth.VectorSparse(V, K, V, 1, np.array([0, 1], np.int32), np.array([7], np.int32), vals, V)
    got = run(vs, B, torch.float32)
    assert np.array_equal(got, np.outer(vals.astype(np.float32), B[7].astype(np.float32)))
    # identity-like pattern with ones: every row of slab i equals B[i]
    m_vec = 8
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, np.arange(m_vec + 1, dtype=np.int32),
                            np.arange(m_vec, dtype=np.int32), np.ones(m_vec * V, np.float16), m_vec * V)
    got = run(vs, B, torch.float16)
    for i in range(m_vec):
        assert np.array_equal(got[i * V:(i + 1) * V], np.tile(B[i], (V, 1)))


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_slab_kernel_at_k1024_v16(oracle, kernel, out_dtype):
    vs = synth.vector_sparse(2048, 1024, 16, 0.95, seed=3, std=0.05)
    check(oracle, vs, synth.dense_rhs(1024, 448, seed=14), out_dtype)


def test_skewed_row_lengths(oracle, kernel):
    """A few very long vector-rows among short ones (what the row counter in the slab kernel balances)."""
    rng = np.random.default_rng(123)
    K, V, N, m_vec = 1000, 8, 192, 96
    lens = rng.integers(0, 20, m_vec)
    lens[[3, 40, 95]] = [1000, 700, 333]
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols,
                            rng.standard_normal(cols.size * V).astype(np.float16), cols.size * V)
    check(oracle, vs, synth.dense_rhs(K, N, seed=15))


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_wide_matrix_with_long_vector_rows(oracle, built_library, V, out_dtype):
    """K above 4096 runs the gather kernel's variant that splits long vector-rows over the four waves of a
    workgroup: rows just below and above the 512-vector limit, thousands of vectors, empty rows, a row count
    that is no multiple of four, a partial last column tile, row_indices, and a batch."""
    from sspmm_amd import _lib
    rng = np.random.default_rng(500 + V)
    K, N, m_vec = 6000, 200, 23
    lens = rng.integers(0, 40, m_vec)
    lens[[0, 5, 6, 7, 13, 22]] = [512, 513, 4100, 0, 1999, 545]
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols,
                            (rng.standard_normal(cols.size * V) * 0.05).astype(np.float16), cols.size * V)
    B = synth.dense_rhs(K, N, seed=16)
    got, _ = check(oracle, vs, B, out_dtype)
    assert _lib.lib().sspmm_last_kernel() == 4
    assert not got[7 * V:8 * V].any()
    perm = rng.permutation(m_vec).astype(np.int32)
    assert np.array_equal(run(vs, B, out_dtype, dev(perm)), got)
    # a batch of three shares the pattern
    vals3 = (rng.standard_normal((3, cols.size * V)) * 0.05).astype(np.float16)
    B3 = np.stack([synth.dense_rhs(K, N, seed=20 + b) for b in range(3)])
    out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals3), dev(B3), V, out_dtype=out_dtype)
    torch.cuda.synchronize()
    for b in range(3):
        one = sspmm_amd.spmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals3[b]), dev(B3[b]), V,
                             out_dtype=out_dtype)
        assert torch.equal(out[b], one)


def test_linearity_at_full_size(built_library):
    """cfg3 at N = 3136 without the oracle: spmm(A, B1 + B2) == spmm(A, B1) + spmm(A, B2) when the
    sums are exact (small integers), and scaling the values by 2 doubles the result exactly."""
    V = 16
    vs = synth.vector_sparse(1024, 2304, V, 0.8, seed=3)
    rng = np.random.default_rng(0)
    vals = rng.integers(-2, 3, vs.values.size).astype(np.float16)
    vs = vs._replace(values=vals)
    B1 = rng.integers(-3, 4, (2304, 3136)).astype(np.float16)
    B2 = rng.integers(-3, 4, (2304, 3136)).astype(np.float16)
    c1, c2, c12 = run(vs, B1, torch.float32), run(vs, B2, torch.float32), run(vs, B1 + B2, torch.float32)
    assert np.array_equal(c12, c1 + c2)
    c1d = run(vs._replace(values=vals * np.float16(2)), B1, torch.float32)
    assert np.array_equal(c1d, 2 * c1)
    # and against an exact dense integer matmul on a slab of rows
    A = np.zeros((vs.m_vec * V, 2304), np.float32)
    vv = vals.reshape(-1, V).astype(np.float32)
    for i in range(4):
        for j in range(vs.row_offsets[i], vs.row_offsets[i + 1]):
            A[i * V:(i + 1) * V, vs.col_idx[j]] = vv[j]
    assert np.array_equal(c1[:4 * V], A[:4 * V] @ B1.astype(np.float32))


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_bspmm_matches_looped_spmm(oracle, kernel, V, out_dtype):
    """Pattern shared by the batch, per-batch values / B / C (reference spmm_kernel.cu:532-534)."""
    batch, K, N = 3, 96, 192
    vs = synth.vector_sparse(12 * V, K, V, 0.75, seed=50)
    rng = np.random.default_rng(51)
    vals = rng.standard_normal((batch, vs.values.size)).astype(np.float16)
    B = rng.standard_normal((batch, K, N)).astype(np.float16)
    out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals), dev(B), V, out_dtype=out_dtype)
    torch.cuda.synchronize()
    out = out.cpu().numpy()
    assert out.shape == (batch, vs.m_vec * V, N)
    for b in range(batch):
        single = run(vs._replace(values=vals[b]), B[b], out_dtype)
        assert np.array_equal(out[b], single)
        want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[b], B[b])
        assert max_rel_err(out[b], want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16)


@pytest.mark.parametrize("V,batch,m_rows,K,N,sparsity", [
    (8, 1, 3000, 96, 64, 0.7),      # one slab, many row blocks: work items that follow each other on the same slab
    (8, 20, 400, 200, 192, 0.8),    # uneven batch elements per XCD, item lists that cross slabs (two slabs in LDS)
    (16, 11, 150, 160, 136, 0.8),   # V = 16, a partial last column tile, batch not a multiple of 8
    (8, 40, 128, 700, 128, 0.9),    # K too tall for two slabs: the single-buffer path with several items per workgroup
    (16, 5, 70, 1000, 64, 0.9),     # fewer than 8 batch elements: slabs dealt round-robin to the XCDs
])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_slab_kernel_work_item_lists(oracle, built_library, V, batch, m_rows, K, N, sparsity, out_dtype):
    """Shapes chosen to walk the persistent slab kernel through every kind of item transition."""
    from sspmm_amd import _lib
    vs = synth.vector_sparse(m_rows * V, K, V, sparsity, seed=60 + batch)
    rng = np.random.default_rng(61)
    vals = rng.standard_normal((batch, vs.values.size)).astype(np.float16)
    B = rng.standard_normal((batch, K, N)).astype(np.float16)
    print("slab items V=%d batch=%d m_vec=%d K=%d N=%d %s" % (V, batch, vs.m_vec, K, N, out_dtype), flush=True)
    _lib.lib().sspmm_select_kernel(3)
    try:
        out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals), dev(B), V, out_dtype=out_dtype)
        torch.cuda.synchronize()
        assert _lib.lib().sspmm_last_kernel() == 3
    finally:
        _lib.lib().sspmm_select_kernel(0)
    out = out.cpu().numpy()
    tol = TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16
    for b in range(batch):
        want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[b], B[b], threads=8)
        assert max_rel_err(out[b], want) <= tol, b


@pytest.mark.parametrize("V,K,expect", [(8, 574, 3), (8, 575, 3), (16, 512, 3), (16, 543, 3), (16, 544, 3), (8, 1150, 3),
                                        (16, 1100, 3), (8, 1300, 5), (16, 1024, 3), (8, 1025, 3), (16, 2286, 5),
                                        (16, 2287, 2), (8, 2410, 5), (8, 2411, 2),
                                        # padded rows: both slabs (K <= 512, and <= 506 for V = 16), one slab (to about 950 / 900)
                                        (8, 512, 3), (8, 513, 3), (16, 506, 3), (16, 507, 3), (8, 950, 3), (8, 960, 3),
                                        (16, 900, 3), (16, 910, 3)])
def test_slab_kernel_around_its_lds_limits(oracle, built_library, V, K, expect):
    """K just below and above what two slabs (then one slab) leave room for in LDS, with padded and with swizzled
    rows, for the 64-column slab and, above its limit, for the 32-column one; beyond that the forced choice falls
    back to the gather kernel."""
    from sspmm_amd import _lib
    vs = synth.vector_sparse(80 * V, K, V, 0.95, seed=K)
    B = synth.dense_rhs(K, 192, seed=K + 1)
    _lib.lib().sspmm_select_kernel(3)
    try:
        check(oracle, vs, B, torch.float32)
        ran = _lib.lib().sspmm_last_kernel()
    finally:
        _lib.lib().sspmm_select_kernel(0)
    assert ran == expect


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("m_vec,N", [(1, 72), (5, 8), (16, 200), (17, 264), (33, 136), (70, 72)])
def test_slab_kernel_writes_nothing_outside_its_columns(oracle, built_library, V, out_dtype, m_vec, N):
    """Column tails of the slab kernel: lanes beyond N must not store.  C lies between two guard areas, a second
    batch element follows it at a stride that leaves a gap, and the vector-rows are processed last to first, so a
    store that strayed into the following row would survive there.  Fewer vector-rows than the workgroup has waves,
    one more than it has, several row blocks."""
    from sspmm_amd import _lib
    L = _lib.lib()
    batch, K, guard = 2, 96, 4096
    vs = synth.vector_sparse(m_vec * V, K, V, 0.7, seed=900 + m_vec)
    rng = np.random.default_rng(901 + N)
    vals = rng.standard_normal((batch, vs.values.size)).astype(np.float16)
    B = rng.standard_normal((batch, K, N)).astype(np.float16)
    M = m_vec * V
    stride_c = M * N + 64  # elements: a gap of 64 behind every batch element
    np_dtype = np.float32 if out_dtype == torch.float32 else np.float16
    sentinel = 12345.0
    buf = torch.full((guard + batch * stride_c + guard,), sentinel, dtype=out_dtype, device="cuda")
    ro, ci, dv, dB = dev(vs.row_offsets), dev(vs.col_idx), dev(vals), dev(B)
    order = dev(np.arange(m_vec - 1, -1, -1, dtype=np.int32))
    fn = L.sspmm_batched_f16_f32 if out_dtype == torch.float32 else L.sspmm_batched_f16_f16
    L.sspmm_select_kernel(3)
    try:
        rc = fn(batch, m_vec, V, N, K, order.data_ptr(), ro.data_ptr(), ci.data_ptr(), dv.data_ptr(), vs.values.size,
                dB.data_ptr(), K * N, buf.data_ptr() + guard * buf.element_size(), stride_c,
                torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        ran = L.sspmm_last_kernel()
    finally:
        L.sspmm_select_kernel(0)
    assert rc == 0 and ran == 3
    got = buf.cpu().numpy().astype(np_dtype)
    assert np.all(got[:guard] == sentinel) and np.all(got[guard + batch * stride_c:] == sentinel)
    for b in range(batch):
        lo = guard + b * stride_c
        assert np.all(got[lo + M * N:lo + stride_c] == sentinel), b
        want = oracle.spmm(m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[b], B[b])
        assert max_rel_err(got[lo:lo + M * N].reshape(M, N), want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16)


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("N", [32, 72, 200, 256])
def test_narrow_slab_kernel(oracle, built_library, V, out_dtype, N):
    """The 32-column slab (K between the 64-column slab's limit and twice that): column tails, ragged and empty
    rows, unsorted columns, row_indices, a batch that shares slabs between row blocks."""
    from sspmm_amd import _lib
    rng = np.random.default_rng(900 + V + N)
    K, m_vec = 2048, 70
    lens = rng.integers(0, 90, m_vec)
    lens[[0, 9, 33]] = [0, 700, 31]
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols,
                            (rng.standard_normal(cols.size * V) * 0.1).astype(np.float16), cols.size * V)
    B = synth.dense_rhs(K, N, seed=N)
    _lib.lib().sspmm_select_kernel(3)
    try:
        got, _ = check(oracle, vs, B, out_dtype)
        assert _lib.lib().sspmm_last_kernel() == 5
        assert not got[:V].any()
        perm = rng.permutation(m_vec).astype(np.int32)
        assert np.array_equal(run(vs, B, out_dtype, dev(perm)), got)
        vals5 = (rng.standard_normal((5, cols.size * V)) * 0.1).astype(np.float16)
        B5 = np.stack([synth.dense_rhs(K, N, seed=40 + b) for b in range(5)])
        out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals5), dev(B5), V, out_dtype=out_dtype)
        torch.cuda.synchronize()
        assert _lib.lib().sspmm_last_kernel() == 5
        for b in range(5):
            want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals5[b], B5[b], threads=8)
            assert max_rel_err(out[b].cpu().numpy(), want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16)
    finally:
        _lib.lib().sspmm_select_kernel(0)


def test_row_swizzle_matches_oracle(oracle, built_library):
    rng = np.random.default_rng(3)
    for m_vec in [1, 5, 255, 256, 257, 3000]:
        lens = rng.integers(0, 50, m_vec)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        got = sspmm_amd.sorted_row_swizzle(dev(off)).cpu().numpy()
        assert np.array_equal(got, oracle.sorted_row_swizzle(off))
    # the radix-sort entry gives the same order, ties included; the wrapper takes it for many rows
    from sspmm_amd import _lib
    from sspmm_amd.spmm import SWIZZLE_SORT_FROM
    L = _lib.lib()
    for m_vec in [1, 300, 70000]:
        lens = rng.integers(0, 40 if m_vec < 1000 else 20000, m_vec)
        lens[::7] = 13  # plenty of ties
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        d_off = dev(off)
        out = torch.empty(m_vec, dtype=torch.int32, device="cuda")
        ws = torch.empty(L.sspmm_sorted_row_swizzle_workspace_bytes(m_vec), dtype=torch.uint8, device="cuda")
        assert L.sspmm_sorted_row_swizzle_ws(m_vec, d_off.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel() - 1, None) != 0
        assert L.sspmm_sorted_row_swizzle_ws(m_vec, d_off.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), None) == 0
        torch.cuda.synchronize()
        want = oracle.sorted_row_swizzle(off)
        assert np.array_equal(out.cpu().numpy(), want)
        if m_vec > SWIZZLE_SORT_FROM:
            assert np.array_equal(sspmm_amd.sorted_row_swizzle(d_off).cpu().numpy(), want)


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("N", [128, 136, 200, 256, 520])
def test_wide_slab_kernel(oracle, built_library, V, out_dtype, N):
    """The 128-column slab: column tails inside the first and the second half of a slab, ragged and empty rows,
    unsorted columns, row_indices, a batch whose row blocks share slabs, and the automatic choice for fp16 outputs."""
    from sspmm_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(700 + V + N)
    K, m_vec = 512, 150
    lens = rng.integers(0, 90, m_vec)
    lens[[0, 9, 33, 149]] = [0, 512, 31, 33]
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)
    vs = synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols,
                            (rng.standard_normal(cols.size * V) * 0.1).astype(np.float16), cols.size * V)
    B = synth.dense_rhs(K, N, seed=N)
    L.sspmm_select_kernel(9)
    try:
        got, _ = check(oracle, vs, B, out_dtype)
        assert L.sspmm_last_kernel() == 9
        assert not got[:V].any()
        perm = rng.permutation(m_vec).astype(np.int32)
        assert np.array_equal(run(vs, B, out_dtype, dev(perm)), got)
        vals9 = (rng.standard_normal((9, cols.size * V)) * 0.1).astype(np.float16)
        B9 = np.stack([synth.dense_rhs(K, N, seed=40 + b) for b in range(9)])
        out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals9), dev(B9), V, out_dtype=out_dtype)
        torch.cuda.synchronize()
        assert L.sspmm_last_kernel() == 9
        for b in range(9):
            want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals9[b], B9[b], threads=8)
            assert max_rel_err(out[b].cpu().numpy(), want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16)
    finally:
        L.sspmm_select_kernel(0)
    # K beyond what a 128-column slab leaves room for: the forced choice is ignored
    tall = synth.vector_sparse(80 * V, 700, V, 0.9, seed=5)
    L.sspmm_select_kernel(9)
    try:
        check(oracle, tall, synth.dense_rhs(700, 256, seed=6), out_dtype)
        assert L.sspmm_last_kernel() != 9
    finally:
        L.sspmm_select_kernel(0)


def test_wide_slab_is_the_choice_for_fp16_outputs_of_large_batches(oracle, built_library):
    from sspmm_amd import _lib
    L = _lib.lib()
    V, K, N, batch = 8, 512, 256, 64
    vs = synth.vector_sparse(2048, K, V, 0.9, seed=2, std=0.02)
    g = torch.Generator("cuda").manual_seed(1)
    vals = (torch.randn(batch, vs.col_idx.size * V, device="cuda", generator=g) * 0.02).half()
    B = torch.randn(batch, K, N, device="cuda", generator=g).half()
    ro, ci = dev(vs.row_offsets), dev(vs.col_idx)
    out16 = sspmm_amd.bspmm(None, ro, ci, vals, B, V, out_dtype=torch.float16)
    assert L.sspmm_last_kernel() == 9
    out32 = sspmm_amd.bspmm(None, ro, ci, vals, B, V, out_dtype=torch.float32)
    assert L.sspmm_last_kernel() == 3
    torch.cuda.synchronize()
    for b in (0, 7, 8, 63):
        want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[b].cpu().numpy(), B[b].cpu().numpy(), threads=8)
        assert max_rel_err(out16[b].cpu().numpy(), want) <= TIGHT_F16
        assert max_rel_err(out32[b].cpu().numpy(), want) <= TIGHT_F32
