"""Pins the CPU oracle (oracle/) without a GPU: against the golden fixtures the reference's own
RowMerge wrote, against the Python runtime's builtin set, against brute force and closed forms."""
import glob
import os
import random

import numpy as np
import pytest

from sspmm_amd import formats, synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = sorted(os.path.basename(p)[:-5] for p in glob.glob(os.path.join(GOLDEN, "*.smtx"))
               if ".v" not in os.path.basename(p))


def test_golden_fixtures_present():
    assert len(CASES) >= 6


@pytest.mark.parametrize("order_keys", [8, 64, 512, 4096, 70000, 1 << 20])
def test_pyset_model_matches_builtin_set(oracle, order_keys):
    rng = random.Random(order_keys)
    for n in [0, 1, 2, 4, 5, 6, 18, 19, 20, 76, 77, 78, 306, 307, 308, 1228, 1229, 1230, 5000, 20000]:
        for _ in range(6):
            keys = [rng.randrange(order_keys) for _ in range(n)]
            assert oracle.pyset_order(keys).tolist() == list(set(keys))


def test_pyset_model_beyond_50000_keys(oracle):
    # growth factor drops from 4x to 2x above 50 000 keys
    rng = random.Random(7)
    keys = rng.sample(range(1 << 22), 120000)
    assert oracle.pyset_order(keys).tolist() == list(set(keys))


def test_pyset_small_keys_are_ascending(oracle):
    # every key below 8 sits in its own slot of the 8-slot table... as long as no rebuild moved it
    assert oracle.pyset_order([3, 1, 2]).tolist() == [1, 2, 3]


@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("V", [8, 16])
def test_svc_oracle_reproduces_reference_files(oracle, name, V):
    """Byte-for-byte: oracle SVC + the package's CVSE writer == the file the reference wrote."""
    M, K, nnz, row_ptr, col_ind = formats.read_smtx(os.path.join(GOLDEN, name + ".smtx"))
    vrp, vcol, _ = oracle.svc(M, K, V, row_ptr, col_ind)
    with open(os.path.join(GOLDEN, "%s.v%d.smtx" % (name, V))) as f:
        want = f.read()
    assert formats.cvse_text(len(vrp) - 1, K, nnz, vrp, vcol) == want


@pytest.mark.parametrize("name", CASES)
def test_python_rowmerge_reproduces_reference_files(oracle, name):
    M, K, nnz, row_ptr, col_ind = formats.read_smtx(os.path.join(GOLDEN, name + ".smtx"))
    ptr, flat = oracle.rowmerge_python(M, 8, oracle.csr_col_lists(M, row_ptr, col_ind))
    want = formats.read_cvse(os.path.join(GOLDEN, name + ".v8.smtx"))
    assert ptr == want.row_offsets.tolist() and flat == want.col_idx.tolist()


def _random_csr(rng, M, K, max_len, sort=True):
    rows = []
    for _ in range(M):
        r = rng.sample(range(K), rng.randrange(0, min(K, max_len) + 1))
        rows.append(sorted(r) if sort else r)
    ptr = [0]
    cols = []
    for r in rows:
        cols += r
        ptr.append(len(cols))
    return rows, np.array(ptr, dtype=np.int32), np.array(cols, dtype=np.int32)


@pytest.mark.parametrize("V", [1, 3, 8, 16])
def test_svc_oracle_vs_python_set_and_bitmap(oracle, V):
    rng = random.Random(100 + V)
    for trial in range(60):
        M = rng.randrange(1, 80)
        K = rng.choice([8, 33, 512, 5000])
        rows, ptr, cols = _random_csr(rng, M, K, 50, sort=bool(trial % 2))
        vals = (np.arange(len(cols)) % 2039 + 1).astype(np.float16)
        vrp, vcol, vval = oracle.svc(M, K, V, ptr, cols, vals)
        want_ptr, want_cols = oracle.rowmerge_python(M, V, rows)
        assert vrp.tolist() == want_ptr and vcol.tolist() == want_cols
        # closed form for the counts: distinct columns per group, from a dense occupancy bitmap
        m_vec = (M + V - 1) // V
        occ = np.zeros((m_vec * V, K), dtype=bool)
        dense = np.zeros((m_vec * V, K), dtype=np.float16)
        for r, row in enumerate(rows):
            occ[r, row] = True
            dense[r, row] = vals[ptr[r]:ptr[r + 1]]
        counts = occ.reshape(m_vec, V, K).any(axis=1).sum(axis=1)
        assert np.array_equal(np.diff(vrp), counts)
        assert m_vec * K - int(counts.sum()) == int((~occ.reshape(m_vec, V, K).any(axis=1)).sum())
        # value packing: densify(svc(A)) == A
        assert np.array_equal(oracle.densify(m_vec, V, K, vrp, vcol, vval), dense)
        # sorted mode: same sets, ascending
        srp, scol, sval = oracle.svc(M, K, V, ptr, cols, vals, order="sorted")
        assert np.array_equal(srp, vrp)
        for i in range(m_vec):
            seg = scol[srp[i]:srp[i + 1]]
            assert np.all(np.diff(seg) > 0) and set(seg.tolist()) == set(vcol[vrp[i]:vrp[i + 1]].tolist())
        assert np.array_equal(oracle.densify(m_vec, V, K, srp, scol, sval), dense)


def test_svc_of_vector_sparse_returns_same_pattern(oracle):
    vs = synth.vector_sparse(64, 512, 8, 0.9, seed=1)
    csr = synth.expand_to_csr(vs)
    vrp, vcol, vval = oracle.svc(csr.M, csr.K, 8, csr.row_ptr, csr.col_ind, csr.values, order="sorted")
    assert np.array_equal(vrp, vs.row_offsets) and np.array_equal(vcol, vs.col_idx)
    assert np.array_equal(vval, vs.values)
    # CPython order: same sets per vector-row
    vrp2, vcol2, _ = oracle.svc(csr.M, csr.K, 8, csr.row_ptr, csr.col_ind)
    assert np.array_equal(vrp2, vs.row_offsets)
    for i in range(vs.m_vec):
        assert sorted(vcol2[vrp2[i]:vrp2[i + 1]].tolist()) == vcol[vrp[i]:vrp[i + 1]].tolist()


@pytest.mark.parametrize("V", [8, 16])
def test_spmm_oracle_vs_dense_matmul(oracle, V):
    vs = synth.vector_sparse(16 * V, 96, V, 0.8, seed=3)
    B = synth.dense_rhs(96, 40, seed=4)
    C = oracle.spmm(vs.m_vec, V, 40, 96, vs.row_offsets, vs.col_idx, vs.values, B)
    A = oracle.densify(vs.m_vec, V, 96, vs.row_offsets, vs.col_idx, vs.values)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.abs(C - want).max() <= 1e-5 * np.abs(want).max()
    # fp16 output = round-to-nearest-even of the fp32 result
    C16 = oracle.spmm(vs.m_vec, V, 40, 96, vs.row_offsets, vs.col_idx, vs.values, B, out_dtype=np.float16)
    assert np.array_equal(C16.view(np.uint16), C.astype(np.float16).view(np.uint16))
    # threads > 1 changes nothing
    C4 = oracle.spmm(vs.m_vec, V, 40, 96, vs.row_offsets, vs.col_idx, vs.values, B, threads=4)
    assert np.array_equal(C4, C)


def test_spmm_oracle_special_cases(oracle):
    V, K, N = 8, 16, 24
    B = synth.dense_rhs(K, N, seed=5)
    # one vector -> outer product
    vals = np.arange(1, V + 1).astype(np.float16)
    C = oracle.spmm(1, V, N, K, [0, 1], [5], vals, B)
    assert np.array_equal(C, np.outer(vals.astype(np.float32), B[5].astype(np.float32)))
    # empty vector-rows -> zeros, written
    C = oracle.spmm(3, V, N, K, [0, 0, 0, 0], np.zeros(0, np.int32), np.zeros(0, np.float16), B)
    assert C.shape == (24, N) and not C.any()
    # "identity" pattern: vector-row i uses column i with all-ones -> every row of the slab = B[i]
    m_vec = 4
    C = oracle.spmm(m_vec, V, N, K, np.arange(m_vec + 1), np.arange(m_vec), np.ones(m_vec * V, np.float16), B)
    for i in range(m_vec):
        assert np.array_equal(C[i * V:(i + 1) * V], np.tile(B[i].astype(np.float32), (V, 1)))
    # accumulation order is j ascending in fp32: 2048 + 1 + 1 ... differs from a pairwise sum
    vals = np.zeros((3, V), np.float16)
    vals[:, 0] = [1.0, 1.0, 1.0]
    Bb = np.zeros((3, 1), np.float16)
    Bb[:, 0] = [16777216.0 if False else 2048.0, 1.0, 1.0]
    C = oracle.spmm(1, V, 1, 3, [0, 3], [0, 1, 2], vals.reshape(-1), Bb)
    assert C[0, 0] == np.float32(2050.0)


def test_half_conversions_exhaustive(oracle):
    L = oracle.lib()
    h = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    f = h.view(np.float16).astype(np.float32)
    for x in range(0, 65536, 3):
        got = L.oracle_h2f(int(x))
        assert (np.isnan(got) and np.isnan(f[x])) or got == f[x]
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 4000),
                         np.array([65504, 65519.99, 65520, 1e9, 2 ** -24, 2 ** -25, 2 ** -25 * 1.0001, 6.1e-5, 0.0, -0.0],
                                  dtype=np.float32)]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.oracle_f2h(float(v)) for v in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_sorted_row_swizzle_invariants(oracle):
    rng = np.random.default_rng(9)
    lens = rng.integers(0, 40, 300)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    perm = oracle.sorted_row_swizzle(off)
    assert sorted(perm.tolist()) == list(range(300))
    assert np.all(np.diff(lens[perm]) <= 0)
    assert np.array_equal(perm, np.argsort(-lens, kind="stable"))


@pytest.mark.parametrize("V", [8, 16])
def test_sddmm_oracle_vs_dense_matmul_sampled_at_the_pattern(oracle, V):
    """out[j*V+v] must be entry (i*V+v, col_j) of lhs @ rhs.T: a transposed operand, a wrong row or a
    wrong vector-major index all show up as O(1) errors."""
    vs = synth.vector_sparse(6 * V, 50, V, 0.7, seed=80 + V)
    rng = np.random.default_rng(81)
    F = 40
    lhs = rng.standard_normal((vs.m_vec * V, F)).astype(np.float16)
    rhs = rng.standard_normal((50, F)).astype(np.float16)
    got = oracle.sddmm(vs.m_vec, V, vs.row_offsets, vs.col_idx, lhs, rhs).astype(np.float64).reshape(-1, V)
    dense = lhs.astype(np.float64) @ rhs.astype(np.float64).T
    for i in range(vs.m_vec):
        for j in range(vs.row_offsets[i], vs.row_offsets[i + 1]):
            want = dense[i * V:(i + 1) * V, vs.col_idx[j]]
            assert np.all(np.abs(got[j] - want) <= 2e-3 * max(1.0, np.abs(want).max()) + 2e-3)
    # exact case: small integers
    lhs_i = rng.integers(-3, 4, lhs.shape).astype(np.float16)
    rhs_i = rng.integers(-3, 4, rhs.shape).astype(np.float16)
    got = oracle.sddmm(vs.m_vec, V, vs.row_offsets, vs.col_idx, lhs_i, rhs_i).astype(np.float64).reshape(-1, V)
    dense = lhs_i.astype(np.float64) @ rhs_i.astype(np.float64).T
    for i in range(vs.m_vec):
        for j in range(vs.row_offsets[i], vs.row_offsets[i + 1]):
            assert np.array_equal(got[j], dense[i * V:(i + 1) * V, vs.col_idx[j]])


@pytest.mark.parametrize("V", [8, 16])
def test_softmax_oracle_vs_dense_softmax_with_minus_inf_fill(oracle, V):
    """The reference's own check: softmax over the dense rows with -inf where nothing is stored."""
    K = 70
    vs = synth.vector_sparse(5 * V, K, V, 0.6, seed=90 + V)
    lens = np.diff(vs.row_offsets)
    rng = np.random.default_rng(91)
    vals = (rng.standard_normal(vs.col_idx.size * V) * 3).astype(np.float16)
    scaler = 0.37
    got = oracle.softmax(vs.m_vec, V, vs.row_offsets, vals, scaler).astype(np.float64).reshape(-1, V)
    dense = np.full((vs.m_vec * V, K), -np.inf)
    vv = vals.reshape(-1, V).astype(np.float64)
    for i in range(vs.m_vec):
        for j in range(vs.row_offsets[i], vs.row_offsets[i + 1]):
            dense[i * V:(i + 1) * V, vs.col_idx[j]] = vv[j]
    x = dense * scaler
    e = np.exp(x - x.max(axis=1, keepdims=True))
    ref = e / e.sum(axis=1, keepdims=True)
    for i in range(vs.m_vec):
        for j in range(vs.row_offsets[i], vs.row_offsets[i + 1]):
            want = ref[i * V:(i + 1) * V, vs.col_idx[j]]
            assert np.all(np.abs(got[j] - want) <= 1e-3 * want + 1e-6)
    assert lens.min() > 0
    # each dense row sums to one; a row with a single entry is exactly one
    sums = np.zeros(vs.m_vec * V)
    for i in range(vs.m_vec):
        sums[i * V:(i + 1) * V] = got[vs.row_offsets[i]:vs.row_offsets[i + 1]].sum(axis=0)
    assert np.all(np.abs(sums - 1) < 5e-3)
    one = oracle.softmax(1, V, np.array([0, 1], np.int32), np.arange(V).astype(np.float16), 2.0)
    assert np.array_equal(one, np.ones(V, np.float16))
    # empty vector-rows write nothing
    assert oracle.softmax(3, V, np.array([0, 0, 1, 1], np.int32), np.zeros(V, np.float16), 1.0).tolist() == [1.0] * V
