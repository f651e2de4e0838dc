"""Seeded synthetic inputs for the benchmark configurations (numpy only, deterministic).

vector_sparse():  a matrix that is already vector-sparse: every group of V rows shares its
                  column set (round((1 - sparsity) * K) distinct columns per vector-row, uniform
                  without replacement, stored ascending), values N(0, std).
zipf_csr():       an unstructured CSR matrix with power-law row lengths, the input of the SVC.
clustered_csr():  rows that are noisy copies of a few prototype rows, in shuffled order: the case
                  a row reordering ahead of the SVC is for.
"""
import collections

import numpy as np

VectorSparse = collections.namedtuple(
    "VectorSparse", ["M", "K", "V", "m_vec", "row_offsets", "col_idx", "values", "nnz"])
Csr = collections.namedtuple("Csr", ["M", "K", "row_ptr", "col_ind", "values"])


def vector_sparse(M, K, V, sparsity, seed, std=1.0):
    rng = np.random.default_rng(seed)
    m_vec = (M + V - 1) // V
    per_row = int(round((1.0 - sparsity) * K))
    per_row = max(0, min(K, per_row))
    col_idx = np.empty(m_vec * per_row, dtype=np.int32)
    for i in range(m_vec):
        col_idx[i * per_row:(i + 1) * per_row] = np.sort(rng.choice(K, size=per_row, replace=False))
    row_offsets = (np.arange(m_vec + 1, dtype=np.int64) * per_row).astype(np.int32)
    values = (rng.standard_normal(m_vec * per_row * V) * std).astype(np.float16)
    return VectorSparse(m_vec * V, K, V, m_vec, row_offsets, col_idx, values, m_vec * per_row * V)


def expand_to_csr(vs):
    """Scalar CSR of a vector-sparse matrix: row i*V+v holds the columns of vector-row i (entries
    whose fp16 value is zero are kept, so RowMerge of the result returns the same pattern)."""
    V = vs.V
    lens = np.repeat(np.diff(vs.row_offsets), V)
    row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col_ind = np.empty(int(row_ptr[-1]), dtype=np.int32)
    values = np.empty(int(row_ptr[-1]), dtype=np.float16)
    vals = vs.values.reshape(-1, V)
    for i in range(vs.m_vec):
        b, e = int(vs.row_offsets[i]), int(vs.row_offsets[i + 1])
        for v in range(V):
            r = i * V + v
            col_ind[row_ptr[r]:row_ptr[r + 1]] = vs.col_idx[b:e]
            values[row_ptr[r]:row_ptr[r + 1]] = vals[b:e, v]
    return Csr(vs.m_vec * V, vs.K, row_ptr, col_ind, values)


def zipf_row_lengths(M, mean, max_len, s, rng):
    raw = rng.zipf(s, size=M).astype(np.float64)
    lo, hi = 0.0, float(max_len)
    for _ in range(60):  # bisection on the scale so that the clipped lengths average `mean`
        f = 0.5 * (lo + hi)
        m = np.minimum(max_len, np.rint(f * raw)).mean()
        if m < mean:
            lo = f
        else:
            hi = f
    return np.minimum(max_len, np.rint(hi * raw)).astype(np.int64)


def zipf_csr(M, K, seed, mean=16, max_len=2048, s=1.5, std=1.0):
    rng = np.random.default_rng(seed)
    lens = np.minimum(zipf_row_lengths(M, mean, max_len, s, rng), K)
    row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col_ind = np.empty(int(row_ptr[-1]), dtype=np.int32)
    for r in range(M):
        n = int(lens[r])
        if n:
            col_ind[row_ptr[r]:row_ptr[r + 1]] = np.sort(rng.choice(K, size=n, replace=False))
    values = (rng.standard_normal(col_ind.size) * std).astype(np.float16)
    # fp16 rounding may produce exact zeros; keep the pattern meaningful for the densify round trip
    values[values == 0] = np.float16(std)
    return Csr(M, K, row_ptr, col_ind, values)


def clustered_csr(M, K, prototypes, cols_per_prototype, seed, keep=0.9, extras=1, std=1.0):
    """Row r copies prototype (r mod prototypes) before the shuffle: each of the prototype's columns
    with probability `keep`, plus `extras` columns drawn from all K."""
    rng = np.random.default_rng(seed)
    protos = [np.sort(rng.choice(K, size=cols_per_prototype, replace=False)) for _ in range(prototypes)]
    rows = []
    for r in range(M):
        p = protos[r % prototypes]
        cols = p[rng.random(p.size) < keep]
        if extras:
            cols = np.union1d(cols, rng.choice(K, size=extras, replace=False))
        rows.append(np.sort(cols))
    rows = [rows[i] for i in rng.permutation(M)]
    lens = np.array([r.size for r in rows], dtype=np.int64)
    row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col_ind = np.concatenate(rows + [np.zeros(0, np.int64)]).astype(np.int32)
    values = (rng.standard_normal(col_ind.size) * std).astype(np.float16)
    values[values == 0] = np.float16(std)
    return Csr(M, K, row_ptr, col_ind, values)


def dense_rhs(K, N, seed, std=1.0):
    return (np.random.default_rng(seed).standard_normal((K, N)) * std).astype(np.float16)


def spmm_algorithmic_bytes(m_vec, V, nvec, K, N, out_bytes, k_touched=None):
    """HBM bytes one SpMM call has to move when every operand is read and written once:
    value vectors, column indices, row offsets, each referenced row of B once, C once."""
    kt = K if k_touched is None else k_touched
    return 2 * V * nvec + 4 * nvec + 4 * (m_vec + 1) + 2 * kt * N + out_bytes * m_vec * V * N


def svc_algorithmic_bytes(M, nnz, m_vec, nvec, V):
    """HBM bytes of one SVC: read the CSR (pointers, columns, fp16 values), write the CVSE."""
    return 4 * (M + 1) + (4 + 2) * nnz + 4 * (m_vec + 1) + (4 + 2 * V) * nvec
