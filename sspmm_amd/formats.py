"""Text formats of the path: the DLMC `.smtx` CSR pattern file the reference's RowMerge reads
(reference RowMerge/sparse_matrix_format.py:8-39) and the CVSE pattern file it writes
(:152-175) and the C++ harness reads back (reference SSpMM/sspmm_test.cpp:28-64).
"""
import collections

import numpy as np

Cvse = collections.namedtuple("Cvse", ["m_vec", "K", "nnz", "row_offsets", "col_idx"])


def read_smtx(path):
    """-> (M, K, nnz, row_ptr[int32 M+1], col_ind[int32 nnz]).  Line 1 "M, K, nnz", line 2 the
    row pointer, line 3 the column indices, both space separated."""
    with open(path) as f:
        head = f.readline()
        ptr_s = f.readline()
        col_s = f.readline()
    M, K, nnz = (int(x) for x in head.split(", "))
    row_ptr = np.array(ptr_s.split(), dtype=np.int64).astype(np.int32)
    col_ind = np.array(col_s.split(), dtype=np.int64).astype(np.int32)
    if row_ptr.size != M + 1:
        raise ValueError("%s: row pointer has %d entries, expected %d" % (path, row_ptr.size, M + 1))
    return M, K, nnz, row_ptr, col_ind


def read_smtx_header(path):
    """-> (M, K, nnz) of a `.smtx` file: its first line alone."""
    with open(path) as f:
        M, K, nnz = (int(x) for x in f.readline().split(", "))
    return M, K, nnz


def write_smtx(path, M, K, row_ptr, col_ind):
    with open(path, "w") as f:
        f.write("%d, %d, %d\n" % (M, K, len(col_ind)))
        f.write(" ".join(str(int(x)) for x in row_ptr) + "\n")
        f.write(" ".join(str(int(x)) for x in col_ind) + "\n")


def cvse_text(m_vec, K, nnz, row_offsets, col_idx):
    """The exact text CVSE_out writes: "<m_vec>, <K>, <nnz>\\n", the row offsets joined by single
    spaces + "\\n", the column indices joined by single spaces and NO trailing newline (an empty
    third line when there is no vector).  nnz is the scalar non-zero count of the original matrix."""
    return "%d, %d, %d\n%s\n%s" % (m_vec, K, nnz, " ".join(str(int(x)) for x in row_offsets),
                                  " ".join(str(int(x)) for x in col_idx))


def write_cvse(path, m_vec, K, nnz, row_offsets, col_idx):
    with open(path, "w") as f:
        f.write(cvse_text(m_vec, K, nnz, row_offsets, col_idx))


def read_cvse(path):
    """Reads a CVSE pattern file the way the reference harness does (sspmm_test.cpp:28-64):
    header "m_vec, K, nnz", m_vec+1 offsets, then row_offsets[m_vec] column indices."""
    with open(path) as f:
        head = f.readline()
        off_s = f.readline()
        col_s = f.readline()
    m_vec, K, nnz = (int(x) for x in head.split(","))
    row_offsets = np.array(off_s.split(), dtype=np.int64).astype(np.int32)
    if row_offsets.size != m_vec + 1:
        raise ValueError("%s: %d row offsets, expected %d" % (path, row_offsets.size, m_vec + 1))
    col_idx = np.array(col_s.split(), dtype=np.int64).astype(np.int32)
    nvec = int(row_offsets[-1])
    if col_idx.size < nvec:
        raise ValueError("%s: %d column indices, expected %d" % (path, col_idx.size, nvec))
    return Cvse(m_vec, K, nnz, row_offsets, col_idx[:nvec])
