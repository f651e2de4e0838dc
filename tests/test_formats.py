"""Text formats: .smtx reader/writer and the CVSE writer against the files the reference wrote."""
import glob
import os

import numpy as np
import pytest

from sspmm_amd import formats

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "*.v*.smtx"))))
def test_cvse_read_write_round_trip_is_byte_exact(path, tmp_path):
    c = formats.read_cvse(path)
    out = tmp_path / "x.smtx"
    formats.write_cvse(str(out), c.m_vec, c.K, c.nnz, c.row_offsets, c.col_idx)
    assert out.read_bytes() == open(path, "rb").read()
    assert c.row_offsets[0] == 0 and np.all(np.diff(c.row_offsets) >= 0)
    assert c.col_idx.size == c.row_offsets[-1]
    assert c.col_idx.size == 0 or (c.col_idx.min() >= 0 and c.col_idx.max() < c.K)


def test_cvse_text_layout():
    assert formats.cvse_text(2, 8, 5, [0, 2, 3], [4, 1, 7]) == "2, 8, 5\n0 2 3\n4 1 7"
    assert formats.cvse_text(1, 8, 0, [0, 0], []) == "1, 8, 0\n0 0\n"


def test_smtx_round_trip(tmp_path):
    p = tmp_path / "a.smtx"
    formats.write_smtx(str(p), 3, 9, [0, 2, 2, 5], [1, 8, 0, 3, 4])
    M, K, nnz, ptr, col = formats.read_smtx(str(p))
    assert (M, K, nnz) == (3, 9, 5) and ptr.tolist() == [0, 2, 2, 5] and col.tolist() == [1, 8, 0, 3, 4]
    assert ptr.dtype == np.int32 and col.dtype == np.int32


def test_smtx_bad_pointer_length(tmp_path):
    p = tmp_path / "bad.smtx"
    p.write_text("3, 9, 2\n0 1 2\n1 2\n")
    with pytest.raises(ValueError):
        formats.read_smtx(str(p))
