"""Dataset tooling (sspmm_amd.rowmerge): the statistics row against the rows the reference published,
and the converter end to end against the files the reference wrote."""
import csv
import glob
import os

import numpy as np
import pytest

from sspmm_amd import formats, rowmerge

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _published_rows(V):
    # the first rows of the reference's result-data/RowMerge_V{8,16}.csv (512 x 512 DLMC matrices)
    with open(os.path.join(GOLDEN, "rowmerge_stats_v%d_head.csv" % V)) as f:
        return list(csv.reader(f))


@pytest.mark.parametrize("V", [8, 16])
def test_statistics_reproduce_the_published_rows(V):
    """The inputs of those rows are not available, but every column is a function of (ROW, COL, NNZ, V),
    the number of vectors and the number of 32-vector tiles: a row pointer with the published vector and
    tile counts must give back the published row, strings included."""
    for row in _published_rows(V):
        no, ROW, COL, NNZ = int(row[0]), int(row[1]), int(row[2]), int(row[3])
        all_zero, srbcsr = int(row[5]), int(row[9])
        m_vec = -(-ROW // V)
        nvec = m_vec * COL - all_zero
        tiles = (srbcsr - nvec * V * 2 - (m_vec + 1) * 4) // 128
        # any vector-row lengths with that total and that many tiles: a row of t tiles has 32 (t - 1) + 1 .. 32 t vectors
        per_row_tiles = np.full(m_vec, tiles // m_vec)
        per_row_tiles[:tiles % m_vec] += 1
        lens = np.where(per_row_tiles > 0, 32 * (per_row_tiles - 1) + 1, 0).astype(np.int64)
        extra = nvec - int(lens.sum())
        for i in range(m_vec):
            take = min(extra, 31) if per_row_tiles[i] > 0 else 0
            lens[i] += take
            extra -= take
        assert extra == 0 and lens.sum() == nvec and ((lens + 31) // 32).sum() == tiles
        ptr = np.concatenate([[0], np.cumsum(lens)])
        assert rowmerge.csv_row(no, rowmerge.statistics(ROW, COL, NNZ, V, ptr)) == row


def test_statistics_closed_forms():
    s = rowmerge.statistics(5, 8, 7, 8, [0, 6])
    assert s["all_zero_vec_cnt"] == 2 and s["CVSE_storage"] == 6 * 16 + 2 * 4 + 6 * 4
    assert s["CSR_storage"] == 7 * 6 + 6 * 4 and s["new_sparsity"] == 1.0 - 7 / 48
    assert s["TCF_storage"] == 7 * 2 + 7 * 12 + 6 * 4 + 128 and s["SR_BCSR_storage"] == 96 + 8 + 128
    empty = rowmerge.statistics(17, 32, 0, 8, [0, 0, 0, 0])
    assert empty["new_sparsity"] == 1.0 and empty["all_zero_vec_cnt"] == 3 * 32


@pytest.mark.gpu
@pytest.mark.parametrize("V", [8, 16])
def test_converter_writes_the_reference_files_and_rows(built_library, tmp_path, V):
    names = sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLDEN, "*.smtx")) if ".v" not in os.path.basename(p))
    paths = tmp_path / "paths.txt"
    paths.write_text("".join("%s extra-token\n" % n for n in names))
    out_csv = tmp_path / "stats.csv"
    rc = rowmerge.main([GOLDEN, str(tmp_path / "out"), str(paths), str(V), "--csv", str(out_csv)])
    assert rc == 0
    rows = list(csv.reader(open(out_csv)))
    assert len(rows) == len(names)
    for i, n in enumerate(names):
        want = os.path.join(GOLDEN, n.replace(".smtx", ".v%d.smtx" % V))
        assert (tmp_path / "out" / n).read_bytes() == open(want, "rb").read()
        M, K, nnz, _, _ = formats.read_smtx(os.path.join(GOLDEN, n))
        c = formats.read_cvse(want)
        assert rows[i] == rowmerge.csv_row(i, rowmerge.statistics(M, K, nnz, V, c.row_offsets))
        assert int(rows[i][5]) == c.m_vec * K - c.col_idx.size  # all-zero vectors = m_vec * COL - nvec
