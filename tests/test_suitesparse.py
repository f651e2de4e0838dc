"""SuiteSparse half of the dataset tooling (sspmm_amd.suitesparse): the Matrix Market reader and the coordinate ->
CSR conversion against scipy (the library the reference calls) and against files the reference wrote, the
converter end to end on the GPU byte for byte, the statistics row against rows the reference published."""
import csv
import glob
import os
import shutil

import numpy as np
import pytest

from sspmm_amd import formats, suitesparse

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = ["general_37x90", "symmetric_48x48", "skew_24x70000"]


def _read_csr_side_file(path):
    with open(path) as f:
        head, ptr, col = f.readline(), f.readline(), f.readline()
    M, K, nnz = (int(x) for x in head.split(", "))
    return M, K, nnz, np.array(ptr.split(), dtype=np.int64), np.array(col.split(), dtype=np.int64)


def _write_mtx(path, banner, M, K, entries, values=None):
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate " + banner + "\n% a comment line\n\n")
        f.write("%d %d %d\n" % (M, K, len(entries)))
        for i, (r, c) in enumerate(entries):
            f.write("%d %d%s\n" % (r + 1, c + 1, "" if values is None else " " + values[i]))


@pytest.mark.parametrize("case", CASES)
def test_reader_and_oracle_conversion_reproduce_the_reference_csr_file(oracle, case):
    M, K, rows, cols = suitesparse.read_mtx(os.path.join(GOLDEN, case + ".mtx"))
    wM, wK, wnnz, wptr, wcol = _read_csr_side_file(os.path.join(GOLDEN, case + "_csr.mtx"))
    assert (M, K, rows.size) == (wM, wK, wnnz)  # the header count is the coordinate list's length
    ptr, col = oracle.coo_to_csr(M, K, rows, cols)
    assert np.array_equal(ptr, wptr) and np.array_equal(col, wcol)
    text = suitesparse.csr_side_file_text(M, K, rows.size, ptr, col)
    assert text.encode() == open(os.path.join(GOLDEN, case + "_csr.mtx"), "rb").read()


@pytest.mark.parametrize("banner,with_values", [("pattern general", False), ("real general", True), ("integer symmetric", True),
                                               ("real skew-symmetric", True), ("complex hermitian", True),
                                               ("pattern symmetric", False)])
def test_reader_matches_scipy_mmread(oracle, tmp_path, banner, with_values):
    """Field and symmetry variants: same shape, same coordinate list (order included), same CSR pattern as
    scipy.io.mmread(...).tocsr()."""
    from scipy.io import mmread
    from scipy.sparse import coo_matrix
    rng = np.random.default_rng(len(banner))
    n = 40
    sym = "general" not in banner
    ent = set()
    while len(ent) < 130:
        r, c = int(rng.integers(n)), int(rng.integers(n))
        if sym:
            r, c = max(r, c), min(r, c)
            if "skew" in banner and r == c:
                continue
        ent.add((r, c))
    ent = list(ent)
    rng.shuffle(ent)
    if with_values:
        fmt = {"complex hermitian": lambda: "%.3f %.3f" % (rng.uniform(-1, 1), 0.0), "integer symmetric": lambda: str(int(rng.integers(1, 9)))}
        values = [fmt.get(banner, lambda: "%.4f" % rng.uniform(0.1, 2))() for _ in ent]
    else:
        values = None
    path = str(tmp_path / "m.mtx")
    _write_mtx(path, banner, n, n, ent, values)
    M, K, rows, cols = suitesparse.read_mtx(path)
    coo = coo_matrix(mmread(path))
    assert (M, K) == coo.shape and rows.size == coo.nnz
    assert np.array_equal(rows, coo.row) and np.array_equal(cols, coo.col)
    csr = coo.tocsr()
    ptr, col = oracle.coo_to_csr(M, K, rows, cols)
    assert np.array_equal(ptr, csr.indptr) and np.array_equal(col, csr.indices)


def test_reader_rejects_what_it_does_not_read(tmp_path):
    p = tmp_path / "a.mtx"
    p.write_text("%%MatrixMarket matrix array real general\n2 2\n1\n2\n3\n4\n")
    with pytest.raises(NotImplementedError):
        suitesparse.read_mtx(str(p))
    p.write_text("%%MatrixMarket matrix coordinate real general\n2 2 1\n3 1 1.0\n")
    with pytest.raises(ValueError):
        suitesparse.read_mtx(str(p))
    p.write_text("2 2 1\n1 1 1.0\n")
    with pytest.raises(ValueError):
        suitesparse.read_mtx(str(p))


@pytest.mark.parametrize("V", [8, 16])
def test_statistics_row_agrees_with_the_published_rows(V):
    """The matrices behind the reference's RowMerge_suit_V*.csv are not available, but its columns are tied to each
    other by the formulas of suit_cvse: from name, NNZ, COL and the CVSE and SR-BCSR sizes the number of vectors,
    vector-rows and tiles follow, and a CVSE pattern with those counts must give back the whole row, strings
    included."""
    with open(os.path.join(GOLDEN, "rowmerge_suit_stats_v%d_head.csv" % V)) as f:
        published = list(csv.reader(f))
    assert len(published) >= 3
    for row in published:
        name, nnz, col = row[0], int(row[1]), int(row[2])
        csr_b, cvse_b, srbcsr_b = int(row[4]), int(row[5]), int(row[7])
        m_vec = ((csr_b - nnz * 6) // 4 - 1) // V
        num_vec = (cvse_b - (m_vec + 1) * 4) // (V * 2 + 4)
        tiles = (srbcsr_b - num_vec * V * 2 - (m_vec + 1) * 4) // 128
        assert tiles >= -(-num_vec // 32)
        # vector-row lengths with that total and that many 32-vector tiles
        per_row_tiles = np.full(m_vec, tiles // m_vec)
        per_row_tiles[:tiles % m_vec] += 1
        lens = np.where(per_row_tiles > 0, 32 * (per_row_tiles - 1) + 1, 0).astype(np.int64)
        extra = num_vec - int(lens.sum())
        for i in range(m_vec):
            take = min(extra, 31) if per_row_tiles[i] > 0 else 0
            lens[i] += take
            extra -= take
        assert extra == 0
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        cvse = formats.Cvse(m_vec, col, nnz, off, np.zeros(num_vec, np.int32))
        assert suitesparse.cvse_statistics(name, cvse, V) == row


@pytest.mark.gpu
@pytest.mark.parametrize("V", [8, 16])
def test_converter_writes_the_reference_files(built_library, tmp_path, V):
    """.mtx -> _csr.mtx side file and CVSE .smtx through the GPU (coordinate -> CSR, then RowMerge): the bytes the
    reference's suite_matrix.coo2csr(1) and CVSE_out wrote; then the CSV of the files just written."""
    src = tmp_path / "src" / "suitesparse"
    src.mkdir(parents=True)
    for c in CASES:
        shutil.copy(os.path.join(GOLDEN, c + ".mtx"), src / (c + ".mtx"))
    paths = tmp_path / "suitpaths.txt"
    paths.write_text("".join("suitesparse/%s.mtx\n" % c for c in CASES))
    dest = tmp_path / ("dlmc-v%d" % V)
    rc = suitesparse.main(["convert", str(tmp_path / "src"), str(dest), str(paths), str(V)])
    assert rc == 0
    for c in CASES:
        assert (src / (c + "_csr.mtx")).read_bytes() == open(os.path.join(GOLDEN, c + "_csr.mtx"), "rb").read(), c
        assert (dest / "suitesparse" / (c + ".smtx")).read_bytes() == open(os.path.join(GOLDEN, "%s.mtx.v%d.smtx" % (c, V)), "rb").read(), c
    out_csv = tmp_path / "RowMerge_suit.csv"
    assert suitesparse.main(["csv", str(dest), str(paths), str(V), str(out_csv)]) == 0
    rows = list(csv.reader(open(out_csv)))
    assert [r[0] for r in rows] == CASES
    for r, c in zip(rows, CASES):
        cv = formats.read_cvse(os.path.join(GOLDEN, "%s.mtx.v%d.smtx" % (c, V)))
        assert r == suitesparse.cvse_statistics(c, cv, V)
        assert int(r[5]) == cv.col_idx.size * (2 * V + 4) + (cv.m_vec + 1) * 4


@pytest.mark.gpu
def test_coordinate_list_to_csr_on_the_gpu(oracle, built_library):
    """Large shuffled lists with repeated pairs, empty rows, entries outside the matrix; an empty list."""
    import torch
    rng = np.random.default_rng(5)
    for M, K, n in [(1000, 3000, 200000), (17, 5, 400), (70000, 70000, 50000), (5, 9, 0), (1, 1, 3)]:
        rows = rng.integers(0, M, n).astype(np.int32)
        cols = rng.integers(0, K, n).astype(np.int32)
        if n > 100:
            rows[rng.integers(0, n, 20)] = M + 3      # outside: dropped
            cols[rng.integers(0, n, 20)] = -1
            rows[rows == 7] = 8                        # an empty row
        print("coo M=%d K=%d n=%d" % (M, K, n), flush=True)
        ptr, col = suitesparse.coo_to_csr(M, K, torch.from_numpy(rows).cuda(), torch.from_numpy(cols).cuda())
        torch.cuda.synchronize()
        wptr, wcol = oracle.coo_to_csr(M, K, rows, cols)
        assert np.array_equal(ptr.cpu().numpy(), wptr) and np.array_equal(col.cpu().numpy(), wcol)
