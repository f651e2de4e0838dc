"""SuiteSparse half of the RowMerge dataset tooling: Matrix Market `.mtx` files -> CSR side file
-> CVSE `.smtx` files, and the statistics row the reference logs for each of them.

Mirrors reference RowMerge/suit_sparse_matrix.py:
  * `suite_matrix` (:87-166): `scipy.io.mmread` + `coo.tocsr()`.  Here the file is parsed by
    read_mtx() and the coordinate list becomes CSR on the GPU (svc_coo_to_csr of the C ABI): rows
    ascending, inside a row the columns ascending, repeated (row, column) pairs merged: what
    scipy's tocsr() returns.  The header count NNZ is the length of the coordinate list (after a
    symmetric file has been mirrored, before merging), as `coo.nnz` is there.
  * `coo2csr(1)` (:108-135): the `<name>_csr.mtx` side file next to the source, "M, K, NNZ" / row
    pointer / column indices, no trailing newline.
  * `generate_suitesparse_CVSE_file(src_dir, dest_dir, paths_txt, vec_len)` (:181-221): every
    file of paths_txt converted, `.mtx` -> `.smtx` in the destination name, the RowMerge itself
    on the GPU (sspmm_amd.svc, CPython set order: byte for byte the reference's files).
  * `suit_cvse` / `generate_suitesparse_csv_file(src_dir, paths_txt, vec_len)` (:279-394): the
    nine CSV columns  name, NNZ, COL, new_sparsity, CSR, CVSE, TCF, SR_BCSR storage, Dense_X.

    python -m sspmm_amd.suitesparse convert <src_dir> <dest_dir> <paths.txt> <vec_len>
    python -m sspmm_amd.suitesparse csv <cvse_dir> <paths.txt> <vec_len> <out.csv>
"""
import argparse
import csv
import math
import os
import re
import sys

import numpy as np

_FIELDS = {"real": 1, "double": 1, "integer": 1, "complex": 2, "pattern": 0}
_SYMMETRIES = ("general", "symmetric", "skew-symmetric", "hermitian")


def read_mtx(path):
    """Matrix Market coordinate file -> (M, K, rows[int32], cols[int32]), zero-based, in file order, with the
    mirrored entries of a symmetric / skew-symmetric / hermitian file appended behind them (off-diagonal entries
    only), as scipy.io.mmread lays its coordinate list out.  Values are not kept: RowMerge uses the pattern."""
    with open(path) as f:
        banner = f.readline().split()
        if len(banner) < 5 or banner[0] != "%%MatrixMarket" or banner[1].lower() != "matrix":
            raise ValueError("%s: not a Matrix Market matrix file" % path)
        layout, field, symmetry = (x.lower() for x in banner[2:5])
        if layout != "coordinate":
            raise NotImplementedError("%s: only coordinate (sparse) files are supported, not %r" % (path, layout))
        if field not in _FIELDS or symmetry not in _SYMMETRIES:
            raise ValueError("%s: unknown field %r or symmetry %r" % (path, field, symmetry))
        line = f.readline()
        while line and (line.startswith("%") or not line.strip()):
            line = f.readline()
        M, K, n = (int(x) for x in line.split())
        body = np.loadtxt(f, dtype=np.float64, ndmin=2, comments="%") if n else np.zeros((0, 2))
    if body.shape[0] != n:
        raise ValueError("%s: %d entries, header says %d" % (path, body.shape[0], n))
    rows = body[:, 0].astype(np.int64) - 1
    cols = body[:, 1].astype(np.int64) - 1
    if n and (rows.min() < 0 or rows.max() >= M or cols.min() < 0 or cols.max() >= K):
        raise ValueError("%s: an entry lies outside the %d x %d matrix" % (path, M, K))
    if symmetry != "general":
        off = rows != cols
        rows, cols = np.concatenate([rows, cols[off]]), np.concatenate([cols, rows[off]])
    return M, K, rows.astype(np.int32), cols.astype(np.int32)


def coo_to_csr(M, K, rows, cols):
    """Coordinate list (int32 GPU tensors) -> (row_ptr[int32 M+1], col_ind[int32]) on the GPU: columns ascending
    inside a row, repeated pairs merged (scipy's coo.tocsr() pattern)."""
    import torch

    from . import _lib
    L = _lib.lib()
    n = rows.numel()
    dev = rows.device
    with torch.cuda.device(dev):
        row_ptr = torch.empty(M + 1, dtype=torch.int32, device=dev)
        col_ind = torch.empty(n, dtype=torch.int32, device=dev)
        nbytes = L.svc_coo_workspace_bytes(n)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
        _lib.check(L.svc_coo_to_csr(M, K, n, rows.data_ptr(), cols.data_ptr(), row_ptr.data_ptr(), col_ind.data_ptr(),
                                    ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream), "svc_coo_to_csr")
        kept = int(row_ptr[-1].item())
    return row_ptr, col_ind[:kept].contiguous()


def csr_side_file_text(M, K, nnz, row_ptr, col_ind):
    """What coo2csr(1) writes (reference suit_sparse_matrix.py:114-133): no newline behind the column indices."""
    return "%d, %d, %d\n%s\n%s" % (M, K, nnz, " ".join(str(int(x)) for x in row_ptr), " ".join(str(int(x)) for x in col_ind))


def convert_file(src_path, dest_path, vec_len, write_csr=True):
    """One `.mtx` file -> its `_csr.mtx` side file and one CVSE file.  Returns (M, K, NNZ, vec_row_ptr)."""
    import torch

    from . import formats
    from .svc import svc
    M, K, rows, cols = read_mtx(src_path)
    nnz = int(rows.size)
    row_ptr, col_ind = coo_to_csr(M, K, torch.from_numpy(rows).cuda(), torch.from_numpy(cols).cuda())
    if write_csr:
        with open(src_path.replace(".mtx", "_csr.mtx"), "w") as f:
            f.write(csr_side_file_text(M, K, nnz, row_ptr.cpu().numpy(), col_ind.cpu().numpy()))
    r = svc(row_ptr, col_ind, None, M, K, vec_len, order="cpython")
    vec_row_ptr = r.vec_row_ptr.cpu().numpy()
    os.makedirs(os.path.dirname(os.path.abspath(dest_path)), exist_ok=True)
    formats.write_cvse(dest_path, vec_row_ptr.size - 1, K, nnz, vec_row_ptr, r.vec_col.cpu().numpy())
    return M, K, nnz, vec_row_ptr


def generate_suitesparse_CVSE_file(src_dir, dest_dir, paths_txt, vec_len, log=None):
    """Every line of paths_txt names a `.mtx` file below src_dir; its CVSE file goes below dest_dir under the same
    name with `.mtx` replaced by `.smtx` (reference suit_sparse_matrix.py:181-221)."""
    with open(paths_txt) as f:
        lines = [line.rstrip("\n") for line in f if line.strip()]
    done = []
    for i, name in enumerate(lines):
        dest = os.path.join(dest_dir, name).replace(".mtx", ".smtx")
        convert_file(os.path.join(src_dir, name), dest, vec_len)
        done.append(dest)
        if log:
            log("File- %d  Finished  %s" % (i, dest))
    return done


def cvse_statistics(name, cvse, vec_len):
    """The reference's CSV row for a CVSE file (suit_cvse, suit_sparse_matrix.py:279-354, row at :378), as it writes
    it: every number through str().  `cvse` is a formats.Cvse."""
    num_vec_row, col, nnz = cvse.m_vec, cvse.K, cvse.nnz
    num_vec = int(cvse.col_idx.size)
    tiles = int(sum(math.ceil((int(cvse.row_offsets[i + 1]) - int(cvse.row_offsets[i])) / 32) for i in range(num_vec_row)))
    index_type, value_type = 4, 2
    new_sparsity = 1.0 - nnz / (num_vec * vec_len)
    csr = nnz * (value_type + index_type) + (num_vec_row * vec_len + 1) * index_type
    cvse_b = num_vec * vec_len * value_type + (num_vec_row + 1) * index_type + num_vec * index_type
    tcf = nnz * value_type + nnz * 3 * index_type + (num_vec_row * vec_len + 1) * index_type + tiles * 32 * index_type
    srbcsr = num_vec * vec_len * value_type + (num_vec_row + 1) * index_type + tiles * 32 * index_type
    dense_x = (col * col) / (num_vec * vec_len)
    return [name, str(nnz), str(col), str(new_sparsity), str(csr), str(cvse_b), str(tcf), str(srbcsr), str(dense_x)]


def generate_suitesparse_csv_file(src_dir, paths_txt, vec_len, csv_path):
    """Appends one row per file of paths_txt (the `.mtx` names; the CVSE files are looked up below src_dir with
    `.smtx`), reference suit_sparse_matrix.py:356-394."""
    from . import formats
    pattern = re.compile(r"/([^/]+)\.mtx$")
    with open(paths_txt) as f:
        lines = [line.rstrip("\n") for line in f if line.strip()]
    rows = []
    for name in lines:
        m = pattern.search("/" + name)
        cvse = formats.read_cvse(os.path.join(src_dir, name).replace(".mtx", ".smtx"))
        rows.append(cvse_statistics(m.group(1), cvse, vec_len))
    with open(csv_path, "a", newline="") as f:  # the reference appends too
        csv.writer(f).writerows(rows)
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    sub = ap.add_subparsers(dest="cmd", required=True)
    c = sub.add_parser("convert")
    for a in ("src_dir", "dest_dir", "paths_txt"):
        c.add_argument(a)
    c.add_argument("vec_len", type=int, choices=[8, 16])
    s = sub.add_parser("csv")
    for a in ("cvse_dir", "paths_txt"):
        s.add_argument(a)
    s.add_argument("vec_len", type=int, choices=[8, 16])
    s.add_argument("out_csv")
    a = ap.parse_args(argv)
    if a.cmd == "convert":
        done = generate_suitesparse_CVSE_file(a.src_dir, a.dest_dir, a.paths_txt, a.vec_len, log=print)
        print("Row-Merge (V = %d) of %d SuiteSparse files finished" % (a.vec_len, len(done)))
    else:
        rows = generate_suitesparse_csv_file(a.cvse_dir, a.paths_txt, a.vec_len, a.out_csv)
        print("%d rows appended to %s" % (len(rows), a.out_csv))
    return 0


if __name__ == "__main__":
    sys.exit(main())
