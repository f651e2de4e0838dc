"""Dataset tooling of the RowMerge step: convert DLMC-style `.smtx` pattern files to CVSE files
on the GPU and write the statistics row the reference logs for each of them.

Mirrors `generate_CVSE_file(src_dir, dest_dir, paths_txt, vec_len)` of the reference
(RowMerge/sparse_matrix_format.py:190-250): same output files (byte for byte, CPython set order)
and the same ten CSV columns
    NO., ROW, COL, NNZ, new_sparsity, all_zero_vec_cnt, CSR_storage, CVSE_storage, TCF_storage, SR_BCSR_storage
(`:193`, storage formulas `:124-150`).  The reference counts the all-zero vectors by scanning a
dense ROW x COL copy of the matrix (`:176-188`); here the count is m_vec * COL - nvec, the same
number, from the merged row pointer.

    python -m sspmm_amd.rowmerge <src_dir> <dest_dir> <paths.txt> <vec_len> [--csv stats.csv] [--order cpython|sorted]
                                 [--reorder]

`--reorder` is the reference's second pass (`python row_merge_reorder.py`, README.md:36, which
writes the dataset-v8 / dataset-v16 folders): the rows are first brought into the order of
sspmm_amd.reorder.minhash_order, then merged; the row order is written next to each output file
as `<file>.perm` (one line of space-separated source row numbers).
"""
import argparse
import csv
import os
import sys

import numpy as np


def statistics(ROW, COL, NNZ, vec_len, vec_row_ptr):
    """The values of the reference's CSV row (without the leading index) as Python numbers."""
    vec_row_ptr = np.asarray(vec_row_ptr, dtype=np.int64)
    m_vec = vec_row_ptr.size - 1
    num_vec = int(vec_row_ptr[-1])
    all_zero_vec_cnt = m_vec * COL - num_vec
    new_sparsity = 1.0 if num_vec == 0 else 1.0 - NNZ / (num_vec * vec_len)
    index_type, value_type = 4, 2
    tiles = int(((np.diff(vec_row_ptr) + 31) // 32).sum())  # tile_num[i] = ceil(len_i / 32), reference :114
    csr = NNZ * (value_type + index_type) + (ROW + 1) * index_type
    cvse = num_vec * vec_len * value_type + (m_vec + 1) * index_type + num_vec * index_type
    tcf = NNZ * value_type + NNZ * 3 * index_type + (ROW + 1) * index_type + tiles * 32 * index_type
    srbcsr = num_vec * vec_len * value_type + (m_vec + 1) * index_type + tiles * 32 * index_type
    return {"ROW": ROW, "COL": COL, "NNZ": NNZ, "new_sparsity": new_sparsity, "all_zero_vec_cnt": all_zero_vec_cnt,
            "CSR_storage": csr, "CVSE_storage": cvse, "TCF_storage": tcf, "SR_BCSR_storage": srbcsr}


CSV_COLUMNS = ["ROW", "COL", "NNZ", "new_sparsity", "all_zero_vec_cnt", "CSR_storage", "CVSE_storage", "TCF_storage",
               "SR_BCSR_storage"]


def csv_row(index, stats):
    """The row as the reference writes it: every field through str()."""
    return [str(index)] + [str(stats[c]) for c in CSV_COLUMNS]


def convert_file(src_path, dest_path, vec_len, order="cpython", reorder=False):
    """One `.smtx` file -> one CVSE file, merged on the GPU.  Returns the statistics dict."""
    import torch

    from . import formats
    from .svc import svc
    M, K, nnz, row_ptr, col_ind = formats.read_smtx(src_path)
    rp, ci = torch.from_numpy(row_ptr).cuda(), torch.from_numpy(col_ind).cuda()
    os.makedirs(os.path.dirname(os.path.abspath(dest_path)), exist_ok=True)
    if reorder:
        from .reorder import minhash_order, permute_csr
        perm = minhash_order(rp, ci, M)
        rp, ci, _ = permute_csr(rp, ci, None, perm)
        with open(dest_path + ".perm", "w") as f:
            f.write(" ".join(map(str, perm.cpu().tolist())))
    r = svc(rp, ci, None, M, K, vec_len, order=order)
    vec_row_ptr = r.vec_row_ptr.cpu().numpy()
    formats.write_cvse(dest_path, vec_row_ptr.size - 1, K, nnz, vec_row_ptr, r.vec_col.cpu().numpy())
    return statistics(M, K, nnz, vec_len, vec_row_ptr)


# entries of one batched call: the stack's CSR, the workspace (16 x) and the outputs stay well inside a GPU's memory
BATCH_NNZ = 32 << 20


def convert_files(src_paths, dest_paths, vec_len, order="cpython"):
    """Many `.smtx` files -> as many CVSE files with ONE chain of GPU launches: the matrices are read, stacked along
    the rows, merged by svc_batched, brought back with one copy and written.  Returns the statistics dicts."""
    import torch

    from . import formats
    from .svc import stack_csr, svc_batched
    mats = []
    for p in src_paths:
        M, K, nnz, row_ptr, col_ind = formats.read_smtx(p)
        mats.append((M, K, row_ptr, col_ind, None))
    mat_rows, K_max, rp, ci, _ = stack_csr(mats)
    batch = svc_batched(mat_rows, K_max, torch.from_numpy(rp).cuda(), torch.from_numpy(ci).cuda(), None, vec_len, order=order)
    stats = []
    for (M, K, row_ptr, col_ind, _), dest, (vec_row_ptr, vec_col, _v) in zip(mats, dest_paths, batch.to_host()):
        os.makedirs(os.path.dirname(os.path.abspath(dest)), exist_ok=True)
        formats.write_cvse(dest, vec_row_ptr.size - 1, K, int(col_ind.size), vec_row_ptr, vec_col)
        stats.append(statistics(M, K, int(col_ind.size), vec_len, vec_row_ptr))
    return stats


def generate_cvse_files(src_dir, dest_dir, paths_txt, vec_len, csv_path=None, order="cpython", log=None,
                        reorder=False):
    """Every file named in paths_txt (first token of each line, relative to src_dir / dest_dir).  Without
    `reorder` the files go through the GPU in stacks (convert_files) of up to BATCH_NNZ entries, so the dataset
    costs a handful of launch chains instead of one per file."""
    with open(paths_txt) as f:
        names = [line.split()[0] for line in f if line.split()]
    rows = []
    if reorder:
        for i, name in enumerate(names):
            stats = convert_file(os.path.join(src_dir, name), os.path.join(dest_dir, name), vec_len, order, reorder)
            rows.append(csv_row(i, stats))
            if log:
                log("No. %d  OK  %s" % (i, os.path.join(dest_dir, name)))
    else:
        from . import formats
        start = 0
        while start < len(names):
            # a stack ends before the file that would take it past BATCH_NNZ entries (the header line names the count)
            end, total = start, 0
            while end < len(names):
                n = formats.read_smtx_header(os.path.join(src_dir, names[end]))[2]
                if end > start and total + n > BATCH_NNZ:
                    break
                total += n
                end += 1
            chunk = names[start:end]
            stats = convert_files([os.path.join(src_dir, n) for n in chunk], [os.path.join(dest_dir, n) for n in chunk],
                                  vec_len, order)
            for k, st in enumerate(stats):
                rows.append(csv_row(start + k, st))
                if log:
                    log("No. %d  OK  %s" % (start + k, os.path.join(dest_dir, chunk[k])))
            start = end
    if csv_path:
        with open(csv_path, "a", newline="") as f:  # the reference appends too
            csv.writer(f).writerows(rows)
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("src_dir")
    ap.add_argument("dest_dir")
    ap.add_argument("paths_txt")
    ap.add_argument("vec_len", type=int, choices=[8, 16])
    ap.add_argument("--csv", default=None, help="append the statistics rows to this file")
    ap.add_argument("--order", default="cpython", choices=["cpython", "sorted"])
    ap.add_argument("--reorder", action="store_true", help="sort the rows by min-hash key before merging")
    a = ap.parse_args(argv)
    rows = generate_cvse_files(a.src_dir, a.dest_dir, a.paths_txt, a.vec_len, a.csv, a.order, log=print,
                               reorder=a.reorder)
    print("Row-Merge (V = %d) format transformation finish: %d files" % (a.vec_len, len(rows)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
