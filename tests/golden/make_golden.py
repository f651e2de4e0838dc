"""Writes the RowMerge golden fixtures in this directory.

Run once, in the development container only, where the reference checkout is at
/root/reference:  python tests/golden/make_golden.py

It imports the reference's RowMerge/sparse_matrix_format.py, feeds it seeded
synthetic .smtx inputs (written here as <case>.smtx) and stores what the
reference's own CVSE class and CVSE_out writer produce:
  <case>.v<V>.smtx   the exact bytes CVSE_out wrote
The fixtures pin the two things no closed form pins: the byte layout of the
output file and the column order on realistic merged rows.  Tests read only the
fixture files; the reference itself is never needed at test time.

The SuiteSparse half (reference RowMerge/suit_sparse_matrix.py) gets the same treatment: seeded
Matrix Market coordinate files <case>.mtx are written here, and the reference's suite_matrix
(scipy.io.mmread, coo.tocsr()), its coo2csr(1) writer and CVSE / CVSE_out produce
  <case>_csr.mtx       the CSR side file, exact bytes
  <case>.mtx.v<V>.smtx the CVSE file, exact bytes
"""
import os
import random
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def write_smtx(path, M, K, rows):
    ptr = [0]
    cols = []
    for r in rows:
        cols += r
        ptr.append(len(cols))
    with open(path, "w") as f:
        f.write("%d, %d, %d\n" % (M, K, len(cols)))
        f.write(" ".join(map(str, ptr)) + "\n")
        f.write(" ".join(map(str, cols)) + "\n")


def cases():
    rng = random.Random(20240601)
    out = {}
    # ragged M (not a multiple of V), tiny K: every key < 8
    out["tiny_5x8"] = (5, 8, [sorted(rng.sample(range(8), rng.randrange(0, 5))) for _ in range(5)])
    # DLMC-like 90 % sparse block
    out["rand_64x512"] = (64, 512, [sorted(rng.sample(range(512), rng.randrange(30, 70))) for _ in range(64)])
    # wide K, V=16-sized groups, some empty rows
    out["wide_50x2048"] = (50, 2048, [sorted(rng.sample(range(2048), rng.choice([0, 0, 5, 40, 200])))
                                      for _ in range(50)])
    # all rows empty -> nvec == 0 (third line of the output is empty)
    out["empty_17x32"] = (17, 32, [[] for _ in range(17)])
    # one heavy vector-row (several table resizes) next to light ones, large keys
    heavy = [sorted(rng.sample(range(70000), 900)) for _ in range(3)]
    light = [sorted(rng.sample(range(70000), rng.randrange(0, 12))) for _ in range(21)]
    out["skew_24x70000"] = (24, 70000, heavy[:2] + light[:9] + heavy[2:] + light[9:])
    # rows stored in descending column order (the reader keeps file order)
    out["desc_16x300"] = (16, 300, [sorted(rng.sample(range(300), rng.randrange(5, 60)), reverse=True)
                                   for _ in range(16)])
    return out


def main():
    sys.path.insert(0, "/root/reference/RowMerge")
    os.environ.setdefault("MPLBACKEND", "Agg")
    import sparse_matrix_format as ref  # the reference itself

    for name, (M, K, rows) in cases().items():
        src = os.path.join(HERE, name + ".smtx")
        write_smtx(src, M, K, rows)
        m = ref.sparse_matrix(src)
        assert (m.M, m.N) == (M, K)
        for V in (8, 16):
            c = ref.CVSE(m.M, m.N, m.nnz, m.colInd_list_array(), V)
            c.CVSE_out(os.path.join(HERE, "%s.v%d.smtx" % (name, V)))
            print(name, V, "num_vec_row", c.num_vec_row, "num_vec", c.num_vec)


def mtx_cases():
    """name -> text of a Matrix Market coordinate file."""
    rng = random.Random(20241125)
    out = {}
    # general, real values, entries in shuffled order, some repeated (row, column) pairs, an explicit zero,
    # empty rows, M not a multiple of 8
    M, K = 37, 90
    ent = [(rng.randrange(M), rng.randrange(K)) for _ in range(260)]
    ent = [e for e in ent if e[0] not in (5, 6, 20)]
    ent += ent[:9]  # duplicates
    rng.shuffle(ent)
    lines = ["%%MatrixMarket matrix coordinate real general", "% shuffled entries with duplicates", "%d %d %d" % (M, K, len(ent))]
    lines += ["%d %d %s" % (r + 1, c + 1, "0.0" if i == 3 else repr(round(rng.uniform(-2, 2), 4))) for i, (r, c) in enumerate(ent)]
    out["general_37x90"] = "\n".join(lines) + "\n"
    # symmetric pattern (lower triangle stored): the reader mirrors the off-diagonal entries
    n = 48
    low = sorted(set((max(a, b), min(a, b)) for a, b in ((rng.randrange(n), rng.randrange(n)) for _ in range(150))))
    rng.shuffle(low)
    lines = ["%%MatrixMarket matrix coordinate pattern symmetric", "%d %d %d" % (n, n, len(low))]
    lines += ["%d %d" % (r + 1, c + 1) for r, c in low]
    out["symmetric_48x48"] = "\n".join(lines) + "\n"
    # wide integer matrix with a heavy row group (set resizes) and large column numbers
    M, K = 24, 70000
    ent = []
    for r in range(M):
        cnt = 900 if r in (1, 2, 13) else rng.randrange(0, 12)
        ent += [(r, c) for c in rng.sample(range(K), cnt)]
    rng.shuffle(ent)
    lines = ["%%MatrixMarket matrix coordinate integer general", "%d %d %d" % (M, K, len(ent))]
    lines += ["%d %d %d" % (r + 1, c + 1, rng.randrange(1, 9)) for r, c in ent]
    out["skew_24x70000"] = "\n".join(lines) + "\n"
    return out


def main_suitesparse():
    sys.path.insert(0, "/root/reference/RowMerge")
    os.environ.setdefault("MPLBACKEND", "Agg")
    import sparse_matrix_format as ref
    import suit_sparse_matrix as ref_suite  # the reference itself

    for name, text in mtx_cases().items():
        src = os.path.join(HERE, name + ".mtx")
        with open(src, "w") as f:
            f.write(text)
        sm = ref_suite.suite_matrix(src)
        sm.coo2csr(1)  # writes <case>_csr.mtx beside the source
        lists = sm.colInd_list_array()
        for V in (8, 16):
            c = ref.CVSE(sm.M, sm.K, sm.nnz, lists, V)
            c.CVSE_out(os.path.join(HERE, "%s.mtx.v%d.smtx" % (name, V)))
            print(name, V, "M", sm.M, "K", sm.K, "nnz", sm.nnz, "num_vec", c.num_vec)


if __name__ == "__main__":
    if "--suitesparse" in sys.argv:
        main_suitesparse()
    else:
        main()
