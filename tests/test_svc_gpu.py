"""GPU parity of the SVC (RowMerge) through the C ABI: bit-exact against the files the reference
wrote, the CPU oracle and the Python runtime's own set."""
import glob
import os

import numpy as np
import pytest
import torch

import sspmm_amd
from sspmm_amd import _lib, formats, synth
from gpu_util import dev

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = sorted(os.path.basename(p)[:-5] for p in glob.glob(os.path.join(GOLDEN, "*.smtx"))
               if ".v" not in os.path.basename(p))


def gpu_svc(M, K, V, row_ptr, col_ind, vals=None, order="cpython"):
    r = sspmm_amd.svc(dev(row_ptr), dev(col_ind), None if vals is None else dev(vals), M, K, V, order=order)
    torch.cuda.synchronize()
    return (r.vec_row_ptr.cpu().numpy(), r.vec_col.cpu().numpy(),
            None if r.vec_val is None else r.vec_val.cpu().numpy(), r.num_vec)


@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("V", [8, 16])
def test_reference_files_byte_for_byte(built_library, name, V):
    print("case", name, V, flush=True)
    M, K, nnz, row_ptr, col_ind = formats.read_smtx(os.path.join(GOLDEN, name + ".smtx"))
    vrp, vcol, _, nvec = gpu_svc(M, K, V, row_ptr, col_ind)
    with open(os.path.join(GOLDEN, "%s.v%d.smtx" % (name, V))) as f:
        want = f.read()
    assert formats.cvse_text(len(vrp) - 1, K, nnz, vrp, vcol) == want
    assert nvec == vcol.size


def _compare_with_oracle(oracle, csr, V, order="cpython"):
    print("case M=%d K=%d nnz=%d V=%d %s" % (csr.M, csr.K, csr.col_ind.size, V, order), flush=True)
    vrp, vcol, vval, _ = gpu_svc(csr.M, csr.K, V, csr.row_ptr, csr.col_ind, csr.values, order)
    wrp, wcol, wval = oracle.svc(csr.M, csr.K, V, csr.row_ptr, csr.col_ind, csr.values, order=order)
    assert np.array_equal(vrp, wrp)
    assert np.array_equal(vcol, wcol)
    assert np.array_equal(vval.view(np.uint16), wval.view(np.uint16))
    return vrp, vcol, vval


def _random_csr(rng, M, K, max_len, sort=True):
    lens = rng.integers(0, min(K, max_len) + 1, M)
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([(np.sort if sort else (lambda x: x))(rng.permutation(K)[:n]) for n in lens] +
                          [np.zeros(0, np.int64)]).astype(np.int32)
    vals = rng.standard_normal(cols.size).astype(np.float16)
    return synth.Csr(M, K, ptr, cols, vals)


@pytest.mark.parametrize("V", [1, 3, 8, 16])
@pytest.mark.parametrize("order", ["cpython", "sorted"])
def test_random_small_matrices(oracle, built_library, V, order):
    rng = np.random.default_rng(1000 + V)
    for trial in range(6):
        csr = _random_csr(rng, int(rng.integers(1, 90)), int(rng.choice([8, 33, 512, 5000])), 60, sort=bool(trial % 2))
        _compare_with_oracle(oracle, csr, V, order)


@pytest.mark.parametrize("V", [8, 16])
def test_against_python_set_directly(oracle, built_library, V):
    """The reference's one-line merge evaluated by the Python runtime itself."""
    rng = np.random.default_rng(5)
    csr = _random_csr(rng, 70, 3000, 120)
    vrp, vcol, _, _ = gpu_svc(csr.M, csr.K, V, csr.row_ptr, csr.col_ind)
    ptr, flat = oracle.rowmerge_python(csr.M, V, oracle.csr_col_lists(csr.M, csr.row_ptr, csr.col_ind))
    assert vrp.tolist() == ptr and vcol.tolist() == flat


@pytest.mark.parametrize("keys", [300, 310, 1200, 1240, 4800, 5000, 7590, 7610, 9000])
def test_every_group_size_class(oracle, built_library, keys):
    """Groups whose distinct-column bound falls into each kernel class (LDS 64 / 256 / 1024 threads,
    and tables in the workspace), next to empty and tiny groups."""
    rng = np.random.default_rng(keys)
    V, K = 8, 40000
    lens = np.zeros(40, np.int64)
    lens[8:16] = keys // 8 + 1
    lens[17] = 3
    lens[24:27] = [keys // 2, 2, keys // 3]
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([np.sort(rng.permutation(K)[:n]) for n in lens]).astype(np.int32)
    csr = synth.Csr(40, K, ptr, cols, rng.standard_normal(cols.size).astype(np.float16))
    _compare_with_oracle(oracle, csr, V)
    _compare_with_oracle(oracle, csr, 16)


@pytest.mark.parametrize("distinct", [3000, 4914, 4915, 5600])
def test_a_groups_class_comes_from_its_distinct_columns(oracle, built_library, distinct):
    """A group with 6400 non-zeros and 3000 .. 5600 distinct columns (its rows repeat columns of one another):
    the table it is merged in is chosen from the distinct count, either side of the 4914-column class limit."""
    rng = np.random.default_rng(distinct)
    V, K, per_row = 8, 16384, 800
    pool = rng.permutation(K)[:distinct]
    rows = []
    covered = 0
    for r in range(V):  # every pool column occurs, rows repeat columns of one another
        must = pool[covered:covered + per_row]
        covered += must.size
        rest = rng.choice(pool, per_row - must.size, replace=False) if must.size < per_row else np.empty(0, np.int64)
        rows.append(np.unique(np.concatenate([must, rest])))
    lens = np.array([0] * 8 + [len(x) for x in rows] + [5] * 8)
    cols = np.concatenate([np.empty(0, np.int64)] * 8 + rows + [rng.permutation(K)[:5] for _ in range(8)]).astype(np.int32)
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    csr = synth.Csr(24, K, ptr, cols, rng.standard_normal(cols.size).astype(np.float16))
    vrp, _, _ = _compare_with_oracle(oracle, csr, V)
    assert vrp[2] - vrp[1] == distinct


@pytest.mark.parametrize("keys", [5, 40, 200, 700, 2500, 4000])
def test_member_rows_that_bring_nothing_new(oracle, built_library, keys):
    """CPython rebuilds the set for every member row, also for an empty row and for a row whose columns are all
    known; the order can change each time, settle, or alternate between two orders.  The kernels skip
    constructions whose result they know: groups whose empty and repeated rows come singly, in runs of even and
    odd length, at the start, between rows with new columns and at the end, in every size class, against the
    Python runtime's own set."""
    rng = np.random.default_rng(keys)
    V, K = 8, 16384
    layouts = ["n.......", "nr......", "n.n.....", "n..n....", "n...n...", "n....n..", ".n.....n", "..n..r.n",
               "nrrrrrrr", "n.r.r.r.", "nn....nn", "n.....rn", "........", "...n....", "n......r", "nr.n.r.n"]
    rows = []
    for layout in layouts:
        seen = np.empty(0, np.int64)
        for ch in layout:
            if ch == "n":    # new columns (and a few known ones)
                fresh = rng.choice(np.setdiff1d(np.arange(K), seen), keys, replace=False)
                again = rng.choice(seen, min(seen.size, 3), replace=False) if seen.size else seen
                row = np.sort(np.concatenate([fresh, again]))
                seen = np.union1d(seen, fresh)
            elif ch == "r":  # only known columns
                row = np.sort(rng.choice(seen, max(1, seen.size // 2), replace=False)) if seen.size else seen
            else:
                row = np.empty(0, np.int64)
            rows.append(row)
    lens = np.array([r.size for r in rows])
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate(rows).astype(np.int32)
    csr = synth.Csr(len(rows), K, ptr, cols, rng.standard_normal(cols.size).astype(np.float16))
    vrp, vcol, _ = _compare_with_oracle(oracle, csr, V)
    want_ptr, want_cols = oracle.rowmerge_python(csr.M, V, oracle.csr_col_lists(csr.M, csr.row_ptr, csr.col_ind))
    assert vrp.tolist() == want_ptr and vcol.tolist() == want_cols


def test_more_groups_of_a_class_than_workgroups_in_its_launch(oracle, built_library):
    """V = 1 makes every row a group: 9000 short rows (the launch of the smallest class has 8192 workgroups),
    and 300 + 260 + 270 rows of 1300, 400 and 5000 columns (one workgroup per CU for those classes), so that
    workgroups walk on to a second group and reuse their tables."""
    rng = np.random.default_rng(77)
    K = 16384
    lens = np.concatenate([rng.integers(0, 20, 9000), np.full(300, 1300), np.full(260, 400), np.full(270, 5000)])
    rng.shuffle(lens)
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens]).astype(np.int32)
    csr = synth.Csr(lens.size, K, ptr, cols, rng.standard_normal(cols.size).astype(np.float16))
    _compare_with_oracle(oracle, csr, 1)


def test_a_row_that_repeats_a_column_stays_inside_its_group(built_library):
    """Invalid input (the contract forbids repeated columns in a row): the column order is then unspecified,
    but the counts are the distinct columns and every write stays inside the group's own vectors."""
    rng = np.random.default_rng(78)
    K, V = 4096, 8
    rows = [np.concatenate([c, c[: len(c) // 2]]) for c in (rng.choice(K, n, replace=False) for n in [5, 300, 0, 1500, 40, 2, 9, 700] * 3)]
    lens = np.array([len(r) for r in rows])
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate(rows).astype(np.int32)
    vals = np.ones(cols.size, np.float16)
    vrp, vcol, vval, nvec = gpu_svc(len(rows), K, V, ptr, cols, vals)
    want = [np.unique(cols[ptr[g]:ptr[min(len(rows), g + V)]]).size for g in range(0, len(rows), V)]
    assert np.array_equal(np.diff(vrp), want)
    assert vcol.size == nvec and vval.size == nvec * V
    assert ((vcol >= 0) & (vcol < K)).all() and np.isin(vval, [0.0, 1.0]).all()


@pytest.mark.parametrize("sizes", [[5, 300, 0, 1500, 40, 2, 9, 700], [3, 12, 0, 25, 7, 1, 30, 16], [2400, 0, 0, 4, 0, 1100, 0, 600],
                                   [9000, 0, 40, 3000, 0, 0, 2, 0]])
def test_a_repeated_column_is_kept_once(built_library, sizes):
    """Invalid input again: whatever the order, a group's vectors are its distinct columns, each once, and every
    non-zero lands in the vector of its column (the placements that pass over slots unseen are given up for the
    group as soon as it holds more keys than distinct columns, and the group is done again with those that look)."""
    rng = np.random.default_rng(sum(sizes))
    K, V = 16384, 8
    rows = []
    for g in range(3):
        for n in sizes:
            c = rng.choice(K, n, replace=False)
            rows.append(np.concatenate([c, c[: (len(c) + 1) // 2]]) if g != 1 else c)  # the middle group is valid
    lens = np.array([len(r) for r in rows])
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate(rows).astype(np.int32)
    vals = np.ones(cols.size, np.float16)
    vrp, vcol, vval, nvec = gpu_svc(len(rows), K, V, ptr, cols, vals)
    for g in range(0, len(rows), V):
        distinct = np.unique(cols[ptr[g]:ptr[g + V]])
        got = vcol[vrp[g // V]:vrp[g // V + 1]]
        assert np.array_equal(np.sort(got), distinct)
        block = vval[vrp[g // V] * V:vrp[g // V + 1] * V].reshape(-1, V)
        for r in range(V):
            assert np.array_equal(np.sort(got[block[:, r] != 0]), np.unique(rows[g + r]))


@pytest.mark.parametrize("K,order", [(4096, "cpython"), (4096, "sorted"), (300000, "cpython")])
def test_columns_outside_the_matrix_are_ignored(oracle, built_library, K, order):
    """Invalid input (the contract wants 0 <= column < K): such non-zeros are dropped, nothing else changes, and
    no kernel indexes a table with them.  The result is that of the matrix without them."""
    rng = np.random.default_rng(80)
    clean = _random_csr(rng, 96, K, 400)
    rows = []
    for r in range(clean.M):
        c = clean.col_ind[clean.row_ptr[r]:clean.row_ptr[r + 1]]
        bad = rng.choice([-1, -7, K, K + 5, 2**31 - 1, -2**31], size=rng.integers(0, 4)).astype(np.int64)
        merged = np.concatenate([c.astype(np.int64), bad])
        rng.shuffle(merged)
        rows.append(merged)
    lens = np.array([len(x) for x in rows])
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate(rows).astype(np.int32)
    vals = rng.standard_normal(cols.size).astype(np.float16)
    keep = (cols >= 0) & (cols < K)
    kept_ptr = np.concatenate([[0], np.cumsum([keep[ptr[r]:ptr[r + 1]].sum() for r in range(len(rows))])]).astype(np.int32)
    want = oracle.svc(len(rows), K, 8, kept_ptr, cols[keep], vals[keep], order=order)
    vrp, vcol, vval, _ = gpu_svc(len(rows), K, 8, ptr, cols, vals, order)
    assert np.array_equal(vrp, want[0]) and np.array_equal(vcol, want[1])
    assert np.array_equal(vval.view(np.uint16), want[2].view(np.uint16))


def test_calls_from_several_host_threads_on_their_own_streams(oracle, built_library):
    """The helper streams and events of the merge are per device: concurrent callers must not mix their
    fork / join sequences."""
    import threading
    rng = np.random.default_rng(79)
    cases = [_random_csr(rng, 600 + 50 * t, 3000, 900) for t in range(4)]
    want = [oracle.svc(c.M, c.K, 8, c.row_ptr, c.col_ind, c.values) for c in cases]
    errors = []

    def worker(t):
        try:
            c = cases[t]
            with torch.cuda.stream(torch.cuda.Stream()):
                args = (dev(c.row_ptr), dev(c.col_ind), dev(c.values), c.M, c.K, 8)
                for _ in range(8):
                    r = sspmm_amd.svc(*args)
                    torch.cuda.current_stream().synchronize()
                    ok = (np.array_equal(r.vec_row_ptr.cpu().numpy(), want[t][0]) and
                          np.array_equal(r.vec_col.cpu().numpy(), want[t][1]) and
                          np.array_equal(r.vec_val.cpu().numpy().view(np.uint16), want[t][2].view(np.uint16)))
                    if not ok:
                        errors.append("thread %d: mismatch" % t)
        except Exception as e:  # noqa: BLE001
            errors.append("thread %d: %r" % (t, e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_cfg1_rowmerge_returns_the_vector_pattern(oracle, built_library):
    vs = synth.vector_sparse(512, 512, 8, 0.9, seed=1)
    csr = synth.expand_to_csr(vs)
    vrp, vcol, vval, _ = gpu_svc(csr.M, csr.K, 8, csr.row_ptr, csr.col_ind, csr.values, "sorted")
    assert np.array_equal(vrp, vs.row_offsets) and np.array_equal(vcol, vs.col_idx)
    assert np.array_equal(vval.view(np.uint16), vs.values.view(np.uint16))
    _compare_with_oracle(oracle, csr, 8)


def test_cfg4_zipf_16384(oracle, built_library):
    csr = synth.zipf_csr(16384, 16384, seed=4)
    vrp, vcol, vval = _compare_with_oracle(oracle, csr, 8)
    # size-independent properties: densify(svc(A)) == A on sampled groups, nvec <= nnz, counts == distinct columns
    assert vrp[-1] <= csr.col_ind.size
    vv = vval.reshape(-1, 8)
    for g in [0, 1, 777, 2047] + list(np.argsort(np.diff(vrp))[-2:]):
        cols = vcol[vrp[g]:vrp[g + 1]]
        assert len(set(cols.tolist())) == cols.size
        for v in range(8):
            r = g * 8 + v
            b, e = csr.row_ptr[r], csr.row_ptr[r + 1]
            where = {c: p for p, c in enumerate(cols.tolist())}
            dense_row = np.zeros(cols.size, np.float16)
            for c, x in zip(csr.col_ind[b:e].tolist(), csr.values[b:e]):
                dense_row[where[c]] = x
            assert np.array_equal(vv[vrp[g]:vrp[g + 1], v], dense_row)
    _compare_with_oracle(oracle, csr, 16, "sorted")


def test_cfg4_svc_then_spmm_at_full_size(oracle, built_library):
    """cfg4 end to end at its real shape: Zipf CSR 16384^2 -> SVC (GPU) -> SpMM (GPU) against the
    oracle's SpMM on the oracle's SVC output (a pattern with vector-rows from 0 to several thousand vectors)."""
    csr = synth.zipf_csr(16384, 16384, seed=4)
    N = 256
    B = synth.dense_rhs(csr.K, N, seed=14)
    r = sspmm_amd.svc(dev(csr.row_ptr), dev(csr.col_ind), dev(csr.values), csr.M, csr.K, 8)
    for out_dtype, tol in ((torch.float32, 2e-5), (torch.float16, 2e-3)):
        out = sspmm_amd.spmm(None, r.vec_row_ptr, r.vec_col, r.vec_val, dev(B), 8, out_dtype=out_dtype)
        torch.cuda.synchronize()
        vrp, vcol, vval = oracle.svc(csr.M, csr.K, 8, csr.row_ptr, csr.col_ind, csr.values)
        want = oracle.spmm(csr.M // 8, 8, N, csr.K, vrp, vcol, vval, B, threads=8)
        got = out.float().cpu().numpy()
        scale = np.abs(want).max()
        assert np.abs(got - want).max() / scale <= tol


def test_svc_then_spmm_equals_csr_matmul(oracle, built_library):
    """End of the pipe: unstructured CSR -> SVC (GPU) -> SpMM (GPU) == dense(A) @ B."""
    rng = np.random.default_rng(8)
    csr = _random_csr(rng, 128, 200, 30)
    B = synth.dense_rhs(200, 64, seed=8)
    r = sspmm_amd.svc(dev(csr.row_ptr), dev(csr.col_ind), dev(csr.values), csr.M, csr.K, 8)
    out = sspmm_amd.spmm(None, r.vec_row_ptr, r.vec_col, r.vec_val, dev(B), 8, out_dtype=torch.float32)
    torch.cuda.synchronize()
    A = np.zeros((csr.M, csr.K), np.float64)
    for i in range(csr.M):
        A[i, csr.col_ind[csr.row_ptr[i]:csr.row_ptr[i + 1]]] = csr.values[csr.row_ptr[i]:csr.row_ptr[i + 1]]
    want = A @ B.astype(np.float64)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("order", ["cpython", "sorted"])
def test_outputs_sized_by_the_bound_need_no_read_back(oracle, built_library, order):
    """exact_size=False: arrays of nnz vectors, the result in their first nvec entries, and the
    SpMM takes them as they are (every kernel reads the extent from the row offsets)."""
    rng = np.random.default_rng(21)
    csr = _random_csr(rng, 256, 300, 40)
    B = synth.dense_rhs(300, 64, seed=21)
    args = (dev(csr.row_ptr), dev(csr.col_ind), dev(csr.values), csr.M, csr.K, 8)
    exact = sspmm_amd.svc(*args, order=order)
    loose = sspmm_amd.svc(*args, order=order, exact_size=False)
    assert loose.num_vec is None and loose.vec_col.numel() == csr.col_ind.size
    assert loose.vec_val.numel() == csr.col_ind.size * 8
    n = exact.num_vec
    assert torch.equal(loose.vec_row_ptr, exact.vec_row_ptr)
    assert torch.equal(loose.vec_col[:n], exact.vec_col) and torch.equal(loose.vec_val[:n * 8], exact.vec_val)
    want = sspmm_amd.spmm(None, exact.vec_row_ptr, exact.vec_col, exact.vec_val, dev(B), 8, out_dtype=torch.float32)
    for force in (0, 1, 2, 6):
        _lib.lib().sspmm_select_kernel(force)
        try:
            got = sspmm_amd.spmm(None, loose.vec_row_ptr, loose.vec_col, loose.vec_val, dev(B), 8, out_dtype=torch.float32)
        finally:
            _lib.lib().sspmm_select_kernel(0)
        assert torch.allclose(got, want, rtol=0, atol=2e-5 * float(want.abs().max())), force


def test_wide_matrices_and_giant_groups_take_the_64_bit_tables(oracle, built_library):
    """K above 2^17 (column indices too wide for 32-bit table entries) and a group above 19 660 keys
    run the kernels with 64-bit entries, the giant group with its table in the workspace."""
    rng = np.random.default_rng(42)
    K = 300000
    lens = np.zeros(24, np.int64)
    lens[:8] = 3000          # 24 000 distinct columns in one group
    lens[8:16] = [0, 5, 700, 1, 0, 90, 2000, 3]
    lens[16:] = 40
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens]).astype(np.int32)
    csr = synth.Csr(24, K, ptr, cols, rng.standard_normal(cols.size).astype(np.float16))
    _compare_with_oracle(oracle, csr, 8)
    # same shape of groups with narrow columns: the giant group is the only one on 64-bit entries
    K2 = 100000
    cols2 = np.concatenate([np.sort(rng.choice(K2, n, replace=False)) for n in lens]).astype(np.int32)
    _compare_with_oracle(oracle, synth.Csr(24, K2, ptr, cols2, csr.values), 8)
