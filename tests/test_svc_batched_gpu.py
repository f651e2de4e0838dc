"""The SVC of a stack of matrices (svc_count_batched / svc_fill_batched through the C ABI): every matrix of the stack
must come out as it does on its own, bit for bit: against the CPU oracle, the files the reference wrote and the
single-matrix entry points."""
import glob
import os

import numpy as np
import pytest
import torch

import sspmm_amd
from sspmm_amd import formats, synth
from gpu_util import dev

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _random_csr(rng, M, K, max_len):
    lens = rng.integers(0, min(K, max_len) + 1, M)
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([np.sort(rng.permutation(K)[:n]) for n in lens] + [np.zeros(0, np.int64)]).astype(np.int32)
    vals = rng.standard_normal(cols.size).astype(np.float16)
    return synth.Csr(M, K, ptr, cols, vals)


def _run(mats, V, order="cpython", with_values=True):
    host = [(c.M, c.K, c.row_ptr, c.col_ind, c.values if with_values else None) for c in mats]
    mat_rows, K_max, rp, ci, cv = sspmm_amd.stack_csr(host)
    print("stack of %d matrices, rows %d, nnz %d, V=%d %s" % (len(mats), mat_rows[-1], ci.size, V, order), flush=True)
    batch = sspmm_amd.svc_batched(mat_rows, K_max, dev(rp), dev(ci), None if cv is None else dev(cv), V, order=order)
    torch.cuda.synchronize()
    return batch


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("order", ["cpython", "sorted"])
def test_stack_equals_every_matrix_on_its_own(oracle, built_library, V, order):
    """Row counts that are and are not multiples of V (a short last group per matrix), an empty matrix, a matrix of
    empty rows, widths from 8 to 5000 columns, groups in every LDS size class."""
    rng = np.random.default_rng(40 + V)
    shapes = [(64, 512, 80), (13, 33, 20), (1, 8, 8), (0, 100, 0), (40, 5000, 900), (17, 700, 0), (128, 2048, 400),
              (5, 4000, 4000), (24, 512, 512)]
    mats = [_random_csr(rng, M, K, mx) for M, K, mx in shapes]
    batch = _run(mats, V, order)
    host = batch.to_host()
    assert len(host) == len(mats)
    for i, (c, (vrp, vcol, vval)) in enumerate(zip(mats, host)):
        wrp, wcol, wval = oracle.svc(c.M, c.K, V, c.row_ptr, c.col_ind, c.values, order=order)
        assert np.array_equal(vrp, wrp), i
        assert np.array_equal(vcol, wcol), i
        assert np.array_equal(vval.view(np.uint16), wval.view(np.uint16)), i
        view = batch.matrix(i)   # the device views agree with the host copies
        assert np.array_equal(view.vec_row_ptr.cpu().numpy(), wrp) and np.array_equal(view.vec_col.cpu().numpy(), wcol)
        assert view.num_vec == wcol.size


@pytest.mark.parametrize("V", [8, 16])
def test_stack_of_the_reference_written_files(built_library, V):
    """All golden `.smtx` inputs in one stack: each comes back as the CVSE file the reference wrote for it."""
    names = sorted(p for p in glob.glob(os.path.join(GOLDEN, "*.smtx")) if ".v" not in os.path.basename(p))
    mats, meta = [], []
    for p in names:
        M, K, nnz, row_ptr, col_ind = formats.read_smtx(p)
        mats.append(synth.Csr(M, K, row_ptr, col_ind, None))
        meta.append((p, K, nnz))
    batch = _run(mats, V, with_values=False)
    for (p, K, nnz), (vrp, vcol, _v) in zip(meta, batch.to_host()):
        with open(p.replace(".smtx", ".v%d.smtx" % V)) as f:
            assert formats.cvse_text(vrp.size - 1, K, nnz, vrp, vcol) == f.read(), p


def test_stack_matches_the_single_matrix_entry_points(built_library):
    """96 matrices of the dataset's shapes in one call against 96 calls of svc()."""
    rng = np.random.default_rng(7)
    mats = []
    for i in range(24):
        M, K = [(512, 512), (2048, 512), (512, 2048)][i % 3]
        s = [0.5, 0.7, 0.9, 0.98][i % 4]
        mask = rng.random((M, K)) >= s
        ptr = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32)
        mats.append(synth.Csr(M, K, ptr, np.nonzero(mask)[1].astype(np.int32), None))
    batch = _run(mats, 8, with_values=False)
    for c, (vrp, vcol, _v) in zip(mats, batch.to_host()):
        r = sspmm_amd.svc(dev(c.row_ptr), dev(c.col_ind), None, c.M, c.K, 8)
        assert np.array_equal(vrp, r.vec_row_ptr.cpu().numpy())
        assert np.array_equal(vcol, r.vec_col.cpu().numpy())


def test_group_count_the_device_arrives_at(built_library):
    """mat_groups[count] is the device's own count of the groups; a caller that passes another count gets a wrong
    answer it can detect, not a write outside its arrays."""
    from sspmm_amd import _lib
    L = _lib.lib()
    V = 8
    rng = np.random.default_rng(9)
    mats = [_random_csr(rng, M, 64, 10) for M in (9, 16, 3)]
    mat_rows, K_max, rp, ci, cv = sspmm_amd.stack_csr([(c.M, c.K, c.row_ptr, c.col_ind, None) for c in mats])
    groups = 2 + 2 + 1
    d_rows, d_rp, d_ci = dev(mat_rows), dev(rp), dev(ci)
    ws = torch.empty(L.svc_batched_workspace_bytes(3, int(mat_rows[-1]), ci.size, V), dtype=torch.uint8, device="cuda")
    d_groups = torch.full((4,), -1, dtype=torch.int32, device="cuda")
    vrp = torch.full((groups + 1 + 4,), -7, dtype=torch.int32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    assert L.svc_count_batched(3, groups, d_rows.data_ptr(), int(mat_rows[-1]), K_max, V, d_rp.data_ptr(), d_ci.data_ptr(),
                               ci.size, 0, d_groups.data_ptr(), vrp.data_ptr(), ws.data_ptr(), s) == 0
    torch.cuda.synchronize()
    assert d_groups.cpu().tolist() == [0, 2, 4, 5]
    assert torch.all(vrp[groups + 1:] == -7)
    # rejected before anything is launched: more groups than the stack can have, no table
    assert L.svc_count_batched(3, 40, d_rows.data_ptr(), int(mat_rows[-1]), K_max, V, d_rp.data_ptr(), d_ci.data_ptr(),
                               ci.size, 0, d_groups.data_ptr(), vrp.data_ptr(), ws.data_ptr(), s) == 1
    assert L.svc_count_batched(3, groups, None, int(mat_rows[-1]), K_max, V, d_rp.data_ptr(), d_ci.data_ptr(),
                               ci.size, 0, d_groups.data_ptr(), vrp.data_ptr(), ws.data_ptr(), s) == 1


def test_converter_takes_the_files_through_one_stack(built_library, tmp_path):
    from sspmm_amd import rowmerge
    names = sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLDEN, "*.smtx")) if ".v" not in os.path.basename(p))
    stats = rowmerge.convert_files([os.path.join(GOLDEN, n) for n in names], [str(tmp_path / n) for n in names], 8)
    assert len(stats) == len(names)
    for n in names:
        assert (tmp_path / n).read_bytes() == open(os.path.join(GOLDEN, n.replace(".smtx", ".v8.smtx")), "rb").read()
