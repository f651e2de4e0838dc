"""Row reordering ahead of the SVC.

The reference's reorder module is not among its sources, so no output of it exists to compare
with: parity against the reference is unpinned for this step.  The CPU statement of the library's
own method (oracle.minhash_order / permute_csr) is checked here by what its definition fixes, and
the GPU path through the C ABI is compared with it bit for bit."""
import os

import numpy as np
import pytest
import torch

from sspmm_amd import synth


def _mix32(x):
    x = np.asarray(x, dtype=np.uint64)
    m = np.uint64(0xffffffff)
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x85ebca6b)) & m
    x ^= x >> np.uint64(13)
    x = (x * np.uint64(0xc2b2ae35)) & m
    x ^= x >> np.uint64(16)
    return x


def _random_csr(rng, M, K, max_len, empty_rows=0.1):
    lens = rng.integers(0, min(K, max_len) + 1, M)
    lens[rng.random(M) < empty_rows] = 0
    rows = [np.unique(rng.integers(0, K, n)) for n in lens]  # distinct, ascending; a few shorter than drawn
    lens = np.array([r.size for r in rows], dtype=np.int64)
    cols = np.concatenate(rows + [np.zeros(0, np.int64)]).astype(np.int32)
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    vals = rng.standard_normal(cols.size).astype(np.float16)
    return synth.Csr(M, K, ptr, cols, vals)


def _union_count(csr, V):
    """nvec of the merged matrix: distinct columns per group of V rows."""
    total = 0
    for g in range(0, csr.M, V):
        total += np.unique(csr.col_ind[csr.row_ptr[g]:csr.row_ptr[min(csr.M, g + V)]]).size
    return total


# ------------------------------------------------------------------ CPU: the oracle itself


def test_mix32_is_a_bijection_on_a_sample():
    x = np.arange(1 << 16, dtype=np.uint64)
    assert np.unique(_mix32(x)).size == x.size
    # murmur3's finaliser maps 0 to 0 and has published avalanche outputs; one known value pins the constants
    assert int(_mix32(np.array([0]))[0]) == 0
    assert int(_mix32(np.array([1]))[0]) == 0x514e28b7


def test_oracle_order_properties(oracle):
    rng = np.random.default_rng(11)
    for M, K, L in [(1, 5, 5), (7, 16, 4), (100, 64, 20), (1000, 4096, 64)]:
        csr = _random_csr(rng, M, K, L)
        perm, keys = oracle.minhash_order(M, csr.row_ptr, csr.col_ind, return_keys=True)
        assert np.array_equal(np.sort(perm), np.arange(M))
        # keys from first principles (vectorised, independent of the C loop), and numpy's stable sort
        want = np.empty(M, dtype=np.uint64)
        for r in range(M):
            c = csr.col_ind[csr.row_ptr[r]:csr.row_ptr[r + 1]].astype(np.uint64)
            h1 = _mix32(c ^ np.uint64(0x9e3779b9)).min() if c.size else np.uint64(0xffffffff)
            h2 = _mix32(c ^ np.uint64(0x7f4a7c15)).min() if c.size else np.uint64(0xffffffff)
            want[r] = (np.uint64(h1) << np.uint64(32)) | np.uint64(h2)
        assert np.array_equal(keys, want)
        assert np.array_equal(perm, np.argsort(keys, kind="stable"))
        # empty rows come last, in source order
        empty = np.flatnonzero(np.diff(csr.row_ptr) == 0)
        assert np.array_equal(perm[M - empty.size:], empty)


def test_oracle_keys_ignore_the_order_of_columns_in_a_row(oracle):
    rng = np.random.default_rng(12)
    csr = _random_csr(rng, 50, 200, 30)
    shuffled = csr.col_ind.copy()
    for r in range(csr.M):
        seg = shuffled[csr.row_ptr[r]:csr.row_ptr[r + 1]]
        rng.shuffle(seg)
    a = oracle.minhash_order(csr.M, csr.row_ptr, csr.col_ind)
    b = oracle.minhash_order(csr.M, csr.row_ptr, shuffled)
    assert np.array_equal(a, b)


def test_oracle_puts_equal_rows_together_and_improves_fill(oracle):
    # exact copies of 13 prototypes: after the reordering every prototype's rows are one contiguous run
    csr = synth.clustered_csr(13 * 24, 512, 13, 40, seed=5, keep=1.0, extras=0)
    perm = oracle.minhash_order(csr.M, csr.row_ptr, csr.col_ind)
    rp, ci, _ = oracle.permute_csr(csr.M, perm, csr.row_ptr, csr.col_ind)
    sig = [tuple(ci[rp[i]:rp[i + 1]]) for i in range(csr.M)]
    runs = 1 + sum(sig[i] != sig[i - 1] for i in range(1, csr.M))
    assert runs == 13
    before = _union_count(csr, 8)
    after = _union_count(synth.Csr(csr.M, csr.K, rp, ci, None), 8)
    assert after * 4 < before  # 24 rows per prototype = 3 full groups of 8: 40 columns instead of up to 320


def test_oracle_permute_csr_is_a_row_gather(oracle):
    rng = np.random.default_rng(13)
    csr = _random_csr(rng, 40, 30, 10)
    perm = rng.permutation(csr.M).astype(np.int32)
    rp, ci, val = oracle.permute_csr(csr.M, perm, csr.row_ptr, csr.col_ind, csr.values)
    for i in range(csr.M):
        s = slice(csr.row_ptr[perm[i]], csr.row_ptr[perm[i] + 1])
        assert np.array_equal(ci[rp[i]:rp[i + 1]], csr.col_ind[s])
        assert np.array_equal(val[rp[i]:rp[i + 1]].view(np.uint16), csr.values[s].view(np.uint16))
    assert rp[-1] == csr.row_ptr[-1]


# ------------------------------------------------------------------ GPU: through the C ABI


def _gpu_order(csr):
    import sspmm_amd
    from gpu_util import dev
    perm = sspmm_amd.minhash_order(dev(csr.row_ptr), dev(csr.col_ind), csr.M)
    torch.cuda.synchronize()
    return perm


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 8, 8), (5, 16, 4), (64, 64, 64), (1000, 512, 100), (4099, 20000, 300),
                                   (70000, 1 << 20, 12)])
def test_gpu_order_matches_the_oracle(built_library, oracle, shape):
    M, K, L = shape
    print("case", shape, flush=True)
    csr = _random_csr(np.random.default_rng(M), M, K, L)
    got = _gpu_order(csr).cpu().numpy()
    assert np.array_equal(got, oracle.minhash_order(M, csr.row_ptr, csr.col_ind))


@pytest.mark.gpu
def test_gpu_order_of_empty_and_all_empty_matrices(built_library, oracle):
    import sspmm_amd
    from gpu_util import dev
    assert sspmm_amd.minhash_order(dev(np.zeros(1, np.int32)), dev(np.zeros(0, np.int32)), 0).numel() == 0
    ptr = np.zeros(301, np.int32)
    got = sspmm_amd.minhash_order(dev(ptr), dev(np.zeros(0, np.int32)), 300).cpu().numpy()
    assert np.array_equal(got, np.arange(300))  # all keys equal: the sort is stable


@pytest.mark.gpu
@pytest.mark.parametrize("with_values", [True, False])
def test_gpu_permute_csr_matches_the_oracle(built_library, oracle, with_values):
    import sspmm_amd
    from gpu_util import dev
    rng = np.random.default_rng(21)
    for M, K, L in [(1, 4, 4), (37, 100, 50), (5000, 3000, 700)]:
        print("case", M, K, L, with_values, flush=True)
        csr = _random_csr(rng, M, K, L)
        perm = rng.permutation(M).astype(np.int32)
        vals = csr.values if with_values else None
        rp, ci, val = sspmm_amd.permute_csr(dev(csr.row_ptr), dev(csr.col_ind), None if vals is None else dev(vals),
                                            dev(perm))
        torch.cuda.synchronize()
        wrp, wci, wval = oracle.permute_csr(M, perm, csr.row_ptr, csr.col_ind, vals)
        assert np.array_equal(rp.cpu().numpy(), wrp)
        assert np.array_equal(ci.cpu().numpy(), wci)
        if with_values:
            assert np.array_equal(val.cpu().numpy().view(np.uint16), wval.view(np.uint16))
        else:
            assert val is None


@pytest.mark.gpu
@pytest.mark.parametrize("V", [8, 16])
def test_reordered_svc_then_spmm_gives_the_permuted_rows(built_library, oracle, V):
    """Clustered rows in shuffled order: the reordering cuts the vector count several times over, and the
    SpMM on the reordered matrix is the SpMM on the source matrix with its output rows in the new order."""
    import sspmm_amd
    from gpu_util import dev
    M, K, N = 2048, 1024, 128
    csr = synth.clustered_csr(M, K, 32, 96, seed=31, keep=0.9, extras=1, std=0.1)
    args = (dev(csr.row_ptr), dev(csr.col_ind), dev(csr.values), M, K, V)
    plain = sspmm_amd.svc(*args, order="sorted")
    r = sspmm_amd.svc_reordered(*args, order="sorted")
    torch.cuda.synchronize()
    perm = r.perm.cpu().numpy()
    assert np.array_equal(perm, oracle.minhash_order(M, csr.row_ptr, csr.col_ind))
    # the merged result is the oracle's merge of the oracle's reordered matrix, bit for bit
    wrp, wci, wval = oracle.permute_csr(M, perm, csr.row_ptr, csr.col_ind, csr.values)
    orp, ocol, oval = oracle.svc(M, K, V, wrp, wci, wval, order="sorted")
    assert np.array_equal(r.svc.vec_row_ptr.cpu().numpy(), orp)
    assert np.array_equal(r.svc.vec_col.cpu().numpy(), ocol)
    assert np.array_equal(r.svc.vec_val.cpu().numpy().view(np.uint16), oval.view(np.uint16))
    print("nvec plain %d reordered %d" % (plain.num_vec, r.svc.num_vec), flush=True)
    assert r.svc.num_vec * 3 < plain.num_vec
    B = dev(synth.dense_rhs(K, N, 32))
    c_plain = sspmm_amd.spmm(None, plain.vec_row_ptr, plain.vec_col, plain.vec_val, B, V, out_dtype=torch.float32)
    c_new = sspmm_amd.spmm(None, r.svc.vec_row_ptr, r.svc.vec_col, r.svc.vec_val, B, V, out_dtype=torch.float32)
    torch.cuda.synchronize()
    want = c_plain[r.perm.long()]
    scale = want.abs().max().item()
    # the same products summed in a different order (the merged column lists differ): fp32 rounding only
    assert (c_new - want).abs().max().item() <= 1e-2 * scale
    dense = np.zeros((M, K), np.float32)
    for i in range(M):
        dense[i, csr.col_ind[csr.row_ptr[i]:csr.row_ptr[i + 1]]] = csr.values[csr.row_ptr[i]:csr.row_ptr[i + 1]]
    ref = dense[perm] @ B.cpu().numpy().astype(np.float32)
    assert np.abs(c_new.cpu().numpy() - ref).max() <= 1e-2 * np.abs(ref).max()


@pytest.mark.gpu
def test_rowmerge_tool_with_reordering(built_library, oracle, tmp_path):
    from sspmm_amd import formats, rowmerge
    csr = synth.clustered_csr(256, 300, 8, 30, seed=41)
    src, dst = tmp_path / "src", tmp_path / "dst"
    os.makedirs(src)
    formats.write_smtx(str(src / "a.smtx"), csr.M, csr.K, csr.row_ptr, csr.col_ind)
    (tmp_path / "paths.txt").write_text("a.smtx\n")
    rows = rowmerge.generate_cvse_files(str(src), str(dst), str(tmp_path / "paths.txt"), 8, reorder=True)
    perm = np.array((dst / "a.smtx.perm").read_text().split(), dtype=np.int32)
    assert np.array_equal(perm, oracle.minhash_order(csr.M, csr.row_ptr, csr.col_ind))
    wrp, wci, _ = oracle.permute_csr(csr.M, perm, csr.row_ptr, csr.col_ind)
    orp, ocol, _ = oracle.svc(csr.M, csr.K, 8, wrp, wci, None, order="cpython")
    assert (dst / "a.smtx").read_text() == formats.cvse_text(len(orp) - 1, csr.K, csr.col_ind.size, orp, ocol)
    assert int(rows[0][3]) == csr.col_ind.size
