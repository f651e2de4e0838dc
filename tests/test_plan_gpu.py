"""Products with a plan: the row-panel schedule that cuts overlong vector-rows into panels processed by
different workgroups, against the CPU oracle and against the product without a plan."""
import numpy as np
import pytest
import torch

import sspmm_amd
from sspmm_amd import _lib, synth
from sspmm_amd.plan import Plan
from gpu_util import PARITY_TOL, TIGHT_F16, TIGHT_F32, dev, max_rel_err

pytestmark = pytest.mark.gpu

BALANCED = 7


def ragged(m_vec, K, V, lens, seed, std=0.1):
    rng = np.random.default_rng(seed)
    lens = np.asarray(lens, dtype=np.int64)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens] + [np.zeros(0, np.int64)]).astype(np.int32)
    vals = (rng.standard_normal(cols.size * V) * std).astype(np.float16)
    return synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols, vals, cols.size * V)


def steps_of(lens):
    lens = np.asarray(lens, dtype=np.int64)
    return np.where(lens > 0, (lens + 31) // 32, 1)


def expected_info(lens, panel_steps=0):
    """The schedule's figures restated from the row lengths (steps of 32 vectors; an empty row is one step)."""
    steps = steps_of(lens)
    total, m_vec = int(steps.sum()), len(steps)
    budget = panel_steps or max(8, -(-total // 512), -(-2 * total // m_vec))
    cut = steps > budget
    panels = int((-(-steps[cut] // budget)).sum())
    return dict(num_vec=int(np.sum(lens)), longest_row_steps=int(steps.max()), total_steps=total, panel_steps=budget,
                cut_rows=int(cut.sum()), panels=panels, items=panels + int((~cut).sum()))


def run(vs, B, out_dtype, plan=None):
    out = sspmm_amd.spmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vs.values), dev(B), vs.V, out_dtype=out_dtype,
                         plan=plan)
    torch.cuda.synchronize()
    return out.cpu().numpy()


SKEWED = [0, 5, 300, 0, 33, 2100, 64, 1, 256, 257, 7, 31, 32, 3000, 12, 0, 95, 640, 20]


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("panel_steps", [0, 1, 3, 8])
@pytest.mark.parametrize("N", [64, 200, 256])
def test_planned_product_matches_the_oracle(oracle, built_library, V, out_dtype, panel_steps, N):
    """Rows of 0 to 3000 vectors (empty, one short of a step, exactly a panel, one more than a panel), every
    panel length from one step up, partial last column tiles."""
    K = 3100
    vs = ragged(len(SKEWED), K, V, SKEWED, seed=V + N)
    B = synth.dense_rhs(K, N, seed=N)
    print("plan case V=%d N=%d panel=%d %s" % (V, N, panel_steps, out_dtype), flush=True)
    plan = Plan(dev(vs.row_offsets), V, K, max_N=N, panel_steps=panel_steps)
    info = plan.info()
    want_info = expected_info(SKEWED, panel_steps)
    for k, v in want_info.items():
        assert getattr(info, k) == v, (k, getattr(info, k), v)
    got = run(vs, B, out_dtype, plan)
    assert _lib.lib().sspmm_last_kernel() == (BALANCED if want_info["cut_rows"] else _lib.lib().sspmm_last_kernel())
    want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vs.values, B, threads=8)
    err = max_rel_err(got, want)
    assert err <= PARITY_TOL and err <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16), err
    for i in np.flatnonzero(np.asarray(SKEWED) == 0):
        assert not got[i * V:(i + 1) * V].any()
    # the same bits from run to run (the partial tiles are added in panel order whichever wave does it), also
    # after the counters have been through a product
    for _ in range(3):
        assert np.array_equal(run(vs, B, out_dtype, plan), got)
    plan.destroy()


@pytest.mark.parametrize("V", [8, 16])
def test_rows_that_are_not_cut_equal_the_staged_gather_kernel_bit_for_bit(oracle, built_library, V):
    """The balanced kernel runs the staged gather kernel's arithmetic: a row that stays whole gets the same bits."""
    K, N = 3100, 264
    vs = ragged(len(SKEWED), K, V, SKEWED, seed=40 + V)
    B = synth.dense_rhs(K, N, seed=41)
    plan = Plan(dev(vs.row_offsets), V, K, max_N=N, panel_steps=8)
    L = _lib.lib()
    got = run(vs, B, torch.float32, plan)
    assert L.sspmm_last_kernel() == BALANCED
    L.sspmm_select_kernel(6)
    try:
        base = run(vs, B, torch.float32)
        assert L.sspmm_last_kernel() == 6
    finally:
        L.sspmm_select_kernel(0)
    cut = steps_of(SKEWED) > 8
    assert cut.any() and not cut.all()
    for i in range(vs.m_vec):
        rows = slice(i * V, (i + 1) * V)
        if cut[i]:
            assert max_rel_err(got[rows], base[rows]) <= TIGHT_F32
        else:
            assert np.array_equal(got[rows], base[rows]), i


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_planned_batch_shares_the_pattern(oracle, built_library, out_dtype):
    V, K, N, batch = 8, 5000, 136, 3
    lens = [40, 0, 1500, 17, 900, 64, 3, 2500, 10]
    vs = ragged(len(lens), K, V, lens, seed=77)
    rng = np.random.default_rng(78)
    vals = (rng.standard_normal((batch, vs.values.size)) * 0.1).astype(np.float16)
    B = rng.standard_normal((batch, K, N)).astype(np.float16)
    plan = Plan(dev(vs.row_offsets), V, K, max_N=N, max_batch=batch)
    assert plan.info().cut_rows > 0
    out = sspmm_amd.bspmm(None, dev(vs.row_offsets), dev(vs.col_idx), dev(vals), dev(B), V, out_dtype=out_dtype, plan=plan)
    torch.cuda.synchronize()
    assert _lib.lib().sspmm_last_kernel() == BALANCED
    out = out.cpu().numpy()
    for b in range(batch):
        want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[b], B[b], threads=8)
        assert max_rel_err(out[b], want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16), b
    # a product wider or larger than the plan was sized for runs without the schedule and is still right
    wide = synth.dense_rhs(K, N + 128, seed=3)
    got = run(vs, wide, out_dtype, plan)
    assert _lib.lib().sspmm_last_kernel() != BALANCED
    want = oracle.spmm(vs.m_vec, V, N + 128, K, vs.row_offsets, vs.col_idx, vs.values, wide, threads=8)
    assert max_rel_err(got, want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16)


@pytest.mark.parametrize("V", [8, 16])
def test_one_plan_many_products_with_changing_operands(oracle, built_library, V):
    """The partial tiles of a product land where the previous product's were: products with different values and
    right-hand sides, enqueued back to back on one plan, each equal to the oracle (a tile or counter left over from
    the product before would show)."""
    K, N = 6000, 256
    rng = np.random.default_rng(9 + V)
    lens = rng.integers(0, 50, 120)
    lens[rng.choice(120, 12, replace=False)] = rng.integers(400, 3000, 12)
    vs = ragged(len(lens), K, V, lens, seed=V)
    ro, ci = dev(vs.row_offsets), dev(vs.col_idx)
    plan = Plan(ro, V, K, max_N=N, panel_steps=2)
    assert plan.info().cut_rows >= 12
    sets = []
    for i in range(4):
        vals = (rng.standard_normal(vs.values.size) * (0.05 * (i + 1))).astype(np.float16)
        B = synth.dense_rhs(K, N, seed=100 + i)
        sets.append((vals, B, dev(vals), dev(B)))
    outs = []
    for rnd in range(3):  # no synchronisation between the twelve products
        for vals, B, dv, dB in sets:
            outs.append(sspmm_amd.spmm(None, ro, ci, dv, dB, V, out_dtype=torch.float32, plan=plan))
    torch.cuda.synchronize()
    wants = [oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals, B, threads=8) for vals, B, _, _ in sets]
    for i, out in enumerate(outs):
        assert max_rel_err(out.cpu().numpy(), wants[i % 4]) <= TIGHT_F32, i
        assert torch.equal(out, outs[i % 4])


def test_even_pattern_keeps_the_kernels_chosen_by_shape(oracle, built_library):
    """No row is much longer than the mean: nothing is cut and the product is the one without a plan, bit for bit."""
    vs = synth.vector_sparse(2048, 512, 8, 0.9, seed=2, std=0.02)
    B = synth.dense_rhs(512, 256, seed=12)
    plan = Plan(dev(vs.row_offsets), 8, 512, max_N=256)
    info = plan.info()
    assert info.cut_rows == 0 and info.panels == 0 and info.items == vs.m_vec and info.num_vec == vs.col_idx.size
    got = run(vs, B, torch.float32, plan)
    assert _lib.lib().sspmm_last_kernel() != BALANCED
    assert np.array_equal(got, run(vs, B, torch.float32))
    # forced, the balanced kernel runs the same rows whole
    L = _lib.lib()
    L.sspmm_select_kernel(BALANCED)
    try:
        forced = run(vs, B, torch.float32, plan)
        assert L.sspmm_last_kernel() == BALANCED
    finally:
        L.sspmm_select_kernel(0)
    want = oracle.spmm(vs.m_vec, 8, 256, 512, vs.row_offsets, vs.col_idx, vs.values, B, threads=8)
    assert max_rel_err(forced, want) <= TIGHT_F32


def test_zipf_matrix_through_svc_and_plan_at_full_size(oracle, built_library):
    """The unstructured 16384 x 16384 configuration end to end: SVC on the GPU, a plan from its row pointer, the
    product against the oracle."""
    V, N = 8, 256
    csr = synth.zipf_csr(16384, 16384, seed=4)
    r = sspmm_amd.svc(dev(csr.row_ptr), dev(csr.col_ind), dev(csr.values), csr.M, csr.K, V)
    plan = Plan(r.vec_row_ptr, V, csr.K, max_N=N)
    info = plan.info()
    lens = np.diff(r.vec_row_ptr.cpu().numpy())
    want_info = expected_info(lens)
    for k, v in want_info.items():
        assert getattr(info, k) == v, (k, getattr(info, k), v)
    assert info.cut_rows > 0
    B = synth.dense_rhs(csr.K, N, seed=14)
    for out_dtype, tol in ((torch.float32, TIGHT_F32), (torch.float16, TIGHT_F16)):
        out = sspmm_amd.spmm(None, r.vec_row_ptr, r.vec_col, r.vec_val, dev(B), V, out_dtype=out_dtype, plan=plan)
        torch.cuda.synchronize()
        assert _lib.lib().sspmm_last_kernel() == BALANCED
        want = oracle.spmm(csr.M // V, V, N, csr.K, r.vec_row_ptr.cpu().numpy(), r.vec_col.cpu().numpy(),
                           r.vec_val.cpu().numpy(), B, threads=8)
        assert max_rel_err(out.cpu().numpy(), want) <= tol


def test_planned_product_in_a_graph(built_library):
    """A product with a plan enqueues one kernel: recorded once, every replay equals the eager result."""
    V, K, N = 8, 4000, 192
    lens = [2000, 3, 0, 700, 45, 1300, 8, 90]
    vs = ragged(len(lens), K, V, lens, seed=5)
    ro, ci, vv, B = dev(vs.row_offsets), dev(vs.col_idx), dev(vs.values), dev(synth.dense_rhs(K, N, seed=6))
    plan = Plan(ro, V, K, max_N=N)
    assert plan.info().cut_rows > 0
    L = _lib.lib()
    C = torch.zeros(vs.m_vec * V, N, device="cuda")

    def launch(stream):
        rc = L.sspmm_plan_batched_f16_f32(plan.handle, 1, N, ro.data_ptr(), ci.data_ptr(), vv.data_ptr(), 0, B.data_ptr(),
                                          0, C.data_ptr(), 0, stream)
        assert rc == 0, rc

    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        launch(s.cuda_stream)
    torch.cuda.synchronize()
    want = C.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        launch(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        C.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, want)
        torch.ones(4096, device="cuda").sum().item()


def test_plan_argument_checks(built_library):
    vs = synth.vector_sparse(64, 128, 8, 0.9, seed=1)
    ro = dev(vs.row_offsets)
    plan = Plan(ro, 8, 128, max_N=64)
    with pytest.raises(ValueError):  # another pattern's shape
        sspmm_amd.spmm(None, ro, dev(vs.col_idx), dev(vs.values), dev(synth.dense_rhs(256, 64, seed=1)), 8, plan=plan)
    plan.destroy()
    with pytest.raises(RuntimeError):
        plan.info()
    empty = Plan(torch.zeros(1, dtype=torch.int32, device="cuda"), 16, 32, max_N=8)
    assert empty.info().items == 0


@pytest.mark.parametrize("M,K,V,sparsity,N,batch,want_plain,want_planned", [
    (1024, 2304, 16, 0.95, 256, 16, 2, 2),   # between the gather kernels the density changes nothing
    (2048, 1024, 16, 0.98, 256, 128, 3, 2),  # one step per row: a gather kernel in place of the slab kernel
    (3072, 768, 8, 0.7, 64, 16, 6, 3),       # dense for this format: the slab kernel from fewer blocks on
    (2048, 512, 8, 0.9, 256, 128, 3, 3),     # the density the thresholds were measured at: no change
    (1024, 2048, 8, 0.7, 256, 32, 2, 5),     # tall and dense: the 32-column slab from half as many vector-rows on
])
def test_plan_of_an_even_pattern_picks_the_kernel_by_density(oracle, built_library, M, K, V, sparsity, N, batch, want_plain,
                                                             want_planned):
    """A plan knows the pattern's vector count; products with it choose between the slab, gather and staged kernels
    by density as well as by shape.  The results agree with the oracle either way."""
    L = _lib.lib()
    vs = synth.vector_sparse(M, K, V, sparsity, seed=M + N, std=0.05)
    g = torch.Generator("cuda").manual_seed(N)
    vals = (torch.randn(batch, vs.col_idx.size * V, device="cuda", generator=g) * 0.05).half()
    B = torch.randn(batch, K, N, device="cuda", generator=g).half()
    ro, ci = dev(vs.row_offsets), dev(vs.col_idx)
    plain = sspmm_amd.bspmm(None, ro, ci, vals, B, V, out_dtype=torch.float32)
    assert L.sspmm_last_kernel() == want_plain
    plan = Plan(ro, V, K, max_N=N, max_batch=batch)
    assert plan.info().cut_rows == 0
    planned = sspmm_amd.bspmm(None, ro, ci, vals, B, V, out_dtype=torch.float32, plan=plan)
    assert L.sspmm_last_kernel() == want_planned
    torch.cuda.synchronize()
    for b in sorted({0, batch - 1}):
        want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[b].cpu().numpy(), B[b].cpu().numpy())
        assert max_rel_err(planned[b].cpu().numpy(), want) <= TIGHT_F32
        assert max_rel_err(plain[b].cpu().numpy(), want) <= TIGHT_F32
    plan.destroy()


def test_many_panels_give_the_same_bits_twenty_times_in_a_row(oracle, built_library):
    """More than 1000 panels over 9 column tiles and 2 batch elements (their partial tiles just fit the plan's 64 MB): the cut rows are added up by whichever wave
    counts itself in last, on whichever XCD it runs, so a hand-over that lets a wave read a partial tile before it
    has arrived shows as a run that differs from the first.  Twenty consecutive products are compared bit for bit
    and the test stops at the first mismatch."""
    V, K, N, batch = 8, 12000, 520, 2
    rng = np.random.default_rng(901)
    lens = rng.integers(0, 40, 600)
    long_rows = rng.choice(600, 150, replace=False)
    lens[long_rows] = rng.integers(900, 3000, 150)
    vs = ragged(len(lens), K, V, lens, seed=902)
    vals = (rng.standard_normal((batch, vs.values.size)) * 0.1).astype(np.float16)
    B = rng.standard_normal((batch, K, N)).astype(np.float16)
    ro, ci, dv, dB = dev(vs.row_offsets), dev(vs.col_idx), dev(vals), dev(B)
    plan = Plan(ro, V, K, max_N=N, max_batch=batch, panel_steps=8)
    info = plan.info()
    assert info.panels >= 1000 and info.cut_rows >= 100, info
    first = None
    for it in range(20):
        out = sspmm_amd.bspmm(None, ro, ci, dv, dB, V, out_dtype=torch.float32, plan=plan)
        torch.cuda.synchronize()
        assert _lib.lib().sspmm_last_kernel() == BALANCED
        if first is None:
            first = out.clone()
        else:
            assert torch.equal(out, first), "run %d differs from the first in %d elements" % (it, int((out != first).sum()))
    # and the first is right: one batch element against the oracle
    want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[1], B[1], threads=8)
    assert max_rel_err(first[1].cpu().numpy(), want) <= TIGHT_F32
    plan.destroy()


@pytest.mark.parametrize("V", [8, 16])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_short_rows_run_in_bundles_with_the_same_bits(oracle, built_library, V, out_dtype):
    """The rows that stay whole are filed in bundles (a wave runs the rows of a bundle as one stream of steps): runs of
    more than 64 one-step rows (a bundle holds at most 64), empty rows at the start, in the middle and at the end of
    bundles, rows of more than half a bundle's steps (bundles of their own), partial last steps, a partial last column
    tile.  Every row that is not cut must equal the staged gather kernel's row bit for bit, and all of it the oracle."""
    K, N = 4000, 200
    rng = np.random.default_rng(31 + V)
    lens = rng.integers(0, 34, 700)
    lens[100:180] = rng.integers(1, 20, 80)          # eighty one-step rows in a row
    lens[300:310] = 0
    lens[rng.choice(700, 40, replace=False)] = rng.integers(130, 330, 40)   # five to eleven steps
    lens[[5, 350, 699]] = [2500, 3100, 1800]         # cut
    lens[[0, 698]] = 0
    vs = ragged(len(lens), K, V, lens, seed=32 + V)
    B = synth.dense_rhs(K, N, seed=33)
    plan = Plan(dev(vs.row_offsets), V, K, max_N=N)
    assert plan.info().cut_rows >= 3
    L = _lib.lib()
    got = run(vs, B, out_dtype, plan)
    assert L.sspmm_last_kernel() == BALANCED
    L.sspmm_select_kernel(6)
    try:
        base = run(vs, B, out_dtype)
        assert L.sspmm_last_kernel() == 6
    finally:
        L.sspmm_select_kernel(0)
    cut = steps_of(lens) > plan.info().panel_steps
    for i in np.flatnonzero(~cut):
        assert np.array_equal(got[i * V:(i + 1) * V], base[i * V:(i + 1) * V]), i
    want = oracle.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vs.values, B, threads=8)
    assert max_rel_err(got, want) <= (TIGHT_F32 if out_dtype == torch.float32 else TIGHT_F16)
    for _ in range(2):
        assert np.array_equal(run(vs, B, out_dtype, plan), got)
    plan.destroy()
