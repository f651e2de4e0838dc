"""The allocation-free entry point (schedule and scratch in a static device array of the library) against the
entry point it is a variant of, the product with a plan."""
import numpy as np
import pytest
import torch

from sspmm_amd import _lib, synth
from sspmm_amd.plan import Plan
from gpu_util import TIGHT_F32, dev, max_rel_err

pytestmark = pytest.mark.gpu


def _pattern(m_vec, K, V, seed, long_rows):
    rng = np.random.default_rng(seed)
    lens = rng.integers(0, 60, m_vec)
    lens[rng.choice(m_vec, long_rows, replace=False)] = rng.integers(500, min(K, 3000), long_rows)
    lens[0] = 0
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(K)[:n] for n in lens]).astype(np.int32)
    vals = (rng.standard_normal(cols.size * V) * 0.1).astype(np.float16)
    return synth.VectorSparse(m_vec * V, K, V, m_vec, off, cols, vals, cols.size * V)


def _both(L, vs, B, N):
    """(allocation-free entry point, product with a plan) on the same operands, through the C ABI."""
    ro, ci, vv, dB = dev(vs.row_offsets), dev(vs.col_idx), dev(vs.values), dev(B)
    stream = torch.cuda.current_stream().cuda_stream
    got = torch.full((vs.m_vec * vs.V, N), 7.0, device="cuda")
    print("noalloc m_vec=%d V=%d K=%d N=%d nvec=%d" % (vs.m_vec, vs.V, vs.K, N, vs.col_idx.size), flush=True)
    rc = L.sspmm_noalloc_f16_f32(vs.m_vec, vs.V, N, vs.K, ro.data_ptr(), ci.data_ptr(), vv.data_ptr(), dB.data_ptr(),
                                 got.data_ptr(), stream)
    assert rc == 0, rc
    plan = Plan(ro, vs.V, vs.K, max_N=N)
    want = torch.full((vs.m_vec * vs.V, N), -7.0, device="cuda")
    rc = L.sspmm_plan_batched_f16_f32(plan.handle, 1, N, ro.data_ptr(), ci.data_ptr(), vv.data_ptr(), 0, dB.data_ptr(), 0,
                                      want.data_ptr(), 0, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    cut = plan.info().cut_rows
    plan.destroy()
    return got, want, cut


@pytest.mark.parametrize("V", [8, 16])
def test_two_calls_in_a_row_the_second_smaller(oracle, built_library, V):
    L = _lib.lib()
    # first call: 300 vector-rows, 24 of them long, four column tiles the last one partial
    big = _pattern(300, 6000, V, seed=V, long_rows=24)
    B1 = synth.dense_rhs(6000, 200, seed=1)
    got1, want1, cut1 = _both(L, big, B1, 200)
    assert cut1 > 0
    assert torch.equal(got1, want1)
    ref1 = oracle.spmm(big.m_vec, V, 200, 6000, big.row_offsets, big.col_idx, big.values, B1, threads=8)
    assert max_rel_err(got1.cpu().numpy(), ref1) <= TIGHT_F32
    # second call: fewer rows, fewer cut rows, one column tile: whatever the first call left in the scratch array
    # (a longer work list, counters, partial tiles) must not show
    small = _pattern(40, 2000, V, seed=100 + V, long_rows=3)
    B2 = synth.dense_rhs(2000, 64, seed=2)
    got2, want2, cut2 = _both(L, small, B2, 64)
    assert 0 < cut2 < cut1
    assert torch.equal(got2, want2)
    ref2 = oracle.spmm(small.m_vec, V, 64, 2000, small.row_offsets, small.col_idx, small.values, B2, threads=8)
    assert max_rel_err(got2.cpu().numpy(), ref2) <= TIGHT_F32
    assert not got2[:V].any()  # the empty first vector-row is written as zeros


@pytest.mark.parametrize("m_vec", [64, 511, 513, 1025, 2049, 4096, 4097, 6000])
def test_row_counts_either_side_of_the_schedule_builders(oracle, built_library, m_vec):
    """Up to 4096 vector-rows the schedule is built from row offsets kept in registers (512 threads x 8), beyond
    that by passes over memory; blocks of 512 or 1024 rows are scanned one after the other."""
    L = _lib.lib()
    vs = _pattern(m_vec, 2500, 8, seed=m_vec, long_rows=19)
    B = synth.dense_rhs(2500, 64, seed=5)
    got, want, cut = _both(L, vs, B, 64)
    assert cut > 0
    assert torch.equal(got, want)
    ref = oracle.spmm(vs.m_vec, 8, 64, 2500, vs.row_offsets, vs.col_idx, vs.values, B, threads=8)
    assert max_rel_err(got.cpu().numpy(), ref) <= TIGHT_F32


def test_budget_doubled_until_the_panels_fit_the_static_scratch(oracle, built_library):
    """With 64 column tiles the static scratch holds 64 partial tiles per column tile: 40 rows of 32 steps in a
    pattern of 200 ask for 3 panels each (120), then 2 (80), and are then left whole."""
    L = _lib.lib()
    rng = np.random.default_rng(77)
    lens = rng.integers(1, 33, 200)
    lens[rng.choice(200, 40, replace=False)] = rng.integers(993, 1025, 40)
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([rng.permutation(1500)[:n] for n in lens]).astype(np.int32)
    vals = (rng.standard_normal(cols.size * 8) * 0.1).astype(np.float16)
    vs = synth.VectorSparse(1600, 1500, 8, 200, off, cols, vals, cols.size * 8)
    B = synth.dense_rhs(1500, 4096, seed=6)
    got, want, cut = _both(L, vs, B, 4096)
    assert cut == 40  # the plan has room for all 120 panels ...
    ref = oracle.spmm(200, 8, 4096, 1500, off, cols, vals, B, threads=8)
    assert max_rel_err(got.cpu().numpy(), ref) <= TIGHT_F32  # ... so the sums differ in their order, not in value
    assert max_rel_err(want.cpu().numpy(), ref) <= TIGHT_F32


def test_sizes_beyond_the_static_scratch_are_rejected(built_library):
    L = _lib.lib()
    one = 1  # rejected calls never dereference their pointers
    too_small = 9001
    assert L.sspmm_noalloc_f16_f32(32769, 8, 64, 64, one, one, one, one, one, None) == too_small
    assert L.sspmm_noalloc_f16_f32(64, 8, 4104, 64, one, one, one, one, one, None) == too_small
    assert b"static scratch" in L.sspmm_error_string(too_small)
    assert L.sspmm_noalloc_f16_f32(64, 4, 64, 64, one, one, one, one, one, None) == 1
    assert L.sspmm_noalloc_f16_f32(0, 8, 64, 64, None, None, None, None, None, None) == 0


def test_two_patterns_recorded_into_one_graph(built_library):
    """The entry point is for callers under graph capture: after one eager call (the array's address is looked up
    outside a capture), two calls with different patterns are recorded on one stream and the graph is replayed several
    times with eager work in between; every replay equals the eager results bit for bit."""
    L = _lib.lib()
    V = 8
    pa = _pattern(300, 6000, V, seed=31, long_rows=24)
    pb = _pattern(90, 3000, V, seed=32, long_rows=5)
    Ba, Bb = dev(synth.dense_rhs(6000, 128, seed=3)), dev(synth.dense_rhs(3000, 64, seed=4))
    arrs = [(p, dev(p.row_offsets), dev(p.col_idx), dev(p.values)) for p in (pa, pb)]

    def call(i, B, N, out, stream):
        p, ro, ci, vv = arrs[i]
        rc = L.sspmm_noalloc_f16_f32(p.m_vec, V, N, p.K, ro.data_ptr(), ci.data_ptr(), vv.data_ptr(), B.data_ptr(),
                                     out.data_ptr(), stream)
        assert rc == 0, rc

    eager = [torch.empty(pa.m_vec * V, 128, device="cuda"), torch.empty(pb.m_vec * V, 64, device="cuda")]
    s0 = torch.cuda.current_stream().cuda_stream
    call(0, Ba, 128, eager[0], s0)
    call(1, Bb, 64, eager[1], s0)
    torch.cuda.synchronize()
    outs = [torch.zeros_like(e) for e in eager]
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        st = torch.cuda.current_stream().cuda_stream
        call(0, Ba, 128, outs[0], st)
        call(1, Bb, 64, outs[1], st)
    for replay in range(4):
        for o in outs:
            o.fill_(float(replay))          # eager work of the program's own between the replays
        call(1, Bb, 64, eager[1], s0)       # ... including a call that leaves another schedule in the array
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(outs[0], eager[0]), replay
        assert torch.equal(outs[1], eager[1]), replay
