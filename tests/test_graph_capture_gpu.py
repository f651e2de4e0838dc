"""The entry points enqueue kernels and events only: a caller may record them into a HIP graph.  Every replay is
checked against the eager result, with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

import sspmm_amd
from sspmm_amd import _lib, synth
from gpu_util import dev

pytestmark = pytest.mark.gpu


def _between_replays():
    torch.ones(4096, device="cuda").sum().item()  # eager work and a synchronisation of the program's own


def test_batched_spmm_in_a_graph(built_library):
    L = _lib.lib()
    V, K, N, batch = 8, 512, 256, 16
    vs = synth.vector_sparse(2048, K, V, 0.9, seed=2, std=0.02)
    ro, ci = dev(vs.row_offsets), dev(vs.col_idx)
    g = torch.Generator(device="cuda").manual_seed(5)
    vals = (torch.randn(batch, vs.col_idx.size * V, generator=g, device="cuda") * 0.02).half()
    B = torch.randn(batch, K, N, generator=g, device="cuda").half()
    C = torch.zeros(batch, vs.m_vec * V, N, device="cuda")

    def launch(stream):
        rc = L.sspmm_batched_f16_f32(batch, vs.m_vec, V, N, K, None, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(),
                                     vs.col_idx.size * V, B.data_ptr(), K * N, C.data_ptr(), vs.m_vec * V * N, stream)
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
        _between_replays()


def test_svc_in_a_graph(built_library):
    """svc_count + svc_fill with their fork / join of the helper stream, recorded once and replayed."""
    L = _lib.lib()
    V = 8
    csr = synth.zipf_csr(4096, 4096, seed=4)
    rp, cc, cv = dev(csr.row_ptr), dev(csr.col_ind), dev(csr.values)
    eager = sspmm_amd.svc(rp, cc, cv, csr.M, csr.K, V)
    nnz = csr.col_ind.size
    ws = torch.empty(L.svc_workspace_bytes(csr.M, nnz, V), dtype=torch.uint8, device="cuda")
    vrp = torch.zeros(csr.M // V + 1, dtype=torch.int32, device="cuda")
    vcol = torch.zeros(eager.num_vec, dtype=torch.int32, device="cuda")
    vval = torch.zeros(eager.num_vec * V, dtype=torch.float16, device="cuda")

    def launch(stream):
        rc = L.svc_count(csr.M, csr.K, V, rp.data_ptr(), cc.data_ptr(), nnz, 0, vrp.data_ptr(), ws.data_ptr(), stream)
        assert rc == 0, rc
        rc = L.svc_fill(csr.M, csr.K, V, rp.data_ptr(), cc.data_ptr(), cv.data_ptr(), nnz, 0, vrp.data_ptr(),
                        ws.data_ptr(), vcol.data_ptr(), vval.data_ptr(), stream)
        assert rc == 0, rc

    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        launch(s.cuda_stream)  # creates the helper stream outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        launch(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        vrp.zero_()
        vcol.zero_()
        vval.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(vrp, eager.vec_row_ptr) and torch.equal(vcol, eager.vec_col) and torch.equal(vval, eager.vec_val)
        _between_replays()
