#!/usr/bin/env python3
"""Benchmark of the SVC -> SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE short JSON line (the contract keys, roofline, cpu_baseline and a dozen scalars) and writes every figure of
the run to bench_extra.json in the working directory (--extras-file).  A "step" is one pass of the SpMM over one batch of synthetic inputs
already resident in HBM: the FFN-shaped configuration (A 2048x512 fp16, V=8, 90 % vector
sparsity, B 512x256 fp16, C fp32), run bspmm-style over a batch of independent value / B / C
sets that share the pattern, so that one launch moves more bytes than the last-level cache
holds.  `value` is useful TFLOP/s = 2 * nnz * N * batch / t (the reference's convention,
SSpMM/sspmm_test.cpp:197, with nnz the scalar non-zeros).

`roofline` prices the SpMM kernel against the 8 TB/s HBM peak with the algorithmic bytes of one
launch (every operand read once, C written once).  `cpu_baseline` times the CPU oracle (a port of
the reference's host loop) on one batch element, single thread.  `extra` carries every other
benchmark configuration as single launches (mean, median and minimum launch time, the dense GEMM
of the same shape beside each), the SVC against the Python RowMerge, the encoder layer and the
sparse attention block.

    python bench.py --only NAME[,NAME...]   runs just those entries of `extra` (what the profiles/ summaries use)
    python bench.py --list                  prints their names
"""
import argparse
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
def measured_traffic(profiles_dir=None):
    """HBM bytes per launch from hardware counters, read from the summaries under profiles/: every line of the form
        traffic: entry=<benchmark entry> kernel=<kernel> fetch_mb=<F> write_mb=<W> [l2_request_mb=<R>] alg_mb=<A>
    (FETCH_SIZE and WRITE_SIZE of separate rocprofv3 runs, each scaled by its reading of a plain 256 MiB copy; measured
    in runs of their own, not in this one).  Returns entry -> {kernel, bytes, alg_bytes, l2_request_bytes, source}."""
    d = profiles_dir or os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")
    table = {}
    if not os.path.isdir(d):
        return table
    for fn in sorted(os.listdir(d)):
        if not fn.endswith(".txt"):
            continue
        with open(os.path.join(d, fn)) as f:
            for ln in f:
                if not ln.startswith("traffic:"):
                    continue
                kv = dict(p.split("=", 1) for p in ln[len("traffic:"):].split() if "=" in p)
                try:
                    row = {"kernel": kv["kernel"], "bytes": (float(kv["fetch_mb"]) + float(kv["write_mb"])) * 1e6,
                           "alg_bytes": float(kv["alg_mb"]) * 1e6, "source": "profiles/" + fn}
                    if "l2_request_mb" in kv:
                        row["l2_request_bytes"] = float(kv["l2_request_mb"]) * 1e6
                    table[kv["entry"]] = row
                except (KeyError, ValueError):
                    continue
    return table


KERNEL_NAMES = {1: "spmm_generic_kernel", 2: "spmm_gather_kernel", 3: "spmm_slab_kernel<*,4>", 4: "spmm_gather_split_kernel",
                5: "spmm_slab_kernel<*,2>", 6: "spmm_stage_kernel", 7: "spmm_balanced_kernel", 9: "spmm_slab_kernel<*,8>"}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The chip needs a few hundred launches (tens of milliseconds) under this load before its clocks settle: launch
    # times start near 58 us, rise to 70-80 us and come back to 57-59 us after about 500 launches.  The default
    # warm-up covers that transient, so that the timed steps measure the sustained rate; the series of chunk
    # averages through warm-up and timed steps is reported as extra.headline_us_per_chunk.
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--batch", type=int, default=128, help="independent value/B/C sets per step")
    ap.add_argument("--quick", action="store_true", help="skip the extra configurations and CPU legs")
    ap.add_argument("--only", default="", help="comma-separated names of extra entries: run only those and print them")
    ap.add_argument("--list", action="store_true", help="print the names --only accepts")
    ap.add_argument("--attention-only", action="store_true",
                    help="run only the sparse attention block (same as --only sparse_attention_seq4096_d64_v8_s0.9_heads48)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (its hardware-counter readings calibrate FETCH_SIZE / "
                         "WRITE_SIZE when the run is profiled)")
    ap.add_argument("--extras-file", default="bench_extra.json",
                    help="where the full dictionary of figures is written (the line on stdout is a short summary of it)")
    ap.add_argument("--kernel", choices=["auto", "generic", "gather", "slab", "slab128"], default="auto",
                    help="force one SpMM kernel (tuning); the default lets the library choose")
    return ap.parse_args()


def time_launches(fn, steps, warmup, series=None, stats=None):
    """Average milliseconds per call over `steps` calls, HIP events on the launch stream.  `stats`, a dict, receives
    the median and the minimum of the averages over chunks of ten launches."""
    import torch
    chunk = 10
    marks = []

    def run(n, keep):
        for i in range(n):
            if keep and i % chunk == 0:
                ev = torch.cuda.Event(enable_timing=True)
                ev.record()
                marks.append((ev, min(chunk, n - i)))
            fn()

    run(warmup, series is not None)
    torch.cuda.synchronize()
    n_warm = len(marks)
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    run(steps, True)
    end.record()
    torch.cuda.synchronize()
    bounds = [m[0] for m in marks] + [end]
    per_chunk = [ev.elapsed_time(bounds[i + 1]) / n for i, (ev, n) in enumerate(marks)]
    if series is not None:
        # (microseconds per launch for every chunk of 10 launches; the chunk that ends the warm-up runs into the host
        # synchronisation and is left out)
        for i, v in enumerate(per_chunk):
            series.append(v * 1e3 if i != n_warm - 1 else None)
    if stats is not None:
        timed = sorted(per_chunk[n_warm:])
        stats["ms_median"] = timed[len(timed) // 2]
        stats["ms_min"] = timed[0]
    return start.elapsed_time(end) / steps


def graph_time(fn, launches=20, replays=20):
    """Milliseconds per launch when `launches` of them are recorded into one HIP graph and the graph is replayed:
    the host's cost of enqueueing a launch is out of the picture."""
    import torch
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        fn(s.cuda_stream)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        for _ in range(launches):
            fn(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        g.replay()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        g.replay()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / (launches * replays)


def figures(ms, alg_bytes, flops):
    return {"ms": ms, "useful_tflops": flops / ms / 1e9, "alg_bytes": alg_bytes, "hbm_gbps": alg_bytes / ms / 1e6,
            "hbm_frac": alg_bytes / ms / 1e6 / HBM_PEAK_GBPS}


def spmm_case(L, torch, synth, M, K, V, sparsity, N, batch, out_f32, std, seed, steps, warmup, dense=False, series=None,
              plan=False, graph=False, vs=None, handles_out=None):
    """Times one SpMM configuration (a seeded vector-sparse pattern unless `vs` is given); returns a dict of figures."""
    from sspmm_amd.plan import Plan
    if vs is None:
        vs = synth.vector_sparse(M, K, V, sparsity, seed=seed, std=std)
    g = torch.Generator(device="cuda").manual_seed(seed)
    ro = torch.from_numpy(vs.row_offsets).cuda()
    ci = torch.from_numpy(vs.col_idx).cuda()
    nv = vs.col_idx.size
    vals = (torch.randn(batch, nv * V, generator=g, device="cuda") * std).half()
    B = torch.randn(batch, K, N, generator=g, device="cuda").half()
    C = torch.empty(batch, vs.m_vec * V, N, dtype=torch.float32 if out_f32 else torch.float16, device="cuda")
    the_plan = Plan(ro, V, K, max_N=N, max_batch=batch) if plan else None
    if the_plan is not None:
        fn = L.sspmm_plan_batched_f16_f32 if out_f32 else L.sspmm_plan_batched_f16_f16
    else:
        fn = L.sspmm_batched_f16_f32 if out_f32 else L.sspmm_batched_f16_f16

    def launch_on(stream):
        if the_plan is not None:
            rc = fn(the_plan.handle, batch, N, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(), nv * V, B.data_ptr(), K * N,
                    C.data_ptr(), vs.m_vec * V * N, stream)
        else:
            rc = fn(batch, vs.m_vec, V, N, K, None, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(), nv * V, B.data_ptr(),
                    K * N, C.data_ptr(), vs.m_vec * V * N, stream)
        if rc:
            raise RuntimeError("sspmm failed: %d" % rc)

    stream = torch.cuda.current_stream().cuda_stream
    stats = {}
    ms = time_launches(lambda: launch_on(stream), steps, warmup, series, stats)
    bytes_alg = batch * synth.spmm_algorithmic_bytes(vs.m_vec, V, nv, K, N, 4 if out_f32 else 2) \
        - (batch - 1) * (4 * nv + 4 * (vs.m_vec + 1))  # the pattern is shared by the batch
    flops = 2.0 * vs.nnz * N * batch
    out = {"workload": "A %dx%d V=%d s=%.2f, B %dx%d, C %s, batch %d%s" % (
        vs.m_vec * V, K, V, sparsity, K, N, "fp32" if out_f32 else "fp16", batch, ", with a plan" if plan else "")}
    out.update(figures(ms, bytes_alg, flops))
    out.update(stats)
    out["hbm_frac_at_min"] = bytes_alg / stats["ms_min"] / 1e6 / HBM_PEAK_GBPS
    out["kernel"] = KERNEL_NAMES.get(L.sspmm_last_kernel(), "unknown")
    out["gather_bytes_no_reuse"] = batch * 2 * nv * N
    if graph:
        gms = graph_time(launch_on)
        out["ms_in_a_graph"] = gms
        out["hbm_frac_in_a_graph"] = bytes_alg / gms / 1e6 / HBM_PEAK_GBPS
        # a plain device copy that moves the same number of bytes (half read, half written), replayed from a graph
        # like the launch above: what one launch of this size can reach at all, start-up and drain included
        src = torch.empty(bytes_alg // 2, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        cms = graph_time(lambda s_: dst.copy_(src))
        out["plain_copy_of_the_same_bytes_ms_in_a_graph"] = cms
        out["time_vs_plain_copy_of_the_same_bytes_in_a_graph"] = gms / cms
        del src, dst
    if dense:
        A = torch.zeros(vs.m_vec * V, K, dtype=torch.float16, device="cuda")
        Ad = A.unsqueeze(0).expand(batch, -1, -1).contiguous()
        dms = time_launches(lambda: torch.bmm(Ad, B), max(10, steps // 4), 3)
        out["dense_gemm_ms"] = dms
        out["dense_gemm_effective_tflops"] = flops / dms / 1e9
        out["speedup_vs_dense"] = dms / ms
        del A, Ad
    if handles_out is not None:
        handles_out.extend([vs, vals, B, C])
    if the_plan is not None:
        out["plan"] = the_plan.info()._asdict()
        the_plan.destroy()
    return out


def attention_block(torch, synth, sspmm_amd, st, wu):
    """Times the three steps of the reference's sparse attention block, one by one and as the one launch that stands
    for the chain; returns a dict of figures."""
    # the sparse attention block of the reference (bsddmm -> bcsr_softmax -> bspmm) on one mask shared by
    # 48 heads: 4096 tokens, head size 64, V=8, 90 % of the vectors masked out
    seqA, dA, VA, bA = 4096, 64, 8, 48
    mk_a = synth.vector_sparse(seqA, seqA, VA, 0.9, seed=7)
    offA, colA = torch.from_numpy(mk_a.row_offsets).cuda(), torch.from_numpy(mk_a.col_idx).cuda()
    qA, kA, vA = (torch.randn(bA, seqA, dA, device="cuda").half() for _ in range(3))
    nvA = mk_a.col_idx.size
    wA = sspmm_amd.bsddmm(None, offA, colA, qA, kA, VA)
    pA = sspmm_amd.bcsr_softmax(None, offA, wA, 0.125, VA, bA)
    t_sddmm = time_launches(lambda: sspmm_amd.bsddmm(None, offA, colA, qA, kA, VA), st, wu)
    t_soft = time_launches(lambda: sspmm_amd.bcsr_softmax(None, offA, wA, 0.125, VA, bA), st, wu)
    t_av = time_launches(lambda: sspmm_amd.bspmm(None, offA, colA, pA, vA, VA), st, wu)
    t_dense = time_launches(lambda: torch.nn.functional.scaled_dot_product_attention(qA, kA, vA), max(5, st // 10), 2)
    t_one = time_launches(lambda: sspmm_amd.fused_sparse_attention(None, offA, colA, qA, kA, vA, 0.125, VA), st, wu)
    chain = sspmm_amd.bspmm(None, offA, colA, pA, vA, VA).float()
    one = sspmm_amd.fused_sparse_attention(None, offA, colA, qA, kA, vA, 0.125, VA).float()
    by_one = bA * 4 * 2 * seqA * dA + 4 * nvA + 4 * (mk_a.m_vec + 1)   # q, k, v read and the output written, once each
    # the same block on a V = 16 mask of the same sparsity: every gathered row of k and v serves 16 queries instead of 8
    mk16 = synth.vector_sparse(seqA, seqA, 16, 0.9, seed=7)
    off16, col16 = torch.from_numpy(mk16.row_offsets).cuda(), torch.from_numpy(mk16.col_idx).cuda()
    t_one16 = time_launches(lambda: sspmm_amd.fused_sparse_attention(None, off16, col16, qA, kA, vA, 0.125, 16), st, wu)
    by_sddmm = bA * (2 * seqA * dA * 2 + 2 * nvA * VA) + 4 * nvA + 4 * (mk_a.m_vec + 1)
    by_soft = bA * 2 * 2 * nvA * VA + 4 * (mk_a.m_vec + 1)
    by_av = bA * (2 * nvA * VA + 2 * seqA * dA + 2 * seqA * dA) + 4 * nvA + 4 * (mk_a.m_vec + 1)
    res = {
        "bsddmm_ms": t_sddmm, "bsddmm_hbm_frac": by_sddmm / t_sddmm / 1e6 / HBM_PEAK_GBPS, "bsddmm_alg_bytes": by_sddmm,
        "bcsr_softmax_ms": t_soft, "bcsr_softmax_hbm_frac": by_soft / t_soft / 1e6 / HBM_PEAK_GBPS,
        "bcsr_softmax_alg_bytes": by_soft,
        "bspmm_ms": t_av, "bspmm_hbm_frac": by_av / t_av / 1e6 / HBM_PEAK_GBPS, "bspmm_alg_bytes": by_av,
        "block_ms": t_sddmm + t_soft + t_av, "dense_sdpa_ms": t_dense, "nvec": int(nvA),
        "one_launch_ms": t_one, "one_launch_alg_bytes": by_one, "one_launch_hbm_frac": by_one / t_one / 1e6 / HBM_PEAK_GBPS,
        # rows of k and of v fetched from the caches, 128 bytes per stored vector each: what bounds the launch
        "one_launch_gathered_tb_per_s": bA * 2 * nvA * 2 * dA / t_one / 1e9,
        "one_launch_speedup_vs_three": (t_sddmm + t_soft + t_av) / t_one,
        "one_launch_v16_mask_ms": t_one16, "one_launch_v16_mask_gathered_tb_per_s": bA * 2 * mk16.col_idx.size * 2 * dA / t_one16 / 1e9,
        "one_launch_max_rel_err_vs_three": float((one - chain).abs().max() / chain.abs().max()),
    }
    del qA, kA, vA, wA, pA
    return res


# ---- the entries of `extra` ------------------------------------------------------------------------------------------

def single_launch_cases(batch):
    """name -> arguments of spmm_case: every benchmark configuration as one launch (and the batched forms)."""
    cases = {}
    for (M, K) in ((2048, 512), (512, 2048)):
        for s in (0.7, 0.9, 0.98):
            cases["cfg2_%dx%d_v8_s%g_n256" % (M, K, s)] = dict(M=M, K=K, V=8, sparsity=s, N=256, batch=1, out_f32=True,
                                                               std=0.02, seed=2)
    # the other points of cfg2's grid as batched launches (the headline is 2048x512 at 0.9): where the format stops
    # paying against the dense GEMM shows here, not in the latency-bound single products
    for (M, K) in ((2048, 512), (512, 2048)):
        for s in (0.7, 0.9, 0.98):
            if (M, K, s) != (2048, 512, 0.9):
                cases["cfg2_%dx%d_v8_s%g_batched" % (M, K, s)] = dict(M=M, K=K, V=8, sparsity=s, N=256, batch=batch,
                                                                      out_f32=True, std=0.02, seed=2)
    # cfg2's shapes at N = 512, the width of the reference's published sweep (SSpMM/Makefile_ampere:55-60)
    for (M, K) in ((2048, 512), (512, 2048), (2048, 2048)):
        cases["dlmc_shape_%dx%d_v8_s0.9_n512_batched" % (M, K)] = dict(M=M, K=K, V=8, sparsity=0.9, N=512, batch=batch // 2,
                                                                       out_f32=False, std=0.02, seed=2)
    cases["cfg2_batched_fp16_out"] = dict(M=2048, K=512, V=8, sparsity=0.9, N=256, batch=batch, out_f32=False, std=0.02, seed=2)
    cases["cfg2_shape_v16_batched"] = dict(M=2048, K=512, V=16, sparsity=0.9, N=256, batch=batch, out_f32=True, std=0.02, seed=2)
    cases["cfg2_shape_v16_batched_fp16_out"] = dict(M=2048, K=512, V=16, sparsity=0.9, N=256, batch=batch, out_f32=False,
                                                    std=0.02, seed=2)
    for (M, K) in ((1024, 2304), (2048, 1024)):
        for s in (0.8, 0.95):
            for N in (256, 3136):
                cases["cfg3_%dx%d_v16_s%g_n%d" % (M, K, s, N)] = dict(M=M, K=K, V=16, sparsity=s, N=N, batch=1, out_f32=True,
                                                                      std=0.05, seed=3)
    for name, (M, K, seed) in (("q", (768, 768, 51)), ("ffn1", (3072, 768, 55)), ("ffn2", (768, 3072, 56))):
        cases["cfg5_%s_%dx%d_v16_s0.9_n4096" % (name, M, K)] = dict(M=M, K=K, V=16, sparsity=0.9, N=4096, batch=1,
                                                                    out_f32=False, std=0.02, seed=seed)
    cases["cfg5_ffn1_batched8"] = dict(M=3072, K=768, V=16, sparsity=0.9, N=4096, batch=8, out_f32=False, std=0.02, seed=55)
    return cases


def run_cfg1(L, torch, synth, sspmm_amd, O, st, wu):
    """The CPU-runnable configuration end to end on both sides: RowMerge then SpMM of a 512x512 matrix (V=8, 90 %),
    B 512x256.  GPU: svc_count + svc_fill + sspmm_f16_f32 (kernels only, outputs sized beforehand).  CPU: the Python
    RowMerge (list(set(...)) per member row, the reference's algorithm) and the host loop in C, single thread."""
    V, K, N = 8, 512, 256
    vs = synth.vector_sparse(512, K, V, 0.9, seed=1)
    csr = synth.expand_to_csr(vs)
    Bh = synth.dense_rhs(K, N, seed=11)
    rp, ci, cv, B = (torch.from_numpy(x).cuda() for x in (csr.row_ptr, csr.col_ind, csr.values, Bh))
    nnz = csr.col_ind.size
    r = sspmm_amd.svc(rp, ci, cv, csr.M, csr.K, V)
    ws = torch.empty(L.svc_workspace_bytes(csr.M, nnz, V), dtype=torch.uint8, device="cuda")
    vrp = torch.zeros(csr.M // V + 1, dtype=torch.int32, device="cuda")
    vcol = torch.empty(r.num_vec, dtype=torch.int32, device="cuda")
    vval = torch.empty(r.num_vec * V, dtype=torch.float16, device="cuda")
    C = torch.empty(csr.M, N, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def svc_only():
        assert L.svc_count(csr.M, K, V, rp.data_ptr(), ci.data_ptr(), nnz, 0, vrp.data_ptr(), ws.data_ptr(), stream) == 0
        assert L.svc_fill(csr.M, K, V, rp.data_ptr(), ci.data_ptr(), cv.data_ptr(), nnz, 0, vrp.data_ptr(), ws.data_ptr(),
                          vcol.data_ptr(), vval.data_ptr(), stream) == 0

    def spmm_only():
        assert L.sspmm_f16_f32(csr.M // V, V, N, K, None, vrp.data_ptr(), vcol.data_ptr(), vval.data_ptr(), B.data_ptr(),
                               C.data_ptr(), stream) == 0

    def pipeline():
        svc_only()
        spmm_only()

    pipeline()
    torch.cuda.synchronize()
    t_svc, t_spmm, t_pipe = (time_launches(f, st, wu) for f in (svc_only, spmm_only, pipeline))
    lists = O.csr_col_lists(csr.M, csr.row_ptr, csr.col_ind)
    py = []
    for _ in range(5):
        t0 = time.perf_counter()
        ptr, flat = O.rowmerge_python(csr.M, V, lists)
        py.append((time.perf_counter() - t0) * 1e3)
    wrp, wcol, wval = O.svc(csr.M, K, V, csr.row_ptr, csr.col_ind, csr.values)
    t0, reps = time.perf_counter(), 0
    while reps < 50 and (time.perf_counter() - t0 < 2.0 or reps < 3):
        want = O.spmm(csr.M // V, V, N, K, wrp, wcol, wval, Bh, threads=1)
        reps += 1
    cpu_spmm_ms = (time.perf_counter() - t0) * 1e3 / reps
    same = vrp.cpu().numpy().tolist() == ptr and vcol.cpu().numpy().tolist() == flat
    err = float(np.abs(C.cpu().numpy() - want).max() / np.abs(want).max())
    nv = int(r.num_vec)
    by = synth.spmm_algorithmic_bytes(csr.M // V, V, nv, K, N, 4)
    res = {"workload": "CSR 512x512 (V=8 vectors, 90 %% sparse, nnz %d) -> SVC -> SpMM with B 512x256, C fp32" % nnz,
           "gpu_svc_ms": t_svc, "gpu_spmm_ms": t_spmm, "gpu_pipeline_ms": t_pipe,
           "cpu_python_rowmerge_ms_samples": py, "cpu_python_rowmerge_ms": sorted(py)[len(py) // 2],
           "cpu_host_spmm_ms": cpu_spmm_ms, "cpu_cores": 1,
           "cpu_pipeline_ms": sorted(py)[len(py) // 2] + cpu_spmm_ms,
           "svc_bit_exact_vs_python": bool(same), "spmm_max_rel_err_vs_host_loop": err}
    res["speedup_pipeline"] = res["cpu_pipeline_ms"] / t_pipe
    res["svc_speedup_vs_python_one_matrix_per_call"] = res["cpu_python_rowmerge_ms"] / t_svc
    # one such matrix is three launches and a chain of LDS round trips on an idle chip; the reference's job is a
    # dataset of them, so: 96 matrices of this configuration (seeds 1 .. 96) as one stack through svc_batched
    many = [synth.expand_to_csr(synth.vector_sparse(512, K, V, 0.9, seed=s)) for s in range(1, 97)]
    mat_rows, K_max, s_rp, s_ci, _ = sspmm_amd.stack_csr([(c.M, c.K, c.row_ptr, c.col_ind, None) for c in many])
    d_rp, d_ci = torch.from_numpy(s_rp).cuda(), torch.from_numpy(s_ci).cuda()
    t_stack = time_launches(lambda: sspmm_amd.svc_batched(mat_rows, K_max, d_rp, d_ci, None, V), 20, 3)
    lists96 = [O.csr_col_lists(c.M, c.row_ptr, c.col_ind) for c in many]
    t0 = time.perf_counter()
    want96 = [O.rowmerge_python(c.M, V, l) for c, l in zip(many, lists96)]
    py96 = (time.perf_counter() - t0) * 1e3
    got96 = sspmm_amd.svc_batched(mat_rows, K_max, d_rp, d_ci, None, V).to_host()
    res["svc_stack_of_96_such_matrices"] = {
        "gpu_ms": t_stack, "gpu_ms_per_matrix": t_stack / 96, "python_rowmerge_ms": py96,
        "speedup_vs_python": py96 / t_stack,
        "bit_exact_vs_python": bool(all(g[0].tolist() == w[0] and g[1].tolist() == w[1] for g, w in zip(got96, want96)))}
    res["spmm"] = figures(t_spmm, by, 2.0 * vs.nnz * N)
    return res


def run_cfg4(L, torch, synth, sspmm_amd, O, st, wu):
    """The unstructured configuration: SVC of a 16384^2 Zipf CSR matrix (both column orders) against the Python
    RowMerge and the C oracle, and the SpMM that consumes its output, without and with a plan."""
    from sspmm_amd.plan import Plan
    V = 8
    csr = synth.zipf_csr(16384, 16384, seed=4)
    rp, ci, cv = (torch.from_numpy(x).cuda() for x in (csr.row_ptr, csr.col_ind, csr.values))
    nnz = csr.col_ind.size
    r = sspmm_amd.svc(rp, ci, cv, csr.M, csr.K, V)
    torch.cuda.synchronize()
    svc_ms = time_launches(lambda: sspmm_amd.svc(rp, ci, cv, csr.M, csr.K, V), 20, 3)
    # the operator as a whole with outputs sized for nvec <= nnz: allocation, no read-back, nothing waits for the device
    svc_loose_ms = time_launches(lambda: sspmm_amd.svc(rp, ci, cv, csr.M, csr.K, V, exact_size=False), 20, 3)
    # kernels only (no allocation, no host read-back): outputs sized beforehand
    ws = torch.empty(L.svc_workspace_bytes(csr.M, nnz, V), dtype=torch.uint8, device="cuda")
    vrp = torch.zeros(csr.M // V + 1, dtype=torch.int32, device="cuda")
    vcol = torch.empty(r.num_vec, dtype=torch.int32, device="cuda")
    vval = torch.empty(r.num_vec * V, dtype=torch.float16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def svc_kernels(order):
        def f():
            assert L.svc_count(csr.M, csr.K, V, rp.data_ptr(), ci.data_ptr(), nnz, order, vrp.data_ptr(), ws.data_ptr(), stream) == 0
            assert L.svc_fill(csr.M, csr.K, V, rp.data_ptr(), ci.data_ptr(), cv.data_ptr(), nnz, order, vrp.data_ptr(),
                              ws.data_ptr(), vcol.data_ptr(), vval.data_ptr(), stream) == 0
        return f

    st_k = {}
    svc_k_ms = time_launches(svc_kernels(0), 30, 5, stats=st_k)
    svc_sorted_ms = time_launches(svc_kernels(1), 30, 5)
    sorted_cols = vcol.cpu().numpy()
    lists = O.csr_col_lists(csr.M, csr.row_ptr, csr.col_ind)
    py = []
    for _ in range(3):
        t0 = time.perf_counter()
        ptr, flat = O.rowmerge_python(csr.M, V, lists)
        py.append((time.perf_counter() - t0) * 1e3)
    py_ms = sorted(py)[1]
    t0 = time.perf_counter()
    O.svc(csr.M, csr.K, V, csr.row_ptr, csr.col_ind, csr.values)
    c_ms = (time.perf_counter() - t0) * 1e3
    same = (r.vec_row_ptr.cpu().numpy().tolist() == ptr) and (r.vec_col.cpu().numpy().tolist() == flat)
    off_h = r.vec_row_ptr.cpu().numpy()
    sorted_ok = all(np.array_equal(sorted_cols[off_h[i]:off_h[i + 1]], np.sort(np.asarray(flat[off_h[i]:off_h[i + 1]])))
                    for i in range(0, csr.M // V, 64))
    svc_bytes = synth.svc_algorithmic_bytes(csr.M, nnz, csr.M // V, r.num_vec, V)
    out = {"svc_cfg4_zipf_16384_v8": {
        "gpu_ms_with_alloc_and_readback": svc_ms, "gpu_ms_with_alloc_sized_by_nnz_no_readback": svc_loose_ms,
        "speedup_vs_python_sized_by_nnz_no_readback": py_ms / svc_loose_ms,
        "gpu_ms_kernels": svc_k_ms, "gpu_ms_kernels_median": st_k["ms_median"],
        "gpu_ms_kernels_min": st_k["ms_min"], "gpu_ms_kernels_sorted_order": svc_sorted_ms,
        "python_rowmerge_ms_samples": py, "python_rowmerge_ms": py_ms, "c_oracle_ms": c_ms,
        "speedup_vs_python": py_ms / svc_k_ms, "speedup_vs_python_with_alloc_and_readback": py_ms / svc_ms,
        "speedup_vs_python_sorted_order": py_ms / svc_sorted_ms, "bit_exact_vs_python": bool(same),
        "sorted_order_is_the_sorted_python_rows": bool(sorted_ok),
        "nnz": int(nnz), "nvec": int(r.num_vec), "fill_ratio": nnz / (r.num_vec * 8.0),
        "max_vector_row": int(np.diff(off_h).max()), "alg_bytes": svc_bytes, "hbm_gbps": svc_bytes / svc_k_ms / 1e6,
        "hbm_frac": svc_bytes / svc_k_ms / 1e6 / HBM_PEAK_GBPS,
        "hbm_frac_sorted_order": svc_bytes / svc_sorted_ms / 1e6 / HBM_PEAK_GBPS}}

    # ... and the SpMM that consumes it: the skewed pattern straight from the SVC, B 16384 x 256
    N4 = 256
    B4 = torch.from_numpy(synth.dense_rhs(csr.K, N4, seed=14)).cuda()
    C4 = torch.empty(csr.M, N4, dtype=torch.float32, device="cuda")
    m_vec4 = csr.M // 8
    plan = Plan(r.vec_row_ptr, V, csr.K, max_N=N4)

    def spmm_cfg4(stream_):
        assert L.sspmm_f16_f32(m_vec4, 8, N4, csr.K, None, r.vec_row_ptr.data_ptr(), r.vec_col.data_ptr(),
                               r.vec_val.data_ptr(), B4.data_ptr(), C4.data_ptr(), stream_) == 0

    def spmm_cfg4_plan(stream_):
        assert L.sspmm_plan_batched_f16_f32(plan.handle, 1, N4, r.vec_row_ptr.data_ptr(), r.vec_col.data_ptr(),
                                            r.vec_val.data_ptr(), 0, B4.data_ptr(), 0, C4.data_ptr(), 0, stream_) == 0

    def spmm_cfg4_noalloc(stream_):
        assert L.sspmm_noalloc_f16_f32(m_vec4, 8, N4, csr.K, r.vec_row_ptr.data_ptr(), r.vec_col.data_ptr(),
                                       r.vec_val.data_ptr(), B4.data_ptr(), C4.data_ptr(), stream_) == 0

    lens = np.diff(off_h)
    touched = int(np.unique(r.vec_col.cpu().numpy()).size)
    bytes4 = synth.spmm_algorithmic_bytes(m_vec4, 8, int(r.num_vec), csr.K, N4, 4, k_touched=touched)
    want = None
    for name, f in (("cfg4_spmm_on_svc_output", spmm_cfg4), ("cfg4_spmm_on_svc_output_with_plan", spmm_cfg4_plan),
                    ("cfg4_spmm_on_svc_output_allocation_free_entry", spmm_cfg4_noalloc)):
        stt = {}
        ms4 = time_launches(lambda: f(stream), st, wu, stats=stt)
        res = {"workload": "A 16384x16384 Zipf rows (nnz %d) after SVC V=8, B 16384x%d, C fp32" % (nnz, N4)}
        res.update(figures(ms4, bytes4, 2.0 * nnz * N4))
        res.update(stt)
        res["kernel"] = KERNEL_NAMES.get(L.sspmm_last_kernel(), "unknown")
        res["ms_in_a_graph"] = graph_time(f)
        res["hbm_frac_in_a_graph"] = bytes4 / res["ms_in_a_graph"] / 1e6 / HBM_PEAK_GBPS
        res.update({"vector_row_len_max": int(lens.max()), "vector_row_len_mean": float(lens.mean()),
                    "steps_of_longest_row": int((lens.max() + 31) // 32), "steps_total": int(((lens + 31) // 32).sum()),
                    "gather_bytes_no_reuse": int(2 * r.num_vec * N4)})
        if want is None:  # parity of all three against the oracle
            want = O.spmm(m_vec4, 8, N4, csr.K, off_h, r.vec_col.cpu().numpy(), r.vec_val.cpu().numpy(), B4.cpu().numpy(),
                          threads=min(os.cpu_count(), 16))
        torch.cuda.synchronize()
        res["max_rel_err_vs_host_loop"] = float(np.abs(C4.cpu().numpy() - want).max() / np.abs(want).max())
        if "plan" in name:
            res["plan"] = plan.info()._asdict()
        out[name] = res
    plan.destroy()

    # the same pass on the shape of the matrices the reference's RowMerge is run on (its dataset of pruned
    # transformer weights): 2048 x 2048, 90 % of the entries zero at random, V = 8 and 16
    rng_d = np.random.default_rng(7)
    mask_d = rng_d.random((2048, 2048)) < 0.1
    d_ptr = np.concatenate([[0], np.cumsum(mask_d.sum(axis=1))]).astype(np.int32)
    d_col = np.nonzero(mask_d)[1].astype(np.int32)
    d_rp, d_ci = torch.from_numpy(d_ptr).cuda(), torch.from_numpy(d_col).cuda()
    d_lists = O.csr_col_lists(2048, d_ptr, d_col)
    for Vd in (8, 16):
        rd = sspmm_amd.svc(d_rp, d_ci, None, 2048, 2048, Vd)
        d_ms = time_launches(lambda: sspmm_amd.svc(d_rp, d_ci, None, 2048, 2048, Vd), 20, 3)
        t0 = time.perf_counter()
        d_want_ptr, d_want_cols = O.rowmerge_python(2048, Vd, d_lists)
        d_py = (time.perf_counter() - t0) * 1e3
        out["svc_pruned_weight_2048x2048_s0.9_v%d" % Vd] = {
            "gpu_ms_with_alloc_and_readback": d_ms, "python_rowmerge_ms": d_py, "speedup_vs_python": d_py / d_ms,
            "bit_exact_vs_python": bool(rd.vec_row_ptr.cpu().numpy().tolist() == d_want_ptr and
                                        rd.vec_col.cpu().numpy().tolist() == d_want_cols),
            "nnz": int(d_col.size), "nvec": int(rd.num_vec),
        }
    return out


def run_svc_batched(L, torch, synth, sspmm_amd, O):
    """The shape of the reference's RowMerge job (a loop over a dataset of small pruned-weight matrices,
    sparse_matrix_format.py:190-250): 96 seeded unstructured matrices of the dataset's shapes (512x512, 2048x512,
    512x2048) at 50 to 98 % sparsity, V = 8 and 16, as ONE stack through svc_batched against the Python RowMerge loop
    over the same matrices, single thread."""
    shapes = [(512, 512), (2048, 512), (512, 2048)]
    sparsities = [0.5, 0.7, 0.8, 0.9, 0.95, 0.98]
    rng = np.random.default_rng(96)
    mats = []
    for i in range(96):
        M, K = shapes[i % 3]
        mask = rng.random((M, K)) >= sparsities[(i // 3) % 6]
        ptr = np.concatenate([[0], np.cumsum(mask.sum(axis=1))]).astype(np.int32)
        mats.append((M, K, ptr, np.nonzero(mask)[1].astype(np.int32), None))
    mat_rows, K_max, rp, ci, _ = sspmm_amd.stack_csr(mats)
    d_rp, d_ci = torch.from_numpy(rp).cuda(), torch.from_numpy(ci).cuda()
    lists = [O.csr_col_lists(m[0], m[2], m[3]) for m in mats]
    out = {"workload": "96 unstructured matrices (512x512, 2048x512, 512x2048; 50-98 %% sparse), nnz %d in all, one stack" % ci.size,
           "matrices": len(mats), "nnz": int(ci.size)}
    for V in (8, 16):
        batch = sspmm_amd.svc_batched(mat_rows, K_max, d_rp, d_ci, None, V)
        torch.cuda.synchronize()
        gpu_ms = time_launches(lambda: sspmm_amd.svc_batched(mat_rows, K_max, d_rp, d_ci, None, V), 10, 2)
        # the whole job as the converter runs it: stack on the host, upload, merge, one copy back, split per matrix
        t0 = time.perf_counter()
        mr2, km2, rp2, ci2, _ = sspmm_amd.stack_csr(mats)
        host = sspmm_amd.svc_batched(mr2, km2, torch.from_numpy(rp2).cuda(), torch.from_numpy(ci2).cuda(), None, V).to_host()
        job_ms = (time.perf_counter() - t0) * 1e3
        # one matrix per call, as before (read-back of nvec per matrix)
        dm = [(torch.from_numpy(m[2]).cuda(), torch.from_numpy(m[3]).cuda()) for m in mats]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for (M, K, _p, _c, _v), (a, b) in zip(mats, dm):
            sspmm_amd.svc(a, b, None, M, K, V)
        torch.cuda.synchronize()
        loop_ms = (time.perf_counter() - t0) * 1e3
        t0 = time.perf_counter()
        want = [O.rowmerge_python(m[0], V, l) for m, l in zip(mats, lists)]
        py_ms = (time.perf_counter() - t0) * 1e3
        same = all(h[0].tolist() == w[0] and h[1].tolist() == w[1] for h, w in zip(host, want))
        nvec = int(sum(len(w[1]) for w in want))
        alg = sum(synth.svc_algorithmic_bytes(m[0], int(m[3].size), -(-m[0] // V), len(w[1]), V) for m, w in zip(mats, want))
        out["v%d" % V] = {"gpu_ms": gpu_ms, "gpu_ms_one_call_per_matrix": loop_ms,
                          "gpu_ms_whole_job_with_stacking_upload_and_copy_back": job_ms,
                          "python_rowmerge_ms": py_ms, "speedup_vs_python": py_ms / gpu_ms,
                          "speedup_vs_python_whole_job": py_ms / job_ms, "bit_exact_vs_python": bool(same), "nvec": nvec,
                          "alg_bytes": alg, "hbm_frac": alg / gpu_ms / 1e6 / HBM_PEAK_GBPS}
        del batch, host, dm
    out["speedup_vs_python"] = min(out["v8"]["speedup_vs_python"], out["v16"]["speedup_vs_python"])
    out["cpu_cores"] = 1
    return out


def run_cfg5_layer(L, torch, synth, st, wu):
    """One BERT-base shaped encoder layer (hidden 768, 12 heads, FFN 3072, 8 x 512 tokens) with six vector-sparse
    weights (V=16, 90 %; query, key and value stacked into one product, the GELU in the epilogue of the first
    feed-forward product) and dense attention on the feature-major activations; the same layer with dense fp16 matmuls
    on the densified weights beside it, eager and replayed from a HIP graph, and the layer written with torch alone."""
    from sspmm_amd.layers import SparseEncoderLayer, SparseLinear
    hid, heads, ffn, V5, bsz, seq = 768, 12, 3072, 16, 8, 512

    def mk(o, i, seed):
        w = synth.vector_sparse(o, i, V5, 0.9, seed=seed, std=0.02)
        return SparseLinear.from_cvse(i, V5, torch.from_numpy(w.row_offsets).cuda(), torch.from_numpy(w.col_idx).cuda(),
                                      torch.from_numpy(w.values).cuda())

    layer = SparseEncoderLayer(hid, heads, ffn, mk(hid, hid, 51), mk(hid, hid, 52), mk(hid, hid, 53), mk(hid, hid, 54),
                               mk(ffn, hid, 55), mk(hid, ffn, 56)).cuda().half()
    x5 = (torch.randn(hid, bsz * seq, device="cuda") * 1.0).half()
    dense_w = {n: getattr(layer, n).dense_weight() for n in ("q", "k", "v", "o", "ffn1", "ffn2")}
    dense_w["qkv"] = torch.cat([dense_w["q"], dense_w["k"], dense_w["v"]])  # the dense layer fuses the three as well
    def graphed(fn):
        """fn recorded into a HIP graph once; returns the replay (the host's per-launch cost is out of the picture)."""
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            fn()
        return g.replay

    dense_w["ffn1_gelu"] = dense_w["ffn1"]
    gelu = torch.nn.functional.gelu
    dense_lin = lambda n, lin, t: gelu(dense_w[n] @ t) if n == "ffn1_gelu" else dense_w[n] @ t  # noqa: E731
    with torch.no_grad():
        y_sp = layer(x5, bsz, seq)
        y_de = layer(x5, bsz, seq, linear=dense_lin)
        sp_ms = time_launches(lambda: layer(x5, bsz, seq), st, wu)
        de_ms = time_launches(lambda: layer(x5, bsz, seq, linear=dense_lin), st, wu)
        sp_g = time_launches(graphed(lambda: layer(x5, bsz, seq)), st, wu)
        de_g = time_launches(graphed(lambda: layer(x5, bsz, seq, linear=dense_lin)), st, wu)
        per = {}
        xin = {768: torch.randn(hid, bsz * seq, device="cuda").half(), 3072: torch.randn(ffn, bsz * seq, device="cuda").half()}
        sparse_sum = dense_sum = 0.0
        for n, lin in (("qkv", layer.qkv), ("o", layer.o), ("ffn1_gelu", layer.ffn1_gelu), ("ffn2", layer.ffn2)):
            xi = xin[lin.in_features]
            dw = dense_w[n]
            dfn = (lambda: gelu(dw @ xi)) if n == "ffn1_gelu" else (lambda: dw @ xi)  # noqa: E731
            # (twenty calls per graph: a graph of one kernel is bound by the cost of launching a graph)
            per[n] = {"sparse_ms_in_a_graph": graph_time(lambda s_: lin(xi)), "dense_ms_in_a_graph": graph_time(lambda s_: dfn())}
            sparse_sum += per[n]["sparse_ms_in_a_graph"]
            dense_sum += per[n]["dense_ms_in_a_graph"]
        per["qkv"]["three_separate_dense_products_ms_in_a_graph"] = graph_time(
            lambda s_: (dense_w["q"] @ xin[768], dense_w["k"] @ xin[768], dense_w["v"] @ xin[768]))
        # the attention step alone: this library's kernel on the feature-major projections against torch's attention
        # between the two relayout copies it needs on them
        import sspmm_amd.layers as layers_mod
        qkv5 = torch.randn(3 * hid, bsz * seq, device="cuda").half()
        att_kernel = graph_time(lambda s_: layer._attention(qkv5, bsz, seq))
        kernel_fn = layers_mod.attention_fm
        layers_mod.attention_fm = lambda *a, **kw: None
        try:
            att_torch = graph_time(lambda s_: layer._attention(qkv5, bsz, seq))
            sp_torch_att = time_launches(graphed(lambda: layer(x5, bsz, seq)), st, wu)
            de_torch_att = time_launches(graphed(lambda: layer(x5, bsz, seq, linear=dense_lin)), st, wu)
        finally:
            layers_mod.attention_fm = kernel_fn
        att_bytes = 4 * 2 * hid * bsz * seq  # q, k, v read, context written
        # the layer as a torch user writes it: token-major activations, dense weights, torch's linear / attention /
        # LayerNorm / GELU (no layout of this library anywhere)
        xt = x5.t().contiguous()
        wt = {n: dense_w[n] for n in ("qkv", "o", "ffn1", "ffn2")}
        F = torch.nn.functional

        def torch_layer():
            q_, k_, v_ = (t.view(bsz, seq, heads, hid // heads).transpose(1, 2) for t in F.linear(xt, wt["qkv"]).chunk(3, dim=-1))
            c = F.scaled_dot_product_attention(q_, k_, v_).transpose(1, 2).reshape(bsz * seq, hid)
            h1 = layer.ln1(xt + F.linear(c, wt["o"]))
            return layer.ln2(h1 + F.linear(F.gelu(F.linear(h1, wt["ffn1"])), wt["ffn2"]))

        y_t = torch_layer()
        torch_ms = time_launches(graphed(torch_layer), st, wu)
    return {"sparse_layer_ms": sp_ms, "dense_layer_ms": de_ms, "speedup_vs_dense_layer": de_ms / sp_ms,
            "sparse_layer_ms_in_a_graph": sp_g, "dense_layer_ms_in_a_graph": de_g, "speedup_vs_dense_layer_in_a_graph": de_g / sp_g,
            "products_sparse_ms_in_a_graph": sparse_sum, "products_dense_ms_in_a_graph": dense_sum,
            "rest_of_the_layer_ms_in_a_graph": {"sparse_layer": sp_g - sparse_sum, "dense_layer": de_g - dense_sum},
            "attention_ms_in_a_graph": {"feature_major_kernel": att_kernel, "torch_between_two_relayout_copies": att_torch,
                                        "kernel_alg_bytes": att_bytes, "kernel_hbm_frac": att_bytes / att_kernel / 1e6 / HBM_PEAK_GBPS},
            "with_torch_attention_ms_in_a_graph": {"sparse_layer": sp_torch_att, "dense_layer": de_torch_att,
                                                   "speedup": de_torch_att / sp_torch_att},
            "torch_token_major_dense_layer_ms_in_a_graph": torch_ms,
            "speedup_vs_torch_token_major_dense_layer_in_a_graph": torch_ms / sp_g,
            "note": "both layers run the same glue around their four products: this library's attention kernel on the "
                    "feature-major projections and the residual add + LayerNorm in one kernel of this library; the "
                    "products are one fused q/k/v, o, ffn1 with its GELU (in the SpMM's epilogue on the sparse side, "
                    "torch's kernel behind the matmul on the dense side), ffn2.  torch_token_major_dense_layer is the "
                    "same arithmetic written with torch alone on token-major activations",
            "max_rel_diff_vs_dense_layer": float((y_sp.float() - y_de.float()).abs().max() / y_de.float().abs().max()),
            "max_rel_diff_vs_torch_token_major_layer": float((y_sp.float() - y_t.t().float()).abs().max() / y_t.float().abs().max()),
            "projections": per}


def run_attention_forward(torch, sparsity, bsz, seq, heads, embed, st, wu, mlp=1024):
    """The forward pass of the reference's end-to-end sparse attention model (end2end/sspmm_e2e/end_to_end.py:123-203:
    4 blocks, fp16, V = 8 masks drawn at random per block) at the configurations its results are published for,
    timed with a device synchronisation either side (the reference's loop has none, end_to_end.py:198-203), eager
    and replayed from a HIP graph; the same model with dense unmasked attention in torch beside it (the reference's
    "PyTorch" column)."""
    from sspmm_amd.attention import SparseAttentionEncoder
    torch.manual_seed(0)
    # (the head is as wide as the MLP, as the reference's driver builds it: end_to_end.py:176-185, num_class=args.mlp_dim)
    model = SparseAttentionEncoder(257, embed, heads, sparsity, seq, mlp, mlp, vec_length=8, layers=4, seed=20).cuda().half().eval()
    tokens = torch.randint(0, 257, (bsz, seq), device="cuda")

    def dense_forward():
        # the same weights with torch's dense attention (no mask): what the reference's dense model computes
        out = model.encoder(tokens) * (embed ** 0.5)
        out = out.transpose(0, 1) + model.pe[:seq].to(out.dtype)
        d = embed // heads
        for blk in model.blocks:
            q, k, v = blk.in_proj(blk.layer_norm1(out)).chunk(3, dim=-1)
            q, k, v = (t.contiguous().view(seq, bsz * heads, d).transpose(0, 1) for t in (q, k, v))
            a = torch.nn.functional.scaled_dot_product_attention(q, k, v).transpose(0, 1).contiguous().view(seq, bsz, embed)
            h1 = blk.out_proj(a) + out
            out = blk.linear2(blk.linear1(blk.layer_norm2(h1))) + out
        return model.linear(model.layer_norm(out))

    def graphed(fn):
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            fn()
        return g.replay

    with torch.no_grad():
        y = model(tokens)
        ms = time_launches(lambda: model(tokens), st, wu)
        ms_g = time_launches(graphed(lambda: model(tokens)), st, wu)
        dense_ms = time_launches(dense_forward, max(3, st // 4), 2)
        blk = model.blocks[0]
        x0 = torch.randn(seq, bsz, embed, device="cuda").half()
        att_ms = time_launches(graphed(lambda: blk.attention(x0)), st, wu)
    nvec = int(model.blocks[0].column_indices.numel())
    return {"workload": "4 blocks, seq %d, %d heads / embed %d, mlp %d, mask sparsity %g (V=8, %d vectors per block), batch %d, fp16"
                        % (seq, heads, embed, mlp, sparsity, nvec, bsz),
            "ms": ms, "ms_in_a_graph": ms_g, "dense_unmasked_torch_ms": dense_ms, "speedup_vs_dense_unmasked_torch": dense_ms / ms_g,
            "attention_of_one_block_ms_in_a_graph": att_ms, "output_is_finite": bool(torch.isfinite(y).all())}


def run_reorder(L, torch, synth, sspmm_amd):
    """Row reordering ahead of the SVC: 16384 rows that are noisy copies of 256 prototype rows, shuffled."""
    rc_csr = synth.clustered_csr(16384, 16384, 256, 128, seed=6, keep=0.9, extras=1)
    rrp, rci, rcv = (torch.from_numpy(x).cuda() for x in (rc_csr.row_ptr, rc_csr.col_ind, rc_csr.values))
    plain = sspmm_amd.svc(rrp, rci, rcv, rc_csr.M, rc_csr.K, 8, order="sorted")
    reo = sspmm_amd.svc_reordered(rrp, rci, rcv, rc_csr.M, rc_csr.K, 8, order="sorted")
    rws = torch.empty(L.svc_reorder_workspace_bytes(rc_csr.M), dtype=torch.uint8, device="cuda")
    rperm = torch.empty(rc_csr.M, dtype=torch.int32, device="cuda")
    o_rp, o_ci, o_cv = torch.empty_like(rrp), torch.empty_like(rci), torch.empty_like(rcv)
    stream = torch.cuda.current_stream().cuda_stream

    def reorder_order():
        rc = L.svc_reorder_minhash(rc_csr.M, rrp.data_ptr(), rci.data_ptr(), rperm.data_ptr(), rws.data_ptr(),
                                   rws.numel(), stream)
        assert rc == 0, rc

    def reorder_apply():
        rc = L.svc_permute_csr(rc_csr.M, rperm.data_ptr(), rrp.data_ptr(), rci.data_ptr(), rcv.data_ptr(),
                               o_rp.data_ptr(), o_ci.data_ptr(), o_cv.data_ptr(), rws.data_ptr(), rws.numel(),
                               stream)
        assert rc == 0, rc

    reorder_order()
    t_order = time_launches(reorder_order, 20, 3)
    t_apply = time_launches(reorder_apply, 20, 3)
    rnnz = int(rc_csr.col_ind.size)
    by_order = 4 * (rc_csr.M + 1) + 4 * rnnz + 4 * rc_csr.M   # row pointer + columns read, order written
    by_apply = 4 * rc_csr.M + 2 * 4 * (rc_csr.M + 1) + 2 * (4 + 2) * rnnz  # CSR read once, written once
    return {
        "workload": "16384 x 16384 CSR, rows = noisy copies of 256 prototypes (nnz %d), shuffled; V=8" % rnnz,
        "order_ms": t_order, "order_alg_bytes": by_order, "order_hbm_gbps": by_order / t_order / 1e6,
        "apply_ms": t_apply, "apply_alg_bytes": by_apply, "apply_hbm_gbps": by_apply / t_apply / 1e6,
        "nvec_without_reordering": int(plain.num_vec), "nvec_with_reordering": int(reo.svc.num_vec),
        "fill_without_reordering": rnnz / (plain.num_vec * 8.0), "fill_with_reordering": rnnz / (reo.svc.num_vec * 8.0),
    }


ATTENTION = "sparse_attention_seq4096_d64_v8_s0.9_heads48"
# the eight published configurations of the reference's end-to-end model (mask sparsity, sequence, heads / embed), batch 2 and 8
ATTENTION_FORWARD = {"sparse_attention_forward_seq%d_h%d_e%d_s%g_b%d_l4" % (seq, h, e, s, b): (s, b, seq, h, e)
                     for s in (0.9, 0.95) for seq in (4096, 8192) for (h, e) in ((4, 256), (8, 512)) for b in (2, 8)}
GROUPS = ["cfg1_rowmerge_then_spmm_512x512", "cfg4", "svc_batched_dlmc_shapes", *ATTENTION_FORWARD, "cfg5_encoder_layer_v16_s0.9_tokens4096", ATTENTION,
          "reorder_clustered_16384_v8", "headline_batched_cold"]


def headline_cold(L, torch, synth, batch, st, wu):
    """The headline launch with nothing left in a cache from the launch before: two complete operand sets (values, B,
    C: 2 x 329 MB, more than the 256 MB memory-side cache) used in turn."""
    M, K, V, N = 2048, 512, 8, 256
    vs = synth.vector_sparse(M, K, V, 0.9, seed=2, std=0.02)
    ro, ci = torch.from_numpy(vs.row_offsets).cuda(), torch.from_numpy(vs.col_idx).cuda()
    nv = vs.col_idx.size
    g = torch.Generator(device="cuda").manual_seed(3)
    sets = []
    for _ in range(2):
        sets.append(((torch.randn(batch, nv * V, generator=g, device="cuda") * 0.02).half(),
                     torch.randn(batch, K, N, generator=g, device="cuda").half(),
                     torch.empty(batch, M, N, dtype=torch.float32, device="cuda")))
    stream = torch.cuda.current_stream().cuda_stream
    turn = [0]

    def launch():
        vals, B, C = sets[turn[0] & 1]
        turn[0] += 1
        rc = L.sspmm_batched_f16_f32(batch, vs.m_vec, V, N, K, None, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(), nv * V,
                                     B.data_ptr(), K * N, C.data_ptr(), M * N, stream)
        assert rc == 0, rc

    stt = {}
    ms = time_launches(launch, st, wu, stats=stt)
    by = batch * synth.spmm_algorithmic_bytes(vs.m_vec, V, nv, K, N, 4) - (batch - 1) * (4 * nv + 4 * (vs.m_vec + 1))
    res = {"workload": "the headline launch (batch %d), two operand sets of %d MB in rotation" % (batch, by // 1000000)}
    res.update(figures(ms, by, 2.0 * vs.nnz * N * batch))
    res.update(stt)
    return res


def run_extra(name, env):
    """One entry (or group of entries) of `extra` by name; returns a dict name -> figures."""
    L, torch, synth, sspmm_amd, O, st, wu, batch = (env[k] for k in ("L", "torch", "synth", "sspmm_amd", "O", "st", "wu", "batch"))
    cases = single_launch_cases(batch)
    if name in cases:
        kw = cases[name]
        res = spmm_case(L, torch, synth, steps=st, warmup=wu, dense=True, graph=kw["batch"] == 1, **kw)
        torch.cuda.empty_cache()
        return {name: res}
    if name == "cfg1_rowmerge_then_spmm_512x512":
        return {name: run_cfg1(L, torch, synth, sspmm_amd, O, st, wu)}
    if name == "cfg4":
        return run_cfg4(L, torch, synth, sspmm_amd, O, st, wu)
    if name in ATTENTION_FORWARD:
        return {name: run_attention_forward(torch, *ATTENTION_FORWARD[name], st=min(st, 50) if ATTENTION_FORWARD[name][2] <= 4096 else min(st, 20),
                                            wu=min(wu, 10))}
    if name == "svc_batched_dlmc_shapes":
        return {name: run_svc_batched(L, torch, synth, sspmm_amd, O)}
    if name == "cfg5_encoder_layer_v16_s0.9_tokens4096":
        return {name: run_cfg5_layer(L, torch, synth, st, wu)}
    if name == ATTENTION:
        return {name: attention_block(torch, synth, sspmm_amd, st, wu)}
    if name == "reorder_clustered_16384_v8":
        return {name: run_reorder(L, torch, synth, sspmm_amd)}
    if name == "headline_batched_cold":
        return {name: headline_cold(L, torch, synth, batch, st, wu)}
    raise SystemExit("unknown entry %r (see --list)" % name)


def main():
    args = parse_args()
    if args.list:
        print("\n".join(list(single_launch_cases(args.batch)) + GROUPS))
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (vector-rows shard without "
              "communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from sspmm_amd import _lib, synth
    import sspmm_amd
    L = _lib.lib()
    torch.cuda.set_device(0)
    L.sspmm_select_kernel({"auto": 0, "generic": 1, "gather": 2, "slab": 3, "slab128": 9}[args.kernel])
    env = {"L": L, "torch": torch, "synth": synth, "sspmm_amd": sspmm_amd, "O": None, "st": args.steps, "wu": args.warmup,
           "batch": args.batch}
    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    only = [ATTENTION] if args.attention_only else [n for n in args.only.split(",") if n]
    if only:
        from oracle import oracle as O
        O.build()
        env["O"] = O
        out = {}
        for n in only:
            out.update(run_extra(n, env))
        print(json.dumps(out))
        return

    M, K, V, sparsity, N = 2048, 512, 8, 0.9, 256
    series, handles = [], []
    main_res = spmm_case(L, torch, synth, M, K, V, sparsity, N, args.batch, True, 0.02, 2, args.steps, args.warmup,
                         dense=not args.quick, series=series, handles_out=handles)
    vs, vals, B, C = handles
    torch.cuda.synchronize()
    main_kernel = {3: "spmm_slab_kernel<8,float,*,4>", 2: "spmm_gather_kernel<8,float>", 1: "spmm_generic_kernel<8,float>",
                   6: "spmm_stage_kernel<8,float>"}.get(L.sspmm_last_kernel(), "unknown")

    # the same workload as 128 separate launches, one batch element each, rotating through the 335 MB of distinct
    # operands (nothing a launch touches is still in a cache from the launch before): per-launch time when
    # launches are small and cold
    cold = None
    if not args.quick and args.batch >= 8:
        ro_d, ci_d = torch.from_numpy(vs.row_offsets).cuda(), torch.from_numpy(vs.col_idx).cuda()
        st0 = torch.cuda.current_stream().cuda_stream
        turn = [0]

        def one_cold():
            i = turn[0] % args.batch
            turn[0] += 1
            rc = L.sspmm_f16_f32(vs.m_vec, V, N, K, None, ro_d.data_ptr(), ci_d.data_ptr(), vals[i].data_ptr(),
                                 B[i].data_ptr(), C[i].data_ptr(), st0)
            assert rc == 0, rc

        cold_ms = time_launches(one_cold, 4 * args.batch, args.batch)
        one_bytes = synth.spmm_algorithmic_bytes(vs.m_vec, V, vs.col_idx.size, K, N, 4)
        cold = {"workload": "one batch element per launch, %d distinct operand sets in rotation" % args.batch}
        cold.update(figures(cold_ms, one_bytes, 2.0 * vs.nnz * N))
        # (leaves C as the batched launch wrote it: same operands, same results)

    # what this box's memory system sustains for plain streams of the same size class, measured the same way
    # (50 launches after warm-up): a device copy (half reads, half writes) and a fill (writes only)
    ceilings = None
    if not args.quick:
        src = torch.ones(256 * 1024 * 1024, dtype=torch.float32, device="cuda")  # 1 GiB: beyond the memory-side cache
        dst = torch.empty_like(src)
        copy_ms = time_launches(lambda: dst.copy_(src), 50, 5)
        fill_ms = time_launches(lambda: dst.fill_(1.0), 50, 5)
        ceilings = {"device_copy_1GiB_gbps": 2 * src.numel() * 4 / copy_ms / 1e6,
                    "device_fill_1GiB_gbps": src.numel() * 4 / fill_ms / 1e6}
        ceilings["frac_of_device_copy"] = main_res["hbm_gbps"] / ceilings["device_copy_1GiB_gbps"]
        del src, dst

    # parity of batch elements spread over the launch (first, last, and one per way the batch is dealt to the XCDs)
    # against the CPU oracle, and the CPU baseline on element 0
    cpu = None
    parity = None
    if not args.quick:
        from oracle import oracle as O
        O.build()
        env["O"] = O
        ncores = os.cpu_count()
        errs = {}
        for b in sorted(set(x for x in (0, 7, 8, 63, args.batch // 2 + 1, args.batch - 1) if 0 <= x < args.batch)):
            want_b = O.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, vals[b].cpu().numpy(), B[b].cpu().numpy(),
                            threads=min(ncores, 16))
            errs[b] = float(np.abs(C[b].cpu().numpy() - want_b).max() / max(np.abs(want_b).max(), 1e-30))
        parity = max(errs.values())
        if not parity <= 1e-2:
            print("bench.py: the timed launch disagrees with the host loop: max relative error per batch element %r"
                  % errs, file=sys.stderr)
            sys.exit(3)
        v0 = vals[0].cpu().numpy()
        b0 = B[0].cpu().numpy()
        t0 = time.perf_counter()
        reps = 0
        while True:
            O.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, v0, b0, threads=1)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 200:
                break
        cpu_s = (time.perf_counter() - t0) / reps
        t0 = time.perf_counter()
        O.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, v0, b0, threads=min(ncores, 16))
        cpu_mt_s = time.perf_counter() - t0
        cpu = {"value": 2.0 * vs.nnz * N / cpu_s / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
               "sample": "%d repeats of one batch element (A 2048x512 V=8 s=0.9, B 512x256), host loop of "
                         "sspmm_test.cpp:75-95 in C, -O2, single thread; %.1f ms each" % (reps, cpu_s * 1e3),
               "all_cores_value": 2.0 * vs.nnz * N / cpu_mt_s / 1e12, "all_cores": min(ncores, 16),
               "host_cpus": ncores, "parity_checked_batch_elements": sorted(errs)}
    del vals, B, C, handles

    extra = {}
    # launch time (us) averaged over chunks of 100 launches, from the first warm-up launch to the last timed one
    per100 = []
    for i in range(0, len(series), 10):
        part = [v for v in series[i:i + 10] if v is not None]
        per100.append(round(sum(part) / len(part), 1) if part else None)
    extra["headline_us_per_chunk"] = {"chunk": 100, "warmup_chunks": (args.warmup + 99) // 100, "us": per100}
    extra["headline_launch_ms_median_min"] = {"ms_median": main_res["ms_median"], "ms_min": main_res["ms_min"],
                                              "hbm_frac_at_min": main_res["hbm_frac_at_min"]}
    # the window the reference's harness times (200 launches after 10 warm-ups, sspmm_test.cpp:22-23,181-195), read
    # from the same series: launches 10..209 of this process, while the clocks are still settling
    if args.warmup >= 220 and all(v is not None for v in series[1:21]):
        us = sum(series[1:21]) / 20.0
        extra["headline_200_launches_after_10"] = {"us": round(us, 2), "hbm_frac": round(main_res["alg_bytes"] / us / 1e3 / HBM_PEAK_GBPS, 4)}
    if cold:
        extra["cfg2_single_launches_cold"] = cold
    if not args.quick:
        for name in list(single_launch_cases(args.batch)) + GROUPS:
            extra.update(run_extra(name, env))
    traffic = measured_traffic()
    if not args.quick:
        extra["measured_hbm_traffic"] = traffic
    head_traffic = traffic.get("headline_batch128") if (args.kernel == "auto" and args.batch == 128) else None

    roofline = {"bound": "hbm", "achieved": main_res["hbm_gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": main_res["hbm_frac"], "traffic": head_traffic["bytes"] if head_traffic else None,
                "kernel": main_kernel, "alg_bytes_per_launch": main_res["alg_bytes"]}
    dense = {k: main_res[k] for k in main_res if k.startswith("dense") or k.startswith("speedup")}
    contract = {
        "metric": "SpMM useful TFLOP/s (2*nnz*N/t), V=8 @90% sparsity, fp16 in / fp32 accumulate",
        "value": main_res["useful_tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": main_res["ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": main_res["workload"] + " (one launch, pattern shared by the batch)",
                   "hbm_gbps": main_res["hbm_gbps"]},
    }

    # Every figure of the run goes to a file; the line on stdout carries the contract and a dozen scalars.
    full = dict(contract)
    full["roofline"] = dict(roofline, traffic_source=head_traffic["source"] if head_traffic else None,
                            operands="warm: the same 329 MB of operands every launch (the cold rotation of two sets is "
                                     "extra.headline_batched_cold)", measured_stream_rates=ceilings)
    full.update({"cpu_baseline": cpu, "parity_max_rel_err": parity, "dense_gemm": dense, "extra": extra})
    try:
        with open(args.extras_file, "w") as f:
            json.dump(full, f, indent=1)
            f.write("\n")
    except OSError as e:
        print("bench.py: could not write %s: %s" % (args.extras_file, e), file=sys.stderr)

    # an entry whose result was compared with the host loop and disagrees fails the run, whichever entry it is
    bad = parity_failures(extra)
    if bad:
        print("bench.py: entries that disagree with the host loop (max relative error > %g): %r" % (PARITY_BAR, bad),
              file=sys.stderr)
        sys.exit(3)

    line = dict(contract)
    line["roofline"] = roofline
    line["cpu_baseline"] = {k: cpu[k] for k in ("value", "unit", "cores", "kind", "sample")} if cpu else None
    line["parity_max_rel_err"] = parity
    line["dense_gemm"] = dense
    line["extra"] = short_extra(extra)
    line["extra_file"] = args.extras_file
    text = json.dumps(line)
    assert len(text) < 4096, "the benchmark line must stay short (%d bytes)" % len(text)
    print(text)


PARITY_BAR = 1e-2


def parity_failures(tree, path=""):
    """Every '...max_rel_err...' figure of the nested result dictionary that exceeds the bar, and every
    '...bit_exact...' flag that is false."""
    bad = {}
    if isinstance(tree, dict):
        for k, v in tree.items():
            p = path + "/" + str(k) if path else str(k)
            if isinstance(v, dict):
                bad.update(parity_failures(v, p))
            elif "max_rel_err" in str(k) and isinstance(v, (int, float)) and not v <= PARITY_BAR:
                bad[p] = v
            elif "bit_exact" in str(k) and v is False:
                bad[p] = v
    return bad


def short_extra(extra):
    """At most a dozen scalars of the full result dictionary for the line on stdout (single-launch fractions of the
    HBM peak, SVC speed-ups over the Python RowMerge); absent entries are left out."""
    def get(*keys):
        node = extra
        for k in keys:
            if not isinstance(node, dict) or k not in node:
                return None
            node = node[k]
        return round(node, 4) if isinstance(node, float) else node

    picks = {
        "headline_cold_hbm_frac": ("headline_batched_cold", "hbm_frac"),
        "cfg3_1024x2304_s0.8_n3136_hbm_frac": ("cfg3_1024x2304_v16_s0.8_n3136", "hbm_frac"),
        "cfg3_1024x2304_s0.8_n3136_ms": ("cfg3_1024x2304_v16_s0.8_n3136", "ms"),
        "cfg5_ffn1_hbm_frac": ("cfg5_ffn1_3072x768_v16_s0.9_n4096", "hbm_frac"),
        "cfg5_ffn2_hbm_frac": ("cfg5_ffn2_768x3072_v16_s0.9_n4096", "hbm_frac"),
        "cfg4_spmm_with_plan_hbm_frac": ("cfg4_spmm_on_svc_output_with_plan", "hbm_frac"),
        "cfg4_spmm_with_plan_ms": ("cfg4_spmm_on_svc_output_with_plan", "ms"),
        "svc_cfg4_speedup_vs_python": ("svc_cfg4_zipf_16384_v8", "speedup_vs_python"),
        "svc_batched_dlmc_shapes_speedup_vs_python": ("svc_batched_dlmc_shapes", "speedup_vs_python"),
        "cfg5_layer_speedup_vs_dense_in_a_graph": ("cfg5_encoder_layer_v16_s0.9_tokens4096", "speedup_vs_dense_layer_in_a_graph"),
        "sparse_attention_forward_s0.9_b2_ms": ("sparse_attention_forward_seq4096_h4_e256_s0.9_b2_l4", "ms_in_a_graph"),
        "sparse_attention_block_one_launch_ms": (ATTENTION, "one_launch_ms"),
    }
    out = {}
    for name, keys in picks.items():
        v = get(*keys)
        if v is not None:
            out[name] = v
    return out


if __name__ == "__main__":
    main()
