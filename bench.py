#!/usr/bin/env python3
"""Benchmark of the SVC -> SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  A "step" is one pass of the SpMM over one batch of synthetic inputs
already resident in HBM: the FFN-shaped configuration (A 2048x512 fp16, V=8, 90 % vector
sparsity, B 512x256 fp16, C fp32), run bspmm-style over a batch of independent value / B / C
sets that share the pattern, so that one launch moves more bytes than the last-level cache
holds.  `value` is useful TFLOP/s = 2 * nnz * N * batch / t (the reference's convention,
SSpMM/sspmm_test.cpp:197, with nnz the scalar non-zeros).

`roofline` prices the SpMM kernel against the 8 TB/s HBM peak with the algorithmic bytes of one
launch (every operand read once, C written once).  `cpu_baseline` times the CPU oracle (a port of
the reference's host loop) on one batch element, single thread.  `extra` carries the other
configurations (single launches, V=16 shapes, the SVC against the Python RowMerge, the dense GEMM
comparator).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
# HBM bytes per launch of the headline workload at the default batch of 128, from hardware counters
# (FETCH_SIZE and WRITE_SIZE, each scaled by its reading for a 256 MiB device copy): see
# profiles/spmm_slab_v8_f32_cfg2_batch128_hbm_traffic.txt.  Other batch sizes report null.
MEASURED_TRAFFIC_BYTES = {128: 66.1e6 + 268.4e6}


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
    ap.add_argument("--attention-only", action="store_true",
                    help="run only the sparse attention block (bsddmm, bcsr_softmax, bspmm) and print its figures")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (its hardware-counter readings calibrate FETCH_SIZE / "
                         "WRITE_SIZE when the run is profiled)")
    ap.add_argument("--kernel", choices=["auto", "generic", "gather", "slab"], default="auto",
                    help="force one SpMM kernel (tuning); the default lets the library choose")
    return ap.parse_args()


def time_launches(fn, steps, warmup, series=None):
    """Average milliseconds per call over `steps` calls, HIP events on the launch stream."""
    import torch
    chunk = 10
    marks = []

    def run(n):
        for i in range(n):
            if series is not None and i % chunk == 0:
                ev = torch.cuda.Event(enable_timing=True)
                ev.record()
                marks.append((ev, min(chunk, n - i)))
            fn()

    run(warmup)
    torch.cuda.synchronize()
    n_warm = len(marks)
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    run(steps)
    end.record()
    torch.cuda.synchronize()
    if series is not None:
        # (events on the launch stream: microseconds per launch for every chunk of 10 launches; the chunk that ends
        # the warm-up runs into the host synchronisation and is left out)
        bounds = [m[0] for m in marks] + [end]
        for i, (ev, n) in enumerate(marks):
            series.append(ev.elapsed_time(bounds[i + 1]) / n * 1e3 if i != n_warm - 1 else None)
    return start.elapsed_time(end) / steps


def spmm_case(L, torch, synth, M, K, V, sparsity, N, batch, out_f32, std, seed, steps, warmup, dense=False, series=None):
    """Times one SpMM configuration; returns a dict of figures."""
    vs = synth.vector_sparse(M, K, V, sparsity, seed=seed, std=std)
    g = torch.Generator(device="cuda").manual_seed(seed)
    ro = torch.from_numpy(vs.row_offsets).cuda()
    ci = torch.from_numpy(vs.col_idx).cuda()
    nv = vs.col_idx.size
    vals = (torch.randn(batch, nv * V, generator=g, device="cuda") * std).half()
    B = torch.randn(batch, K, N, generator=g, device="cuda").half()
    C = torch.empty(batch, vs.m_vec * V, N, dtype=torch.float32 if out_f32 else torch.float16, device="cuda")
    fn = L.sspmm_batched_f16_f32 if out_f32 else L.sspmm_batched_f16_f16
    stream = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = fn(batch, vs.m_vec, V, N, K, None, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(), nv * V, B.data_ptr(),
                K * N, C.data_ptr(), vs.m_vec * V * N, stream)
        if rc:
            raise RuntimeError("sspmm failed: %d" % rc)

    ms = time_launches(launch, steps, warmup, series)
    bytes_alg = batch * synth.spmm_algorithmic_bytes(vs.m_vec, V, nv, K, N, 4 if out_f32 else 2) \
        - (batch - 1) * (4 * nv + 4 * (vs.m_vec + 1))  # the pattern is shared by the batch
    flops = 2.0 * vs.nnz * N * batch
    out = {
        "workload": "A %dx%d V=%d s=%.2f, B %dx%d, C %s, batch %d" % (M, K, V, sparsity, K, N,
                                                                       "fp32" if out_f32 else "fp16", batch),
        "ms": ms, "useful_tflops": flops / ms / 1e9, "alg_bytes": bytes_alg, "hbm_gbps": bytes_alg / ms / 1e6,
        "hbm_frac": bytes_alg / ms / 1e6 / HBM_PEAK_GBPS,
        "gather_bytes_no_reuse": batch * 2 * nv * N,
    }
    if dense:
        A = torch.zeros(vs.m_vec * V, K, dtype=torch.float16, device="cuda")
        Ad = A.unsqueeze(0).expand(batch, -1, -1).contiguous()
        dms = time_launches(lambda: torch.bmm(Ad, B), max(10, steps // 4), 3)
        out["dense_gemm_ms"] = dms
        out["dense_gemm_effective_tflops"] = flops / dms / 1e9
        out["speedup_vs_dense"] = dms / ms
        del A, Ad
    handles = (vs, vals, B, C)
    return out, handles


def attention_block(torch, synth, sspmm_amd, st, wu):
    """Times the three steps of the reference's sparse attention block; returns a dict of figures."""
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
    t_dense = time_launches(lambda: torch.nn.functional.scaled_dot_product_attention(qA, kA, vA), st, wu)
    by_sddmm = bA * (2 * seqA * dA * 2 + 2 * nvA * VA) + 4 * nvA + 4 * (mk_a.m_vec + 1)
    by_soft = bA * 2 * 2 * nvA * VA + 4 * (mk_a.m_vec + 1)
    by_av = bA * (2 * nvA * VA + 2 * seqA * dA + 2 * seqA * dA) + 4 * nvA + 4 * (mk_a.m_vec + 1)
    res = {
        "bsddmm_ms": t_sddmm, "bsddmm_hbm_frac": by_sddmm / t_sddmm / 1e6 / HBM_PEAK_GBPS, "bsddmm_alg_bytes": by_sddmm,
        "bcsr_softmax_ms": t_soft, "bcsr_softmax_hbm_frac": by_soft / t_soft / 1e6 / HBM_PEAK_GBPS,
        "bcsr_softmax_alg_bytes": by_soft,
        "bspmm_ms": t_av, "bspmm_hbm_frac": by_av / t_av / 1e6 / HBM_PEAK_GBPS, "bspmm_alg_bytes": by_av,
        "block_ms": t_sddmm + t_soft + t_av, "dense_sdpa_ms": t_dense, "nvec": int(nvA),
    }
    del qA, kA, vA, wA, pA
    return res


def main():
    args = parse_args()
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
    L.sspmm_select_kernel({"auto": 0, "generic": 1, "gather": 2, "slab": 3}[args.kernel])
    if args.attention_only:
        print(json.dumps({"sparse_attention_seq4096_d64_v8_s0.9_heads48":
                          attention_block(torch, synth, sspmm_amd, args.steps, args.warmup)}))
        return

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    M, K, V, sparsity, N = 2048, 512, 8, 0.9, 256
    kernel_names = {1: "spmm_generic_kernel<8,float>", 2: "spmm_gather_kernel<8,float>", 3: "spmm_slab_kernel<8,float,*,4>",
                    4: "spmm_gather_split_kernel<8,float>", 5: "spmm_slab_kernel<8,float,*,2>", 6: "spmm_stage_kernel<8,float>"}
    series = []
    main_res, (vs, vals, B, C) = spmm_case(L, torch, synth, M, K, V, sparsity, N, args.batch, True, 0.02, 2,
                                           args.steps, args.warmup, dense=not args.quick, series=series)
    torch.cuda.synchronize()
    main_kernel = kernel_names.get(L.sspmm_last_kernel(), "unknown")

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
        cold = {"workload": "one batch element per launch, %d distinct operand sets in rotation" % args.batch,
                "ms": cold_ms, "useful_tflops": 2.0 * vs.nnz * N / cold_ms / 1e9, "alg_bytes": one_bytes,
                "hbm_gbps": one_bytes / cold_ms / 1e6, "hbm_frac": one_bytes / cold_ms / 1e6 / HBM_PEAK_GBPS}

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

    # parity of batch element 0 against the CPU oracle, and the CPU baseline on the same element
    cpu = None
    parity = None
    if not args.quick:
        from oracle import oracle as O
        O.build()
        v0 = vals[0].cpu().numpy()
        b0 = B[0].cpu().numpy()
        t0 = time.perf_counter()
        reps = 0
        while True:
            want = O.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, v0, b0, threads=1)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 200:
                break
        cpu_s = (time.perf_counter() - t0) / reps
        got = C[0].cpu().numpy()
        parity = float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))
        ncores = os.cpu_count()
        t0 = time.perf_counter()
        O.spmm(vs.m_vec, V, N, K, vs.row_offsets, vs.col_idx, v0, b0, threads=min(ncores, 16))
        cpu_mt_s = time.perf_counter() - t0
        cpu = {"value": 2.0 * vs.nnz * N / cpu_s / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
               "sample": "%d repeats of one batch element (A 2048x512 V=8 s=0.9, B 512x256), host loop of "
                         "sspmm_test.cpp:75-95 in C, -O2, single thread; %.1f ms each" % (reps, cpu_s * 1e3),
               "all_cores_value": 2.0 * vs.nnz * N / cpu_mt_s / 1e12, "all_cores": min(ncores, 16),
               "host_cpus": ncores}
    del vals, B, C

    extra = {}
    # launch time (us) averaged over chunks of 100 launches, from the first warm-up launch to the last timed one
    per100 = []
    for i in range(0, len(series), 10):
        part = [v for v in series[i:i + 10] if v is not None]
        per100.append(round(sum(part) / len(part), 1) if part else None)
    extra["headline_us_per_chunk"] = {"chunk": 100, "warmup_chunks": (args.warmup + 99) // 100, "us": per100}
    # the window the reference's harness times (200 launches after 10 warm-ups, sspmm_test.cpp:22-23,181-195), read
    # from the same series: launches 10..209 of this process, while the clocks are still settling
    if args.warmup >= 220 and all(v is not None for v in series[1:21]):
        us = sum(series[1:21]) / 20.0
        extra["headline_200_launches_after_10"] = {"us": round(us, 2), "hbm_frac": round(main_res["alg_bytes"] / us / 1e3 / HBM_PEAK_GBPS, 4)}
    if cold:
        extra["cfg2_single_launches_cold"] = cold
    if not args.quick:
        st, wu = args.steps, args.warmup  # (the other shapes meet the same clock transient)
        cases = {
            "cfg2_single_launch": dict(M=2048, K=512, V=8, sparsity=0.9, N=256, batch=1, out_f32=True, std=0.02, seed=2),
            "cfg2_batched_fp16_out": dict(M=2048, K=512, V=8, sparsity=0.9, N=256, batch=args.batch, out_f32=False,
                                          std=0.02, seed=2),
            "cfg2_shape_v16_batched": dict(M=2048, K=512, V=16, sparsity=0.9, N=256, batch=args.batch, out_f32=True,
                                           std=0.02, seed=2),
            "cfg2_shape_v16_batched_fp16_out": dict(M=2048, K=512, V=16, sparsity=0.9, N=256, batch=args.batch,
                                                    out_f32=False, std=0.02, seed=2),
            "cfg3_1024x2304_v16_s0.8_n3136": dict(M=1024, K=2304, V=16, sparsity=0.8, N=3136, batch=1, out_f32=True,
                                                  std=0.05, seed=3),
            "cfg3_2048x1024_v16_s0.95_n3136": dict(M=2048, K=1024, V=16, sparsity=0.95, N=3136, batch=1,
                                                   out_f32=True, std=0.05, seed=3),
            "cfg5_ffn1_3072x768_v16_s0.9_n4096": dict(M=3072, K=768, V=16, sparsity=0.9, N=4096, batch=1,
                                                      out_f32=False, std=0.02, seed=5),
            "cfg5_ffn2_768x3072_v16_s0.9_n4096": dict(M=768, K=3072, V=16, sparsity=0.9, N=4096, batch=1,
                                                      out_f32=False, std=0.02, seed=5),
            "cfg5_ffn1_batched8": dict(M=3072, K=768, V=16, sparsity=0.9, N=4096, batch=8, out_f32=False, std=0.02,
                                       seed=5),
        }
        for name, kw in cases.items():
            res, handles = spmm_case(L, torch, synth, steps=st, warmup=wu, dense=True, **kw)
            del handles
            torch.cuda.empty_cache()
            extra[name] = res

        # SVC: cfg4 (Zipf CSR 16384^2) on the GPU against the Python RowMerge and the C oracle
        from oracle import oracle as O
        csr = synth.zipf_csr(16384, 16384, seed=4)
        rp, ci, cv = (torch.from_numpy(x).cuda() for x in (csr.row_ptr, csr.col_ind, csr.values))
        r = sspmm_amd.svc(rp, ci, cv, csr.M, csr.K, 8)
        torch.cuda.synchronize()
        svc_ms = time_launches(lambda: sspmm_amd.svc(rp, ci, cv, csr.M, csr.K, 8), 20, 3)
        # kernels only (no allocation, no host read-back)
        ws = torch.empty(L.svc_workspace_bytes(csr.M, csr.col_ind.size, 8), dtype=torch.uint8, device="cuda")
        vrp = torch.zeros(csr.M // 8 + 1, dtype=torch.int32, device="cuda")
        vcol = torch.empty(r.num_vec, dtype=torch.int32, device="cuda")
        vval = torch.empty(r.num_vec * 8, dtype=torch.float16, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream

        def svc_kernels():
            L.svc_count(csr.M, csr.K, 8, rp.data_ptr(), ci.data_ptr(), csr.col_ind.size, 0, vrp.data_ptr(),
                        ws.data_ptr(), stream)
            L.svc_fill(csr.M, csr.K, 8, rp.data_ptr(), ci.data_ptr(), cv.data_ptr(), csr.col_ind.size, 0,
                       vrp.data_ptr(), ws.data_ptr(), vcol.data_ptr(), vval.data_ptr(), stream)

        svc_k_ms = time_launches(svc_kernels, 20, 3)
        lists = O.csr_col_lists(csr.M, csr.row_ptr, csr.col_ind)
        t0 = time.perf_counter()
        ptr, flat = O.rowmerge_python(csr.M, 8, lists)
        py_ms = (time.perf_counter() - t0) * 1e3
        t0 = time.perf_counter()
        O.svc(csr.M, csr.K, 8, csr.row_ptr, csr.col_ind, csr.values)
        c_ms = (time.perf_counter() - t0) * 1e3
        same = (r.vec_row_ptr.cpu().numpy().tolist() == ptr) and (r.vec_col.cpu().numpy().tolist() == flat)
        nnz = csr.col_ind.size
        svc_bytes = synth.svc_algorithmic_bytes(csr.M, nnz, csr.M // 8, r.num_vec, 8)
        extra["svc_cfg4_zipf_16384_v8"] = {
            "gpu_ms_with_alloc_and_readback": svc_ms, "gpu_ms_kernels": svc_k_ms, "python_rowmerge_ms": py_ms,
            "c_oracle_ms": c_ms, "speedup_vs_python": py_ms / svc_k_ms, "bit_exact_vs_python": bool(same),
            "nnz": int(nnz), "nvec": int(r.num_vec), "fill_ratio": nnz / (r.num_vec * 8.0),
            "max_vector_row": int(np.diff(r.vec_row_ptr.cpu().numpy()).max()),
            "alg_bytes": svc_bytes, "hbm_gbps": svc_bytes / svc_k_ms / 1e6,
        }

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
            extra["svc_pruned_weight_2048x2048_s0.9_v%d" % Vd] = {
                "gpu_ms_with_alloc_and_readback": d_ms, "python_rowmerge_ms": d_py, "speedup_vs_python": d_py / d_ms,
                "bit_exact_vs_python": bool(rd.vec_row_ptr.cpu().numpy().tolist() == d_want_ptr and
                                            rd.vec_col.cpu().numpy().tolist() == d_want_cols),
                "nnz": int(d_col.size), "nvec": int(rd.num_vec),
            }

        # ... and the SpMM that consumes it: the skewed pattern straight from the SVC, B 16384 x 256
        N4 = 256
        B4 = torch.from_numpy(synth.dense_rhs(csr.K, N4, seed=14)).cuda()
        C4 = torch.empty(csr.M, N4, dtype=torch.float32, device="cuda")
        m_vec4 = csr.M // 8

        def spmm_cfg4():
            rc = L.sspmm_f16_f32(m_vec4, 8, N4, csr.K, None, r.vec_row_ptr.data_ptr(), r.vec_col.data_ptr(),
                                 r.vec_val.data_ptr(), B4.data_ptr(), C4.data_ptr(), stream)
            assert rc == 0, rc

        ms4 = time_launches(spmm_cfg4, st, wu)
        lens = np.diff(r.vec_row_ptr.cpu().numpy())
        touched = int(np.unique(r.vec_col.cpu().numpy()).size)
        bytes4 = synth.spmm_algorithmic_bytes(m_vec4, 8, int(r.num_vec), csr.K, N4, 4, k_touched=touched)
        extra["cfg4_spmm_on_svc_output"] = {
            "workload": "A 16384x16384 Zipf rows (nnz %d) after SVC V=8, B 16384x%d, C fp32" % (nnz, N4),
            "ms": ms4, "useful_tflops": 2.0 * nnz * N4 / ms4 / 1e9, "alg_bytes": bytes4,
            "hbm_gbps": bytes4 / ms4 / 1e6, "hbm_frac": bytes4 / ms4 / 1e6 / HBM_PEAK_GBPS,
            "kernel": kernel_names.get(L.sspmm_last_kernel(), "unknown"),
            "vector_row_len_max": int(lens.max()), "vector_row_len_mean": float(lens.mean()),
            "steps_of_longest_row": int((lens.max() + 31) // 32), "steps_total": int(((lens + 31) // 32).sum()),
        }

        # cfg5: one BERT-base shaped encoder layer (hidden 768, 12 heads, FFN 3072, 8 x 512 tokens) with
        # six vector-sparse weights (V=16, 90 %) and dense attention in torch; the same layer with dense fp16
        # matmuls on the densified weights beside it
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
        with torch.no_grad():
            y_sp = layer(x5, bsz, seq)
            y_de = layer(x5, bsz, seq, linear=lambda n, lin, t: dense_w[n] @ t)
            sp_ms = time_launches(lambda: layer(x5, bsz, seq), st, wu)
            de_ms = time_launches(lambda: layer(x5, bsz, seq, linear=lambda n, lin, t: dense_w[n] @ t), st, wu)
            per = {}
            for n in ("q", "o", "ffn1", "ffn2"):
                lin = getattr(layer, n)
                xin = torch.randn(lin.in_features, bsz * seq, device="cuda").half()
                per[n] = {"sparse_ms": time_launches(lambda: lin(xin), st, wu),
                          "dense_ms": time_launches(lambda: dense_w[n] @ xin, st, wu)}
        extra["cfg5_encoder_layer_v16_s0.9_tokens4096"] = {
            "sparse_layer_ms": sp_ms, "dense_layer_ms": de_ms, "speedup_vs_dense_layer": de_ms / sp_ms,
            "max_rel_diff_vs_dense_layer": float((y_sp.float() - y_de.float()).abs().max() / y_de.float().abs().max()),
            "projections": per,
        }

        extra["sparse_attention_seq4096_d64_v8_s0.9_heads48"] = attention_block(torch, synth, sspmm_amd, st, wu)

        # row reordering ahead of the SVC: 16384 rows that are noisy copies of 256 prototype rows, shuffled
        rc_csr = synth.clustered_csr(16384, 16384, 256, 128, seed=6, keep=0.9, extras=1)
        rrp, rci, rcv = (torch.from_numpy(x).cuda() for x in (rc_csr.row_ptr, rc_csr.col_ind, rc_csr.values))
        plain = sspmm_amd.svc(rrp, rci, rcv, rc_csr.M, rc_csr.K, 8, order="sorted")
        reo = sspmm_amd.svc_reordered(rrp, rci, rcv, rc_csr.M, rc_csr.K, 8, order="sorted")
        rws = torch.empty(L.svc_reorder_workspace_bytes(rc_csr.M), dtype=torch.uint8, device="cuda")
        rperm = torch.empty(rc_csr.M, dtype=torch.int32, device="cuda")
        o_rp, o_ci, o_cv = torch.empty_like(rrp), torch.empty_like(rci), torch.empty_like(rcv)

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
        extra["reorder_clustered_16384_v8"] = {
            "workload": "16384 x 16384 CSR, rows = noisy copies of 256 prototypes (nnz %d), shuffled; V=8" % rnnz,
            "order_ms": t_order, "order_alg_bytes": by_order, "order_hbm_gbps": by_order / t_order / 1e6,
            "apply_ms": t_apply, "apply_alg_bytes": by_apply, "apply_hbm_gbps": by_apply / t_apply / 1e6,
            "nvec_without_reordering": int(plain.num_vec), "nvec_with_reordering": int(reo.svc.num_vec),
            "fill_without_reordering": rnnz / (plain.num_vec * 8.0), "fill_with_reordering": rnnz / (reo.svc.num_vec * 8.0),
        }

    line = {
        "metric": "SpMM useful TFLOP/s (2*nnz*N/t), V=8 @90% sparsity, fp16 in / fp32 accumulate",
        "value": main_res["useful_tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": main_res["ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": main_res["workload"] + " (one launch, pattern shared by the batch)",
                   "hbm_gbps": main_res["hbm_gbps"]},
        "roofline": {"bound": "hbm", "achieved": main_res["hbm_gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": main_res["hbm_frac"],
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.batch) if args.kernel == "auto" else None,
                     "kernel": main_kernel, "alg_bytes_per_launch": main_res["alg_bytes"],
                     "measured_stream_rates": ceilings},
        "cpu_baseline": cpu,
        "parity_max_rel_err": parity,
        "dense_gemm": {k: main_res[k] for k in main_res if k.startswith("dense") or k.startswith("speedup")},
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
