"""Benchmark of the fused decompress + mean-aggregation hot path on one MI355X.

    python bench.py [--steps K] [--warmup W] [--workload c2|c1|c3|c4|c5 [--scatter]] [--idx int64|int32]

Prints ONE JSON line.  A step is one launch of the fused operator over one synthetic CSC
block, inputs resident in HBM, through the C ABI (caller-allocated output).  `value` is
edges aggregated per second over the K timed steps (wall clock between device
synchronisations); `roofline.achieved` is algorithmic bytes per launch divided by the
average launch duration measured with HIP events on the launch stream; `cpu_baseline`
is the reference's unfused CPU flow (torch dequantise + torch sparse mm) timed on this
box's host cores on a bounded sample of the same workload.

Every benchmark configuration is in that one line: next to the headline workload's `roofline`,
`configs` holds the other fused workloads (C1, C3, C3 with scattered ids, C4, C5) and the C5 encode
step, each with its own launch count, `launch_us` (and, for C3 / C4 / C5, `cold_launch_us` / `frac_cold`,
for C3 / C5 also `cold_streaming_launch_us` / `frac_cold_streaming` in the streaming store mode
with three blocks and outputs in rotation), `edges_per_s`, `algorithmic_bytes`,
`compulsory_bytes`, measured HBM `traffic` and four fractions of the 8 TB/s peak:
`frac_algorithmic` (every edge charged its source row), `frac_traffic` (the bytes the counters saw
move through HBM in such a launch: a physical rate, so it cannot exceed 1), `frac_compulsory` (every
distinct source row charged once: what no cache can avoid) and `frac`, the lesser of
`frac_algorithmic` and `frac_traffic` (a launch whose hot rows hit in cache is not credited with
bytes it never moved; one that re-reads is not credited with its re-reads).  Without a traffic
figure for these kernel sources `frac` is `min(frac_algorithmic, 1)` when the distinct rows make up
>= 0.9 of the algorithmic bytes and `frac_compulsory` otherwise.  The headline's `roofline.frac_cold` is the same kernel
with six CSC blocks and six outputs in rotation (> 600 MB pass before a buffer comes round again,
more than the 256 MB last-level cache); `frac_cold_streaming` is that rotation with the output
written by non-temporal stores (`f2cgt_set_store_mode(F2CGT_STORE_STREAM)`), which also takes the
same time on one buffer (`cold.streaming_stores.one_buffer_launch_us`).  `--workload X` measures X alone (what the rocprofv3
runs use); `--configs off` drops the extra objects.

    python bench.py --all            adds the other workloads and the streaming/encode ops
                                     under "others" (same JSON line)
    python bench.py --calibrate-copy runs plain device copies of a known size (for scaling the
                                     rocprofv3 FETCH_SIZE / WRITE_SIZE counters), no JSON
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F32_PEAK_TFLOPS = 157.3
MFMA_BF16_PEAK_TFLOPS = 2500.0



def _measured_traffic(workload, idx):
    """HBM bytes per launch from profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, each
    scaled by what the same counter reads for a plain copy of known size; written by
    `python3 -m f2cgt_amd.profile_summary`).  A figure only counts for the kernel sources it was
    measured on: None when the record is missing or the sources have changed since."""
    try:
        from f2cgt_amd import profile_summary
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as fh:
            rec = json.load(fh)
        sha = profile_summary.csrc_sha16()
        for e in rec.get("entries", []):
            if e.get("workload") == workload and e.get("idx") == idx and e.get("csrc_sha16") == sha:
                return int(e["bytes"])
    except (OSError, ValueError, KeyError):
        pass
    return None


def _launcher(capi, wl, out):
    """Returns a zero-argument callable that enqueues one fused launch (pre-bound C ABI call)."""
    import torch

    lib = capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    tag = capi.DT_I64 if wl["indptr"].dtype == torch.int64 else capi.DT_I32
    R, E = wl["R"], wl["E"]
    if wl["kind"] == "sq_affine":
        c, p = wl["codes"], wl["params"]
        args = (c.data_ptr(), p.data_ptr(), p.shape[1], wl["indptr"].data_ptr(), wl["indices"].data_ptr(), tag,
                out.data_ptr(), R, E, c.shape[0], c.shape[1], wl["feat_dim"], wl["bits"], stream)
        fn = lib.f2cgt_sq_affine_decompress_spmm_csr
    elif wl["kind"] == "vq":
        c, cb = wl["codes"], wl["codebooks"]
        args = (c.data_ptr(), capi.DT_U8, cb.data_ptr(), wl["indptr"].data_ptr(), wl["indices"].data_ptr(), tag,
                out.data_ptr(), R, E, c.shape[0], wl["feat_dim"], cb.shape[0], cb.shape[1], cb.shape[2], stream)
        fn = lib.f2cgt_vq_decompress_spmm_csr
    else:
        cb = wl["vq_codebooks"]
        args = (wl["row_map"].data_ptr(), wl["sq_codes"].data_ptr(), wl["sq_params"].data_ptr(),
                wl["sq_params"].shape[1], wl["vq_codes"].data_ptr(), cb.data_ptr(), wl["indptr"].data_ptr(),
                wl["indices"].data_ptr(), tag, out.data_ptr(), R, E, wl["row_map"].numel(),
                wl["sq_codes"].shape[0], wl["vq_codes"].shape[0], wl["feat_dim"], cb.shape[0], cb.shape[1],
                cb.shape[2], stream)
        fn = lib.f2cgt_hybrid_decompress_spmm_csr

    def step():
        rc = fn(*args)
        if rc != 0:
            raise RuntimeError("launch failed (%d): %s" % (rc, lib.f2cgt_last_error().decode()))
    return step


def _time_steps(step, steps, warmup):
    """-> (wall ms per step, HIP-event ms per launch)."""
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()           # torch's current stream: the one the C ABI launches on
    for _ in range(steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall * 1e3 / steps, ev0.elapsed_time(ev1) / steps


def _run_workload(name, idx, steps, warmup, scattered=False):
    import torch
    from f2cgt_amd import capi, synth

    idx_dtype = torch.int64 if idx == "int64" else torch.int32
    wl = synth.WORKLOADS[name](device="cuda", idx_dtype=idx_dtype)
    if scattered:
        wl = synth.scatter_ids(wl)
    out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
    ms_step, ms_launch = _time_steps(_launcher(capi, wl, out), steps, warmup)
    return wl, ms_step, ms_launch


def _fractions(wl, launch_ms, traffic):
    """The fractions of the HBM peak for one fused launch (see the module docstring)."""
    from f2cgt_amd import synth

    secs = launch_ms * 1e-3
    algo, comp = wl["algo_bytes"], synth.compulsory_bytes(wl)
    f_algo = algo / secs / 1e9 / HBM_PEAK_GBS
    f_comp = comp / secs / 1e9 / HBM_PEAK_GBS
    f_traffic = traffic / secs / 1e9 / HBM_PEAK_GBS if traffic is not None else None
    if f_traffic is not None:
        frac = min(f_algo, f_traffic)
    else:
        frac = min(f_algo, 1.0) if comp / algo >= 0.9 else f_comp
    return {"algorithmic_bytes": algo, "compulsory_bytes": comp, "traffic": traffic,
            "frac_algorithmic": f_algo, "frac_traffic": f_traffic, "frac_compulsory": f_comp, "frac": frac}


def _cold_launch_ms(name, idx, wl, blocks=6, rounds=40, warm_rounds=10):
    """Launch time with `blocks` CSC blocks and as many outputs in rotation: between two uses of
    the same graph or output buffer the other launches write blocks-1 whole outputs, so neither
    is still in the last-level cache (the tables' hot rows are, as they are in use)."""
    import torch
    from f2cgt_amd import capi, synth

    graphs = [wl] + synth.extra_blocks(wl, blocks - 1)
    steps = []
    for g in graphs:
        out = torch.empty((g["R"], g["feat_dim"]), dtype=torch.float32, device="cuda")
        steps.append(_launcher(capi, g, out))

    def one_round():
        for st in steps:
            st()

    _, ms = _time_steps(one_round, rounds, warm_rounds)
    algo = sum(g["algo_bytes"] for g in graphs) / len(graphs)
    return ms / len(graphs), algo, len(graphs)


# the other configurations in the default line: (workload, timed launches, warm-up launches, scattered ids)
CONFIG_RUNS = (("c1", 2000, 2000, False), ("c3", 300, 300, False), ("c3", 300, 300, True),
               ("c4", 100, 100, False), ("c5", 60, 60, False))


def _configs(idx):
    import torch
    from f2cgt_amd import capi, synth

    idx_dtype = torch.int64 if idx == "int64" else torch.int32
    res = {}
    for name, steps, warmup, scattered in CONFIG_RUNS:
        key = name + ("_scattered" if scattered else "")
        try:        # a failure here is reported in its entry; the headline line is printed regardless
            wl = synth.WORKLOADS[name](device="cuda", idx_dtype=idx_dtype)
            if scattered:
                wl = synth.scatter_ids(wl)
            key = wl["name"]
            out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
            ms_step, ms_launch = _time_steps(_launcher(capi, wl, out), steps, warmup)
            entry = {"steps": steps, "warmup": warmup, "launch_us": ms_launch * 1e3,
                     "edges_per_s": wl["E"] / (ms_launch * 1e-3), "bound": "hbm"}
            entry.update(_fractions(wl, ms_launch, _measured_traffic(wl["name"], idx)))
            if name in ("c3", "c4", "c5") and not scattered:
                # three blocks and outputs in rotation (each output is 256 MB or more, so more than
                # the last-level cache passes before a buffer comes round again)
                del out
                cold_ms, cold_bytes, nblk = _cold_launch_ms(name, idx, wl, blocks=3, rounds=max(4, steps // 6),
                                                            warm_rounds=max(2, warmup // 6))
                entry["cold_launch_us"] = cold_ms * 1e3
                # the warm fraction scaled by the launch times (the blocks in rotation are the same size)
                entry["frac_cold"] = entry["frac"] * ms_launch / cold_ms
                if name in ("c3", "c5"):
                    # the same rotation in the streaming store mode, which for the fused VQ operator selects the
                    # form whose store instructions write whole lines at every row length up to 16 edges
                    was = capi.set_store_mode(capi.STORE_STREAM)
                    try:
                        s_ms, _, _ = _cold_launch_ms(name, idx, wl, blocks=3, rounds=max(4, steps // 6),
                                                     warm_rounds=max(2, warmup // 6))
                    finally:
                        capi.set_store_mode(was)
                    entry["cold_streaming_launch_us"] = s_ms * 1e3
                    entry["frac_cold_streaming"] = entry["frac"] * ms_launch / s_ms
                out = None
            res[key] = entry
            del wl, out
        except RuntimeError as exc:
            res[key] = {"error": str(exc)[:200]}
        torch.cuda.empty_cache()
    enc = synth.c5_encode(device="cuda")
    labels = torch.empty((enc["m"],), dtype=torch.uint8, device="cuda")
    _, ms = _time_steps(lambda: capi.kmeans_predict(enc["x"], enc["centers"], "l2", u8=True, out=labels), 50, 20)
    tf = enc["flops"] / (ms * 1e-3) / 1e12
    res["c5_encode_l2_argmin"] = {
        "steps": 50, "warmup": 20, "launch_us": ms * 1e3, "vectors_per_s": enc["m"] / (ms * 1e-3), "bound": "mfma",
        "algorithmic_flops": enc["flops"], "algorithmic_TFLOPps": tf, "executed_bf16_mfma_TFLOPps": 6 * tf,
        "frac": 6 * tf / MFMA_BF16_PEAK_TFLOPS, "algorithmic_over_f32_mfma_peak": tf / MFMA_F32_PEAK_TFLOPS}
    return res


def _others(idx):
    """Secondary measurements: the remaining workloads, the encode step and the streaming ops."""
    import torch
    from f2cgt_amd import capi, synth

    res = {}
    for name, steps in (("c1", 2000), ("c3", 300), ("c4", 100), ("c5", 60)):
        wl, ms_step, ms_launch = _run_workload(name, idx, steps, steps)   # as many warm-up launches as timed ones
        gbs = wl["algo_bytes"] / (ms_launch * 1e-3) / 1e9
        res[wl["name"]] = {"launch_us": ms_launch * 1e3, "edges_per_s": wl["E"] / (ms_step * 1e-3),
                           "algorithmic_GBps": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS}
        del wl
        torch.cuda.empty_cache()
    # the operator at the size of a sampled minibatch block: the first R destination rows of the same
    # graphs (the reference's own test block is batch 1024 with fanout 15,
    # tests/test_fusion_decompress_spmm.py:36-90; the first layer of a three-layer sampler sees ~5e4 rows)
    for name in ("c2", "c3"):
        wl = synth.WORKLOADS[name](device="cuda", idx_dtype=torch.int64)
        row_bytes = wl["codes"].shape[1]
        fixed = wl["codebooks"].numel() * 4 if "codebooks" in wl else 2 * wl["feat_dim"] * 4
        for rows in (1024, 4096, 16384, 65536):
            small = dict(wl)
            small["indptr"] = wl["indptr"][:rows + 1].contiguous()
            small["E"] = int(small["indptr"][-1])
            small["indices"] = wl["indices"][:small["E"]].contiguous()
            small["R"] = rows
            nbytes = small["E"] * (row_bytes + 8) + (rows + 1) * 8 + rows * wl["feat_dim"] * 4 + fixed
            out = torch.empty((rows, wl["feat_dim"]), dtype=torch.float32, device="cuda")
            _, ms_launch = _time_steps(_launcher(capi, small, out), 1000, 200)
            res["%s_first_%d_rows" % (wl["name"], rows)] = {
                "launch_us": ms_launch * 1e3, "edges": small["E"], "algorithmic_GBps": nbytes / (ms_launch * 1e-3) / 1e9,
                "frac_hbm_peak": nbytes / (ms_launch * 1e-3) / 1e9 / HBM_PEAK_GBS}
            del small, out
        del wl
        torch.cuda.empty_cache()
    # source ids passed through a fixed bijection (hot rows no longer contiguous), and int32 indices
    for name, steps in (("c2", 500), ("c3", 300)):
        wl = synth.scatter_ids(synth.WORKLOADS[name](device="cuda", idx_dtype=torch.int64))
        out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
        _, ms_launch = _time_steps(_launcher(capi, wl, out), steps, steps)
        gbs = wl["algo_bytes"] / (ms_launch * 1e-3) / 1e9
        res[wl["name"]] = {"launch_us": ms_launch * 1e3, "algorithmic_GBps": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS}
        del wl, out
        torch.cuda.empty_cache()
    other_idx = "int32" if idx == "int64" else "int64"
    for name, steps in (("c2", 500), ("c3", 300), ("c4", 100)):
        wl, ms_step, ms_launch = _run_workload(name, other_idx, steps, steps)
        gbs = wl["algo_bytes"] / (ms_launch * 1e-3) / 1e9
        res[wl["name"] + "_" + other_idx] = {"launch_us": ms_launch * 1e3, "algorithmic_GBps": gbs,
                                             "frac_hbm_peak": gbs / HBM_PEAK_GBS}
        del wl
        torch.cuda.empty_cache()
    # the reference's own fused SQ operator (log-domain codes, [n,5] codebooks) on the C2 graph
    wl = synth.WORKLOADS["c2"](device="cuda", idx_dtype=torch.int64)
    out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
    logcb2 = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
    _, ms = _time_steps(lambda: capi.sq_decompress_spmm_csr(wl["codes"], logcb2, wl["indptr"], wl["indices"], 4,
                                                            wl["feat_dim"], wl["feat_dim"], out=out), 300, 30)
    res["c2_graph_log_sq4_fused"] = {"launch_us": ms * 1e3, "algorithmic_GBps": wl["algo_bytes"] / (ms * 1e-3) / 1e9,
                                     "frac_hbm_peak": wl["algo_bytes"] / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    # the headline step replayed from a captured graph of 100 launches (what a captured training step
    # sees: no host launch gap between consecutive kernels); best effort, the eager figure is the headline
    try:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            gstep = _launcher(capi, wl, out)     # binds the launches to the capture stream
            for _ in range(3):
                gstep()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(100):
                gstep()
        torch.cuda.synchronize()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        g0.record()
        for _ in range(10):
            graph.replay()
        g1.record()
        torch.cuda.synchronize()
        us = g0.elapsed_time(g1) * 1e3 / 1000
        res["c2_sq4_affine_graph_replay"] = {"launch_us": us, "algorithmic_GBps": wl["algo_bytes"] / (us * 1e-6) / 1e9,
                                             "frac_hbm_peak": wl["algo_bytes"] / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
        del graph
    except Exception as exc:  # a capture problem must not take the other measurements down
        res["c2_sq4_affine_graph_replay"] = {"error": str(exc)[:200]}
    # the uncompressed baseline operator (spmm_csr) on the same graph: fp32 rows, 400 B per edge
    feat = torch.randn((wl["N"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
    _, ms = _time_steps(lambda: capi.spmm_csr(feat, wl["indptr"], wl["indices"], out=out), 300, 30)
    nbytes = wl["E"] * (wl["feat_dim"] * 4 + 8) + (wl["R"] + 1) * 8 + wl["R"] * wl["feat_dim"] * 4
    res["c2_graph_spmm_csr_fp32"] = {"launch_us": ms * 1e3, "algorithmic_GBps": nbytes / (ms * 1e-3) / 1e9,
                                     "frac_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    del wl, out, feat
    torch.cuda.empty_cache()
    # Reddit's width, 602 columns: rows of 4 k + 2 columns start at multiples of 8 bytes only and end with a group of two
    # columns.  2e6 edges at 10 per row from 1e6 source rows, next to the same launch at 600 columns.
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    rows602, fan602, src602 = 200_000, 10, 1_000_000
    ptr602 = synth.csc_from_degrees(torch.full((rows602,), fan602, dtype=torch.int64, device="cuda"), torch.int64)
    ids602 = synth.zipf_ids(src602, (rows602 * fan602,), 1.1, gen, "cuda", torch.int64)
    cb5 = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
    for dim in (602, 600):
        o = torch.empty((rows602, dim), dtype=torch.float32, device="cuda")
        c4 = torch.randint(0, 256, (src602, dim // 2), generator=gen, device="cuda", dtype=torch.uint8)
        par = torch.stack([torch.randn(dim, device="cuda"), torch.rand(dim, device="cuda")]).contiguous()
        vc = torch.randint(0, 256, (src602, 19), generator=gen, device="cuda", dtype=torch.uint8)
        vcb = torch.randn((19, 256, 32), device="cuda")
        entry = {}
        _, ms = _time_steps(lambda: capi.sq_affine_decompress_spmm_csr(c4, par, ptr602, ids602, 4, dim, out=o), 30, 10)
        entry["affine_sq4_us"] = ms * 1e3
        _, ms = _time_steps(lambda: capi.sq_decompress_spmm_csr(c4, cb5, ptr602, ids602, 4, dim, dim, out=o), 30, 10)
        entry["log_sq4_us"] = ms * 1e3
        _, ms = _time_steps(lambda: capi.vq_decompress_spmm_csr(vc, vcb, ptr602, ids602, dim, out=o), 30, 10)
        entry["vq_19x32_us"] = ms * 1e3
        f32 = torch.randn((src602, dim), device="cuda")
        _, ms = _time_steps(lambda: capi.spmm_csr(f32, ptr602, ids602, out=o), 30, 10)
        entry["spmm_csr_fp32_us"] = ms * 1e3
        del f32
        _, ms = _time_steps(lambda: capi.sq_decompress(c4[:400_000], cb5, 4, dim, dim), 30, 10)
        entry["sq_decompress4_4e5_rows_us"] = ms * 1e3
        res["fused_and_decode_at_%d_columns" % dim] = entry
        del o, c4, par, vc, vcb
        torch.cuda.empty_cache()
    # the aggregation together with the dense layer that consumes it, at the widest shape (768
    # features -> 256 hidden units, fp32 like the reference's model): the aggregation alone, the GEMM
    # alone, the module's *_linear op (one aggregation, one GEMM), its row-blocked form (bounded
    # staging memory) and the blocked form with the next block's aggregation on a second stream
    import f2cgt_amd
    shim = f2cgt_amd.load()
    wl = synth.WORKLOADS["c5"](device="cuda", idx_dtype=torch.int64)
    hidden = 256
    weight = torch.randn((hidden, wl["feat_dim"]), device="cuda") * 0.03
    bias = torch.randn((hidden,), device="cuda")
    agg = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
    hid = torch.empty((wl["R"], hidden), dtype=torch.float32, device="cuda")
    agg_only = _launcher(capi, wl, agg)
    _, t_agg = _time_steps(agg_only, 30, 5)
    _, t_gemm = _time_steps(lambda: torch.addmm(bias, agg, weight.t(), out=hid), 30, 5)

    def two_pass():
        agg_only()
        torch.addmm(bias, agg, weight.t(), out=hid)

    _, t_two = _time_steps(two_pass, 30, 5)
    layer = {"aggregation_us": t_agg * 1e3, "gemm_fp32_us": t_gemm * 1e3, "aggregate_then_gemm_us": t_two * 1e3,
             "gemm_TFLOPps": 2 * wl["R"] * wl["feat_dim"] * hidden / (t_gemm * 1e-3) / 1e12}
    for block_rows, overlap in ((0, False), (65536, False), (131072, False), (65536, True), (131072, True)):
        _, t = _time_steps(lambda: shim.vq_decompress_spmm_csr_linear(
            wl["codes"], wl["codebooks"], wl["indptr"], wl["indices"], wl["feat_dim"], weight, bias, block_rows,
            overlap), 30, 5)
        layer["linear_op_block_%d%s_us" % (block_rows, "_overlap" if overlap else "")] = t * 1e3
    res["c5_first_layer_768_to_256"] = layer
    del wl, agg, hid, weight
    torch.cuda.empty_cache()
    enc = synth.c5_encode(device="cuda")
    labels = torch.empty((enc["m"],), dtype=torch.uint8, device="cuda")
    _, ms = _time_steps(lambda: capi.kmeans_predict(enc["x"], enc["centers"], "l2", u8=True, out=labels), 50, 5)
    tf = enc["flops"] / (ms * 1e-3) / 1e12
    # the assignment evaluates x.c from three bf16 pieces per value: six bf16 MFMAs of 2*32*32*16
    # flops per 16 dimensions and 32x32 tile, i.e. six times the algorithmic 2*m*n*k flops
    res["c5_encode_l2_argmin"] = {"launch_us": ms * 1e3, "vectors_per_s": enc["m"] / (ms * 1e-3),
                                  "algorithmic_TFLOPps": tf, "executed_bf16_mfma_TFLOPps": 6 * tf,
                                  "frac_mfma_bf16_peak": 6 * tf / MFMA_BF16_PEAK_TFLOPS,
                                  "algorithmic_over_f32_mfma_peak": tf / MFMA_F32_PEAK_TFLOPS}
    # the distance matrix itself (pairwise_distance): 9..64 dimensions go through the same split-bf16
    # matrix-core evaluation as the assignment; the 1.02 GB matrix write is the bound
    for metric in ("l2", "cosine"):
        _, t = _time_steps(lambda: capi.pairwise_distance(enc["x"], enc["centers"], metric), 20, 3)
        res["c5_pairwise_distance_" + metric] = {"launch_us": t * 1e3,
                                                 "matrix_write_GBps": enc["m"] * enc["n"] * 4 / (t * 1e-3) / 1e9,
                                                 "frac_hbm_peak": enc["m"] * enc["n"] * 4 / (t * 1e-3) / 1e9 / HBM_PEAK_GBS}
    # streaming ops at the C2 table shape
    n, d = 2_400_000, 100
    codes = torch.randint(0, 16, (n, d), dtype=torch.uint8, device="cuda")
    _, ms = _time_steps(lambda: capi.packbits(codes, 4), 50, 5)
    res["packbits_4bit_2.4Mx100"] = {"launch_us": ms * 1e3, "GBps": n * d * 1.5 / (ms * 1e-3) / 1e9}
    packed = capi.packbits(codes, 4)
    _, ms = _time_steps(lambda: capi.unpackbits(packed, 4, d), 50, 5)
    res["unpackbits_4bit_2.4Mx100"] = {"launch_us": ms * 1e3, "GBps": n * d * 1.5 / (ms * 1e-3) / 1e9}
    params = torch.rand((2, d), device="cuda")
    _, ms = _time_steps(lambda: capi.sq_affine_decompress(packed, params, 4, d), 20, 3)
    res["sq_affine_decompress_4bit_2.4Mx100"] = {"launch_us": ms * 1e3, "GBps": n * d * 4.5 / (ms * 1e-3) / 1e9}
    logcb = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
    _, ms = _time_steps(lambda: capi.sq_decompress(packed, logcb, 4, d, d), 20, 3)
    res["sq_decompress_4bit_2.4Mx100"] = {"launch_us": ms * 1e3, "GBps": n * d * 4.5 / (ms * 1e-3) / 1e9}
    # encode to storage: one pass against the callers' three (sq_compress -> cast -> packbits)
    xf = torch.randn((n, d), device="cuda")
    _, ms = _time_steps(lambda: capi.sq_encode(xf, logcb, 4, d), 20, 3)
    res["sq_encode_4bit_2.4Mx100"] = {"launch_us": ms * 1e3, "GBps": n * d * 4.5 / (ms * 1e-3) / 1e9}
    _, ms = _time_steps(lambda: capi.packbits(capi.sq_compress(xf, logcb, 4, d).to(torch.uint8), 4), 10, 2)
    res["sq_compress_cast_packbits_4bit_2.4Mx100"] = {"launch_us": ms * 1e3}
    del xf
    cb = torch.randn((16, 256, 8), device="cuda")
    vq = torch.randint(0, 256, (n, 16), dtype=torch.uint8, device="cuda")
    _, ms = _time_steps(lambda: capi.vq_decompress(vq, cb, 128), 20, 3)
    res["vq_decompress_16x8_2.4M"] = {"launch_us": ms * 1e3, "GBps": n * (16 + 512) / (ms * 1e-3) / 1e9}
    del vq, codes
    # the row fetch in front of the operators: uniform random ids (no reuse to speak of), device
    # tables; bytes = ids + rows read + rows written (+ the slot array with a cache of hot rows)
    m = 4_000_000
    ids = torch.randint(0, n, (m,), device="cuda")

    def fetch_case(name, table, hot=None, slot=None, count=m):
        idx = ids[:count]
        out = torch.empty((count, table.shape[1]), dtype=table.dtype, device="cuda")
        _, t = _time_steps(lambda: capi.fetch_rows(table, idx, hot, slot, out=out), 20, 3)
        rb = table.shape[1] * table.element_size()
        nbytes = count * (8 + 2 * rb + (4 if slot is not None else 0))
        res[name] = {"launch_us": t * 1e3, "rows_per_s": count / (t * 1e-3), "GBps": nbytes / (t * 1e-3) / 1e9}

    fetch_case("fetch_rows_16B_4M_of_2.4M", torch.randint(0, 256, (n, 16), dtype=torch.uint8, device="cuda"))
    fetch_case("fetch_rows_50B_4M_of_2.4M", packed)
    hot_ids = torch.randperm(n, device="cuda")[:n // 4]
    slot = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    slot[hot_ids] = torch.arange(hot_ids.numel(), dtype=torch.int32, device="cuda")
    fetch_case("fetch_rows_50B_4M_quarter_cached", packed, packed[hot_ids].contiguous(), slot)
    feats = torch.randn((n, d), device="cuda")
    fetch_case("fetch_rows_400B_4M_of_2.4M", feats)
    host_table = torch.empty((n, 50), dtype=torch.uint8, pin_memory=True)
    host_table.copy_(packed)
    fetch_case("fetch_rows_50B_pinned_host_1M", host_table, count=1_000_000)
    fetch_case("fetch_rows_50B_pinned_host_1M_quarter_cached", host_table, packed[hot_ids].contiguous(), slot,
               count=1_000_000)
    del host_table, feats, packed, slot, hot_ids
    torch.cuda.empty_cache()
    # a minibatch as the training loop sees it (examples/tensor_cache.py:49-58 then the fused operator):
    # the block's distinct source ids are fetched into a gathered copy and aggregated through block-local
    # ids, against the fused operator reading the device-resident table through global ids
    for name in ("c2", "c3"):
        wl = synth.WORKLOADS[name](device="cuda", idx_dtype=torch.int64)
        input_nodes, local = torch.unique(wl["indices"], return_inverse=True)
        codes = wl["codes"]
        gathered = torch.empty((input_nodes.numel(), codes.shape[1]), dtype=codes.dtype, device="cuda")
        out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
        local_wl = dict(wl, codes=gathered, indices=local.contiguous(), N=int(input_nodes.numel()))
        fused_local, fused_global = _launcher(capi, local_wl, out), _launcher(capi, wl, out)
        ids = torch.empty_like(wl["indices"])

        def two_step():
            capi.fetch_rows(codes, input_nodes, None, None, out=gathered)
            fused_local()

        def on_global_ids():
            torch.index_select(input_nodes, 0, local, out=ids)      # compose block-local ids into global ones
            fused_global()

        _, t2 = _time_steps(two_step, 200, 50)
        _, tg = _time_steps(on_global_ids, 200, 50)
        _, t0 = _time_steps(fused_global, 200, 50)
        res[wl["name"] + "_minibatch_flow"] = {
            "distinct_source_rows": int(input_nodes.numel()), "fetch_then_aggregate_us": t2 * 1e3,
            "compose_ids_then_aggregate_global_us": tg * 1e3, "aggregate_on_given_global_ids_us": t0 * 1e3}
        del wl, local_wl, gathered, out, ids, local, input_nodes, codes
        torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    # 5000 launches of ~25 us: the card's clocks and caches settle over ~100 ms, and a warm-up of
    # 100 launches (2.5 ms) leaves the timed region ~2 % slower on the same box.
    ap.add_argument("--warmup", type=int, default=5000)
    ap.add_argument("--workload", default=None, choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--configs", default="auto", choices=["auto", "on", "off"],
                    help="the other configurations and the cold-cache headline in the same line "
                         "(auto: on unless --workload is given)")
    ap.add_argument("--scatter", action="store_true",
                    help="with --workload: pass the source ids through a fixed bijection (hot rows no longer neighbours)")
    ap.add_argument("--idx", default="int64", choices=["int64", "int32"])
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the cpu_baseline leg (0 = skip)")
    ap.add_argument("--all", action="store_true", help="also measure the other workloads and ops")
    ap.add_argument("--calibrate-copy", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print("calibration: 5 device copies of %d bytes each (read %d, write %d per dispatch)"
              % (src.numel(), src.numel(), src.numel()))
        return

    with_configs = args.configs == "on" or (args.configs == "auto" and args.workload is None)
    if args.scatter and args.workload is None:
        ap.error("--scatter needs --workload (the headline line is measured on the workload as generated)")
    args.workload = args.workload or "c2"
    wl, ms_per_step, launch_ms = _run_workload(args.workload, args.idx, args.steps, args.warmup, args.scatter)
    achieved = wl["algo_bytes"] / (launch_ms * 1e-3) / 1e9
    traffic = _measured_traffic(wl["name"], args.idx)
    fr = _fractions(wl, launch_ms, traffic)
    result = {
        "metric": "edges aggregated/sec, fused decompress-SpMM",
        "value": wl["E"] / (ms_per_step * 1e-3),
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": wl["name"], "index_dtype": args.idx, "dst_rows": wl["R"], "edges": wl["E"],
                   "src_rows": wl["N"], "feat_dim": wl["feat_dim"], "algorithmic_bytes": wl["algo_bytes"]},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": fr["frac"], "traffic": traffic, "launch_us": launch_ms * 1e3,
                     "frac_algorithmic": fr["frac_algorithmic"], "frac_traffic": fr["frac_traffic"],
                     "frac_compulsory": fr["frac_compulsory"],
                     "compulsory_bytes": fr["compulsory_bytes"]},
        "cpu_baseline": None,
    }
    if with_configs:
        from f2cgt_amd import capi

        cold_ms, cold_bytes, nblk = _cold_launch_ms(args.workload, args.idx, wl)
        result["roofline"]["frac_cold"] = cold_bytes / (cold_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        result["roofline"]["cold"] = {"launch_us": cold_ms * 1e3, "blocks_in_rotation": nblk,
                                      "algorithmic_bytes": cold_bytes}
        # the same rotation, and the one-buffer loop, with the output streamed past the caches
        was = capi.set_store_mode(capi.STORE_STREAM)
        try:
            s_cold_ms, _, _ = _cold_launch_ms(args.workload, args.idx, wl)
            out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
            _, s_warm_ms = _time_steps(_launcher(capi, wl, out), 1000, 300)
            del out
        finally:
            capi.set_store_mode(was)
        result["roofline"]["frac_cold_streaming"] = cold_bytes / (s_cold_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        result["roofline"]["cold"]["streaming_stores"] = {"launch_us": s_cold_ms * 1e3,
                                                          "one_buffer_launch_us": s_warm_ms * 1e3}

    if args.cpu_seconds > 0:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import f2cgt_cpu_path as cp

        cores = os.cpu_count() or 1
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        torch.set_num_threads(cores)
        host = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in wl.items()}
        rows = min(wl["R"], 250_000)
        _, secs, relabel_secs = cp.run(host, rows)        # warm-up, also sizes the sample
        edges = int(host["indptr"][rows])
        # repeat the sample until the budget (default 15 s of CPU work) is used, at least 3 times
        reps = max(3, min(500, int(args.cpu_seconds / max(secs + relabel_secs, 1e-3))))
        times = sorted(cp.run(host, rows)[1] for _ in range(reps))
        med = times[len(times) // 2]
        result["cpu_baseline"] = {
            "value": edges / med, "unit": "edges/s", "cores": cores, "kind": "port",
            "sample": "first %d of %d destination rows (%d edges), torch gather+dequantise+sparse mm, "
                      "median of %d; unique+relabel (%.3f s) timed separately and excluded"
                      % (rows, wl["R"], edges, reps, relabel_secs),
        }
    del wl
    torch.cuda.empty_cache()
    if with_configs:
        result["configs"] = _configs(args.idx)
    if args.all:
        result["others"] = _others(args.idx)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
