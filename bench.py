"""Benchmark of the fused decompress + mean-aggregation hot path on one MI355X.

    python bench.py [--steps K] [--warmup W] [--workload c2|c1|c3|c4|c5] [--idx int64|int32]

Prints ONE JSON line.  A step is one launch of the fused operator over one synthetic CSC
block, inputs resident in HBM, through the C ABI (caller-allocated output).  `value` is
edges aggregated per second over the K timed steps (wall clock between device
synchronisations); `roofline.achieved` is algorithmic bytes per launch divided by the
average launch duration measured with HIP events on the launch stream; `cpu_baseline`
is the reference's unfused CPU flow (torch dequantise + torch sparse mm) timed on this
box's host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, scaled by the
# same counters on a plain copy kernel of known size); see profiles/.  None = not measured.
MEASURED_TRAFFIC_BYTES = {}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--idx", default="int64", choices=["int64", "int32"])
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the cpu_baseline leg (0 = skip)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch
    from f2cgt_amd import capi, synth

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    idx_dtype = torch.int64 if args.idx == "int64" else torch.int32
    wl = synth.WORKLOADS[args.workload](device="cuda", idx_dtype=idx_dtype)
    out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")

    if wl["kind"] == "sq_affine":
        def step():
            capi.sq_affine_decompress_spmm_csr(wl["codes"], wl["params"], wl["indptr"], wl["indices"],
                                               wl["bits"], wl["feat_dim"], out=out)
    elif wl["kind"] == "vq":
        def step():
            capi.vq_decompress_spmm_csr(wl["codes"], wl["codebooks"], wl["indptr"], wl["indices"],
                                        wl["feat_dim"], out=out)
    else:
        def step():
            capi.hybrid_decompress_spmm_csr(wl["row_map"], wl["sq_codes"], wl["sq_params"], wl["vq_codes"],
                                            wl["vq_codebooks"], wl["indptr"], wl["indices"], wl["feat_dim"],
                                            out=out)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()           # same stream the C ABI launches on (torch's current stream)
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    launch_ms = ev0.elapsed_time(ev1) / args.steps
    ms_per_step = wall * 1e3 / args.steps

    achieved = wl["algo_bytes"] / (launch_ms * 1e-3) / 1e9
    traffic = MEASURED_TRAFFIC_BYTES.get((wl["name"], args.idx))
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
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "launch_us": launch_ms * 1e3},
        "cpu_baseline": None,
    }

    if args.cpu_seconds > 0:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import f2cgt_cpu_path as cp

        cores = os.cpu_count() or 1
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        torch.set_num_threads(cores)
        host = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in wl.items()}
        rows = min(wl["R"], 100_000)
        _, secs, relabel_secs = cp.run(host, rows)        # warm-up, also sizes the sample
        edges = int(host["indptr"][rows])
        reps = max(1, min(5, int(args.cpu_seconds / max(secs + relabel_secs, 1e-3))))
        times = sorted(cp.run(host, rows)[1] for _ in range(reps))
        med = times[len(times) // 2]
        result["cpu_baseline"] = {
            "value": edges / med, "unit": "edges/s", "cores": cores, "kind": "port",
            "sample": "first %d of %d destination rows (%d edges), torch gather+dequantise+sparse mm, "
                      "median of %d; unique+relabel (%.3f s) timed separately and excluded"
                      % (rows, wl["R"], edges, reps, relabel_secs),
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
