"""Time-stamp traces of two kernels, for the library built with `python -m f2cgt_amd.build --experiments`
(the shipped build has neither the time-stamped kernel forms nor the entry points used here).

    python3 -m f2cgt_amd.experiments wave-age c3|c5      per-wave start / first step / end of vq_wave_kernel
    python3 -m f2cgt_amd.experiments block-phases c1|c2|c4  per-workgroup phase times of sq_affine_acc_kernel / hybrid_acc_kernel
    python3 -m f2cgt_amd.experiments mfma-overlap x      fp32 MFMA and LDS-gather work on one SIMD: side by side or one after the other?
    python3 -m f2cgt_amd.experiments dispatch-cost c4    the two-table kernel's grid with workgroups that return at once
    python3 -m f2cgt_amd.experiments hot-rows c4         the two-table kernel with the hottest source rows copied to LDS
    python3 -m f2cgt_amd.experiments affine-geometry x   the affine kernel by edges per row: edge mapping, accumulator sizing, block rows, workgroup size
    python3 -m f2cgt_amd.experiments hybrid-geometry x   the two-table kernel by edges per row: workgroup size and edge batch
    python3 -m f2cgt_amd.experiments vq-degrees x        the fused VQ kernel on uniform and ragged rows: rows per mini-block
    python3 -m f2cgt_amd.experiments vq-store-forms warm|rotate   the fused VQ kernel's store forms by shape
    python3 -m f2cgt_amd.experiments store-form x        plain against non-temporal output stores by shape (any build)
    python3 -m f2cgt_amd.experiments lds-rate x          bytes per clock and CU that conflict-free LDS reads return
    python3 -m f2cgt_amd.experiments cold-parts c2|c3|c4|c5   launch time by what of the input is still cached (any build)

The first two run the workload of `bench.py --workload <w>` warm, switch the trace buffer on for a few launches and
print percentiles of the last one (times in us from the earliest stamp of the launch; the stamps are
`wall_clock64()`, 100 MHz).
"""
from __future__ import annotations

import ctypes
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _q(x):
    return " ".join("%7.2f" % v for v in np.percentile(x, [0, 5, 25, 50, 75, 95, 100]))


def _setup(name):
    import torch

    sys.path.insert(0, ROOT)
    import bench
    from f2cgt_amd import capi, synth

    lib = capi.lib()
    wl = synth.WORKLOADS[name](device="cuda", idx_dtype=torch.int64)
    out = torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda")
    return torch, lib, wl, bench._launcher(capi, wl, out), out


def wave_age(name):
    os.environ["F2CGT_VQ_DEFER"] = "9"   # selects the time-stamped form of vq_wave_kernel
    torch, lib, wl, step, _ = _setup(name)
    if not hasattr(lib, "f2cgt_experiment_set_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    lib.f2cgt_experiment_set_trace.argtypes = [ctypes.c_void_p]
    lib.f2cgt_experiment_set_trace.restype = None
    trace = torch.zeros((4096 * 4,), dtype=torch.int64, device="cuda")   # 256 workgroups x 16 waves x 4 words
    for _ in range(50):
        step()
    torch.cuda.synchronize()
    lib.f2cgt_experiment_set_trace(ctypes.c_void_p(trace.data_ptr()))
    for _ in range(20):
        step()
    torch.cuda.synchronize()
    lib.f2cgt_experiment_set_trace(None)
    full = trace.cpu().numpy().reshape(-1, 4).astype(np.float64)
    valid = full[:, 2] > 0
    t = full[valid]
    t0 = t[:, 0].min()
    start, first, end = (t[:, 0] - t0) / 100.0, (t[:, 1] - t0) / 100.0, (t[:, 2] - t0) / 100.0
    print(name, "waves with rows:", len(t), " steps per wave: %d .. %d" % (t[:, 3].min(), t[:, 3].max()))
    print("  percentiles                0      5     25     50     75     95    100")
    print("  wave start us        :", _q(start))
    print("  first step us        :", _q(first))
    print("  wave end us          :", _q(end))
    print("  busy fraction of the wave slots (mean wave lifetime / launch): %.3f" % ((end - start).mean() / end.max()))
    ends = np.where(valid, (full[:, 2] - t0) / 100.0, np.nan).reshape(-1, 16)
    rows = ~np.isnan(ends).all(axis=1)
    wg_end, wg_min = np.nanmax(ends[rows], axis=1), np.nanmin(ends[rows], axis=1)
    print("  workgroup end us     :", _q(wg_end))
    print("  spread in a workgroup:", _q(wg_end - wg_min))
    print("  mean end by wave index in the workgroup:", " ".join("%.0f" % v for v in np.nanmean(ends[rows], axis=0)))
    for x in range(8):
        sub = ends[x::8]
        sub = sub[~np.isnan(sub).all(axis=1)]
        print("   workgroups with id %% 8 == %d (one XCD): mean wave end %.1f, last %.1f" % (x, np.nanmean(sub), np.nanmax(sub)))


def block_phases(name):
    torch, lib, wl, step, _ = _setup(name)
    if not hasattr(lib, "f2cgt_experiment_set_acc_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    lib.f2cgt_experiment_set_acc_trace.argtypes = [ctypes.c_void_p]
    lib.f2cgt_experiment_set_acc_trace.restype = None
    # 8 words per workgroup; the two-table kernel runs workgroups of at least 8 rows
    trace = torch.zeros((max(65536, wl["R"] // 8 + 1) * 8,), dtype=torch.int64, device="cuda")
    for _ in range(3000 if wl["R"] <= 300_000 else 100):
        step()
    torch.cuda.synchronize()
    lib.f2cgt_experiment_set_acc_trace(ctypes.c_void_p(trace.data_ptr()))
    for _ in range(50 if wl["R"] <= 300_000 else 5):
        step()
    torch.cuda.synchronize()
    lib.f2cgt_experiment_set_acc_trace(None)
    t = trace.cpu().numpy().reshape(-1, 8)
    t = t[t[:, 4] > 0].astype(np.float64)
    T = (t[:, :5] - t[:, 0].min()) / 100.0
    print(name, "workgroups:", len(t), " launch length %.2f us (first stamp to last)" % T[:, 4].max())
    print("  percentiles                        0      5     25     50     75     95    100")
    print("  workgroup start us           :", _q(T[:, 0]))
    print("  workgroup end us             :", _q(T[:, 4]))
    print("  workgroup duration us        :", _q(T[:, 4] - T[:, 0]))
    print("  phase: row offsets           :", _q(T[:, 1] - T[:, 0]))
    print("  phase: source ids and tags   :", _q(T[:, 2] - T[:, 1]))
    print("  phase: gather of the code rows:", _q(T[:, 3] - T[:, 2]))
    print("  phase: finalize and store    :", _q(T[:, 4] - T[:, 3]))
    width = 1.0 if T[:, 4].max() < 60 else 10.0
    for lo in np.arange(0.0, T[:, 4].max(), width):
        hi = lo + width
        print("  t = %3.0f .. %3.0f us: %5d workgroups resident, %5d started, %5d ended"
              % (lo, hi, ((T[:, 0] < hi) & (T[:, 4] > lo)).sum(), ((T[:, 0] >= lo) & (T[:, 0] < hi)).sum(),
                 ((T[:, 4] >= lo) & (T[:, 4] < hi)).sum()))
    hw, xcc = t[:, 5].astype(np.int64), t[:, 6].astype(np.int64) & 0xf
    key = xcc * 4096 + ((hw >> 13) & 7) * 512 + ((hw >> 12) & 1) * 16 + ((hw >> 8) & 0xf)
    _, count = np.unique(key, return_counts=True)
    print("  distinct CUs: %d, workgroups per CU min / mean / max: %d / %.1f / %d" % (len(count), count.min(), count.mean(), count.max()))
    # Residency per CU from the stamps themselves: time-weighted mean, the most ever resident, and how long a
    # CU waits from the end of one workgroup to the start of its next one.
    dur = T[:, 4] - T[:, 0]
    print("  workgroups resident per CU, time-weighted mean over the launch: %.1f" % (dur.sum() / T[:, 4].max() / len(count)))
    peak, refill, steady = [], [], []
    for k in np.unique(key)[:: max(1, len(count) // 64)]:
        sel = key == k
        st, en = np.sort(T[sel, 0]), np.sort(T[sel, 4])
        ev = np.concatenate([np.stack([st, np.ones_like(st)], 1), np.stack([en, -np.ones_like(en)], 1)])
        ev = ev[np.lexsort((ev[:, 1], ev[:, 0]))]
        level = np.cumsum(ev[:, 1])
        peak.append(level.max())
        mid = (ev[:-1, 0] > 0.2 * T[:, 4].max()) & (ev[:-1, 0] < 0.8 * T[:, 4].max())
        steady.append((level[:-1][mid] * np.diff(ev[:, 0])[mid]).sum() / max(np.diff(ev[:, 0])[mid].sum(), 1e-9))
        nxt = np.searchsorted(st, en, side="left")
        ok = nxt < len(st)
        refill.append(st[nxt[ok]] - en[ok])
    refill = np.concatenate(refill)
    print("  (every %d-th CU) most resident at once min / median / max: %d / %d / %d; mean resident in the middle 60 %% of the launch: %.1f"
          % (max(1, len(count) // 64), min(peak), int(np.median(peak)), max(peak), float(np.mean(steady))))
    print("  from a workgroup's last stamp to the next start on its CU, us:", _q(refill))


def dispatch_cost(name):
    """What the grid of the two-table kernel costs to dispatch: the same launch with workgroups that return at
    their first instruction (the trace pointer 1 asks for that), next to the full launch."""
    torch, lib, wl, step, _ = _setup(name)
    if not hasattr(lib, "f2cgt_experiment_set_acc_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    sys.path.insert(0, ROOT)
    import bench

    lib.f2cgt_experiment_set_acc_trace.argtypes = [ctypes.c_void_p]
    lib.f2cgt_experiment_set_acc_trace.restype = None
    _, ms = bench._time_steps(step, 40, 10)
    print("%s launch %.1f us" % (name, ms * 1e3))
    lib.f2cgt_experiment_set_acc_trace(ctypes.c_void_p(1))
    _, ms = bench._time_steps(step, 40, 10)
    lib.f2cgt_experiment_set_acc_trace(None)
    print("the same grid, every workgroup returning at once: %.1f us" % (ms * 1e3))


def hot_rows(name):
    """The two-table kernel with the first 32 / 64 rows of the SQ table (the hottest ones of the synthetic
    workloads) copied into every workgroup's LDS and gathered from there (F2CGT_HYB_HOT), against the shipped
    gather through L1: launch times, and that the results are the same."""
    torch, lib, wl, step, out = _setup(name)
    if not hasattr(lib, "f2cgt_experiment_set_acc_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    sys.path.insert(0, ROOT)
    import bench

    ids = wl["indices"]
    m = wl["row_map"][ids.long()]
    for h in (32, 64):
        print("%s: %.3f of the edges name one of the first %d rows of the SQ table"
              % (name, float(((m >= 0) & (m < h)).float().mean()), h))
    os.environ.pop("F2CGT_HYB_HOT", None)
    step()
    torch.cuda.synchronize()
    ref = out.clone()
    for rnd in range(2):
        for h in (0, 32, 64):
            if h:
                os.environ["F2CGT_HYB_HOT"] = str(h)
            else:
                os.environ.pop("F2CGT_HYB_HOT", None)
            out.zero_()
            step()
            torch.cuda.synchronize()
            same = bool(torch.equal(out, ref))
            _, ms = bench._time_steps(step, 40, 10)
            print("  hot rows in LDS: %2d   launch %.1f us   result identical: %s" % (h, ms * 1e3, same), flush=True)
    os.environ.pop("F2CGT_HYB_HOT", None)


def _affine_case(torch, synth, gen, n_src, bits, dim, rows, fanout):
    """Codes, parameters and a fixed-fanout CSC block with Zipf(1.1) source ids for the affine kernel."""
    codes = torch.randint(0, 256, (n_src, dim * bits // 8), generator=gen, device="cuda", dtype=torch.uint8)
    params = torch.stack([torch.randn(dim, device="cuda"), torch.rand(dim, device="cuda") * 0.05 + 0.01]).contiguous()
    deg = torch.full((rows,), fanout, dtype=torch.int64, device="cuda")
    indptr = synth.csc_from_degrees(deg, torch.int64)
    ids = synth.zipf_ids(n_src, (rows * fanout,), 1.1, gen, "cuda", torch.int64)
    return codes, params, indptr, ids


def affine_geometry(_):
    """The affine row-block kernel at 3e6 edges over a range of edges per row: the shipped choices against the
    interleaved edge-to-lane-group mapping, the accumulators sized for the narrow layout (4-bit codes: long
    rows then take two passes), eight rows per block, and 64-thread workgroups (F2CGT_ACC_CHUNK,
    F2CGT_ACC_WIDE_FULL, F2CGT_ACC_RB, F2CGT_ACC_TB; experiments build)."""
    import torch

    sys.path.insert(0, ROOT)
    import bench
    from f2cgt_amd import capi, synth

    if not hasattr(capi.lib(), "f2cgt_experiment_set_acc_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    knobs = ("F2CGT_ACC_TB", "F2CGT_ACC_RB", "F2CGT_ACC_CHUNK", "F2CGT_ACC_WIDE_FULL")
    cases = (("shipped", {}), ("interleaved", {"F2CGT_ACC_CHUNK": "0"}), ("narrow-sized", {"F2CGT_ACC_WIDE_FULL": "0"}),
             ("8 rows", {"F2CGT_ACC_RB": "8"}), ("64 threads, 8 rows", {"F2CGT_ACC_TB": "64", "F2CGT_ACC_RB": "8"}))
    print("us per launch, 2.4e6 source rows, 3e6 edges: " + " | ".join(name for name, _ in cases))
    for bits in (4, 8):
        for dim in (100, 128):
            for fanout in (3, 5, 8, 10, 12, 14, 17, 18, 20, 25, 30, 40):
                rows = 3_000_000 // fanout
                codes, params, indptr, ids = _affine_case(torch, synth, gen, 2_400_000, bits, dim, rows, fanout)
                out = torch.empty((rows, dim), dtype=torch.float32, device="cuda")
                step = lambda: capi.sq_affine_decompress_spmm_csr(codes, params, indptr, ids, bits, dim, out=out)
                best = {}
                for _ in range(2):
                    for name, env in cases:
                        for k in knobs:
                            os.environ.pop(k, None)
                        os.environ.update(env)
                        _, ms = bench._time_steps(step, 30, 10)
                        best[name] = min(best.get(name, 1e9), ms * 1e3)
                for k in knobs:
                    os.environ.pop(k, None)
                print("  %d bit, %3d columns, %2d edges per row: " % (bits, dim, fanout)
                      + " | ".join("%6.1f" % best[name] for name, _ in cases), flush=True)


def hybrid_geometry(_):
    """The two-table kernel over edges per row and row width: the shipped choice of workgroup size and edge batch
    against fixed ones (F2CGT_HYB_TB threads x F2CGT_HYB_BATCH edges per thread; experiments build)."""
    import torch

    sys.path.insert(0, ROOT)
    import bench
    from f2cgt_amd import capi, synth

    if not hasattr(capi.lib(), "f2cgt_experiment_set_acc_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    cases = (("shipped", None), ("64x4", ("64", "4")), ("128x4", ("128", "4")), ("128x8", ("128", "8")),
             ("128x16", ("128", "16")), ("256x4", ("256", "4")), ("256x8", ("256", "8")))
    print("us per launch, 2e7-node tables, 1.2e7 edges x 128 / columns: " + " | ".join(name for name, _ in cases))
    for dim, n_cb in ((64, 4), (128, 8), (256, 16)):
        for fanout in (2, 5, 12, 20, 32, 48, 64, 80, 128, 200):
            rows = int(12_000_000 / fanout / (dim / 128))
            wl = synth.c4_hybrid(device="cuda", idx_dtype=torch.int64, N=20_000_000, D=dim, n_cb=n_cb, w=16, R=rows,
                                 fanout=fanout)
            out = torch.empty((rows, dim), dtype=torch.float32, device="cuda")
            step = bench._launcher(capi, wl, out)
            best = {}
            for _ in range(2):
                for name, env in cases:
                    os.environ.pop("F2CGT_HYB_TB", None)
                    os.environ.pop("F2CGT_HYB_BATCH", None)
                    if env:
                        if env[0] == "64" and fanout * 8 > 64 * int(env[1]):
                            continue   # several batches per block: minutes per launch at the large sizes
                        os.environ["F2CGT_HYB_TB"], os.environ["F2CGT_HYB_BATCH"] = env
                    _, ms = bench._time_steps(step, 15, 4)
                    best[name] = min(best.get(name, 1e9), ms * 1e3)
            os.environ.pop("F2CGT_HYB_TB", None)
            os.environ.pop("F2CGT_HYB_BATCH", None)
            print("  %3d columns, %3d edges per row: " % (dim, fanout)
                  + " | ".join(("%6.1f" % best[name]) if name in best else "     -" for name, _ in cases), flush=True)
            del wl, out
            torch.cuda.empty_cache()


def vq_degrees(_):
    """The fused VQ kernel (16 codebooks of 8 columns) on uniform rows and on rows capped at a fanout whose degrees
    come from a heavy-tailed distribution: the shipped choice of rows per mini-block against four, two and one
    (F2CGT_VQ_RPM; experiments build).  Mini-blocks above 64 edges go through the staging in slices."""
    import torch

    sys.path.insert(0, ROOT)
    import bench
    from f2cgt_amd import capi, synth

    if not hasattr(capi.lib(), "f2cgt_experiment_set_acc_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    base = synth.c3_vq(device="cuda", idx_dtype=torch.int64, N=10_000_000, n_cb=16, K=256, w=8, R=1000, fanout=2)

    def case(name, deg):
        rows = deg.numel()
        indptr = synth.csc_from_degrees(deg.to(torch.int64), torch.int64)
        edges = int(indptr[-1])
        wl = dict(base)
        wl.update(indptr=indptr, indices=synth.zipf_ids(10_000_000, (edges,), 1.1, gen, "cuda", torch.int64), R=rows, E=edges)
        out = torch.empty((rows, 128), dtype=torch.float32, device="cuda")
        step = bench._launcher(capi, wl, out)
        res = []
        for rpm in ("", "4", "2", "1"):
            os.environ.pop("F2CGT_VQ_RPM", None)
            if rpm:
                os.environ["F2CGT_VQ_RPM"] = rpm
            _, ms = bench._time_steps(step, 10, 3)
            res.append(ms * 1e3)
        os.environ.pop("F2CGT_VQ_RPM", None)
        print("  %-38s mean %6.2f, longest %4d, %8d edges: %7.1f | %7.1f | %7.1f | %7.1f"
              % (name, edges / rows, int(deg.max()), edges, *res), flush=True)

    print("us per launch: shipped | four | two | one row per mini-block")
    rows = 400_000
    for fanout in (15, 16, 20, 25, 32, 40, 64, 80, 200):
        n = rows if fanout <= 80 else rows // 4
        case("every row %d edges" % fanout, torch.full((n,), fanout, device="cuda"))
        if fanout > 80:
            continue
        u = torch.rand((rows,), generator=gen, device="cuda")
        for scale in (0.5, 1.0, 3.0):
            raw = (scale * fanout * (1.0 - u).pow(-1.0 / 1.5)).floor().clamp(min=1)
            raw = (raw * torch.rand((rows,), generator=gen, device="cuda")).ceil()
            case("capped at %d, scale %.1f" % (fanout, scale), raw.clamp(max=fanout))


def vq_store_forms(how):
    """The fused VQ kernel's ways of storing a lane's eight columns (F2CGT_VQ_STORE; experiments build): as they are
    (two 16-byte stores that each write 16 of every 32 bytes), turned round in LDS (256 contiguous bytes per row and
    instruction), halves exchanged inside lane quads (64 contiguous bytes), columns owned by groups of four lanes
    (codebooks of 32 columns: 64 contiguous bytes at no cost in instructions), and one float4 per lane (32 lanes per
    row).  `warm`: one graph and one output; `rotate`: five graphs and outputs in turn, so that neither the source ids
    nor the output lines of a launch are cached when it starts."""
    import torch

    sys.path.insert(0, ROOT)
    from f2cgt_amd import capi, synth

    if not hasattr(capi.lib(), "f2cgt_experiment_set_acc_trace"):
        raise SystemExit("the library in tree was built without --experiments")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    copies = 5 if how == "rotate" else 1

    def timed(fns, steps=30, warm=10):
        for i in range(warm):
            fns[i % len(fns)]()
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for i in range(steps):
            fns[i % len(fns)]()
        t1.record()
        torch.cuda.synchronize()
        return t0.elapsed_time(t1) / steps * 1e3

    forms = ("", "plain", "lds", "quad", "own", "h1")
    print("us per launch (%s): shipped | plain | through LDS | quad exchange | groups of four lanes | one float4 per lane"
          % how)
    shapes = [(1_000_000, d, w, f, 3_000_000 if d <= 256 else 2_000_000)
              for w, d in ((8, 128), (8, 256), (8, 512), (8, 768), (16, 128), (16, 256), (16, 512), (32, 128), (32, 256),
                           (32, 768), (8, 64), (8, 200), (32, 600))
              for f in (5, 8, 10, 12, 14, 16)]
    shapes += [(10_000_000, 128, 8, 15, 7_500_000), (10_000_000, 128, 8, 10, 5_000_000), (10_000_000, 256, 16, 10, 3_000_000),
               (240_000_000, 768, 32, 10, 6_000_000)]
    for n_src, dim, w, fanout, edges in shapes:
        rows = edges // fanout
        n_cb = (dim + w - 1) // w
        codes = torch.randint(0, 256, (n_src, n_cb), generator=gen, device="cuda", dtype=torch.uint8)
        cbs = torch.randn((n_cb, 256, w), device="cuda")
        indptr = synth.csc_from_degrees(torch.full((rows,), fanout, dtype=torch.int64, device="cuda"), torch.int64)
        ids = [synth.zipf_ids(n_src, (rows * fanout,), 1.1, gen, "cuda", torch.int64) for _ in range(copies)]
        outs = [torch.empty((rows, dim), dtype=torch.float32, device="cuda") for _ in range(copies)]
        fns = [(lambda i=i: capi.vq_decompress_spmm_csr(codes, cbs, indptr, ids[i], dim, out=outs[i])) for i in range(copies)]
        res = []
        for form in forms:
            os.environ.pop("F2CGT_VQ_STORE", None)
            if form == "own" and not (w == 32 and dim % 32 == 0):
                res.append(float("nan"))
                continue
            if form:
                os.environ["F2CGT_VQ_STORE"] = form
            res.append(timed(fns))
        os.environ.pop("F2CGT_VQ_STORE", None)
        print("  %9d source rows, %3d columns as %2d x %-2d, %2d edges per row, %4d MB out: " % (
            n_src, dim, n_cb, w, fanout, rows * dim * 4 // 1_000_000)
            + " | ".join("     -" if r != r else "%6.1f" % r for r in res), flush=True)
        del codes, ids, outs, fns
        torch.cuda.empty_cache()


def store_form(_):
    """Plain against non-temporal output stores of the two SQ row-block kernels by output size, row width and
    edges per row, and what the default picks (f2cgt_set_store_mode; any build)."""
    import torch

    sys.path.insert(0, ROOT)
    import bench
    from f2cgt_amd import capi, synth

    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    logcb = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
    print("us per launch: default | plain | non-temporal")
    for bits, dim in ((8, 128), (4, 100)):
        for fanout in (3, 10):
            for out_mb in (64, 100, 128, 160, 200, 240):
                rows = int(out_mb * 1e6 / (dim * 4))
                codes, params, indptr, ids = _affine_case(torch, synth, gen, 2_400_000, bits, dim, rows, fanout)
                out = torch.empty((rows, dim), dtype=torch.float32, device="cuda")
                signed = codes.view(torch.int8) if bits == 8 else codes
                forms = (("affine", lambda: capi.sq_affine_decompress_spmm_csr(codes, params, indptr, ids, bits, dim, out=out)),
                         ("log", lambda: capi.sq_decompress_spmm_csr(signed, logcb, indptr, ids, bits, dim, dim, out=out)))
                for form, step in forms:
                    best = {}
                    for _ in range(2):
                        for name, mode in (("default", capi.STORE_AUTO), ("plain", capi.STORE_CACHED), ("nt", capi.STORE_STREAM)):
                            capi.set_store_mode(mode)
                            _, ms = bench._time_steps(step, 30, 10)
                            best[name] = min(best.get(name, 1e9), ms * 1e3)
                    capi.set_store_mode(capi.STORE_AUTO)
                    print("  %-6s %d bit, %3d columns, %2d edges per row, %3d MB of output: %6.1f | %6.1f | %6.1f"
                          % (form, bits, dim, fanout, out_mb, best["default"], best["plain"], best["nt"]), flush=True)


def mfma_overlap(_):
    """Times the four arrangements of csrc/overlap_probe.hip on every CU and prints what each costs."""
    import torch

    sys.path.insert(0, ROOT)
    from f2cgt_amd import capi

    lib = capi.lib()
    if not hasattr(lib, "f2cgt_experiment_overlap_probe"):
        raise SystemExit("the library in tree was built without --experiments")
    fn = lib.f2cgt_experiment_overlap_probe
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    fn.restype = ctypes.c_int
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.zeros((cus,), device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    iters = 4000
    names = ["mfma        (4 waves: 8 x v_mfma_f32_32x32x2_f32 per trip)", "gather      (4 waves: 8 x ds_read_b128 + 32 adds per trip)",
             "split       (8 waves: 4 mfma + 4 gather, sharing the SIMDs)", "mixed       (4 waves, both kinds from one loop)",
             "lds         (4 waves: the 8 reads alone)", "adds        (4 waves: the 32 adds alone)",
             "split-lds   (8 waves: 4 mfma + 4 lds)", "split-adds  (8 waves: 4 mfma + 4 adds)"]
    times = []
    for arr in range(8):
        for _ in range(3):
            assert fn(out.data_ptr(), cus, iters, arr, stream) == 0
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            assert fn(out.data_ptr(), cus, iters, arr, stream) == 0
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / 5 * 1e3)
    for name, t in zip(names, times):
        print("  %-62s %8.1f us  (%.0f ns per trip)" % (name, t, t * 1e3 / iters))
    print("  sum of mfma and gather %.1f us, larger of the two %.1f us: split is %.2f of the sum, mixed %.2f"
          % (times[0] + times[1], max(times[0], times[1]), times[2] / (times[0] + times[1]), times[3] / (times[0] + times[1])))
    print("  mfma + lds: %.2f of the sum; mfma + adds: %.2f of the sum"
          % (times[6] / (times[0] + times[4]), times[7] / (times[0] + times[5])))
    flops = 2.0 * 32 * 32 * 2 * 8 * iters * 4 * cus
    print("  mfma alone: %.1f TFLOP/s fp32; in split: %.1f" % (flops / times[0] / 1e6, flops / times[2] / 1e6))


def lds_rate(_):
    """Bytes per clock that the LDS of a CU returns to conflict-free reads of 16, 8 and 4 bytes per lane
    (csrc/lds_rate_probe.hip: 16 waves per CU, the aggregation kernel's access shape)."""
    import torch

    sys.path.insert(0, ROOT)
    from f2cgt_amd import capi

    lib = capi.lib()
    if not hasattr(lib, "f2cgt_experiment_lds_rate_probe"):
        raise SystemExit("the library in tree was built without --experiments")
    fn = lib.f2cgt_experiment_lds_rate_probe
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    fn.restype = ctypes.c_int
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.zeros((cus,), dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    iters = 2000
    for width, name in ((16, "ds_read_b128"), (8, "ds_read_b64"), (4, "ds_read_b32")):
        for _ in range(2):
            assert fn(out.data_ptr(), cus, iters, width, stream) == 0
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        assert fn(out.data_ptr(), cus, iters, width, stream) == 0
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3
        clocks = out.cpu().numpy().astype("int64")
        nbytes = 16 * 8 * iters * 64 * width                      # per CU: 16 waves x 8 reads per trip x 64 lanes
        print("  %-13s launch %8.1f us; workgroup loop %d .. %d shader clocks (median %d): %.1f bytes per clock and CU, "
              "%.2f clocks per wave instruction"
              % (name, us, clocks.min(), clocks.max(), int(sorted(clocks)[len(clocks) // 2]),
                 nbytes / float(sorted(clocks)[len(clocks) // 2]), float(sorted(clocks)[len(clocks) // 2]) / (16 * 8 * iters)))


def cold_parts(name):
    """Which part of a launch's input has to be cached for the warm figure of a fused workload: the launch
    with its graph in one or several copies of the index arrays, with other graphs, with other outputs, and
    with a large unrelated read between two launches.  Needs no experiments build."""
    import torch

    sys.path.insert(0, ROOT)
    import bench
    from f2cgt_amd import capi, synth

    wl = synth.WORKLOADS[name](device="cuda", idx_dtype=torch.int64)
    outs = [torch.empty((wl["R"], wl["feat_dim"]), dtype=torch.float32, device="cuda") for _ in range(3)]

    def timed(pairs, rounds=30, warm=8):
        steps = [bench._launcher(capi, g, o) for g, o in pairs]

        def one_round():
            for st in steps:
                st()

        _, ms = bench._time_steps(one_round, rounds, warm)
        return ms / len(steps) * 1e3

    def copies(n, ids=True, ptr=True):
        res = [wl]
        for _ in range(n - 1):
            g = dict(wl)
            if ids:
                g["indices"] = wl["indices"].clone()
            if ptr:
                g["indptr"] = wl["indptr"].clone()
            res.append(g)
        return res

    timed([(wl, outs[0])] * 3, rounds=200)  # brings the clocks up before the first figure
    print(name, "launch times in us")
    print("  one graph, one output                          %7.1f" % timed([(wl, outs[0])] * 3))
    print("  one graph, three outputs in rotation           %7.1f" % timed([(wl, o) for o in outs]))
    for n in (2, 3, 4, 6):
        print("  the graph in %d copies of indices and indptr     %7.1f" % (n, timed([(g, outs[0]) for g in copies(n)])))
    print("  the graph in 6 copies of indptr only           %7.1f" % timed([(g, outs[0]) for g in copies(6, ids=False)]))
    print("  the graph in 6 copies of indices only          %7.1f" % timed([(g, outs[0]) for g in copies(6, ptr=False)]))
    others = synth.extra_blocks(wl, 2)
    print("  three different graphs, one output             %7.1f" % timed([(g, outs[0]) for g in [wl] + others]))
    print("  three different graphs, three outputs          %7.1f" % timed(list(zip([wl] + others, outs))))
    del others
    junk = torch.empty(512 * 1024 * 1024 // 4, dtype=torch.float32, device="cuda")
    step = bench._launcher(capi, wl, outs[0])

    def with_junk():
        junk.sum()
        step()

    _, both = bench._time_steps(with_junk, 20, 5)
    _, alone = bench._time_steps(lambda: junk.sum(), 20, 5)
    print("  one graph, a 512 MB read between two launches  %7.1f" % ((both - alone) * 1e3))


if __name__ == "__main__":
    modes = {"wave-age": wave_age, "block-phases": block_phases, "dispatch-cost": dispatch_cost, "hot-rows": hot_rows,
             "affine-geometry": affine_geometry, "hybrid-geometry": hybrid_geometry, "vq-degrees": vq_degrees, "vq-store-forms": vq_store_forms, "store-form": store_form, "mfma-overlap": mfma_overlap, "lds-rate": lds_rate,
             "cold-parts": cold_parts}
    if len(sys.argv) != 3 or sys.argv[1] not in modes:
        print(__doc__)
        sys.exit(2)
    modes[sys.argv[1]](sys.argv[2])
