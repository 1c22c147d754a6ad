"""Turns a directory of rocprofv3 CSV output into the text summaries under profiles/ and the
HBM-traffic record profiles/traffic.json that bench.py reads.

    python3 -m f2cgt_amd.profile_summary <rocprof_out_dir> [<profiles_dir>]

Nothing is run here.  <rocprof_out_dir> is expected to hold, per workload w in c1..c5 and c3s (c3 with
`--scatter`), the output
directories of these runs (`cd /tmp && export TMPDIR=/tmp` first, every run on its own, from the
repository root; B = `python3 bench.py --workload <w> --steps 2000 --warmup 200 --cpu-seconds 0`,
with 300 steps for c4 and c5 (30 and 100 warm-up launches); T = B except for c2, where T = `python3 bench.py --workload c2
--cpu-seconds 0` and T20 = `python3 bench.py --workload c2 --steps 20 --warmup 5 --cpu-seconds 0`):

    trace_<w>   rocprofv3 --kernel-trace --stats --output-format csv -d <dir>/trace_<w> -o t -- T
    trace20_c2  rocprofv3 --kernel-trace --stats --output-format csv -d <dir>/trace20_c2 -o t -- T20
    fetch_<w>   rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir>/fetch_<w> -o t -- B
    write_<w>   rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir>/write_<w> -o t -- B
    sqa_<w>     rocprofv3 --pmc SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_LDS SQ_ACTIVE_INST_LDS
                    SQ_LDS_BANK_CONFLICT SQ_WAIT_INST_ANY SQ_BUSY_CYCLES SQ_WAVE_CYCLES ... -- B
    sqb_<w>     rocprofv3 --pmc SQ_LDS_IDX_ACTIVE SQ_WAIT_INST_LDS SQ_ACTIVE_INST_VALU SQ_INSTS_VMEM_RD
                    SQ_INSTS_VMEM_WR SQ_INST_LEVEL_VMEM SQ_WAVES GRBM_GUI_ACTIVE ... -- B
    tcc_<w>     rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCC_EA_RDREQ_sum TCC_EA_WRREQ_sum ... -- B
    tcp_<w>     rocprofv3 --pmc TCP_TCC_READ_REQ_sum TCP_TCC_WRITE_REQ_sum TCP_PENDING_STALL_CYCLES_sum
                    TCP_TA_TCP_STATE_READ_sum ... -- B
    fetch_copy / write_copy   the FETCH_SIZE / WRITE_SIZE runs of `python3 bench.py --calibrate-copy`
    trace_all   rocprofv3 --kernel-trace --stats ... -- python3 bench.py --all --steps 200 --warmup 20 --cpu-seconds 0
    mfma_all    rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_BF16 SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES
                    SQ_INSTS_MFMA SQ_INSTS_VALU GRBM_GUI_ACTIVE ... -- (the --all command)

Missing directories are skipped.  Counter values are means per dispatch of the named kernel.
"""
from __future__ import annotations

import csv
import glob
import hashlib
import json
import os
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)

WORKLOADS = {
    "c1": ("sq_affine_acc_kernel", "c1_sq8_affine"),
    "c2": ("sq_affine_acc_kernel", "c2_sq4_affine"),
    "c3": ("vq_wave_kernel", "c3_vq_16x8"),
    "c4": ("hybrid_acc_kernel", "c4_hybrid"),
    "c5": ("vq_wave_kernel", "c5_vq_24x32"),
    "c3s": ("vq_wave_kernel", "c3_vq_16x8_scattered"),
}
STEPS = {"c1": (2000, 200), "c2": (2000, 200), "c3": (2000, 200), "c4": (300, 30), "c5": (300, 100),
         "c3s": (2000, 200)}
N_SIMD, N_XCD, N_CU = 1024, 8, 256


FUSED_SOURCES = ("common.hpp", "spmm.hip", "spmm_fast.hip", "spmm_fast.hpp", "vq_fast.hip")


def csrc_sha16():
    """Content hash of the sources of the fused aggregation kernels and their dispatch: a traffic
    figure belongs to the kernels it was measured on."""
    h = hashlib.sha256()
    for name in FUSED_SOURCES:
        h.update(name.encode())
        h.update(open(os.path.join(PKG, "csrc", name), "rb").read())
    return h.hexdigest()[:16]


def bench_cmd(w, short=False):
    if w == "c2" and short:
        return "python3 bench.py --workload c2 --steps 20 --warmup 5 --cpu-seconds 0"
    steps, warm = STEPS[w]
    name = "c3 --scatter" if w == "c3s" else w
    return "python3 bench.py --workload %s --steps %d --warmup %d --cpu-seconds 0" % (name, steps, warm)


def kstats(d, match):
    for f in glob.glob(d + "/**/*kernel_stats.csv", recursive=True):
        for r in csv.DictReader(open(f)):
            if match in r["Name"]:
                return (r["Name"].replace("f2cgt::(anonymous namespace)::", ""), int(r["Calls"]),
                        float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3, float(r["MaxNs"]) / 1e3)
    return None


def durations(d, match):
    out = []
    for f in glob.glob(d + "/**/*kernel_trace.csv", recursive=True):
        for r in csv.DictReader(open(f)):
            if match in r["Kernel_Name"]:
                out.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"])))
    return [(b - a) / 1e3 for a, b in sorted(out)]


def counters(d, match):
    """-> {counter: (mean per dispatch, dispatches)} of the kernels whose name contains `match`."""
    acc = {}
    for f in glob.glob(d + "/**/*counter_collection.csv", recursive=True):
        for r in csv.DictReader(open(f)):
            if match in r["Kernel_Name"]:
                s = acc.setdefault(r["Counter_Name"], [0.0, 0])
                s[0] += float(r["Counter_Value"])
                s[1] += 1
    return {k: (v[0] / v[1], v[1]) for k, v in acc.items() if v[1]}


def bench_line(d):
    for f in glob.glob(d + "*.out") + glob.glob(d + "/*.out"):
        for line in open(f, errors="replace"):
            if line.startswith('{"metric"'):
                return json.loads(line)
    return None


def write_workload(O, P, w, scales, traffic_out):
    kern, wl = WORKLOADS[w]
    tdir = os.path.join(O, "trace_" + w)
    k = kstats(tdir, kern)
    if k is None:
        return
    b = bench_line(tdir)
    cf, cw, fs, ws = scales
    fc = counters(os.path.join(O, "fetch_" + w), kern).get("FETCH_SIZE")
    wc = counters(os.path.join(O, "write_" + w), kern).get("WRITE_SIZE")
    B = bench_cmd(w)
    T = "python3 bench.py --workload c2 --cpu-seconds 0" if w == "c2" else B
    with open(os.path.join(P, "%s_%s.md" % (kern, wl)), "w") as fh:
        fh.write("# %s on workload %s (MI355X, gfx950)\n\n" % (kern, wl))
        fh.write("Commands (each a separate run; `cd /tmp && export TMPDIR=/tmp` first, from the repo root;\n"
                 "summarised by `python3 -m f2cgt_amd.profile_summary out profiles`):\n\n")
        fh.write("    rocprofv3 --kernel-trace --stats --output-format csv -d out/trace_%s -o t -- %s\n" % (w, T))
        if w == "c2":
            fh.write("    rocprofv3 --kernel-trace --stats --output-format csv -d out/trace20_c2 -o t -- %s\n" % bench_cmd(w, True))
        fh.write("    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out/fetch_%s -o t -- %s\n" % (w, B))
        fh.write("    rocprofv3 --pmc WRITE_SIZE --output-format csv -d out/write_%s -o t -- %s\n" % (w, B))
        fh.write("    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out/fetch_copy -o t -- python3 bench.py --calibrate-copy\n")
        fh.write("    rocprofv3 --pmc WRITE_SIZE --output-format csv -d out/write_copy -o t -- python3 bench.py --calibrate-copy\n")
        extra = [(n, counters(os.path.join(O, "%s_%s" % (n, w)), kern)) for n in ("sqa", "sqb", "tcc", "tcp")]
        for n, c in extra:
            if c:
                fh.write("    rocprofv3 --pmc %s --output-format csv -d out/%s_%s -o t -- %s\n" % (" ".join(sorted(c)), n, w, B))
        fh.write("\n## kernel trace (`t_kernel_stats.csv`)\n\n")
        fh.write("| kernel | calls | avg us | min us | max us |\n|---|---|---|---|---|\n")
        fh.write("| `%s` | %d | %.2f | %.2f | %.2f |\n\n" % (k[0][:90], k[1], k[2], k[3], k[4]))
        if w == "c2":
            ds = durations(tdir, kern)
            if len(ds) >= 1000:
                last = ds[-1000:]
                fh.write("The run is the default one (5000 warm-up launches, 1000 timed).  The last 1000 dispatches of "
                         "`t_kernel_trace.csv`, i.e. the timed region: avg %.2f us, min %.2f, max %.2f.\n\n"
                         % (sum(last) / len(last), min(last), max(last)))
            d20 = durations(os.path.join(O, "trace20_c2"), kern)
            b20 = bench_line(os.path.join(O, "trace20_c2"))
            if len(d20) >= 20:
                last = d20[-20:]
                fh.write("Short run (`--warmup 5 --steps 20`, what a fresh process sees): the 20 timed dispatches avg %.2f us, "
                         "min %.2f, max %.2f" % (sum(last) / len(last), min(last), max(last)))
                if b20:
                    fh.write("; bench.py in that run: launch %.2f us" % b20["roofline"]["launch_us"])
                fh.write(".\n\n")
        if b:
            fh.write("bench.py in the same run (HIP events on the launch stream): launch %.2f us, %.0f GB/s algorithmic, "
                     "%.3f of the 8 TB/s peak\n\n" % (b["roofline"]["launch_us"], b["roofline"]["achieved"],
                                                      b["roofline"]["achieved"] / 8000.0))
        if fc and wc and b:
            algo = b["config"]["algorithmic_bytes"]
            traffic = (fc[0] * fs + wc[0] * ws) * 1024
            fh.write("## HBM traffic per dispatch (`t_counter_collection.csv`, mean over %d dispatches)\n\n" % fc[1])
            fh.write("Calibration: a plain 1 GiB device copy (`__amd_rocclr_copyBuffer`, 1048576 KiB read and written) reads\n")
            fh.write("FETCH_SIZE = %.0f KiB and WRITE_SIZE = %.0f KiB per dispatch, so the scale factors are x%.4f (fetch) "
                     "and x%.4f (write).\n\n" % (cf, cw, fs, ws))
            fh.write("| counter | raw KiB/dispatch | scaled MB |\n|---|---|---|\n")
            fh.write("| FETCH_SIZE | %.0f | %.1f |\n| WRITE_SIZE | %.0f | %.1f |\n\n"
                     % (fc[0], fc[0] * fs * 1024 / 1e6, wc[0], wc[0] * ws * 1024 / 1e6))
            fh.write("Measured traffic %.1f MB per launch against %.1f MB algorithmic (ratio %.2f).\n\n"
                     % (traffic / 1e6, algo / 1e6, traffic / algo))
            traffic_out.append({"workload": wl, "idx": b["config"]["index_dtype"], "bytes": int(traffic),
                                "csrc_sha16": csrc_sha16()})
        merged = {}
        for _, c in extra:
            merged.update(c)
        if merged:
            fh.write("## issue and memory-pipeline counters (mean per dispatch, summed over the device)\n\n")
            fh.write("| counter | value |\n|---|---|\n")
            for name in sorted(merged):
                fh.write("| %s | %.4g |\n" % (name, merged[name][0]))
            g = merged.get("GRBM_GUI_ACTIVE")
            if g:
                clk = g[0] / N_XCD
                fh.write("\nKernel length %.0f clk (GRBM_GUI_ACTIVE / %d XCDs)" % (clk, N_XCD))
                v = merged.get("SQ_ACTIVE_INST_VALU") or merged.get("SQ_INSTS_VALU")
                if v:
                    fh.write("; vector ALU busy %.2f (4 clk per wave instruction on %d SIMDs)" % (v[0] * 4 / N_SIMD / clk, N_SIMD))
                l = merged.get("SQ_LDS_IDX_ACTIVE")
                if l:
                    fh.write("; LDS address pipeline busy %.2f (SQ_LDS_IDX_ACTIVE / %d CUs; a `ds_read_b128` counts 4 clocks there "
                             "and occupies the data return for 8, `profiles/lds_rate_probe_kernel_ds_read_widths.md`)" % (l[0] / N_CU / clk, N_CU))
                fh.write(".\n")
    print(w, wl, "written")


def main(argv):
    O = argv[1]
    P = argv[2] if len(argv) > 2 else os.path.join(ROOT, "profiles")
    os.makedirs(P, exist_ok=True)
    cf = counters(os.path.join(O, "fetch_copy"), "copyBuffer").get("FETCH_SIZE")
    cw = counters(os.path.join(O, "write_copy"), "copyBuffer").get("WRITE_SIZE")
    scales = (cf[0], cw[0], 1048576.0 / cf[0], 1048576.0 / cw[0]) if cf and cw else (float("nan"),) * 4
    traffic = []
    for w in WORKLOADS:
        write_workload(O, P, w, scales, traffic)
    if traffic:
        with open(os.path.join(P, "traffic.json"), "w") as fh:
            json.dump({"note": "HBM bytes per launch = FETCH_SIZE x %.4f + WRITE_SIZE x %.4f (KiB, rocprofv3 --pmc), "
                               "valid for the kernel sources with this content hash" % (scales[2], scales[3]),
                       "entries": traffic}, fh, indent=1)
            fh.write("\n")
    A = "python3 bench.py --all --steps 200 --warmup 20 --cpu-seconds 0"
    tall = os.path.join(O, "trace_all")
    k = kstats(tall, "predict_split_kernel<2, 2, false>")
    if k:
        with open(os.path.join(P, "predict_split_kernel_c5_encode.md"), "w") as fh:
            fh.write("# predict_split_kernel<2, 2, false> on the C5 encode step (1e6 x 32 fp32 vs 256 centres, squared L2 + arg-min)\n\n")
            fh.write("Commands (separate runs):\n\n")
            fh.write("    rocprofv3 --kernel-trace --stats --output-format csv -d out/trace_all -o t -- %s\n" % A)
            fh.write("    rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_BF16 SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_INSTS_MFMA "
                     "SQ_INSTS_VALU GRBM_GUI_ACTIVE --output-format csv -d out/mfma_all -o t -- %s\n\n" % A)
            fh.write("| kernel | calls | avg us | min us | max us |\n|---|---|---|---|---|\n")
            fh.write("| `%s` | %d | %.2f | %.2f | %.2f |\n\n" % (k[0][:60], k[1], k[2], k[3], k[4]))
            fl = 2.0 * 1e6 * 256 * 32
            fh.write("2*m*n*k = %.4g flop per launch -> %.1f TFLOP/s algorithmic; the kernel executes six bf16 MFMAs per fp32 "
                     "product block (three bf16 pieces per value), i.e. %.0f TFLOP/s of bf16 MFMA = %.3f of the 2500 TFLOP/s "
                     "bf16 peak.\n\n" % (fl, fl / (k[2] * 1e-6) / 1e12, 6 * fl / (k[2] * 1e-6) / 1e12,
                                         6 * fl / (k[2] * 1e-6) / 1e12 / 2500))
            vals = counters(os.path.join(O, "mfma_all"), "predict_split_kernel<2, 2, false>")
            if vals:
                fh.write("| counter (mean per dispatch) | value |\n|---|---|\n")
                for cn in sorted(vals):
                    fh.write("| %s | %.4g |\n" % (cn, vals[cn][0]))
                if "SQ_VALU_MFMA_BUSY_CYCLES" in vals and "GRBM_GUI_ACTIVE" in vals:
                    util = vals["SQ_VALU_MFMA_BUSY_CYCLES"][0] / N_SIMD / (vals["GRBM_GUI_ACTIVE"][0] / N_XCD)
                    fh.write("\nMFMA utilisation = SQ_VALU_MFMA_BUSY_CYCLES / %d SIMDs / (GRBM_GUI_ACTIVE / %d XCDs) = %.3f\n"
                             % (N_SIMD, N_XCD, util))
        k = kstats(tall, "predict_split_kernel<2, 2, true>")
        if k:
            with open(os.path.join(P, "predict_split_kernel_pairwise_c5_encode_shape.md"), "w") as fh:
                fh.write("# predict_split_kernel<2, 2, true> (pairwise_distance) at the C5 encode shape: 1e6 x 32 against 256 rows, L2 and cosine\n\n")
                fh.write("    rocprofv3 --kernel-trace --stats --output-format csv -d out/trace_all -o t -- %s\n\n" % A)
                fh.write("| kernel | calls | avg us | min us | max us |\n|---|---|---|---|---|\n")
                fh.write("| `%s` | %d | %.2f | %.2f | %.2f |\n\n" % (k[0][:60], k[1], k[2], k[3], k[4]))
                nb = 1e6 * 256 * 4
                fh.write("The [1e6, 256] fp32 matrix is %.0f MB: %.0f GB/s of matrix write = %.2f of the 8 TB/s peak (both "
                         "metrics in one average).\n" % (nb / 1e6, nb / (k[2] * 1e-6) / 1e9, nb / (k[2] * 1e-6) / 8e12))
        with open(os.path.join(P, "streaming_ops_c2_table_shape.md"), "w") as fh:
            fh.write("# Streaming kernels at the C2 table shape (2.4e6 rows), from the `bench.py --all` kernel trace\n\n")
            fh.write("    rocprofv3 --kernel-trace --stats --output-format csv -d out/trace_all -o t -- %s\n\n" % A)
            fh.write("| kernel | calls | avg us | bytes moved (algorithmic) | GB/s |\n|---|---|---|---|---|\n")
            n, d = 2400000, 100
            for name, nbytes in (("::pack_flat_kernel", n * d * 1.5), ("::unpack_flat_kernel", n * d * 1.5),
                                 ("sq_decode_f4_kernel<4, true>", n * d * 4.5), ("sq_decode_f4_kernel<4, false>", n * d * 4.5),
                                 ("vq_decompress_tile_kernel", n * (16 + 512)), ("sq_encode_f4_kernel<4, true", n * d * 4.5),
                                 ("sq_encode_f4_kernel<4, false", n * d * 8.0)):
                k = kstats(tall, name)
                if k:
                    fh.write("| `%s` | %d | %.2f | %.0f MB | %.0f |\n" % (k[0][:60], k[1], k[2], nbytes / 1e6,
                                                                          nbytes / (k[2] * 1e-6) / 1e9))


if __name__ == "__main__":
    if len(sys.argv) < 2:
        print(__doc__)
        sys.exit(2)
    main(sys.argv)
