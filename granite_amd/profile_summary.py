"""Collects rocprofv3 evidence for the benchmark workloads and writes the short summaries that
live under profiles/ (one markdown file per workload, plus profiles/traffic.json, which
bench.py reads for `roofline.traffic`).

    python -m granite_amd.profile_summary collect [workload ...]    # on the GPU box
    python -m granite_amd.profile_summary summarise [workload ...]  # anywhere, from the raw files

`mfma_calibration` (the matrix-core rate kernel, what an MFMA-bound kernel is compared with
beside the published peak) is collected and summarised like a workload when named: kernel
trace, the instruction counters and the clock, per instruction mix.

`collect` runs, per workload, one `rocprofv3 --kernel-trace --stats` pass and one `--pmc`
pass per counter group (every pass is its own process: rocprofv3 does not split counters
over passes, and a group holds at most 8 SQ counters), always with `python3 bench.py ...`
as the profiled program.  Raw output goes to $GRANITE_PROFILE_RAW/<workload>/ (default
build/prof_raw/, which git ignores); only the summaries are meant to be kept.
"""
from __future__ import annotations

import collections
import csv
import glob
import json
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
RAW = Path(os.environ.get("GRANITE_PROFILE_RAW", ROOT / "build" / "prof_raw")).resolve()
PROFILES = ROOT / "profiles"

WORKLOADS = ["paged_decode", "prefill", "chunked_prefill", "tree", "decode_contiguous", "rope_append",
             "qkv_q4k", "copy_calibration"]
MFMA_BOUND = {"prefill", "chunked_prefill"}
DOMINANT = {"paged_decode": "decode_stream_kernel", "prefill": "attention_tiles_dma_kernel",
            "chunked_prefill": "attention_tiles_dma_kernel", "tree": "attention_tiles_dma_kernel",
            "decode_contiguous": "decode_splitk_kernel", "rope_append": "rope_append_kernel",
            "qkv_q4k": "matvec_q4k_kernel", "copy_calibration": "kv_gather_kernel"}

# counter groups: (tag, counters); HBM traffic for every workload, the SQ groups for the
# MFMA-bound ones (matrix-core utilisation, LDS behaviour, instruction mix, clock)
TRAFFIC_GROUPS = [("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")]
SQ_GROUPS = [
    ("sq1", "SQ_WAVES SQ_WAVE_CYCLES SQ_BUSY_CU_CYCLES SQ_VALU_MFMA_BUSY_CYCLES "
            "SQ_VALU_MFMA_COEXEC_CYCLES SQ_WAIT_INST_LDS SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_VALU"),
    ("sq2", "SQ_INSTS_VALU SQ_INSTS_MFMA SQ_INSTS_SALU SQ_INSTS_LDS SQ_INSTS_VMEM_RD "
            "SQ_INSTS_VALU_TRANS_F32 SQ_LDS_IDX_ACTIVE SQ_ACTIVE_INST_LDS"),
    ("grbm", "GRBM_GUI_ACTIVE"),
]
COPY_BYTES = 2 * 65536 * 8 * 128 * 2  # read (and written) by one launch of copy_calibration
XCDS = 8  # GRBM counters are summed over the part's 8 XCDs


CAL = "mfma_calibration"
CAL_GROUPS = [
    ("sq1", "SQ_WAVES SQ_BUSY_CU_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU SQ_INSTS_MFMA SQ_INSTS_SALU "
            "SQ_INSTS_LDS SQ_INSTS_VALU_TRANS_F32"),
    ("grbm", "GRBM_GUI_ACTIVE"),
]


def trace_cmd(w: str, out: Path) -> list[str]:
    if w == CAL:
        return ["rocprofv3", "--kernel-trace", "--stats", "-d", str(out / "trace"), "-o", "t", "--output-format",
                "csv", "--", "python3", "bench.py", "--workload", w, "--steps", "2", "--no-cpu"]
    return ["rocprofv3", "--kernel-trace", "--stats", "-d", str(out / "trace"), "-o", "t", "--output-format",
            "csv", "--", "python3", "bench.py", "--workload", w, "--steps", "20", "--warmup", "3", "--no-cpu",
            *(["--no-float-queries"] if w in MFMA_BOUND else [])]


def pmc_cmd(w: str, out: Path, tag: str, counters: str) -> list[str]:
    if w == CAL:
        return ["rocprofv3", "--pmc", *counters.split(), "-d", str(out / tag), "-o", "p", "--output-format", "csv",
                "--", "python3", "bench.py", "--workload", w, "--steps", "1", "--no-cpu"]
    return ["rocprofv3", "--pmc", *counters.split(), "-d", str(out / tag), "-o", "p", "--output-format", "csv",
            "--", "python3", "bench.py", "--workload", w, "--steps", "5", "--warmup", "2", "--no-cpu",
            "--ramp-ms", "0", *(["--no-float-queries"] if w in MFMA_BOUND else [])]


def shown(cmd: list[str]) -> str:
    """The command as typed from the repository root (raw output under OUT/)."""
    return " ".join(c.replace(str(RAW) + "/", "OUT/") for c in cmd)


def collect(workloads: list[str]) -> int:
    env = dict(os.environ, TMPDIR="/tmp")
    for w in workloads:
        out = RAW / w
        subprocess.run(["rm", "-rf", str(out)], check=True)
        out.mkdir(parents=True)
        groups = CAL_GROUPS if w == CAL else TRAFFIC_GROUPS + (SQ_GROUPS if w in MFMA_BOUND else [])
        cmds = [("trace", trace_cmd(w, out))] + [(tag, pmc_cmd(w, out, tag, c)) for tag, c in groups]
        for tag, cmd in cmds:
            print(f"== {w} / {tag}", flush=True)
            with open(out / f"{tag}.log", "w") as log:
                # a pass over a short program takes seconds; a hung one is killed, not retried
                res = subprocess.run(["timeout", "-s", "KILL", "240", *cmd], cwd=ROOT, env=env, stdout=log,
                                     stderr=subprocess.STDOUT)
            if res.returncode != 0:
                print((out / f"{tag}.log").read_text()[-1500:], flush=True)
                print(f"{w} / {tag} failed with {res.returncode}; stopping", flush=True)
                return 1
        for big in glob.glob(str(out / "**" / "*.csv"), recursive=True):
            if os.path.getsize(big) > 3 << 20:
                os.remove(big)
    return 0


def short(name: str) -> str:
    return (name.replace("(anonymous namespace)::", "").replace("ghip::", "").replace("void ", "")).split("(")[0]


def counters(w: str, tag: str) -> dict:
    """{(kernel, counter): values of the dispatches with the kernel's largest grid} -- a
    workload that also launches its kernel on a small side shape (rope_append's 512-token
    chunk) is counted on its main shape only."""
    rows = collections.defaultdict(list)
    for f in glob.glob(str(RAW / w / tag / "**" / "*counter_collection.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            rows[(short(r["Kernel_Name"]).split("<")[0], r["Counter_Name"])].append(
                (int(r["Grid_Size"]), float(r["Counter_Value"])))
    agg = {}
    for key, vals in rows.items():
        biggest = max(g for g, _ in vals)
        agg[key] = [v for g, v in vals if g == biggest]
    return agg


def main_shape_duration(w: str):
    """(calls, mean ns) of the dominant kernel's largest-grid dispatches in the kernel trace."""
    rows = []
    for f in glob.glob(str(RAW / w / "trace" / "**" / "*kernel_trace.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            if short(r["Kernel_Name"]).split("<")[0] == DOMINANT.get(w):
                grid = int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"])
                rows.append((grid, float(r["End_Timestamp"]) - float(r["Start_Timestamp"])))
    if not rows:
        return None
    biggest = max(g for g, _ in rows)
    ns = [d for g, d in rows if g == biggest]
    return len(ns), mean(ns)


def resources(w: str) -> dict:
    """Registers, LDS and scratch per kernel: from the kernel trace, or from the FETCH_SIZE pass
    (the same columns) when the trace of a workload with many launches was too large to keep."""
    res = {}
    for f in glob.glob(str(RAW / w / "trace" / "**" / "*kernel_trace.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            res[short(r["Kernel_Name"])] = (r["VGPR_Count"], r["Accum_VGPR_Count"], r["SGPR_Count"],
                                            r["LDS_Block_Size"], r["Scratch_Size"], r["Workgroup_Size_X"])
    if not res:
        for f in glob.glob(str(RAW / w / "fetch" / "**" / "*counter_collection.csv"), recursive=True):
            for r in csv.DictReader(open(f)):
                res[short(r["Kernel_Name"])] = (r["VGPR_Count"], r["Accum_VGPR_Count"], r["SGPR_Count"],
                                                r["LDS_Block_Size"], r["Scratch_Size"], r["Workgroup_Size"])
    return res


def clock_ghz(w: str):
    """GRBM_GUI_ACTIVE cycles over the dispatch's own duration, for the dominant kernel."""
    ratios = []
    for f in glob.glob(str(RAW / w / "grbm" / "**" / "*counter_collection.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            if r["Counter_Name"] == "GRBM_GUI_ACTIVE" and short(r["Kernel_Name"]).split("<")[0] == DOMINANT[w]:
                ns = float(r["End_Timestamp"]) - float(r["Start_Timestamp"])
                if ns > 0:
                    ratios.append(float(r["Counter_Value"]) / XCDS / ns)  # the counter sums the 8 XCDs
    return mean(ratios) if ratios else None


def bench_line(w: str) -> dict:
    for line in open(RAW / w / "trace.log"):
        if line.startswith("{"):
            return json.loads(line)
    raise RuntimeError(f"no bench line in {RAW / w / 'trace.log'}")


def mean(v):
    return sum(v) / len(v)


def calibration():
    f, wr = counters("copy_calibration", "fetch"), counters("copy_calibration", "write")
    fk = mean([v for (k, c), v in f.items() if "kv_gather" in k][0])
    wk = mean([v for (k, c), v in wr.items() if "kv_gather" in k][0])
    return COPY_BYTES / 1024 / fk, COPY_BYTES / 1024 / wk, fk, wk


def cal_kernel(name: str):
    """(wide shape?, (fma, exp, lds, salu) per pair of MFMAs, zero operands?) from
    `mfma_rate_kernel<true, 6, 2, 3, 0, false>`."""
    args = [a.strip() for a in name[name.index("<") + 1:name.rindex(">")].split(",")]
    return args[0] == "true", tuple(int(a) for a in args[1:5]), args[5] == "true"


def summarise_calibration() -> None:
    """profiles/mfma_calibration.md: per instruction mix the kernel-trace duration (the timed
    launches: the longest grid of 512-thread or 256-thread workgroups), the TFLOP/s that
    follows from it, the instructions a wave issues per MFMA (counters) and the clock."""
    out = RAW / CAL
    res = bench_line(CAL)["workloads"][CAL]
    flops_per_wave = 20000 * 16 * 2.0 * 32 * 32 * 16
    trace = collections.defaultdict(list)  # (kernel, workgroup size) -> durations
    for f in glob.glob(str(out / "trace" / "**" / "*kernel_trace.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            k = short(r["Kernel_Name"])
            if k.startswith("mfma_rate_kernel"):
                trace[(k, int(r["Workgroup_Size_X"]))].append(float(r["End_Timestamp"]) - float(r["Start_Timestamp"]))
    cnt = collections.defaultdict(lambda: collections.defaultdict(list))
    clock = collections.defaultdict(list)
    for tag, _ in CAL_GROUPS:
        for f in glob.glob(str(out / tag / "**" / "*counter_collection.csv"), recursive=True):
            for r in csv.DictReader(open(f)):
                k = short(r["Kernel_Name"])
                if not k.startswith("mfma_rate_kernel"):
                    continue
                key = (k, int(r["Workgroup_Size"]) if "Workgroup_Size" in r else int(r["Workgroup_Size_X"]))
                cnt[key][r["Counter_Name"]].append(float(r["Counter_Value"]))
                if r["Counter_Name"] == "GRBM_GUI_ACTIVE":
                    ns = float(r["End_Timestamp"]) - float(r["Start_Timestamp"])
                    if ns > 0:
                        clock[key].append(float(r["Counter_Value"]) / XCDS / ns)
    L = [f"# {CAL}: what the matrix cores reach, by instruction mix ({res['workload']})", "",
         "Commands (from the repository root on one MI355X, `export TMPDIR=/tmp` first; OUT is any scratch folder):",
         "", "```", shown(trace_cmd(CAL, out))]
    L += [shown(pmc_cmd(CAL, out, tag, c)) for tag, c in CAL_GROUPS] + ["```", ""]
    L += ["`mfma_rate_kernel<wide, fma, exp, lds, salu>` of `libgranite_hip_calibration.so`: one workgroup per "
          "compute unit, one (256 threads) or two (512) waves per SIMD, 20000 passes of 16 `v_mfma_f32_32x32x16_f16` "
          "per wave on register operands (normally distributed fp16 unless said otherwise), and per pair of MFMAs "
          "`fma` float FMAs, `exp` `v_exp_f32`, `lds` LDS operand reads whose data feeds later MFMAs and `salu` "
          "scalar additions.  Every launch is preceded by three untimed ones; durations are the kernel trace's, "
          "the best launch per mix.  TFLOP/s counts MFMA flops only; the published peak is 2500.", "",
          "| mix per MFMA | waves per SIMD | best ns | TFLOP/s | of 2500 | VALU per MFMA | of them exp | LDS per MFMA | "
          "SALU per MFMA | MFMA busy | clock GHz |", "|---|---|---|---|---|---|---|---|---|---|---|"]
    rows = {}
    for (k, wg), durs in sorted(trace.items()):
        wide, mix, zeros = cal_kernel(k)
        if not wide:
            continue
        best = min(durs)
        waves = wg // 256
        tf = 256 * 4 * waves * flops_per_wave / (best * 1e-9) / 1e12
        c = {n: mean(v) for n, v in cnt.get((k, wg), {}).items()}
        per = lambda n: (c[n] / c["SQ_INSTS_MFMA"]) if c.get("SQ_INSTS_MFMA") else float("nan")
        valu = per("SQ_INSTS_VALU") - 1 if c.get("SQ_INSTS_VALU") else float("nan")  # the counter includes the MFMAs
        busy = (c["SQ_VALU_MFMA_BUSY_CYCLES"] / (4 * c["SQ_BUSY_CU_CYCLES"])) if c.get("SQ_BUSY_CU_CYCLES") else float("nan")
        ghz = mean(clock[(k, wg)]) if clock.get((k, wg)) else float("nan")
        label = (f"{mix[0] / 2:g} fma, {mix[1] / 2:g} exp, {mix[2] / 2:g} lds, {mix[3] / 2:g} salu" if any(mix) else "none")
        if zeros:
            label += " (all-zero operands)"
        else:
            rows[(mix, waves)] = tf
        L.append(f"| {label} | {waves} | {best:.0f} | {tf:.0f} | {tf / 2500:.3f} | {valu:.2f} | "
                 f"{per('SQ_INSTS_VALU_TRANS_F32'):.2f} | {per('SQ_INSTS_LDS'):.2f} | {per('SQ_INSTS_SALU'):.2f} | "
                 f"{busy:.3f} | {ghz:.2f} |")
    L += ["", "(All-zero operands and the 16x16x32 shape run in the same command; bench.py's own HIP-event figures "
          f"of this run: `{json.dumps(res['rates_TFLOPs'])}`.)"]
    # the prefill kernels against the rows that carry their instruction mix
    notes = []
    for w, mix, kernel in (("chunked_prefill", (6, 2, 3, 4), "attention_tiles_dma_kernel"),):
        md = PROFILES / f"{w}.md"
        if md.exists() and (mix, 2) in rows:
            for line in md.read_text().splitlines():
                if line.startswith("Roofline from the event timing:"):
                    ach = json.loads(line[line.index("`") + 1:line.rindex("`")])["achieved"]
                    notes.append(f"`{kernel}` on {w}: {ach:.0f} TFLOP/s by `profiles/{w}.md` = "
                                 f"**{ach / rows[(mix, 2)]:.2f}** of the {rows[(mix, 2)]:.0f} TFLOP/s of the row that "
                                 f"carries its instruction mix ({mix[0] / 2:g} fma, {mix[1] / 2:g} exp, {mix[2] / 2:g} lds, "
                                 f"{mix[3] / 2:g} salu per MFMA, two waves per SIMD), and {ach / 2500:.3f} of the published "
                                 f"peak.  (Different boxes differ by several per cent; both files should come from one "
                                 f"`collect` call.)")
    if notes:
        L += ["", "## The prefill kernel against its own mix", ""] + notes
    (PROFILES / f"{CAL}.md").write_text("\n".join(L) + "\n")
    print(f"wrote profiles/{CAL}.md", flush=True)


def summarise(workloads: list[str]) -> int:
    PROFILES.mkdir(exist_ok=True)
    if CAL in workloads:
        workloads = [w for w in workloads if w != CAL]
        cal_last = True
    else:
        cal_last = False
    fetch_kib, write_kib, fetch_raw, write_raw = calibration()
    traffic_path = PROFILES / "traffic.json"
    traffic = json.loads(traffic_path.read_text()) if traffic_path.exists() else {}
    for w in workloads:
        res = bench_line(w)["workloads"][w]
        out = RAW / w
        L = [f"# {w}: rocprofv3 summary ({res['workload']})", "",
             "Commands (from the repository root on one MI355X, `export TMPDIR=/tmp` first; OUT is any scratch "
             "folder):", "", "```", shown(trace_cmd(w, out))]
        groups = TRAFFIC_GROUPS + (SQ_GROUPS if w in MFMA_BOUND else [])
        L += [shown(pmc_cmd(w, out, tag, c)) for tag, c in groups] + ["```", ""]
        L += ["## Kernel trace (`*_kernel_stats.csv`: the clock ramp, the warm-up and both timed passes of "
              "bench.py)", "", "| kernel | calls | avg ns | min ns | max ns | % of GPU time |", "|---|---|---|---|---|---|"]
        for f in glob.glob(str(out / "trace" / "**" / "*kernel_stats.csv"), recursive=True):
            for r in csv.DictReader(open(f)):
                L.append(f"| `{short(r['Name'])[:70]}` | {r['Calls']} | {float(r['AverageNs']):.0f} | {r['MinNs']} | "
                         f"{r['MaxNs']} | {float(r['Percentage']):.1f} |")
        main = main_shape_duration(w)
        if main:
            L += ["", f"`{DOMINANT[w]}` on the workload's main shape (largest grid): {main[0]} launches, mean "
                      f"{main[1]:.0f} ns."]
        L += ["", f"bench.py's own HIP-event timing in the same run, ms per launch: `{json.dumps(res['kernels_ms'])}`; "
                  f"whole step {res['ms_per_step']} ms."]
        if "roofline" in res:
            L += ["", f"Roofline from the event timing: `{json.dumps(res['roofline'])}`"]
        L += ["", "## Registers, LDS, scratch (kernel trace; LDS is the static part, the K/V tile buffers of "
              "`attention_tiles_dma_kernel` are 141312 B and those of `attention_tiles_kernel` 101376 B of "
              "dynamic LDS on top)", "",
              "| kernel | VGPRs | AGPRs | SGPRs | LDS bytes | scratch bytes | workgroup |", "|---|---|---|---|---|---|---|"]
        for k, v in sorted(resources(w).items()):
            L.append(f"| `{k[:70]}` | " + " | ".join(v) + " |")
        L += ["", "## HBM traffic (`FETCH_SIZE`, `WRITE_SIZE`: KiB per dispatch, mean over dispatches)", "",
              f"Calibration: the identity block-table gather (`--workload copy_calibration`, {COPY_BYTES} B read and "
              f"as many written per launch) reads FETCH_SIZE = {fetch_raw:.0f} and WRITE_SIZE = {write_raw:.0f}, so one "
              f"counter unit is {fetch_kib:.3f} KiB of reads and {write_kib:.3f} KiB of writes.", "",
              "| kernel | FETCH_SIZE | WRITE_SIZE | read bytes (scaled) | written bytes (scaled) |", "|---|---|---|---|---|"]
        f, wr = counters(w, "fetch"), counters(w, "write")
        dominant = None
        for (k, c), v in sorted(f.items()):
            wv = wr.get((k, "WRITE_SIZE"), [0])
            rb, wb = mean(v) * fetch_kib * 1024, mean(wv) * write_kib * 1024
            if k == DOMINANT.get(w):
                dominant = int(rb + wb)
            L.append(f"| `{k[:60]}` | {mean(v):.0f} | {mean(wv):.0f} | {rb:.4g} | {wb:.4g} |")
        if "algorithmic_bytes" in res and dominant is not None:
            L += ["", f"Algorithmic bytes of the workload: {res['algorithmic_bytes']} per step; traffic of "
                      f"`{DOMINANT[w]}`: {dominant} B per launch ({dominant / res['algorithmic_bytes']:.3f} x)."]
            traffic[w] = {"workload": res["workload"], "kernel": DOMINANT[w], "traffic_bytes": dominant,
                          "summary": f"profiles/{w}.md"}
        if w in MFMA_BOUND:
            c = {}
            for tag, _ in SQ_GROUPS:
                for (k, name), v in counters(w, tag).items():
                    if k == DOMINANT[w]:
                        c[name] = mean(v)
            L += ["", f"## Matrix-core and LDS counters of `{DOMINANT[w]}` (mean per dispatch)", "",
                  "| counter | value |", "|---|---|"]
            L += [f"| {name} | {value:.4g} |" for name, value in sorted(c.items())]
            if "SQ_BUSY_CU_CYCLES" in c and "SQ_VALU_MFMA_BUSY_CYCLES" in c:
                busy = c["SQ_VALU_MFMA_BUSY_CYCLES"] / (4 * c["SQ_BUSY_CU_CYCLES"])
                L += ["", f"Matrix cores busy: SQ_VALU_MFMA_BUSY_CYCLES / (4 SIMDs x SQ_BUSY_CU_CYCLES) = "
                          f"**{busy:.3f}**"]
                if "SQ_VALU_MFMA_COEXEC_CYCLES" in c:
                    L[-1] += (f"; vector ALU running beside them: "
                              f"{c['SQ_VALU_MFMA_COEXEC_CYCLES'] / (4 * c['SQ_BUSY_CU_CYCLES']):.3f} of the cycles")
            if "SQ_WAIT_INST_LDS" in c and "SQ_WAVE_CYCLES" in c:
                L += [f"Waves waiting for LDS: SQ_WAIT_INST_LDS / SQ_WAVE_CYCLES = "
                      f"{c['SQ_WAIT_INST_LDS'] / c['SQ_WAVE_CYCLES']:.3f}; bank conflicts "
                      f"{c.get('SQ_LDS_BANK_CONFLICT', 0):.0f} cycles."]
            if "SQ_WAVES" in c and "SQ_INSTS_MFMA" in c:
                per = {n: c[n] / c["SQ_WAVES"] for n in c if n.startswith("SQ_INSTS")}
                L += ["Instructions per wave: " + ", ".join(f"{n[9:]} {v:.0f}" for n, v in sorted(per.items())) + "."]
            ghz = clock_ghz(w)
            if ghz:
                L += [f"Clock under this kernel: GRBM_GUI_ACTIVE / 8 XCDs over the dispatch's own duration (counter "
                      f"pass: launches serialised, no clock ramp in front) = {ghz:.2f} GHz."]
        (PROFILES / f"{w}.md").write_text("\n".join(L) + "\n")
        print(f"wrote profiles/{w}.md", flush=True)
    traffic_path.write_text(json.dumps(traffic, indent=2) + "\n")
    if cal_last:
        summarise_calibration()  # after the workloads: it quotes profiles/chunked_prefill.md
    return 0


def main() -> int:
    if len(sys.argv) < 2 or sys.argv[1] not in ("collect", "summarise"):
        print(__doc__)
        return 2
    names = sys.argv[2:] or WORKLOADS + [CAL]
    if sys.argv[1] == "collect":
        if "copy_calibration" not in names:
            names = names + ["copy_calibration"]
        return collect(names)
    return summarise([n for n in names if n != "copy_calibration"] + (["copy_calibration"] if "copy_calibration" in names else []))


if __name__ == "__main__":
    sys.exit(main())
