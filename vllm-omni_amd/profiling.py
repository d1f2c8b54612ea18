"""Turns raw rocprofv3 output into the short text summaries kept under profiles/, and reads them back.

Every summary ends with one line ``bench.py reads: {...}`` (JSON): the figures ``bench.py`` quotes in its
``roofline`` object together with the attention launch plan (kernel names and unit counts, as
``kernels.attn_plan`` reports them) that was profiled. ``bench.py`` compares that plan with the one the
library dispatches now and refuses to quote figures measured on other kernels.

    python -m vllm_omni_amd.profiling counters <dir of pass a> <dir of pass b> <probe stdout>
    python -m vllm_omni_amd.profiling traffic  <dir of FETCH_SIZE pass> <dir of WRITE_SIZE pass> <probe stdout>
    python -m vllm_omni_amd.profiling step     <dir of the kernel trace> <bench.py stdout> <qwen_image|flux|wan>

The commands that make the inputs are written at the top of each summary.
"""

from __future__ import annotations

import collections
import csv
import glob
import json
import os
import sys
from pathlib import Path

PROFILES = Path(__file__).resolve().parent.parent / "profiles"
COUNTERS_FILE = "kernels_qwen_shape_sq_counters_pmc.txt"
TRAFFIC_FILE = "attn_fwd_qwen_shape_hbm_traffic_pmc.txt"
MARK = "bench.py reads: "

SIMDS, CUS, XCDS = 1024, 256, 8

PASS_A = ("SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES SQ_INSTS_VALU_MFMA_MOPS_BF16 SQ_INSTS_MFMA SQ_VALU_MFMA_COEXEC_CYCLES "
          "SQ_ACTIVE_INST_VALU SQ_WAVE_CYCLES GRBM_GUI_ACTIVE")
PASS_B = ("SQ_LDS_IDX_ACTIVE SQ_LDS_BANK_CONFLICT SQ_INSTS_LDS SQ_ACTIVE_INST_LDS SQ_WAIT_INST_LDS SQ_WAIT_INST_ANY SQ_INSTS_VALU "
          "SQ_INSTS_VALU_TRANS_F32 GRBM_GUI_ACTIVE")


# ------------------------------------------------------------------------------------------ reading
def read_record(name: str) -> dict:
    """The JSON record at the end of profiles/<name>; raises when the file or the record is missing."""
    path = PROFILES / name
    for line in reversed(path.read_text().splitlines()):
        if line.startswith(MARK):
            return json.loads(line[len(MARK):])
    raise ValueError(f"{path} has no '{MARK.strip()}' line: re-create it with python -m vllm_omni_amd.profiling")


def attention_figures(current_plan: str) -> dict:
    """HBM traffic, MFMA-busy share and in-kernel clock of the attention call at the headline shape from the
    committed counter summaries, after checking that they were measured on the launches ``current_plan``
    names (``kernels.attn_plan`` of the headline shape)."""
    traffic, counters = read_record(TRAFFIC_FILE), read_record(COUNTERS_FILE)
    for name, rec in ((TRAFFIC_FILE, traffic), (COUNTERS_FILE, counters)):
        if rec["attention_plan"] != current_plan:
            raise RuntimeError(
                f"profiles/{name} was measured on the attention launches\n    {rec['attention_plan']}\n"
                f"but this build dispatches\n    {current_plan}\nre-run the counter passes named at the top of that file")
    return {"traffic_bytes": traffic["traffic_bytes"], "mfma_busy_frac": counters["mfma_busy_frac"],
            "clock_MHz": counters["clock_MHz"], "profiled_kernel": counters["main_kernel"]}


# ------------------------------------------------------------------------------------------ helpers
def _one(pattern: str) -> str:
    hits = glob.glob(pattern, recursive=True)
    if len(hits) != 1:
        raise FileNotFoundError(f"expected one file matching {pattern}, found {len(hits)}")
    return hits[0]


def _probe_json(path: str) -> dict:
    lines = [l for l in Path(path).read_text().splitlines() if l.startswith("{")]
    if not lines:
        raise ValueError(f"{path} holds no JSON line (the stdout of the probe run is expected there)")
    return json.loads(lines[-1])


def _dispatches(directory: str) -> "collections.OrderedDict[str, dict]":
    rows = list(csv.DictReader(open(_one(os.path.join(directory, "**", "*counter_collection.csv")))))
    d: collections.OrderedDict[str, dict] = collections.OrderedDict()
    for r in rows:
        e = d.setdefault(r["Dispatch_Id"], {"name": r["Kernel_Name"], "dur": int(r["End_Timestamp"]) - int(r["Start_Timestamp"]),
                                            "lds": r["LDS_Block_Size"], "scratch": r["Scratch_Size"]})
        e[r["Counter_Name"]] = float(r["Counter_Value"])
    return d


def _ours(name: str) -> bool:
    return "odit" in name or "Cijk" in name


def _short(name: str) -> str:
    n = name.replace("void odit::", "").replace("odit::", "").replace("(anonymous namespace)::", "")
    if n.startswith("Custom_Cijk") or n.startswith("Cijk"):
        return "hipBLASLt " + n[n.index("MT"):].split("_")[0]
    return n.split("(")[0]


def _plan_kernels(plan: str) -> list[str]:
    """Kernel names of a launch plan: each "; "-separated part is "<kernel name> <counts>"."""
    return [part.strip()[:part.strip().index(">") + 1] if ">" in part else part.strip().split(" ")[0] for part in plan.split(";")]


def _is_kernel(kern: str, name: str) -> bool:
    """Whether the profiler's kernel name `name` is the plan's kernel `kern` (which writes T for the element type)."""
    head, _, tail = kern.partition("<T, ")
    return (head + "<") in name and tail in name if tail else kern in name


def _check_plan_in_trace(plan: str, names: list[str], what: str) -> None:
    for kern in _plan_kernels(plan):
        if not any(_is_kernel(kern, n) for n in names):
            raise RuntimeError(f"{what}: the probe reports the launch plan\n    {plan}\nbut no dispatch of '{kern}' was recorded")


# ------------------------------------------------------------------------------------------ counters
def summarise_counters(dir_a: str, dir_b: str, probe_stdout: str) -> str:
    probe = _probe_json(probe_stdout)
    plan = probe["attention_plan"]

    def load(directory):
        per: collections.OrderedDict[str, list] = collections.OrderedDict()
        for e in _dispatches(directory).values():
            if _ours(e["name"]):
                per.setdefault(e["name"], []).append(e)
        out = collections.OrderedDict()
        for n, es in per.items():  # mean of the launches after the first (the first carries one-off costs)
            es = es[1:] if len(es) > 1 else es
            out[n] = {k: (sum(e[k] for e in es) / len(es) if isinstance(es[0][k], (int, float)) else es[0][k]) for k in es[0]}
        return out

    a, b = load(dir_a), load(dir_b)
    _check_plan_in_trace(plan, list(a), "counter pass a")
    L = ["# rocprofv3 hardware-counter summary (SQ block): every hand-written kernel of the path and the two large library GEMMs at the",
         "# Qwen-Image shape (B=2, 4096 image + 256 text tokens, 24 heads x 128, hidden 3072, MLP 12288), bf16, N(0,1) data, MI355X.",
         "# commands (from the repo root, on the GPU box; one counter set per run):",
         "#   export TMPDIR=/tmp OUT=<a scratch directory>",
         f"#   rocprofv3 --pmc {PASS_A} --output-format csv -d $OUT/pmc_sq_a -o a -- python3 bench.py --counter-probe > $OUT/pmc_sq_probe.log",
         f"#   rocprofv3 --pmc {PASS_B} --output-format csv -d $OUT/pmc_sq_b -o b -- python3 bench.py --counter-probe",
         "#   python3 -m vllm_omni_amd.profiling counters $OUT/pmc_sq_a $OUT/pmc_sq_b $OUT/pmc_sq_probe.log",
         "# Three launches per kernel; figures are the mean of launches 2 and 3. Counters are summed over 8 XCDs x 4 shader engines.",
         "# cycles = GRBM_GUI_ACTIVE / 8 (per XCD). clock = cycles / duration: only meaningful for the long kernels (GUI_ACTIVE also",
         "#   counts ~15-25 k cycles around a dispatch, which dominates a 20 us kernel).",
         "# MFMA busy = SQ_VALU_MFMA_BUSY_CYCLES / (cycles x 1024 SIMDs)  (rocprofv3's MfmaUtil expression).",
         "# co-exec = SQ_VALU_MFMA_COEXEC_CYCLES / (cycles x 1024): share of time a SIMD had the matrix pipe busy AND issued another VALU op.",
         "# VALU/MFMA = (SQ_INSTS_VALU - SQ_INSTS_MFMA) / SQ_INSTS_MFMA; trans/MFMA = SQ_INSTS_VALU_TRANS_F32 / SQ_INSTS_MFMA (exp2).",
         "# occupancy = 4 x SQ_WAVE_CYCLES / (cycles x 1024)  waves per SIMD (SQ_WAVE_CYCLES counts in units of 4 cycles).",
         "# issue-wait = SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES: share of wave time spent waiting for an issue slot.",
         "# LDS busy = SQ_LDS_IDX_ACTIVE / (cycles x 256 CUs) (rocprofv3's LdsUtil); bank conflicts = SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE.",
         f"# attention launch plan at this shape: {plan}",
         "#",
         f"# {'kernel':58s} {'us':>7s} {'cycles':>8s} {'MHz':>6s} {'MFMA busy':>9s} {'co-exec':>8s} {'MFMA insts':>11s} {'VALU/MFMA':>9s} "
         f"{'trans/MFMA':>10s} {'occup.':>6s} {'issue-wait':>10s} {'LDS busy':>8s} {'LDS confl.':>10s} {'LDS B/WG':>8s} {'scratch':>7s}"]
    nan = float("nan")
    for n in a:
        if n not in b:
            continue
        x, y = a[n], b[n]
        cyc, cyc_b = x["GRBM_GUI_ACTIVE"] / XCDS, y["GRBM_GUI_ACTIVE"] / XCDS
        mf = x["SQ_INSTS_MFMA"]
        long_k = x["dur"] > 200e3
        L.append(f"  {_short(n)[:58]:58s} {x['dur'] / 1e3:7.1f} {cyc:8.0f} {(cyc / (x['dur'] / 1e3) if long_k else nan):6.0f} "
                 f"{100 * x['SQ_VALU_MFMA_BUSY_CYCLES'] / (cyc * SIMDS):8.1f}% {100 * x['SQ_VALU_MFMA_COEXEC_CYCLES'] / (cyc * SIMDS):7.1f}% {mf:11.3e} "
                 f"{((y['SQ_INSTS_VALU'] - mf) / mf if mf else nan):9.2f} {(y['SQ_INSTS_VALU_TRANS_F32'] / mf if mf else nan):10.2f} "
                 f"{4 * x['SQ_WAVE_CYCLES'] / (cyc * SIMDS):6.2f} {100 * y['SQ_WAIT_INST_ANY'] / x['SQ_WAVE_CYCLES']:9.1f}% "
                 f"{100 * y['SQ_LDS_IDX_ACTIVE'] / (cyc_b * CUS):7.1f}% "
                 f"{(100 * y['SQ_LDS_BANK_CONFLICT'] / y['SQ_LDS_IDX_ACTIVE'] if y['SQ_LDS_IDX_ACTIVE'] else 0):9.1f}% {x['lds']:>8s} {x['scratch']:>7s}")
    main = _plan_kernels(plan)[0]
    at = [n for n in a if _is_kernel(main, n)][0]
    x = a[at]
    cyc = x["GRBM_GUI_ACTIVE"] / XCDS
    busy = x["SQ_VALU_MFMA_BUSY_CYCLES"] / (cyc * SIMDS)
    mhz = cyc / (x["dur"] / 1e3)
    L += ["#",
          "# Reading, attention main launch (the first launch of the plan; the key-split last round and its merge are the next two lines):",
          f"#   {x['SQ_INSTS_MFMA']:.4g} v_mfma_f32_32x32x16_bf16 x 32768 flop = {x['SQ_INSTS_MFMA'] * 32768 / 1e12:.4f} TFLOP, each busy 32 cycles "
          f"({x['SQ_VALU_MFMA_BUSY_CYCLES'] / x['SQ_INSTS_MFMA']:.1f} measured);",
          f"#   the matrix pipe is busy {100 * busy:.1f} % of the kernel's cycles, and the kernel's cycles run at {mhz:.0f} MHz, not the 2400 MHz "
          "the 2.5 PFLOP/s peak assumes",
          f"#   ({100 * busy:.1f} % x {mhz:.0f}/2400 = {100 * busy * mhz / 2400:.1f} % of nominal peak for this launch). The library GEMMs run at the "
          "same reduced clock.",
          MARK + json.dumps({"attention_plan": plan, "main_kernel": at, "mfma_busy_frac": round(busy, 4), "clock_MHz": round(mhz, 1)})]
    text = "\n".join(L) + "\n"
    (PROFILES / COUNTERS_FILE).write_text(text)
    return text


# ------------------------------------------------------------------------------------------ traffic
def summarise_traffic(dir_fetch: str, dir_write: str, probe_stdout: str) -> str:
    probe = _probe_json(probe_stdout)
    plan = probe["attention_plan"]
    copy_kib = probe["copy_bytes_each_way"] / 1024.0
    readings: dict[str, dict[str, list[float]]] = {"FETCH_SIZE": collections.OrderedDict(), "WRITE_SIZE": collections.OrderedDict()}
    for counter, directory in (("FETCH_SIZE", dir_fetch), ("WRITE_SIZE", dir_write)):
        for e in _dispatches(directory).values():
            if (_ours(e["name"]) or "copyBuffer" in e["name"]) and counter in e:
                readings[counter].setdefault(e["name"], []).append(e[counter])
    _check_plan_in_trace(plan, list(readings["FETCH_SIZE"]), "FETCH_SIZE pass")
    copy = [n for n in readings["FETCH_SIZE"] if "copyBuffer" in n][0]
    scale = {c: copy_kib / (sum(readings[c][copy]) / len(readings[c][copy])) for c in readings}
    L = ["HBM traffic of one joint-attention call at the headline shape (B=2, 24 heads x 128, S=4352, bf16),",
         "from two rocprofv3 counter passes on one MI355X (each pass in a run of its own, no trace domains):",
         "",
         "  export TMPDIR=/tmp OUT=<a scratch directory>",
         "  rocprofv3 --pmc FETCH_SIZE --output-format csv -d $OUT/pmc_fetch -o f -- python3 bench.py --traffic-probe > $OUT/pmc_traffic_probe.log",
         "  rocprofv3 --pmc WRITE_SIZE --output-format csv -d $OUT/pmc_write -o w -- python3 bench.py --traffic-probe",
         "  python3 -m vllm_omni_amd.profiling traffic $OUT/pmc_fetch $OUT/pmc_write $OUT/pmc_traffic_probe.log",
         "",
         f"bench.py --traffic-probe makes the attention call 4 times and a plain {copy_kib / 1024:.0f} MiB device-to-device copy 4 times",
         f"(known traffic: {copy_kib:.0f} KiB read, {copy_kib:.0f} KiB written), nothing else. Launch plan of one call at this shape:",
         f"  {plan}",
         "(the units that fill whole rounds of the 512 workgroup slots, the left-over units cut into key ranges that write",
         "fp32 partial results, and the merge of those partials).",
         "",
         f"{'counter':12s} {'kernel':60s} per-dispatch readings (KiB as reported)"]
    for c in ("FETCH_SIZE", "WRITE_SIZE"):
        for n, vals in readings[c].items():
            L.append(f"{c:12s} {_short(n)[:60]:60s} " + " ".join(f"{v:.0f}" for v in vals))
    L += ["", f"Scale factors from the copy (known KiB / reading): FETCH_SIZE x{scale['FETCH_SIZE']:.3f}, WRITE_SIZE x{scale['WRITE_SIZE']:.3f}.",
          "", f"{'mean of the dispatches, scaled:':60s} {'fetched':>10s} {'written':>10s}"]
    total = {"FETCH_SIZE": 0.0, "WRITE_SIZE": 0.0}
    for kern in _plan_kernels(plan):
        row = {}
        for c in ("FETCH_SIZE", "WRITE_SIZE"):
            n = [k for k in readings[c] if _is_kernel(kern, k)][0]
            row[c] = sum(readings[c][n]) / len(readings[c][n]) * scale[c] * 1024.0
            total[c] += row[c]
        L.append(f"  {kern[:58]:58s} {row['FETCH_SIZE'] / 1e6:8.1f} MB {row['WRITE_SIZE'] / 1e6:8.1f} MB")
    both = total["FETCH_SIZE"] + total["WRITE_SIZE"]
    algo = probe["attention_min_bytes"]
    L += [f"  {'one call':58s} {total['FETCH_SIZE'] / 1e6:8.1f} MB {total['WRITE_SIZE'] / 1e6:8.1f} MB   = {both / 1e6:.1f} MB",
          "",
          f"algorithmic minimum (q, k, v read once, o written once): {algo / 1e6:.1f} MB; ratio {both / algo:.2f}. The excess is K/V re-reads",
          "that miss L2 (K and V of a head are re-read by the 34 query blocks of that head; the XCD-contiguous workgroup order",
          "keeps most of them in L2) and the key split (partials written and read back, K/V ranges read again). The call is",
          f"MFMA-bound: {both / 1e6:.0f} MB in about 0.455 ms is {both / 0.455e-3 / 1e12:.1f} TB/s, {100 * both / 0.455e-3 / 8e12:.0f} % of HBM peak.",
          MARK + json.dumps({"attention_plan": plan, "traffic_bytes": round(both), "fetched_bytes": round(total["FETCH_SIZE"]),
                             "written_bytes": round(total["WRITE_SIZE"]), "scale_fetch": round(scale["FETCH_SIZE"], 4),
                             "scale_write": round(scale["WRITE_SIZE"], 4)})]
    text = "\n".join(L) + "\n"
    (PROFILES / TRAFFIC_FILE).write_text(text)
    return text


# ------------------------------------------------------------------------------------------ step trace
_STEP_NOTES = {
    "qwen_image": ("Qwen-Image-shape denoise step (60 blocks, B=2, 4096+256 tokens)", "",
                   ["# GELU and the image stream's gated residuals run inside the GEMM epilogues (odit_linear -> the Cijk_* kernels); the",
                    "# text stream's MLP down-projection with its gated residual is gemm_bf16_streamk_kernel, its other gated residual the",
                    "# gated_residual_kernel rows."]),
    "flux": ("FLUX.1-shape denoise step (19 dual-stream + 38 single-stream blocks, B=1, 4096+512 tokens)", " --workload flux", []),
    "wan": ("Wan2.2-shape denoise step (40 blocks, B=2, 32760 video tokens, 512 text tokens)", " --workload wan", []),
}


def summarise_step(directory: str, bench_stdout: str, workload: str) -> str:
    title, flag, notes = _STEP_NOTES[workload]
    rows = list(csv.DictReader(open(_one(os.path.join(directory, "**", "*kernel_stats.csv")))))
    d = _probe_json(bench_stdout)
    r = d["roofline"]
    steps = d["steps"] + d["warmup"]
    out = [f"# rocprofv3 kernel-trace summary: bench.py, {title}, MI355X",
           "# commands (from the repo root, on the GPU box):",
           f"#   export TMPDIR=/tmp OUT=<a scratch directory>; rocprofv3 --kernel-trace --stats --output-format csv -d $OUT/prof_{workload} -o bench -- "
           f"python3 bench.py{flag} --steps {d['steps']} --warmup {d['warmup']} --no-cpu --no-kernels --no-in-step --no-teacache > $OUT/prof_{workload}.log",
           f"#   python3 -m vllm_omni_amd.profiling step $OUT/prof_{workload} $OUT/prof_{workload}.log {workload}",
           f"# {steps} steps recorded ({d['warmup']} warm-up + {d['steps']} timed) => per-step time = total / {steps}. Weight-initialisation kernels of the",
           "# synthetic model (at::native::distribution_* = normal_ init, FillFunctor = zero_ init, __amd_rocclr_copyBuffer = stacking the",
           "# modulation weights) are part of the run but not of a step."] + notes + [
           f"# bench.py line of this run (under the profiler): {d['value']:.3f} steps/s, {d['ms_per_step']:.1f} ms/step; attention avg "
           f"{r['avg_ms'] * 1e3:.0f} us/call by HIP events",
           f"#   = {r['achieved']:.0f} TFLOP/s = {r['frac']:.3f} of 2500 TFLOP/s."]
    attn = [x for x in rows if "attn_" in x["Name"]]
    if attn:
        out.append("# attention kernels, average under the profiler: " +
                   " + ".join(f"{float(x['AverageNs']) / 1e3:.1f} us ({_short(x['Name'])}, {int(x['Calls']) // steps} per step)" for x in attn))
    out += ["#", "#  total ms      %  calls    avg us    min us  kernel"]
    for x in rows[:26]:
        out.append(f"{int(x['TotalDurationNs']) / 1e6:10.2f} {float(x['Percentage']):6.2f} {int(x['Calls']):6d} {float(x['AverageNs']) / 1e3:9.1f} "
                   f"{int(x['MinNs']) / 1e3:9.1f}  {x['Name'][:120]}")
    text = "\n".join(out) + "\n"
    (PROFILES / f"bench_{workload}_step_kernel_stats.txt").write_text(text)
    return text


def main(argv: list[str]) -> int:
    if len(argv) == 4 and argv[0] == "counters":
        print(summarise_counters(*argv[1:]))
    elif len(argv) == 4 and argv[0] == "traffic":
        print(summarise_traffic(*argv[1:]))
    elif len(argv) == 4 and argv[0] == "step" and argv[3] in _STEP_NOTES:
        print(summarise_step(*argv[1:]))
    else:
        sys.stderr.write(__doc__)
        return 2
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
