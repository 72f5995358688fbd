"""Two-pass rocprofv3 capture of the attention kernels and the table built from it.

Counterpart of the reference's ``scripts/profile.sh`` (a timing pass and a
counter pass per case around the standalone programs, ``profile.sh:143-185``)
and ``scripts/extract_ncu.py`` (the per-kernel duration / DRAM traffic /
throughput / registers / spills table, ``extract_ncu.py:193-326``), on rocprofv3:

    python -m dscuda_amd.profiler.capture {metric|mla|flash_attention} [quick|full] [profile|extract]
        [--out DIR] [--profiles DIR] [--only STEM] [--passes time,fetch,write,mfma,cache,waits,lds]
        [--no-gate] [--commit HASH]

``profile`` first runs the family's GPU correctness tests (the reference gates
its captures on its tests the same way, ``scripts/profile.sh:109-113``;
``--no-gate`` skips that), then runs every case of the family once per pass,
each pass a rocprofv3 process of its own (a kernel trace, or one ``--pmc``
group that fits the hardware's counter blocks), raw CSV under ``--out``; then
extracts.  ``extract`` only rebuilds the tables from raw output that is already
there.  The tables go to ``--profiles`` as one ``<stem>.md`` per case plus
``capture_<family>.md`` and ``<family>_environment.md`` (GPU, ROCm, compiler,
commit: the counterpart of ``scripts/profile.sh:129-141``).

What a row holds, per kernel of a case:

* launches and duration: mean over the second half of the launches of the
  timing pass (the chip's clock needs some tens of back-to-back launches to
  settle, so the first launches are reported separately);
* bytes the L2 caches fetched from / wrote to the fabric per launch:
  ``FETCH_SIZE`` / ``WRITE_SIZE`` (KiB per dispatch) times the factor the same
  counter shows for a plain device copy of known size (the ``copy`` case of
  the metric family).  These are L2 misses and write-backs: the Infinity Cache
  may serve them, so they bound the HBM bytes from above;
* L2 hit rate ``TCC_HIT_sum / (TCC_HIT_sum + TCC_MISS_sum)`` (the reference's
  table carries L1 / L2 hit rates, ``scripts/extract_ncu.py:227-231``) and the
  read requests the L2s sent on (``TCC_EA0_RDREQ_sum``);
* matrix-pipe utilisation ``SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / XCDS *
  SIMDS)`` and the shader clock ``GRBM_GUI_ACTIVE / XCDS / duration`` of the
  counter pass, LDS bank-conflict cycles;
* registers per lane (rocprofv3's VGPR_Count is in units of two registers of
  the unified arch + accumulator file on this part, so it is doubled here),
  scratch bytes per lane (spills) and the statically declared LDS bytes per
  workgroup as the dispatch packets report them (dynamic LDS is not in them).
"""

from __future__ import annotations

import argparse
import collections
import csv
import os
import shlex
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[2]
BUILD = ROOT / "build"
CASE_SCRIPT = ROOT / "dscuda_amd" / "harness" / "profile_case.py"

XCDS = 8
SIMDS = 256 * 4
COPY_KIB = float(1 << 20)   # the copy case moves 1 GiB each way

PASSES = {
    "time": ["--kernel-trace", "--stats"],
    "fetch": ["--pmc", "FETCH_SIZE"],
    "write": ["--pmc", "WRITE_SIZE"],
    "mfma": ["--pmc", "SQ_VALU_MFMA_BUSY_CYCLES", "SQ_BUSY_CU_CYCLES", "SQ_WAVE_CYCLES", "SQ_INSTS_LDS",
             "SQ_LDS_BANK_CONFLICT", "SQ_INSTS_VALU", "GRBM_GUI_ACTIVE"],
    "waits": ["--pmc", "SQ_WAIT_ANY", "SQ_WAIT_INST_ANY", "SQ_WAIT_INST_LDS", "SQ_ACTIVE_INST_ANY",
              "SQ_ACTIVE_INST_VALU", "SQ_ACTIVE_INST_LDS", "SQ_WAVE_CYCLES", "SQ_INSTS_VMEM"],
    "lds": ["--pmc", "SQ_INSTS_LDS_LOAD", "SQ_INSTS_LDS_LOAD_BANDWIDTH", "SQ_LDS_IDX_ACTIVE", "SQ_LDS_DATA_FIFO_FULL",
            "SQ_LDS_CMD_FIFO_FULL", "SQ_INST_LEVEL_LDS", "SQ_INSTS_MFMA", "SQ_BUSY_CYCLES"],
}
PASSES["cache"] = ["--pmc", "TCC_HIT_sum", "TCC_MISS_sum", "TCC_EA0_RDREQ_sum"]
EXTRA_PASSES = ("waits", "lds", "cache")   # reported counter by counter below the table; a failing one is skipped
DEFAULT_PASSES = ("time", "fetch", "write", "mfma", "cache", "waits", "lds")

# GPU correctness tests that must pass before a family is captured
GATES = {
    "metric": ["tests/test_gpu_forward.py", "tests/test_gpu_backward.py", "tests/test_gpu_decode.py"],
    "mla": ["tests/test_gpu_decode.py", "tests/test_gpu_backward.py", "tests/test_gpu_profiler_programs.py"],
    "flash_attention": ["tests/test_gpu_forward.py", "tests/test_gpu_profiler_programs.py"],
}

Case = collections.namedtuple("Case", "stem label command counter_command kernels")


def _python_case(workload, steps, counter_steps, *extra):
    base = [sys.executable, str(CASE_SCRIPT), workload, *map(str, extra)]
    return base + ["--steps", str(steps)], base + ["--steps", str(counter_steps)]


def copy_case():
    """A plain device copy of 1 GiB: what FETCH_SIZE / WRITE_SIZE read for a known amount of traffic."""
    command, counter_command = _python_case("copy", 12, 6)
    return Case("copy_1GiB", "device copy of 1 GiB (FETCH_SIZE / WRITE_SIZE calibration)", command, counter_command,
                ["copyBuffer"])


def metric_cases(suite):
    """The workloads of the headline metric (synthetic inputs drawn on the GPU) and the copy calibration."""
    cases = []

    def add(stem, label, workload, steps, counter_steps, kernels, *extra):
        command, counter_command = _python_case(workload, steps, counter_steps, *extra)
        cases.append(Case(stem, label, command, counter_command, kernels))

    add("mla_prefill_forward_S4096_H128", "MLA prefill forward B=1 S=4096 H=128 192/128", "forward", 160, 60,
        ["attention_forward"])
    add("mla_prefill_backward_S4096_H128", "MLA prefill backward B=1 S=4096 H=128 192/128", "backward", 80, 30,
        ["attention_backward", "attention_key_value", "attention_query"])
    add("mla_decode_B64_H128", "absorbed MLA decode B=64 H=128 lengths U[1024,8192] seed 3", "decode", 300, 100,
        ["mla_decode"])
    add("flash_forward_S512_H8_D64", "flash forward B=1 H=8 S=512 D=64", "flash", 300, 100, ["attention_forward"])
    add("mla_absorbed_T4096_H128", "absorbed MLA prefill forward + backward (dscuda_mla_forward / _backward) B=1 T=4096 H=128",
        "absorbed", 6, 3, ["mla_absorbed"])
    add("mla_projection_T4096_H128", "W_UK absorb and W_UV un-absorb of 4096 tokens x 128 heads", "projection", 60, 20,
        ["mla_absorb_query", "mla_unabsorb_output"])
    if suite == "full":
        add("mla_prefill_forward_S16384_H128", "MLA prefill forward B=1 S=16384 H=128 192/128", "forward", 16, 8,
            ["attention_forward"], "--seq", 16384)
        add("mla_prefill_backward_S16384_H128", "MLA prefill backward B=1 S=16384 H=128 192/128", "backward", 8, 4,
            ["attention_backward", "attention_key_value", "attention_query"], "--seq", 16384)
        # the same launches on all-zero inputs: same instruction streams, operands that do not toggle
        add("mla_prefill_forward_S4096_H128_zero_inputs", "MLA prefill forward B=1 S=4096 H=128 192/128, all inputs zero",
            "forward", 160, 60, ["attention_forward"], "--data", "zero")
        add("mla_prefill_backward_S4096_H128_zero_inputs", "MLA prefill backward B=1 S=4096 H=128 192/128, all inputs zero",
            "backward", 80, 30, ["attention_backward", "attention_key_value", "attention_query"], "--data", "zero")
        add("mla_decode_B64_H128_zero_inputs", "absorbed MLA decode B=64 H=128 lengths U[1024,8192] seed 3, query and cache zero",
            "decode", 300, 100, ["mla_decode"], "--data", "zero")
    return cases


def mla_cases(suite):
    """The reference's profile_mla cases (scripts/profile.sh:281-296) on the standalone programs."""
    cases = []
    for sequence in ((128,) if suite == "quick" else (128, 256, 512)):
        command = [str(BUILD / "benchmark_mla"), "1", str(sequence), "8", "512", "64"]
        cases.append(Case(f"mla_T{sequence}_forward_backward", f"B=1,T={sequence},H=8,D=512,R=64/custom/forward_backward",
                          command, command, ["mla_absorbed"]))
        command = [str(BUILD / "benchmark_mla_decode"), "2", str(sequence), "16", "512", "64", "8"]
        cases.append(Case(f"mla_KV{sequence}_decode", f"B=2,KV={sequence},H=16,D=512,R=64/custom/decode", command, command,
                          ["mla_decode"]))
    return cases


def flash_cases(suite):
    """The reference's profile_flash_attention shapes (scripts/profile.sh:232-279), custom side."""
    cases = []
    shapes = [(2, 512, 8, 128)] if suite == "quick" else [(2, 512, 8, 128), (1, 2048, 8, 128), (1, 512, 8, 64)]
    for batch, sequence, heads, dimension in shapes:
        command = [str(BUILD / "benchmark_flash_attention"), *map(str, (batch, sequence, heads, dimension)), "forward"]
        cases.append(Case(f"flash_B{batch}_T{sequence}_H{heads}_D{dimension}_forward",
                          f"B={batch},T={sequence},H={heads},D={dimension}/custom/forward", command, command,
                          ["attention_forward"]))
    return cases


FAMILIES = {"metric": metric_cases, "mla": mla_cases, "flash_attention": flash_cases}


def rocprof_command(pass_name, directory, program):
    return ["rocprofv3", *PASSES[pass_name], "--output-format", "csv", "-d", str(directory), "-o", "x", "--", *program]


def run_pass(case, pass_name, out, limit):
    directory = out / case.stem / pass_name
    directory.mkdir(parents=True, exist_ok=True)
    program = case.command if pass_name == "time" else case.counter_command
    command = rocprof_command(pass_name, directory, program)
    (directory / "command.txt").write_text(shlex.join(command) + "\n")
    print(f"[capture] {case.stem} / {pass_name}", flush=True)
    environment = dict(os.environ, TMPDIR="/tmp", PYTHONPATH=str(ROOT))
    # a rocprofv3 that asks for more counters than a block holds hangs after its error line: hard limit
    result = subprocess.run(["timeout", "-s", "KILL", str(limit), *command], cwd="/tmp", env=environment,
                            capture_output=True, text=True)
    (directory / "log.txt").write_text(result.stdout[-4000:] + "\n--- stderr ---\n" + result.stderr[-4000:])
    if result.returncode != 0:
        message = f"{case.stem}/{pass_name}: rocprofv3 exited with {result.returncode}; see {directory / 'log.txt'}"
        if pass_name in EXTRA_PASSES:
            print(f"[capture] skipped: {message}", flush=True)   # a counter this rocprofv3 does not know
            return
        raise RuntimeError(message)


def run_gate(family):
    """The family's GPU tests, as the reference runs its own before a capture."""
    command = [sys.executable, "-u", "-m", "pytest", *GATES[family], "-m", "gpu", "-x", "-q", "--timeout", "300",
               "--timeout-method", "thread"]
    print("[capture] gate: " + shlex.join(command), flush=True)
    result = subprocess.run(command, cwd=ROOT, capture_output=True, text=True)
    tail = (result.stdout + result.stderr).strip().splitlines()[-1:]
    print("[capture] gate: " + " ".join(tail), flush=True)
    if result.returncode != 0:
        raise RuntimeError("the correctness gate failed; nothing was captured\n" + result.stdout[-3000:] + result.stderr[-2000:])


def _first_line(command):
    try:
        result = subprocess.run(command, capture_output=True, text=True, timeout=60)
    except (OSError, subprocess.TimeoutExpired):
        return "unavailable"
    lines = [line.strip() for line in (result.stdout + result.stderr).splitlines() if line.strip()]
    return lines[0] if lines else "unavailable"


def write_environment(family, suite, profiles, commit, gate):
    """What the capture ran on: `<family>_environment.md`."""
    gpu = "unavailable"
    try:
        result = subprocess.run(["rocminfo"], capture_output=True, text=True, timeout=60)
        # one block per agent: "Name:", "Marketing Name:", ..., "Device Type:"
        # (a GPU's "Compute Unit:" line follows its "Device Type:")
        found, name, marketing, is_gpu = [], "", "", False
        for line in result.stdout.splitlines():
            text = line.strip()
            if text.startswith("Name:"):
                name, is_gpu = text.split(":", 1)[1].strip(), False
            elif text.startswith("Marketing Name:"):
                marketing = text.split(":", 1)[1].strip()
            elif text.startswith("Device Type:"):
                is_gpu = "GPU" in text
            elif text.startswith("Compute Unit:") and is_gpu:
                found.append(f"{marketing or 'no marketing name'} ({name}, {text.split(':', 1)[1].strip()} compute units)")
                is_gpu = False
        gpu = "; ".join(dict.fromkeys(found)) or "unavailable"
    except (OSError, subprocess.TimeoutExpired):
        pass
    try:
        import torch
        if torch.cuda.is_available():
            properties = torch.cuda.get_device_properties(0)
            gpu += f"; as PyTorch names device 0: {properties.name or 'no name'}, {properties.total_memory / 2 ** 30:.0f} GiB"
    except Exception:   # noqa: BLE001 -- the record is written with or without it
        pass
    version_file = Path("/opt/rocm/.info/version")
    rocm = version_file.read_text().strip() if version_file.exists() else "unavailable"
    hipcc = [line for line in [_first_line(["/opt/rocm/bin/hipcc", "--version"])]][0]
    rocprof = _first_line(["rocprofv3", "--version"])
    try:
        import torch
        framework = f"{torch.__version__} (HIP {torch.version.hip})"
    except Exception:   # noqa: BLE001 -- the standalone programs need no PyTorch
        framework = "unavailable"
    lines = [f"# capture environment: family `{family}`, suite `{suite}`", "",
             f"- GPU: {gpu}", f"- ROCm: {rocm}", f"- compiler: {hipcc}", f"- profiler: {rocprof}",
             f"- PyTorch (device memory and streams of the Python cases): {framework}",
             f"- commit: {commit or 'not given (--commit)'}",
             f"- correctness gate before the capture: {gate}", ""]
    (profiles / f"{family}_environment.md").write_text("\n".join(lines))


# ---- extraction ---------------------------------------------------------------------------------------------

def short_name(name: str) -> str:
    name = name.replace("void ", "").replace("(anonymous namespace)::", "").replace("dscuda::", "")
    cut = name.find("(")
    return name if cut < 0 else name[:cut]


def mean(values):
    values = list(values)
    return sum(values) / len(values) if values else float("nan")


def settled(values):
    """Mean of the second half (all of them when there are fewer than four)."""
    values = list(values)
    return mean(values[len(values) // 2:] if len(values) >= 4 else values)


def read_trace(directory, wanted):
    rows = collections.OrderedDict()
    for path in sorted(directory.rglob("*_kernel_trace.csv")):
        with open(path, newline="") as handle:
            for row in csv.DictReader(handle):
                name = short_name(row["Kernel_Name"])
                if not any(text in name for text in wanted):
                    continue
                entry = rows.setdefault(name, {"durations": [], "vgpr": 0, "scratch": 0, "lds": 0})
                entry["durations"].append((int(row["End_Timestamp"]) - int(row["Start_Timestamp"])) / 1e3)
                entry["vgpr"] = 2 * int(row["VGPR_Count"]) + int(row["Accum_VGPR_Count"])
                entry["scratch"] = int(row["Scratch_Size"])
                entry["lds"] = int(row["LDS_Block_Size"])
    return rows


def read_counters(directory, wanted):
    """kernel -> counter -> list of per-dispatch values; kernel -> list of dispatch durations (us)."""
    table = collections.OrderedDict()
    spans = {}
    for path in sorted(directory.rglob("*_counter_collection.csv")):
        with open(path, newline="") as handle:
            seen = set()
            for row in csv.DictReader(handle):
                name = short_name(row["Kernel_Name"])
                if not any(text in name for text in wanted):
                    continue
                table.setdefault(name, collections.OrderedDict()).setdefault(row["Counter_Name"], []).append(
                    float(row["Counter_Value"]))
                key = (name, row["Dispatch_Id"])
                if key not in seen and row.get("Start_Timestamp") and row.get("End_Timestamp"):
                    seen.add(key)
                    spans.setdefault(name, []).append((int(row["End_Timestamp"]) - int(row["Start_Timestamp"])) / 1e3)
    return table, spans


def calibration(out):
    """(fetch factor, write factor) from the copy case: bytes moved / bytes the counter reports."""
    factors = []
    for pass_name, counter in (("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")):
        table, _ = read_counters(out / "copy_1GiB" / pass_name, ["copyBuffer"])
        values = [settled(counters[counter]) for counters in table.values() if counter in counters]
        values = [value for value in values if value > COPY_KIB / 8]   # the 1 GiB copy, not the fills around it
        factors.append(COPY_KIB / mean(values) if values else float("nan"))
    return tuple(factors)


def extract_case(case, out, factors):
    directory = out / case.stem
    trace = read_trace(directory / "time", case.kernels)
    fetch, _ = read_counters(directory / "fetch", case.kernels)
    write, _ = read_counters(directory / "write", case.kernels)
    mfma, mfma_spans = read_counters(directory / "mfma", case.kernels)
    rows = []
    for kernel, entry in trace.items():
        durations = entry["durations"]
        row = {"kernel": kernel, "launches": len(durations), "first_us": mean(durations[:5]), "time_us": settled(durations),
               "vgpr": entry["vgpr"], "scratch": entry["scratch"], "lds": entry["lds"],
               "read_mb": float("nan"), "write_mb": float("nan"), "l2_hit_pct": float("nan"), "mfma_pct": float("nan"),
               "clock_ghz": float("nan"),
               "bank_conflict": float("nan"), "counter_us": float("nan")}
        if kernel in fetch and "FETCH_SIZE" in fetch[kernel]:
            row["read_mb"] = settled(fetch[kernel]["FETCH_SIZE"]) * factors[0] * 1024 / 1e6
        if kernel in write and "WRITE_SIZE" in write[kernel]:
            row["write_mb"] = settled(write[kernel]["WRITE_SIZE"]) * factors[1] * 1024 / 1e6
        if kernel in mfma:
            counters = mfma[kernel]
            span = settled(mfma_spans.get(kernel, []))
            row["counter_us"] = span
            if "GRBM_GUI_ACTIVE" in counters:
                cycles = settled(counters["GRBM_GUI_ACTIVE"]) / XCDS
                row["clock_ghz"] = cycles / span / 1e3 if span == span else float("nan")
                if "SQ_VALU_MFMA_BUSY_CYCLES" in counters:
                    row["mfma_pct"] = 100.0 * settled(counters["SQ_VALU_MFMA_BUSY_CYCLES"]) / (cycles * SIMDS)
            if "SQ_LDS_BANK_CONFLICT" in counters:
                row["bank_conflict"] = settled(counters["SQ_LDS_BANK_CONFLICT"])
        cache, _ = read_counters(directory / "cache", case.kernels)
        if kernel in cache and "TCC_HIT_sum" in cache[kernel] and "TCC_MISS_sum" in cache[kernel]:
            hits, misses = settled(cache[kernel]["TCC_HIT_sum"]), settled(cache[kernel]["TCC_MISS_sum"])
            if hits + misses > 0:
                row["l2_hit_pct"] = 100.0 * hits / (hits + misses)
        row["more"] = collections.OrderedDict()
        for pass_name in EXTRA_PASSES:
            table, _ = read_counters(directory / pass_name, case.kernels)
            for counter, values in table.get(kernel, {}).items():
                row["more"][f"{pass_name}:{counter}"] = settled(values)
        rows.append(row)
    return rows


COLUMNS = [("kernel", "kernel", "{}"), ("launches", "launches", "{:d}"), ("first_us", "first 5 us", "{:.1f}"),
           ("time_us", "settled us", "{:.1f}"), ("read_mb", "L2 fetch MB", "{:.1f}"), ("write_mb", "L2 write-back MB", "{:.1f}"),
           ("l2_hit_pct", "L2 hit %", "{:.1f}"), ("mfma_pct", "MFMA busy %", "{:.1f}"), ("clock_ghz", "clock GHz", "{:.2f}"),
           ("counter_us", "us in counter pass", "{:.1f}"), ("bank_conflict", "LDS bank conflict cycles", "{:.0f}"),
           ("vgpr", "registers/lane", "{:d}"), ("scratch", "scratch B/lane", "{:d}"),
           ("lds", "static LDS B", "{:d}")]


def cell(pattern, value):
    if isinstance(value, float) and value != value:
        return "-"
    return pattern.format(value)


def markdown_table(rows):
    lines = ["| " + " | ".join(title for _, title, _ in COLUMNS) + " |", "|" + "---|" * len(COLUMNS)]
    for row in rows:
        lines.append("| " + " | ".join(cell(pattern, row[key]) for key, _, pattern in COLUMNS) + " |")
    return lines


def portable(command: str, out: Path) -> str:
    """The recorded command with the checkout's location taken out: paths relative to the repository root
    (recognised by the top-level folder of the raw output `out`, the package and the build folder), the
    interpreter as `python3`."""
    try:
        raw = out.resolve().relative_to(ROOT.resolve()).parts[0]
    except (ValueError, IndexError):
        raw = out.name
    words = []
    for word in shlex.split(command):
        for anchor in (raw + "/", "dscuda_amd/", "build/"):
            cut = word.find("/" + anchor)
            if cut >= 0:
                word = word[cut + 1:]
                break
        if word.rsplit("/", 1)[-1] in ("python", "python3") or word.rsplit("/", 1)[-1].startswith("python3."):
            word = "python3"
        words.append(word)
    return shlex.join(words)


def write_case(case, rows, out, profiles, factors):
    lines = [f"# {case.label}", ""]
    lines.append("Commands (one rocprofv3 process per pass; raw CSV is not kept in the repository):")
    lines.append("")
    for pass_name in PASSES:
        recorded = out / case.stem / pass_name / "command.txt"
        if recorded.exists():
            lines.append(f"- {pass_name}: `{portable(recorded.read_text().strip(), out)}`")
    lines += ["", f"Counter calibration from the 1 GiB copy: FETCH_SIZE x {factors[0]:.3f}, WRITE_SIZE x {factors[1]:.3f}.",
              "Durations are the mean of the second half of the launches of the timing pass.",
              "L2 fetch / write-back: what the L2 caches exchanged with the fabric (Infinity Cache or HBM behind it): an upper",
              "bound of the HBM bytes.", ""]
    lines += markdown_table(rows)
    if any(row.get("more") for row in rows):
        lines += ["", "Further counters, mean per launch over the second half of the launches (summed over the chip as "
                      "rocprofv3 reports them):", ""]
        for row in rows:
            for name, value in row.get("more", {}).items():
                lines.append(f"    {row['kernel']} :: {name} = {value:.0f}")
    lines += ["", "Machine-readable (bytes per launch from the two traffic columns, microseconds from the settled column):", ""]
    for row in rows:
        total = (row["read_mb"] + row["write_mb"]) * 1e6
        lines.append(f"    {row['kernel']} :: time_us = {row['time_us']:.3f} ; fabric_bytes = "
                     f"{'nan' if total != total else format(total, '.0f')}")
    (profiles / f"{case.stem}.md").write_text("\n".join(lines) + "\n")


def write_overview(family, suite, cases, results, profiles):
    lines = [f"# rocprofv3 capture: family `{family}`, suite `{suite}`", "",
             "One row per kernel of each case; `python -m dscuda_amd.profiler.capture " + family + " " + suite +
             "` reproduces it.  The per-case files carry the exact commands.", ""]
    for case in cases:
        rows = results[case.stem]
        if not rows:
            continue
        lines += [f"## {case.label}", ""] + markdown_table(rows)
        total = sum(row["time_us"] for row in rows)
        read = sum(row["read_mb"] for row in rows)
        wrote = sum(row["write_mb"] for row in rows)
        lines += ["", f"total: {len(rows)} kernels, {total:.1f} us, L2 fetch {cell('{:.1f}', read)} MB, "
                      f"write-back {cell('{:.1f}', wrote)} MB", ""]
    (profiles / f"capture_{family}.md").write_text("\n".join(lines) + "\n")


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("family", choices=sorted(FAMILIES))
    parser.add_argument("suite", nargs="?", default="quick", choices=("quick", "full"))
    parser.add_argument("mode", nargs="?", default="profile", choices=("profile", "extract"))
    parser.add_argument("--out", type=Path, default=ROOT / "profiler_out" / "capture", help="raw profiler output")
    parser.add_argument("--profiles", type=Path, default=ROOT / "profiles")
    parser.add_argument("--only", action="append", default=[], help="case stems to run (default: all)")
    parser.add_argument("--passes", default=",".join(DEFAULT_PASSES))
    parser.add_argument("--limit", type=int, default=240, help="seconds before a pass is killed")
    parser.add_argument("--no-gate", action="store_true", help="do not run the family's GPU tests before the capture")
    parser.add_argument("--commit", default=os.environ.get("DSCUDA_AMD_COMMIT", ""), help="recorded in the environment file")
    args = parser.parse_args(argv)

    passes = [name for name in args.passes.split(",") if name]
    for name in passes:
        if name not in PASSES:
            parser.error(f"unknown pass {name}")
    cases = [copy_case()] + FAMILIES[args.family](args.suite)
    if args.only:
        cases = [case for case in cases if case.stem in args.only or case.stem == "copy_1GiB"]
    out = args.out.resolve()
    args.profiles.mkdir(parents=True, exist_ok=True)
    if args.mode == "profile":
        gate = "skipped (--no-gate)"
        if not args.no_gate:
            run_gate(args.family)
            gate = "passed: " + " ".join(GATES[args.family])
        write_environment(args.family, args.suite, args.profiles, args.commit, gate)
        for case in cases:
            for name in passes:
                run_pass(case, name, out, args.limit)
    factors = calibration(out) if (out / "copy_1GiB").exists() else (float("nan"), float("nan"))
    args.profiles.mkdir(parents=True, exist_ok=True)
    results = {}
    for case in cases:
        rows = extract_case(case, out, factors)
        results[case.stem] = rows
        if rows:
            write_case(case, rows, out, args.profiles, factors)
            for line in markdown_table(rows):
                print(line)
    write_overview(args.family, args.suite, cases, results, args.profiles)


if __name__ == "__main__":
    main()
