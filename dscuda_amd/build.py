"""Builds the two drop-in shared libraries with hipcc for gfx950.

Outputs ``build/libdscuda_mla_bench.so`` and
``build/libdscuda_flash_attention_bench.so`` under the repository root: the
file names the reference's harness loads (``benchmarks/common.py:19-20``,
``CMakeLists.txt:56-61``).  Objects are compiled in parallel, one hipcc
process per translation unit.  The standalone profiler programs
(``dscuda_amd/profiler/*.cpp``, the counterparts of the reference's
``benchmarks/attention/benchmark_*.cu`` launchers, ``CMakeLists.txt:43-50``) are
linked against them into ``build/`` as well.

Run ``python -m dscuda_amd.build`` (add ``--resource-usage`` to print the
compiler's per-kernel register / LDS / spill report).
"""

from __future__ import annotations

import argparse
import concurrent.futures
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]
CSRC = ROOT / "dscuda_amd" / "csrc"
BUILD = ROOT / "build"

ARCH = "gfx950"
# Packed fp32 VALU ops are switched off for every device compile.
COMMON_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]

LIBRARIES = {
    "libdscuda_mla_bench.so": ["api_mla", "attn_fwd", "attn_bwd", "mla_absorbed", "mla_decode", "mla_projection", "rope"],
    "libdscuda_flash_attention_bench.so": ["api_flash", "attn_fwd", "attn_bwd"],
}


# executable -> (source under dscuda_amd/profiler, library it links)
PROGRAMS = {
    "benchmark_mla": ("benchmark_mla.cpp", "libdscuda_mla_bench.so"),
    "benchmark_mla_decode": ("benchmark_mla_decode.cpp", "libdscuda_mla_bench.so"),
    "benchmark_mla_prefill": ("benchmark_mla_prefill.cpp", "libdscuda_mla_bench.so"),
    "benchmark_flash_attention": ("benchmark_flash_attention.cpp", "libdscuda_flash_attention_bench.so"),
}
PROFILER = ROOT / "dscuda_amd" / "profiler"


def _hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _run(command, quiet_pattern="packed-fp32-ops"):
    result = subprocess.run(command, capture_output=True, text=True)
    noise = ("is not a recognized feature for this target", "1 warning generated", "warnings generated")
    lines = [line for line in (result.stdout + result.stderr).splitlines()
             if line.strip() and not any(n in line for n in noise)]
    if result.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(map(str, command)) + "\n" + "\n".join(lines))
    return lines


def compile_object(name: str, resource_usage: bool = False) -> Path:
    source = CSRC / f"{name}.hip"
    obj_dir = BUILD / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    target = obj_dir / f"{name}.o"
    command = [_hipcc(), *COMMON_FLAGS, "-c", str(source), "-o", str(target)]
    if resource_usage:
        command.insert(1, "-Rpass-analysis=kernel-resource-usage")
    lines = _run(command)
    if lines:
        print(f"[{name}]\n" + "\n".join(lines), file=sys.stderr)
    return target


def build_all(resource_usage: bool = False, jobs: int | None = None) -> dict[str, Path]:
    """Compile every translation unit and link both libraries.  Always recompiles."""
    names = sorted({name for parts in LIBRARIES.values() for name in parts})
    jobs = jobs or min(len(names), max(1, (os.cpu_count() or 2) - 1))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = dict(zip(names, pool.map(lambda n: compile_object(n, resource_usage), names)))
    outputs = {}
    for library, parts in LIBRARIES.items():
        target = BUILD / library
        _run([_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(target),
              *[str(objects[p]) for p in parts]])
        outputs[library] = target

    def link_program(item):
        program, (source, library) = item
        target = BUILD / program
        _run([_hipcc(), *COMMON_FLAGS, f"-I{PROFILER}", str(PROFILER / source), "-o", str(target),
              f"-L{BUILD}", f"-l:{library}", "-Wl,-rpath,$ORIGIN"])
        return program, target

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        outputs.update(dict(pool.map(link_program, PROGRAMS.items())))
    return outputs


def main():
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("--resource-usage", action="store_true")
    parser.add_argument("--jobs", type=int, default=None)
    args = parser.parse_args()
    for name, path in build_all(args.resource_usage, args.jobs).items():
        print(f"built {path}")


if __name__ == "__main__":
    main()
