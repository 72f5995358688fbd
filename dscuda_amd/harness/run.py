"""Runtime tables, correctness checks and profiler launches of the library's operations, one entry point.

    python -m dscuda_amd.harness.run mla --suite quick
    python -m dscuda_amd.harness.run all --suite full --output /tmp/runtime
    python -m dscuda_amd.harness.run mla --test
    python -m dscuda_amd.harness.run mla_prefill --suite metric --operation forward --reference none
    rocprofv3 --kernel-trace --stats -- python3 -m dscuda_amd.harness.run mla --suite h100 --profile --backend custom

The command line is the reference's (``benchmarks/run.py:13-27``): family, ``--suite quick|full|h100``, ``--test``
(check the library against PyTorch on the small ragged shapes, no timing), ``--reference``, ``--operation``,
``--profile`` with ``--backend`` (one uncaptured call per backend, for a profiler wrapped around the process), and
the four timing knobs.  Additions: the family ``mla_prefill``, the suite ``metric`` and ``--output``.  The only
reference backend on this platform is PyTorch (``--reference pytorch``, the default); ``--reference none`` times the
library alone, which the ``metric`` suite needs where fp32 PyTorch would take tens of gigabytes.

Per family the run prints the Markdown table and writes ``<family>.csv``, ``<family>.md`` and
``<family>_samples.json`` (``tables.py``).  What is run is decided by ``catalogue.py``, how it is timed by
``replay.py``.
"""

from __future__ import annotations

import argparse
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[2]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

from dscuda_amd.harness import catalogue, replay, tables  # noqa: E402

UNAVAILABLE = ("cublas", "deepgemm", "fa2", "fa3", "fa4", "flash_attention_2", "flashmla", "both", "all")


def parse(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("family", choices=(*catalogue.FAMILIES, "all"))
    parser.add_argument("--suite", choices=catalogue.SUITES, default="quick")
    parser.add_argument("--test", action="store_true", help="check the library against PyTorch on the test shapes; no timing")
    parser.add_argument("--reference", default="pytorch", help="pytorch (default) or none")
    parser.add_argument("--operation", help="only this operation: forward, backward or decode")
    parser.add_argument("--profile", action="store_true", help="one uncaptured, synchronised call per backend; no timing")
    parser.add_argument("--backend", choices=("custom", "reference", "all"), default="all", help="backend(s) to profile")
    parser.add_argument("--graph-operations", type=int, default=10, help="calls recorded into one graph")
    parser.add_argument("--warmup-ms", type=float, default=1000)
    parser.add_argument("--sample-ms", type=float, default=20)
    parser.add_argument("--trials", type=int, default=9)
    parser.add_argument("--output", default=str(ROOT / "build" / "runtime"), help="directory of the report files")
    args = parser.parse_args(argv)
    reference = args.reference.lower()
    if reference in UNAVAILABLE:
        parser.error(f"--reference {args.reference}: that library does not exist on this platform; use pytorch or none")
    if reference not in ("pytorch", "none"):
        parser.error(f"--reference {args.reference}: unknown; use pytorch or none")
    if args.test and reference == "none":
        parser.error("--test compares with PyTorch: it cannot run with --reference none")
    args.with_reference = reference == "pytorch"
    try:
        args.settings = replay.Settings(args.graph_operations, args.warmup_ms, args.sample_ms, args.trials)
    except ValueError as error:
        parser.error(str(error))
    return parser, args


def _described(workload, backend, error):
    return type(error)(f"{workload.family}: {workload.label}, bf16, {workload.operation}, {backend}\n{error}")


def check_once(bound, only_custom: bool) -> None:
    """Every backend once, eagerly, synchronised (so that an asynchronous fault surfaces here and names its
    workload), compared with the expected tensors."""
    import torch
    for backend, call in bound.backends.items():
        if only_custom and backend != "custom":
            continue
        try:
            outputs = call()
            torch.cuda.current_stream().synchronize()
            bound.verify(backend, outputs)
        except (AssertionError, RuntimeError) as error:
            raise _described(bound.workload, backend, error) from error


def profile_once(bound, which: str) -> None:
    """One call per chosen backend between two synchronisations, announced on stdout: the profiler around the
    process sees exactly the kernels of that call after the announcement."""
    import torch
    for backend, call in bound.backends.items():
        kind = "custom" if backend == "custom" else "reference"
        if which not in ("all", kind):
            continue
        torch.cuda.synchronize()
        print(f"profile: {bound.workload.label}/{bound.dtype}/{backend}/{bound.workload.operation}", flush=True)
        with torch.no_grad():
            call()
        torch.cuda.synchronize()


def run_family(family: str, args) -> str | None:
    """Returns what to print for the family."""
    import torch
    workloads = catalogue.select(family, args.suite, args.test, args.operation)
    rows, samples = [], []
    # A profiler run of the library alone binds no PyTorch expression: nothing but the library's kernels runs in
    # the process, and no autograd worker thread is ever started in it (see `finish`).
    library_only = args.profile and args.backend == "custom"
    for workload in workloads:
        bound = catalogue.bind(workload, args.with_reference and not library_only)
        if args.test and bound.expected is None:
            raise RuntimeError(f"{family}: {workload.label}: a correctness test needs a PyTorch result to compare with")
        check_once(bound, only_custom=args.test or library_only)
        if args.test:
            del bound
            continue
        if args.profile:
            profile_once(bound, args.backend)
            del bound
            continue
        try:
            timings = replay.time_backends(bound.backends, args.settings, bound.verify)
        except (AssertionError, RuntimeError) as error:
            raise _described(workload, "graph replay", error) from error
        rows += tables.summarise(workload.label, bound.dtype, workload.operation, timings)
        samples.append(dict(size=workload.label, dtype=bound.dtype, operation=workload.operation, samples_us=timings,
                            **bound.facts))
        del bound
        torch.cuda.empty_cache()
    if not workloads:
        return None
    if args.test:
        return f"{family}: {len(workloads)} correctness checks passed\n"
    if args.profile:
        return ""
    environment = {"gpu": torch.cuda.get_device_name(), "torch": torch.__version__, "hip": torch.version.hip}
    return tables.write(args.output, family, rows, samples, environment)


def finish(profile: bool) -> None:
    """Orderly end of a run: nothing of this process is left in flight or alive on the device side before the
    interpreter starts taking itself apart.

    One run of ``mla_prefill --test`` ended, after all results were printed and with every check passed, in
    ``terminate called without an active exception`` (abort at interpreter exit); runs of the same command before and
    after did not.  That message is the C++ runtime's for std::terminate() reached with no exception in flight: a
    joinable std::thread destroyed, or a thread unwound by force through a noexcept frame, which is what CPython 3.10
    does (pthread_exit) to a non-Python thread that asks for the GIL while the interpreter finalises.  This library
    starts no threads and registers no exit handlers; the process that aborted had, unlike the runs of the other
    families' ``--test`` that day, used PyTorch's autograd worker thread within milliseconds of its exit (the last
    workload of that family is a backward check whose expected gradients come from ``torch.autograd.grad``).  The
    cause has not been shown beyond that, so the exit is made as quiet as this module can make it: references
    dropped and collected, the device idle and its cached blocks returned, output flushed; then a timed run leaves
    through ``common.leave`` (no exit-time teardown at all), while a profiler run, whose tool writes its trace from
    an exit handler, takes the ordinary exit, having started no autograd thread when only the library is profiled.
    ``faulthandler`` is armed in ``main`` so that an abort, should one come again, names the threads alive in it."""
    import gc

    import torch
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    sys.stdout.flush()
    sys.stderr.flush()
    if not profile:
        from dscuda_amd.harness import common
        common.leave()


def main(argv=None):
    parser, args = parse(argv)
    import faulthandler

    import torch
    faulthandler.enable()
    if not torch.cuda.is_available():
        sys.exit("dscuda_amd.harness.run needs a GPU")
    torch.manual_seed(2026)
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    side = torch.cuda.Stream()          # graphs are captured on a stream of their own, never the default one
    side.wait_stream(torch.cuda.current_stream())
    families = catalogue.FAMILIES if args.family == "all" else (args.family,)
    with torch.cuda.stream(side):
        for family in families:
            text = run_family(family, args)
            side.synchronize()
            if text is None:
                if args.family != "all":
                    parser.error("No matching operations.")
                continue
            print(text, end="")
    torch.cuda.current_stream().wait_stream(side)
    del side
    return args


if __name__ == "__main__":
    finish(main().profile)
