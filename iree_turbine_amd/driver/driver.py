"""Command-line driver: runs MIOpen-driver-style commands on the MI355X kernels, times them and
optionally checks their numerics.

    python -m iree_turbine_amd.driver gemmfp16 --a_w 8192 --a_h 8192 --b_w 8192 --transB 1 --iter 20
    python -m iree_turbine_amd.driver --commands-file cmds.txt --csv out.csv --backend mi355 --backend torch
    python -m iree_turbine_amd.driver --verify-numerics aten::mm "[[512, 256], [256, 384]]" \\
        "['c10::Half', 'c10::Half']" "[[256, 1], [384, 1]]" "['', '']"

Command grammar, options, CSV layout (header `arguments`, then `<backend> min|max|mean|stddev|num_dispatches`
per backend, then the numerics columns), "N.A." rows and the exit code follow the reference driver
(iree/turbine/kernel/boo/driver/driver.py:40-61,176-458).  Differences, by design: the default backend is
this library's kernels, and device time is taken with HIP events on the launch stream (one pair per
iteration, microseconds) instead of a profiler trace, so a launch that needs a layout copy is timed as one
zone whose `num_dispatches` counts the copy kernels too.
"""

from __future__ import annotations

import argparse
import csv
import enum
import gc
import os
import shlex
import statistics
import sys
import traceback
from typing import Callable, NamedTuple, Sequence

import torch

from .backends import BACKEND_TO_FUNC_GENERATOR, DEFAULT_BACKEND, CountingCallable
from .numerics import (MEAN_CHECK_ATOL_DEFAULT, MEAN_CHECK_RTOL_DEFAULT, MIN_SAMPLES_DEFAULT, STDDEV_CHECK_ATOL_DEFAULT,
                       STDDEV_CHECK_RTOL_DEFAULT)
from .signatures import OpSignature, parse_command

ALL_STATS = ["min", "max", "mean", "stddev", "num_dispatches"]
NUMERICS_CSV_COLUMNS = ["numerics_pass", "boo_vs_ref_mean", "boo_vs_ref_stddev", "boo_vs_ref_max", "pytorch_vs_ref_mean",
                        "pytorch_vs_ref_stddev", "pytorch_vs_ref_max", "boo_vs_pytorch_mean", "boo_vs_pytorch_stddev",
                        "boo_vs_pytorch_max", "structured_test"]


class ZoneStats(NamedTuple):
    min: float | str = "N.A."
    max: float | str = "N.A."
    mean: float | str = "N.A."
    stddev: float | str = "N.A."
    num_dispatches: int | str = "N.A."


class Action(enum.Enum):
    """What the measurement does with one step of the launch loop."""
    NONE = 0             # run, do not time (first launch on a device, clean-up steps)
    RECORD = 1           # time it
    RECORD_AND_SAVE = 2  # time it; the last timed step before a pause


def get_timing_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(add_help=False)
    p.add_argument("--time", "-t", type=int, default=1, help="Enable timing")
    p.add_argument("--iter", type=int, default=100, help="Number of iterations to run")
    return p


def make_measurement_schedule(timing_iter: int, num_devices: int, iter_thresh: int):
    """(schedule_fn, total_num_iters, needs_cleanup).  The first launch on every device is not timed; after
    every `iter_thresh` launches per device all devices are synchronised and garbage is collected on an
    untimed step, and the step before such a pause closes the current recording window
    (driver.py:471-528; the same sequences as the reference's profiler schedule)."""
    num_cleanups = (timing_iter // num_devices + 1) // (iter_thresh - 1)
    total_num_iters = timing_iter + (num_cleanups + 1) * num_devices

    def needs_cleanup(step: int) -> bool:
        return (step // num_devices + 1) % iter_thresh == 0

    def schedule_fn(step: int) -> Action:
        if step < num_devices:
            return Action.NONE
        if step == total_num_iters - 1:
            return Action.RECORD_AND_SAVE
        if step >= total_num_iters:
            return Action.NONE
        if needs_cleanup(step):
            return Action.NONE
        if needs_cleanup(step + 1):
            return Action.RECORD_AND_SAVE
        return Action.RECORD

    return schedule_fn, total_num_iters, needs_cleanup


def _get_main_driver_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(
        prog="python -m iree_turbine_amd.driver",
        usage="%(prog)s [-h] [... MIOpenDriver command ...] [--commands-file COMMANDS_FILE]",
        description="Run a GEMM / attention command on the MI355X kernels.  With --commands-file every line of the "
                    "file is one command (tab-separated if the file ends in .tsv); other arguments are appended to each.",
    )
    p.add_argument("--commands-file", type=str, help="read commands from file")
    p.add_argument("--backend", dest="backends", type=str, choices=list(BACKEND_TO_FUNC_GENERATOR), action="append",
                   default=[], help=f"backend to run; may be repeated (default '{DEFAULT_BACKEND}')")
    p.add_argument("--csv", type=str, default=None, help="file to output timing information in csv format")
    p.add_argument("--gpu-id", default=0, type=int, help="torch.device('cuda:<gpu-id>') to run on; -1 = all visible devices")
    p.add_argument("--splat-input-value", default=None, type=float, help="use one value for all inputs (default: random)")
    p.add_argument("--verbose", action="store_true", default=None, help="print command/output on stdout")
    p.add_argument("--no-verbose", action="store_false", dest="verbose")
    p.add_argument("--verify-numerics", action="store_true", help="run the statistical numerics check as well")
    p.add_argument("--numerics-verbose", action="store_true", help="print the error statistics, not just PASS/FAIL")
    p.add_argument("--numerics-min-samples", type=int, default=MIN_SAMPLES_DEFAULT)
    p.add_argument("--numerics-stddev-rtol", type=float, default=STDDEV_CHECK_RTOL_DEFAULT)
    p.add_argument("--numerics-mean-atol", type=float, default=MEAN_CHECK_ATOL_DEFAULT)
    p.add_argument("--numerics-mean-rtol", type=float, default=MEAN_CHECK_RTOL_DEFAULT)
    p.add_argument("--numerics-stddev-atol", type=float, default=STDDEV_CHECK_ATOL_DEFAULT)
    p.add_argument("--numerics-reference-dtype", type=str, choices=["float32", "float64"], default="float64")
    p.add_argument("--skip-structured-tests", action="store_true")
    return p


def _get_devices(gpu_id: int) -> list[torch.device]:
    if gpu_id != -1:
        return [torch.device(f"cuda:{gpu_id}")]
    return [torch.device(f"cuda:{i}") for i in range(torch.cuda.device_count())]


def _as_tuple(result) -> tuple[torch.Tensor, ...]:
    if result is None:
        return ()
    return (result,) if isinstance(result, torch.Tensor) else tuple(result)


def run(func: CountingCallable, timing_args: argparse.Namespace, per_device_args: Sequence[tuple[torch.Tensor, ...]],
        devices: Sequence[torch.device], verbose: bool) -> list[float] | None:
    """Applies `func` `iter` times round-robin over the devices; returns the device time of every timed launch
    in microseconds (None when timing is off)."""

    def pause_and_collect():
        for d in devices:
            torch.cuda.synchronize(d)
        gc.collect()

    pause_and_collect()
    torch.cuda.empty_cache()
    example = _as_tuple(func(*per_device_args[0]))
    out_bytes = max(1, sum(x.element_size() * x.numel() for x in example))
    in_bytes = sum(x.element_size() * x.numel() for x in per_device_args[0])
    num_devices = len(per_device_args)
    # outputs are freed asynchronously: pause before half of the device memory could be queued up
    iter_thresh = (torch.cuda.get_device_properties(devices[0]).total_memory // 2 - in_bytes) // out_bytes
    if timing_args.time and iter_thresh <= 1:
        raise RuntimeError("Cannot reliably time if cleanup is needed after every step.")
    if timing_args.time:
        schedule_fn, total, needs_cleanup = make_measurement_schedule(timing_args.iter, num_devices, iter_thresh)
    else:
        schedule_fn, total, needs_cleanup = (lambda step: Action.NONE), timing_args.iter, (lambda step: False)
    events: list[tuple[torch.cuda.Event, torch.cuda.Event]] = []
    results = example
    for step in range(total):
        dev_idx = step % num_devices
        timed = schedule_fn(step) is not Action.NONE
        with torch.cuda.device(devices[dev_idx]):
            if timed:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            results = func(*per_device_args[dev_idx])
            if timed:
                e1.record()
                events.append((e0, e1))
        if needs_cleanup(step):
            if verbose:
                print(f">>>\tSynchronizing all devices on iter {step} and collecting garbage.")
            pause_and_collect()
    pause_and_collect()
    for i, r in enumerate(_as_tuple(results)):
        if verbose:
            print(f">>>\tresult #{i} shape: {list(r.shape)}; stride: {list(r.stride())}; dtype: {r.dtype}; "
                  f"device type: {r.device.type}")
    if not timing_args.time:
        return None
    return [e0.elapsed_time(e1) * 1e3 for e0, e1 in events]


def _zone_stats(times: list[float], dispatches_per_call: int) -> ZoneStats:
    return ZoneStats(min=min(times), max=max(times), mean=statistics.mean(times),
                     stddev=statistics.stdev(times) if len(times) > 1 else 0, num_dispatches=dispatches_per_call * len(times))


def _print_zone_stats(name: str, stats: ZoneStats) -> None:
    deco = lambda v: f"{v:.2f}us" if isinstance(v, float) else str(v)
    print(f">>>\t{name}\n>>>\t\t" + " ".join(f"{k}={deco(v)}" for k, v in stats._asdict().items()))


def main(args: list[str] | None = None) -> int:
    args = sys.argv[1:] if args is None else args
    meta, extra = _get_main_driver_parser().parse_known_args(args)
    if meta.verbose is None:
        meta.verbose = meta.csv is None
    # tabs separate arguments too, so that a row pasted from a .tsv file works as one argument
    extra = [a for arg in extra for a in arg.split("\t")]
    if meta.commands_file:
        tsv = meta.commands_file.endswith(".tsv")
        split: Callable[[str], list[str]] = (lambda s: s.strip().split("\t")) if tsv else shlex.split
        with open(meta.commands_file) as f:
            commands = [split(line) + extra for line in f.readlines() if line.strip() and not line.startswith("#")]
    else:
        commands = [extra]

    backends: list[str] = meta.backends or [DEFAULT_BACKEND]
    out = open(meta.csv if meta.csv is not None else os.devnull, "w", newline="")
    writer = csv.writer(out)
    numerics_cols = NUMERICS_CSV_COLUMNS if meta.verify_numerics else []
    writer.writerow(["arguments"] + [f"{b} {s}" for b in backends for s in ALL_STATS] + numerics_cols)

    timing_parser = get_timing_parser()
    test_count = test_error = 0
    devices: list[torch.device] | None = None
    for cmd in commands:
        test_count += 1
        if meta.verbose:
            print(f"\n>>> {shlex.join(cmd)}\n")
        else:
            print("Running test :", test_count)
        timing_args, runner_args = timing_parser.parse_known_args(cmd)
        row: list[str] = [shlex.join(cmd)]
        sig = parse_command(runner_args)
        if sig is None:
            if meta.verbose:
                print(f">>> Failed to parse '{shlex.join(runner_args)}'.")
            writer.writerow(row + ["N.A."] + ["N.A."] * len(numerics_cols))
            test_error += 1
            continue
        if devices is None:
            if not torch.cuda.is_available():
                print("driver: no GPU visible; the kernels have no CPU fallback", file=sys.stderr)
                out.close()
                return 1
            devices = _get_devices(meta.gpu_id)

        for backend in backends:
            try:
                func = BACKEND_TO_FUNC_GENERATOR[backend](sig)
                sample = [sig.get_sample_args(seed=10, device=d, splat_value=meta.splat_input_value) for d in devices]
                times = run(func, timing_args, sample, devices, meta.verbose)
            except Exception as exc:
                if meta.verbose:
                    traceback.print_exception(exc)
                row += ["N.A."] * len(ALL_STATS)
                test_error += 1
                continue
            if not timing_args.time:
                row += ["untimed"] * len(ALL_STATS)
                test_error += 1
                continue
            if not times:
                row += ["failed to collect timing info"] * len(ALL_STATS)
                test_error += 1
                continue
            stats = _zone_stats(times, func.dispatches_per_call or 1)
            if meta.verbose:
                _print_zone_stats(f"{backend}::{sig.func_name[:60]}", stats)
                print(f">>>\tPer-launch # GPU kernel dispatches ({backend}): {stats.num_dispatches / timing_args.iter}")
                print(f">>>\tPer-launch GPU mean time ({backend}): {stats.mean}us")
            row += [f"{stats._asdict()[s]}" for s in ALL_STATS]

        if meta.verify_numerics:
            from .numerics import format_verdict_simple, format_verdict_verbose, verify_signature

            ref_dtype = {"float32": torch.float32, "float64": torch.float64}[meta.numerics_reference_dtype]
            try:
                verdict = verify_signature(
                    sig, shlex.join(runner_args), devices[0], backend=DEFAULT_BACKEND, min_samples=meta.numerics_min_samples,
                    stddev_check_rtol=meta.numerics_stddev_rtol, stddev_check_atol=meta.numerics_stddev_atol,
                    mean_check_atol=meta.numerics_mean_atol, mean_check_rtol=meta.numerics_mean_rtol,
                    run_structured_tests=not meta.skip_structured_tests, reference_dtype=ref_dtype)
            except Exception as exc:
                if meta.numerics_verbose:
                    traceback.print_exception(exc)
                writer.writerow(row + ["N.A."] * len(numerics_cols))
                test_error += 1
                continue
            row.append("PASS" if verdict.passed else "FAIL")
            for s in (verdict.boo_gpu_err, verdict.pytorch_gpu_err, verdict.boo_pytorch_diff):
                row += [f"{s.mean:.6e}", f"{s.stddev:.6e}", f"{s.max_abs_err:.6e}"] if s is not None else ["N.A."] * 3
            row.append("N.A." if verdict.structured_test_passed is None else ("PASS" if verdict.structured_test_passed else "FAIL"))
            print(format_verdict_verbose(verdict) if meta.numerics_verbose else format_verdict_simple(verdict))
            if not verdict.passed:
                test_error += 1
        writer.writerow(row)
    out.close()
    return 0 if test_error == 0 else 1


if __name__ == "__main__":
    sys.exit(main())
