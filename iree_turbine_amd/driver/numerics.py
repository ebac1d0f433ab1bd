"""Statistical check of a kernel's numerics, after the reference's three-way comparison
(iree/turbine/kernel/boo/driver/numerics.py):

  kernel_err  : this library's GPU output  vs a high-precision CPU result (the ground truth)
  pytorch_err : PyTorch's GPU output       vs the same CPU result
  diff        : this library's GPU output  vs PyTorch's GPU output

A command passes when the kernel's signed error has no detectable bias (|mean| <= atol + rtol * its own
stddev), its spread is comparable to PyTorch's (stddev <= atol + rtol * PyTorch's stddev), NaNs sit where
the reference has them, and a structured 0/1 input (which exposes indexing mistakes) reproduces PyTorch's
GPU result to 1e-7.  Thresholds and messages follow numerics.py:30-36,258-316.
"""

from __future__ import annotations

import math
import shlex
from dataclasses import dataclass, field
from typing import Callable, Optional, Sequence

import torch

from .backends import BACKEND_TO_FUNC_GENERATOR, DEFAULT_BACKEND
from .signatures import OpSignature, parse_command

MIN_SAMPLES_DEFAULT = 1000
STDDEV_CHECK_RTOL_DEFAULT = 1.2
MEAN_CHECK_ATOL_DEFAULT = 1e-5
MEAN_CHECK_RTOL_DEFAULT = 0.2
STDDEV_CHECK_ATOL_DEFAULT = 1e-5
STRUCTURED_TEST_ATOL = 1e-7
STRUCTURED_BLOCK_SIZE_LIMIT = 128


@dataclass
class ErrorStatistics:
    mean: float
    stddev: float
    max_abs_err: float
    num_samples: int


@dataclass
class NumericsVerdict:
    command: str
    passed: bool
    boo_gpu_err: Optional[ErrorStatistics] = None      # this library's kernel vs the CPU reference
    pytorch_gpu_err: Optional[ErrorStatistics] = None
    boo_pytorch_diff: Optional[ErrorStatistics] = None
    mean_near_zero: bool = True
    stddev_ratio_ok: bool = True
    structured_test_passed: Optional[bool] = None
    boo_nan_mismatch: bool = False
    pytorch_nan_mismatch: bool = False
    boo_pytorch_nan_mismatch: bool = False
    failure_reasons: list[str] = field(default_factory=list)
    error_message: Optional[str] = None
    reference_dtype: torch.dtype = torch.float64


def compute_cpu_reference(sig: OpSignature, sample_args: Sequence[torch.Tensor], dtype: torch.dtype = torch.float64):
    """The eager PyTorch op on CPU with floating-point inputs widened to `dtype`."""
    cpu = torch.device("cpu")
    ref_args = tuple(a.to(device=cpu, dtype=dtype) if a.is_floating_point() else a.to(device=cpu) for a in sample_args)
    with torch.no_grad():
        result = sig.get_nn_module()(*ref_args)
    return (result,) if isinstance(result, torch.Tensor) else tuple(result)


def element_errors(comparee: torch.Tensor, reference: torch.Tensor) -> tuple[torch.Tensor, bool]:
    """Signed errors comparee - reference (in the reference's dtype and device) where not both are NaN, and
    whether the NaN patterns differ."""
    c = comparee.to(device=reference.device)
    c_nan, r_nan = torch.isnan(c), torch.isnan(reference)
    mismatch = bool((c_nan != r_nan).any().item())
    valid = ~(c_nan & r_nan)
    return (c[valid] - reference[valid]).flatten(), mismatch


def compute_error_statistics(errors: torch.Tensor) -> ErrorStatistics:
    """Moments of a 1-D tensor of signed errors, accumulated once in float64: the sample standard deviation
    divides by n - 1, so one sample has none (NaN)."""
    n = errors.numel()
    e = errors.detach().to(torch.float64)
    total = float(e.sum())
    mean = total / n
    spread = float("nan") if n < 2 else math.sqrt(max(float((e * e).sum()) - total * mean, 0.0) / (n - 1))
    return ErrorStatistics(mean=mean, stddev=spread, max_abs_err=float(e.abs().max()), num_samples=n)


@dataclass(frozen=True)
class _Bound:
    """One acceptance rule `|value| <= atol + rtol * |scale|`, with what its failure line reports."""
    atol: float
    rtol: float

    def limit(self, scale: float) -> float:
        return self.atol + self.rtol * abs(scale)

    def holds(self, value: float, scale: float) -> bool:
        return abs(value) <= self.limit(scale)

    def describe(self, scale_name: str, scale: float) -> str:
        return f"threshold (atol={self.atol:.6e} + rtol={self.rtol:.6e} * {scale_name}={scale:.6e})"


def is_approximately_negligible(value: float, reference: float, atol: float, rtol: float) -> bool:
    return _Bound(atol, rtol).holds(value, reference)


def evaluate_statistical_criteria(boo_stats: ErrorStatistics, pytorch_stats: ErrorStatistics, mean_check_atol: float,
                                  mean_check_rtol: float, stddev_check_rtol: float = STDDEV_CHECK_RTOL_DEFAULT,
                                  stddev_check_atol: float = STDDEV_CHECK_ATOL_DEFAULT) -> tuple[bool, bool, list[str]]:
    """(mean_near_zero, stddev_ok, failure reasons): the bias is judged against the kernel's own spread, the
    spread against PyTorch's spread on the same inputs."""
    bias_rule, spread_rule = _Bound(mean_check_atol, mean_check_rtol), _Bound(stddev_check_atol, stddev_check_rtol)
    verdicts = (
        (bias_rule.holds(boo_stats.mean, boo_stats.stddev),
         f"Mean error |{boo_stats.mean:.6e}| > " + bias_rule.describe("boo_stddev", boo_stats.stddev)),
        (spread_rule.holds(boo_stats.stddev, pytorch_stats.stddev),
         f"BOO stddev {boo_stats.stddev:.6e} > " + spread_rule.describe("pytorch_stddev", pytorch_stats.stddev)),
    )
    return verdicts[0][0], verdicts[1][0], [line for ok, line in verdicts if not ok]


def _block_span(numel: int, seed: int, block_size_limit: int) -> tuple[int, int]:
    """[begin, end) of the run of ones in a tensor of `numel` elements: at most a quarter of it and at most
    `block_size_limit` long, at an offset drawn from a CPU generator seeded with `seed`."""
    length = min(max(numel // 4, 1), block_size_limit)
    draw = torch.randint(0, max(numel - length, 1), (1,), generator=torch.Generator("cpu").manual_seed(seed))
    return int(draw), int(draw) + length


def _apply_block_pattern(tensor: torch.Tensor, seed: int = 0, block_size_limit: int = STRUCTURED_BLOCK_SIZE_LIMIT) -> None:
    """Sets one run of consecutive elements (in row-major order) of `tensor` to 1, in place, whatever its strides."""
    if tensor.numel() == 0:
        return
    begin, end = _block_span(tensor.numel(), seed, block_size_limit)
    where = torch.unravel_index(torch.arange(begin, end, device=tensor.device), tensor.shape)
    tensor[where] = 1.0


def generate_structured_test_pattern(shape, dtype: torch.dtype, device, seed: int = 0,
                                     block_size_limit: int = STRUCTURED_BLOCK_SIZE_LIMIT) -> torch.Tensor:
    pattern = torch.zeros(shape, dtype=dtype, device=device)
    _apply_block_pattern(pattern, seed, block_size_limit)
    return pattern


def _as_tuple(result):
    return (result,) if isinstance(result, torch.Tensor) else tuple(result)


def run_structured_test(sig: OpSignature, kernel_fn: Callable, device: torch.device,
                        atol: float = STRUCTURED_TEST_ATOL) -> tuple[bool, Optional[str]]:
    """All-zero operands carrying one run of ones each (operand i seeded with i) make every output an exact small
    integer, so an indexing mistake shows as a whole-number difference: the kernel must match PyTorch's GPU result."""
    operands = [a.to(device) for a in sig.get_sample_args(device=torch.device("cpu"), splat_value=0)]
    for i, a in enumerate(operands):
        if a.is_floating_point():
            _apply_block_pattern(a, seed=i)
    pick = sig.main_result_index
    with torch.no_grad():
        try:
            got = _as_tuple(kernel_fn(*operands))[pick]
        except Exception as e:  # the verdict carries the failure
            return False, f"BOO runtime failed: {e}"
        want = _as_tuple(sig.get_nn_module()(*operands))[pick]
    worst = float((got.double() - want.double()).abs().max()) if got.numel() else 0.0
    if not worst <= atol:  # also catches NaN
        return False, f"Structured test failed: max_diff={worst:.6e} > atol={atol:.6e}"
    return True, None


def verify_signature(sig: OpSignature, command: str, device: torch.device, *, backend: str = DEFAULT_BACKEND,
                     min_samples: int = MIN_SAMPLES_DEFAULT, stddev_check_rtol: float = STDDEV_CHECK_RTOL_DEFAULT,
                     stddev_check_atol: float = STDDEV_CHECK_ATOL_DEFAULT, mean_check_atol: float = MEAN_CHECK_ATOL_DEFAULT,
                     mean_check_rtol: float = MEAN_CHECK_RTOL_DEFAULT, run_structured_tests: bool = True,
                     reference_dtype: torch.dtype = torch.float64) -> NumericsVerdict:
    try:
        kernel_fn = BACKEND_TO_FUNC_GENERATOR[backend](sig)
    except Exception as e:
        return NumericsVerdict(command=command, passed=False, error_message=f"BOO compilation failed: {e}",
                               failure_reasons=["Execution error"], reference_dtype=reference_dtype)
    reference_module = sig.get_nn_module()
    idx = sig.main_result_index
    kernel_errs, torch_errs, diff_errs = [], [], []
    kernel_nan = torch_nan = diff_nan = False
    num_batches, batch = None, 0
    while num_batches is None or batch < num_batches:
        gpu_args = sig.get_sample_args(device=device, seed=batch)  # one seed per batch
        cpu_ref = compute_cpu_reference(sig, tuple(a.cpu() for a in gpu_args), dtype=reference_dtype)[idx]
        if num_batches is None:
            num_batches = max(1, (min_samples + cpu_ref.numel() - 1) // cpu_ref.numel())
        with torch.no_grad():
            torch_out = _as_tuple(reference_module(*gpu_args))[idx]
            try:
                kernel_out = _as_tuple(kernel_fn(*gpu_args))[idx]
            except Exception as e:
                return NumericsVerdict(command=command, passed=False, error_message=f"BOO runtime failed: {e}",
                                       failure_reasons=["Execution error"], reference_dtype=reference_dtype)
        e, n = element_errors(kernel_out, cpu_ref)
        kernel_errs.append(e)
        kernel_nan |= n
        e, n = element_errors(torch_out, cpu_ref)
        torch_errs.append(e)
        torch_nan |= n
        e, n = element_errors(kernel_out, torch_out)
        diff_errs.append(e)
        diff_nan |= n
        batch += 1
    boo_stats = compute_error_statistics(torch.cat(kernel_errs))
    pytorch_stats = compute_error_statistics(torch.cat(torch_errs))
    diff_stats = compute_error_statistics(torch.cat(diff_errs))
    mean_ok, stddev_ok, reasons = evaluate_statistical_criteria(boo_stats, pytorch_stats, mean_check_atol, mean_check_rtol,
                                                               stddev_check_rtol, stddev_check_atol)
    # only a NaN mismatch of the kernel against the ground truth fails the command
    if kernel_nan:
        reasons.append("NaN mismatch: BOO vs CPU reference")
    if torch_nan:
        reasons.append("NaN mismatch [warning]: PyTorch GPU vs CPU reference")
    if diff_nan:
        reasons.append("NaN mismatch [warning]: BOO vs PyTorch GPU")
    structured: Optional[bool] = None
    if run_structured_tests:
        structured, err = run_structured_test(sig, kernel_fn, device)
        if not structured and err:
            reasons.append(err)
    passed = mean_ok and stddev_ok and not kernel_nan and (structured is None or structured)
    return NumericsVerdict(command=command, passed=passed, boo_gpu_err=boo_stats, pytorch_gpu_err=pytorch_stats,
                           boo_pytorch_diff=diff_stats, mean_near_zero=mean_ok, stddev_ratio_ok=stddev_ok,
                           structured_test_passed=structured, boo_nan_mismatch=kernel_nan, pytorch_nan_mismatch=torch_nan,
                           boo_pytorch_nan_mismatch=diff_nan, failure_reasons=reasons, reference_dtype=reference_dtype)


def verify_numerics(commands: Sequence[str], *, device: int = 0, **kwargs) -> list[NumericsVerdict]:
    """One verdict per command string."""
    if not torch.cuda.is_available():
        raise RuntimeError("CUDA is not available. Cannot verify numerics.")
    dev = torch.device(f"cuda:{device}")
    verdicts = []
    for cmd in commands:
        sig = parse_command(shlex.split(cmd))
        if sig is None:
            verdicts.append(NumericsVerdict(command=cmd, passed=False, error_message=f"Failed to parse command: {cmd}",
                                            failure_reasons=["Parse error"],
                                            reference_dtype=kwargs.get("reference_dtype", torch.float64)))
            continue
        verdicts.append(verify_signature(sig, cmd, dev, **kwargs))
    return verdicts


# One line per verdict: the labels of whatever failed, in the order the CSV consumers expect them.
_FAILURE_LABELS = (
    ("mean bias", lambda v: not v.mean_near_zero),
    ("stddev", lambda v: not v.stddev_ratio_ok),
    ("NaN mismatch", lambda v: bool(v.boo_nan_mismatch)),
    ("structured test", lambda v: v.structured_test_passed is False),
    ("error", lambda v: bool(v.error_message)),
)


def format_verdict_simple(verdict: NumericsVerdict) -> str:
    if verdict.passed:
        return "Numerics: PASS"
    labels = [label for label, failed in _FAILURE_LABELS if failed(verdict)] or ["unknown"]
    return "Numerics: FAIL (" + ", ".join(labels) + ")"


def format_verdict_verbose(verdict: NumericsVerdict) -> str:
    lines = [f"=== {verdict.command} ===", ""]
    if verdict.error_message:
        lines += [f"ERROR: {verdict.error_message}", "", f"VERDICT: {'PASS' if verdict.passed else 'FAIL'}"]
        return "\n".join(lines)
    lines.append("Error Statistics:")

    def fmt(name, s: Optional[ErrorStatistics]):
        if s is None:
            return [f"  {name}: N/A"]
        return [f"  {name}:", f"    mean:     {s.mean:.6e}", f"    stddev:   {s.stddev:.6e}",
                f"    max_abs:  {s.max_abs_err:.6e}", f"    samples:  {s.num_samples}"]

    ref = str(verdict.reference_dtype).replace("torch.", "")
    lines += fmt(f"BOO GPU vs {ref} Reference", verdict.boo_gpu_err) + [""]
    lines += fmt(f"PyTorch GPU vs {ref} Reference", verdict.pytorch_gpu_err) + [""]
    lines += fmt("BOO GPU vs PyTorch GPU", verdict.boo_pytorch_diff) + [""]
    lines += ["Statistical Tests:", f"  Mean near zero:    {'PASS' if verdict.mean_near_zero else 'FAIL'}",
              f"  Stddev check:      {'PASS' if verdict.stddev_ratio_ok else 'FAIL'}", ""]
    if verdict.structured_test_passed is not None:
        lines += [f"Structured Test:    {'PASS' if verdict.structured_test_passed else 'FAIL'}", ""]
    if verdict.failure_reasons:
        lines.append("Failure Reasons:")
        lines += [f"  - {r}" for r in verdict.failure_reasons]
        lines.append("")
    lines.append(f"VERDICT: {'PASS' if verdict.passed else 'FAIL'}")
    return "\n".join(lines)


def format_results_table(verdicts: list[NumericsVerdict]) -> str:
    return "\n".join(format_verdict_simple(v) for v in verdicts)
