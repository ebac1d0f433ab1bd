"""Error statistics and pass criteria of the reference's numerics harness
(iree/turbine/kernel/boo/driver/numerics.py:30-36,115-142,245-316), restated.  Test infrastructure only."""

from __future__ import annotations

from dataclasses import dataclass

import torch

MEAN_CHECK_ATOL = 1e-5
MEAN_CHECK_RTOL = 0.2
STDDEV_CHECK_ATOL = 1e-5
STDDEV_CHECK_RTOL = 1.2


@dataclass
class ErrorStatistics:
    mean: float
    stddev: float
    max_abs_err: float
    num_samples: int


def element_errors(comparee: torch.Tensor, reference: torch.Tensor) -> tuple[torch.Tensor, bool]:
    """Signed errors (comparee - reference) where not both NaN, and whether NaNs mismatch
    (numerics.py:115-142)."""
    c = comparee.detach().to(device=reference.device)
    cn, rn = torch.isnan(c), torch.isnan(reference)
    mismatch = bool((cn != rn).any().item())
    valid = ~(cn & rn)
    return (c[valid] - reference[valid]).flatten(), mismatch


def error_statistics(errors: torch.Tensor) -> ErrorStatistics:
    """mean, Bessel-corrected stddev (NaN for one sample), max |err|, count (numerics.py:245-256)."""
    e = errors.double()
    return ErrorStatistics(
        mean=e.mean().item(),
        stddev=e.std(unbiased=True).item() if e.numel() > 1 else float("nan"),
        max_abs_err=e.abs().max().item(),
        num_samples=e.numel(),
    )


def mean_near_zero(ours: ErrorStatistics) -> bool:
    """|mean| <= atol + rtol * stddev: no systematic drift (numerics.py:266-289)."""
    return abs(ours.mean) <= MEAN_CHECK_ATOL + MEAN_CHECK_RTOL * ours.stddev


def stddev_ratio_ok(ours: ErrorStatistics, baseline: ErrorStatistics) -> bool:
    """our error spread is at most 1.2x the baseline implementation's (numerics.py:292-316)."""
    return ours.stddev <= STDDEV_CHECK_ATOL + STDDEV_CHECK_RTOL * baseline.stddev
