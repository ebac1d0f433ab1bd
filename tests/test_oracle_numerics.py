"""The reference's own known-answer tests for its error statistics, restated as literal numbers
(tests/kernel/boo/driver/numerics_smoke_test.py:24-56) plus the pass criteria of numerics.py:266-316."""

import math

import torch

from oracle import numerics as on


def test_error_statistics_kat():
    s = on.error_statistics(torch.tensor([-2.0, -1.0, 0.0, 1.0, 2.0]))
    assert s.mean == 0.0 and s.num_samples == 5 and s.max_abs_err == 2.0
    assert abs(s.stddev - 1.5811388) < 1e-6  # Bessel-corrected


def test_single_sample_stddev_is_nan():
    s = on.error_statistics(torch.tensor([3.0]))
    assert s.mean == 3.0 and math.isnan(s.stddev) and s.num_samples == 1


def test_element_errors_nan_handling():
    a = torch.tensor([1.0, float("nan"), 3.0, float("nan")])
    b = torch.tensor([1.5, float("nan"), 3.0, 4.0], dtype=torch.float64)
    e, mismatch = on.element_errors(a, b)
    assert mismatch  # NaN on one side only
    assert e.dtype == torch.float64 and e.numel() == 3 and e[0].item() == -0.5
    e2, mismatch2 = on.element_errors(torch.tensor([1.0, float("nan")]), torch.tensor([1.0, float("nan")]))
    assert not mismatch2 and e2.tolist() == [0.0]


def test_criteria():
    ok = on.ErrorStatistics(mean=1e-4, stddev=1e-3, max_abs_err=5e-3, num_samples=1000)
    assert on.mean_near_zero(ok)  # |mean| <= 1e-5 + 0.2 * stddev
    biased = on.ErrorStatistics(mean=5e-4, stddev=1e-3, max_abs_err=5e-3, num_samples=1000)
    assert not on.mean_near_zero(biased)
    base = on.ErrorStatistics(mean=0.0, stddev=1e-3, max_abs_err=4e-3, num_samples=1000)
    assert on.stddev_ratio_ok(ok, base)
    wide = on.ErrorStatistics(mean=0.0, stddev=1.3e-3, max_abs_err=4e-3, num_samples=1000)
    assert not on.stddev_ratio_ok(wide, base)  # more than 1.2x the baseline spread
