"""Host-side behaviour of the command-line driver (no GPU): command grammar, measurement schedule,
error statistics and verdict criteria, CSV layout.  Expected values are the ones the reference's own
tests pin (tests/kernel/boo/driver/parser_test.py, profiler_schedule_test.py, numerics_smoke_test.py,
csv_output_test.py), restated as literals."""

import csv
import math

import pytest
import torch

from iree_turbine_amd.driver import AtenSignature, GEMMSignature, parse_command
from iree_turbine_amd.driver import driver
from iree_turbine_amd.driver.backends import UnsupportedSignature, mi355_backend
from iree_turbine_amd.driver.numerics import (ErrorStatistics, NumericsVerdict, compute_error_statistics,
                                             evaluate_statistical_criteria, format_results_table, format_verdict_simple,
                                             format_verdict_verbose, generate_structured_test_pattern)

A = driver.Action


def test_gemm_command_flag_quirk_and_name():
    # --a_w is the ROW count of A, --a_h the contraction size (op_exports/gemm.py:173-180)
    sig = parse_command(["gemmfp16", "--a_w", "32", "--a_h", "64", "--b_w", "128", "--transB", "1"])
    assert isinstance(sig, GEMMSignature)
    assert sig.a_shape == [32, 64] and sig.b_shape == [64, 128] and sig.dtype == torch.float16
    assert sig.func_name == "gemm_float16_forward_32x64x128_transB"
    a, b = sig.get_sample_args(seed=10)
    assert list(a.shape) == [32, 64] and list(b.shape) == [128, 64]  # B is stored transposed
    assert parse_command(["gemm", "-k", "8", "-m", "4", "-n", "2", "-u", "1"]).func_name == "gemm_float32_forward_8x4x2_transA"
    assert parse_command(["gemm"]).a_shape == [256, 256]
    # seeded draws are reproducible, splat overrides them
    a2, _ = sig.get_sample_args(seed=10)
    assert torch.equal(a, a2)
    s, _ = sig.get_sample_args(splat_value=3)
    assert (s == 3).all()
    out = sig.get_nn_module()(a.float(), b.float())
    assert list(out.shape) == [32, 128]


@pytest.mark.parametrize("cmd", [["invalid-command"], [], ["gemmfp16", "--a_w", "0"], ["gemmfp16", "-F", "2"],
                                 ["gemmfp16", "--bogus", "1"], ["aten::no_such_op", "[]", "[]", "[]", "[]"],
                                 ["aten::mm", "[[2, 2]", "[]", "[]", "[]"]])
def test_unparseable_commands_give_none(cmd):
    assert parse_command(cmd) is None


def test_aten_parser_addmm():
    sig = parse_command(["aten::addmm", "[[512], [24576, 512], [512, 512], [], []]",
                         "['c10::BFloat16', 'c10::BFloat16', 'float', 'Scalar', 'Scalar']",
                         "[[1], [512, 1], [1, 512], [], []]", "['', '', '', '10', '20']"])
    assert isinstance(sig, AtenSignature)
    a0, a1, a2 = sig.get_sample_args()
    assert list(a0.shape) == [512] and list(a0.stride()) == [1] and a0.dtype == torch.bfloat16
    assert list(a1.shape) == [24576, 512] and list(a1.stride()) == [512, 1] and a1.dtype == torch.bfloat16
    assert list(a2.shape) == [512, 512] and list(a2.stride()) == [1, 512] and a2.dtype == torch.float32
    (beta, bv), (alpha, av) = sig.get_concrete_args()
    assert (beta.name, bv, alpha.name, av) == ("beta", 10, "alpha", 20)


@pytest.mark.parametrize("aten_dtype, expected", [("float", torch.float32), ("double", torch.float64),
                                                  ("c10::Half", torch.float16), ("c10::BFloat16", torch.bfloat16)])
def test_aten_dtype_mapping(aten_dtype, expected):
    sig = parse_command(["aten::bmm", "[[2, 3, 4], [2, 4, 5]]", f"['{aten_dtype}', '{aten_dtype}']",
                         "[[12, 4, 1], [20, 5, 1]]", "['', '']"])
    a0, a1 = sig.get_sample_args()
    assert a0.dtype == expected and a1.dtype == expected


def test_aten_parser_sdpa_and_strides():
    sig = parse_command(["aten::scaled_dot_product_attention",
                         "[[32, 8, 128, 64], [32, 8, 128, 64], [32, 8, 128, 64], [], [], [], [], []]",
                         "['c10::Half', 'c10::Half', 'c10::Half', '', 'Scalar', 'Scalar', '', 'Scalar']",
                         "[[65536, 8192, 64, 1], [65536, 8192, 64, 1], [65536, 8192, 64, 1], [], [], [], [], []]",
                         "['', '', '', 'None', '0.0', 'False', 'None', 'False']"])
    q, k, v = sig.get_sample_args()
    assert list(q.shape) == [32, 8, 128, 64] and list(q.stride()) == [65536, 8192, 64, 1] and q.dtype == torch.float16
    assert sig.concrete_kwargs() == {"attn_mask": None, "dropout_p": 0.0, "is_causal": False, "scale": None, "enable_gqa": False}
    # non-contiguous strides may address more elements than prod(dims): 671*16 + 2*1 + 2*4 + 1 = 10747
    sig = parse_command(["aten::bmm", "[[672, 3, 3], [672, 3, 250]]", "['float', 'float']", "[[16, 1, 4], [750, 250, 1]]", "['', '']"])
    a0, a1 = sig.get_sample_args()
    assert list(a0.shape) == [672, 3, 3] and list(a0.stride()) == [16, 1, 4]
    assert a0.untyped_storage().nbytes() == 10747 * 4


def test_backend_rejects_what_the_kernels_do_not_cover():
    with pytest.raises(UnsupportedSignature):
        mi355_backend(parse_command(["gemm", "--a_w", "64"]))  # fp32 operands
    # bf16 products are covered, mixed or fp32 operands are not
    mi355_backend(parse_command(["aten::mm", "[[8, 8], [8, 8]]", "['c10::BFloat16', 'c10::BFloat16']", "[[8, 1], [8, 1]]", "['', '']"]))
    with pytest.raises(UnsupportedSignature):
        mi355_backend(parse_command(["aten::mm", "[[8, 8], [8, 8]]", "['c10::BFloat16', 'c10::Half']", "[[8, 1], [8, 1]]", "['', '']"]))
    with pytest.raises(UnsupportedSignature):
        mi355_backend(parse_command(["aten::mm", "[[8, 8], [8, 8]]", "['float', 'float']", "[[8, 1], [8, 1]]", "['', '']"]))
    with pytest.raises(UnsupportedSignature):  # head dim 64
        mi355_backend(parse_command(["aten::scaled_dot_product_attention",
                                     "[[2, 2, 16, 64], [2, 2, 16, 64], [2, 2, 16, 64], [], [], [], [], []]",
                                     "['c10::Half', 'c10::Half', 'c10::Half', '', 'Scalar', 'Scalar', '', 'Scalar']",
                                     "[[2048, 1024, 64, 1], [2048, 1024, 64, 1], [2048, 1024, 64, 1], [], [], [], [], []]",
                                     "['', '', '', 'None', '0.0', 'False', 'None', 'False']"]))
    with pytest.raises(UnsupportedSignature):
        mi355_backend(parse_command(["aten::bmm", "[[2, 3, 4], [2, 4, 5]]", "['c10::Half', 'c10::Half']", "[[12, 4, 1], [20, 5, 1]]", "['', '']"]))


def test_schedule_no_cleanup():
    fn, total, _ = driver.make_measurement_schedule(timing_iter=10, num_devices=1, iter_thresh=100)
    assert total == 11
    assert [fn(s) for s in range(total)] == [A.NONE] + [A.RECORD] * 9 + [A.RECORD_AND_SAVE]


def test_schedule_with_cleanup():
    fn, total, needs_cleanup = driver.make_measurement_schedule(timing_iter=12, num_devices=1, iter_thresh=4)
    expected = [A.NONE, A.RECORD, A.RECORD_AND_SAVE, A.NONE, A.RECORD, A.RECORD, A.RECORD_AND_SAVE, A.NONE, A.RECORD, A.RECORD,
                A.RECORD_AND_SAVE, A.NONE, A.RECORD, A.RECORD, A.RECORD_AND_SAVE, A.NONE, A.RECORD_AND_SAVE]
    assert [fn(s) for s in range(total)] == expected
    assert sum(a is not A.NONE for a in expected) == 12
    assert [s for s in range(total) if needs_cleanup(s)] == [3, 7, 11, 15]


def test_schedule_four_devices():
    fn, total, _ = driver.make_measurement_schedule(timing_iter=4, num_devices=4, iter_thresh=100)
    assert [fn(s) for s in range(total)] == [A.NONE] * 4 + [A.RECORD] * 3 + [A.RECORD_AND_SAVE]


def test_error_statistics_kats():
    s = compute_error_statistics(torch.tensor([-2.0, -1.0, 0.0, 1.0, 2.0]))
    assert s.mean == pytest.approx(0.0) and s.stddev == pytest.approx(1.5811388, rel=1e-5)
    assert s.max_abs_err == pytest.approx(2.0) and s.num_samples == 5
    z = compute_error_statistics(torch.zeros(100))
    assert (z.mean, z.stddev, z.max_abs_err, z.num_samples) == (0.0, 0.0, 0.0, 100)
    one = compute_error_statistics(torch.tensor([-0.5]))
    assert one.mean == pytest.approx(-0.5) and math.isnan(one.stddev) and one.max_abs_err == pytest.approx(0.5)


def _st(mean, stddev, mx=1e-4):
    return ErrorStatistics(mean=mean, stddev=stddev, max_abs_err=mx, num_samples=1000)


def test_criteria_kats():
    ok = evaluate_statistical_criteria(_st(1e-8, 1e-5), _st(1e-8, 1e-5), mean_check_atol=1e-6, mean_check_rtol=0.0)
    assert ok == (True, True, [])
    m, _, r = evaluate_statistical_criteria(_st(1e-4, 1e-5), _st(1e-8, 1e-5), mean_check_atol=1e-6, mean_check_rtol=0.0)
    assert m is False and any("Mean error" in x for x in r)
    _, s, r = evaluate_statistical_criteria(_st(1e-8, 2e-4), _st(1e-8, 1e-4), mean_check_atol=1e-6, mean_check_rtol=0.0,
                                            stddev_check_rtol=1.2)
    assert s is False and any("BOO stddev" in x for x in r)
    _, s, _ = evaluate_statistical_criteria(_st(1e-8, 0.0), _st(0.0, 0.0), mean_check_atol=1e-6, mean_check_rtol=0.0)
    assert s is True  # both below the absolute floor
    m, s, _ = evaluate_statistical_criteria(_st(5e-5, 1e-4), _st(1e-8, 5e-5), mean_check_atol=1e-6, mean_check_rtol=0.0)
    assert (m, s) == (False, False)
    m, s, _ = evaluate_statistical_criteria(_st(5e-5, 1e-4), _st(1e-8, 5e-5), mean_check_atol=1e-4, mean_check_rtol=0.0,
                                            stddev_check_rtol=3.0)
    assert (m, s) == (True, True)
    # the mean threshold scales with the kernel's own error spread: 1e-5 + 0.2 * stddev
    m, _, _ = evaluate_statistical_criteria(_st(5e-2, 1e-3), _st(1e-8, 1e-3), mean_check_atol=1e-5, mean_check_rtol=0.2)
    assert m is False
    m, _, _ = evaluate_statistical_criteria(_st(5e-2, 1.0), _st(1e-8, 1e-3), mean_check_atol=1e-5, mean_check_rtol=0.2)
    assert m is True


def test_structured_pattern():
    t = generate_structured_test_pattern((16, 64), torch.float32, "cpu", seed=3)
    flat = t.flatten()
    ones = torch.nonzero(flat).flatten()
    assert len(ones) == 128 and (flat[ones] == 1).all()            # min(1024 // 4, 128)
    assert ones[-1] - ones[0] == 127                               # one contiguous block
    assert torch.equal(t, generate_structured_test_pattern((16, 64), torch.float32, "cpu", seed=3))
    small = generate_structured_test_pattern((2, 3), torch.float16, "cpu")
    assert small.sum() == 1                                        # 6 // 4 = 1 element
    assert generate_structured_test_pattern((0,), torch.float32, "cpu").numel() == 0


def test_verdict_formatting():
    good = NumericsVerdict(command="gemmfp16", passed=True, boo_gpu_err=_st(0, 1e-4), pytorch_gpu_err=_st(0, 1e-4),
                           boo_pytorch_diff=_st(0, 1e-5), structured_test_passed=True)
    bad = NumericsVerdict(command="x", passed=False, mean_near_zero=False, stddev_ratio_ok=False, boo_nan_mismatch=True,
                          structured_test_passed=False, failure_reasons=["Mean error ..."])
    err = NumericsVerdict(command="y", passed=False, error_message="boom")
    assert format_verdict_simple(good) == "Numerics: PASS"
    assert format_verdict_simple(bad) == "Numerics: FAIL (mean bias, stddev, NaN mismatch, structured test)"
    assert format_verdict_simple(err) == "Numerics: FAIL (error)"
    assert format_verdict_simple(NumericsVerdict(command="z", passed=False)) == "Numerics: FAIL (unknown)"
    text = format_verdict_verbose(good)
    assert "=== gemmfp16 ===" in text and "BOO GPU vs float64 Reference" in text and text.endswith("VERDICT: PASS")
    assert "ERROR: boom" in format_verdict_verbose(err)
    assert format_results_table([good, bad]).splitlines() == [format_verdict_simple(good), format_verdict_simple(bad)]


def test_csv_header_and_unparseable_row(tmp_path):
    out = tmp_path / "stats.csv"
    assert driver.main([f"--csv={out}", "--backend", "mi355", "--backend", "torch", "--verify-numerics", "invalid-command", "--iter=3"]) == 1
    rows = list(csv.reader(out.read_text().splitlines()))
    assert rows[0] == ["arguments"] + [f"{b} {s}" for b in ("mi355", "torch") for s in driver.ALL_STATS] + driver.NUMERICS_CSV_COLUMNS
    assert driver.ALL_STATS == ["min", "max", "mean", "stddev", "num_dispatches"]
    assert rows[1][0] == "invalid-command --iter=3" and set(rows[1][1:]) == {"N.A."}
    assert len(rows) == 2


def test_commands_file_splitting(tmp_path):
    f = tmp_path / "cmds.txt"
    f.write_text("nope one\n# comment\n\nnope 'two words'\n")
    out = tmp_path / "o.csv"
    assert driver.main(["--commands-file", str(f), f"--csv={out}", "extra"]) == 1
    rows = list(csv.reader(out.read_text().splitlines()))
    assert [r[0] for r in rows[1:]] == ["nope one extra", "nope 'two words' extra"]
    tsv = tmp_path / "cmds.tsv"
    tsv.write_text("nope\ta b\n")
    assert driver.main(["--commands-file", str(tsv), f"--csv={out}"]) == 1
    assert list(csv.reader(out.read_text().splitlines()))[1][0] == "nope 'a b'"
