"""GPU: the command-line driver end to end -- CSV round trip, dispatch counts, three-way numerics verdicts
on GEMM and attention commands (the reference's csv_output_test.py / cli_test.py shapes, with the commands
this kernel path covers)."""

import csv
import shlex

import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

MM_BF16 = ["aten::mm", "[[256, 512], [512, 384]]", "['c10::BFloat16', 'c10::BFloat16']", "[[512, 1], [384, 1]]", "['', '']"]
SDPA_128 = ["aten::scaled_dot_product_attention",
            "[[2, 4, 256, 128], [2, 4, 256, 128], [2, 4, 256, 128], [], [], [], [], []]",
            "['c10::Half', 'c10::Half', 'c10::Half', '', 'Scalar', 'Scalar', '', 'Scalar']",
            "[[131072, 32768, 128, 1], [131072, 32768, 128, 1], [131072, 32768, 128, 1], [], [], [], [], []]",
            "['', '', '', 'None', '0.0', 'True', 'None', 'False']"]
MM_HALF = ["aten::mm", "[[512, 256], [256, 384]]", "['c10::Half', 'c10::Half']", "[[256, 1], [1, 256]]", "['', '']"]


def _rows(path, backends):
    from iree_turbine_amd.driver import driver

    lines = path.read_text().splitlines()
    headers = ["arguments"] + [f"{b} {s}" for b in backends for s in driver.ALL_STATS]
    assert lines[0].split(",")[:len(headers)] == headers
    return list(csv.DictReader(lines[1:], fieldnames=lines[0].split(",")))


def test_csv_single_command(dev, tmp_path):
    from iree_turbine_amd.driver import driver

    announce("driver csv single command")
    out = tmp_path / "gemm.csv"
    cmd = ["gemmfp16", "--a_w", "512", "--a_h", "256", "--b_w", "768", "--transB", "1", "--iter=4"]
    assert driver.main([f"--csv={out}"] + cmd) == 0
    (row,) = _rows(out, ["mi355"])
    assert row["arguments"] == shlex.join(cmd)
    assert row["mi355 num_dispatches"] == "4"  # one kernel per launch in the native NT layout
    assert 0 < float(row["mi355 min"]) <= float(row["mi355 mean"]) <= float(row["mi355 max"])


def test_commands_file_two_backends_and_layout_copy(dev, tmp_path):
    from iree_turbine_amd.driver import driver

    announce("driver commands file")
    f = tmp_path / "cmds.txt"
    f.write_text("\n".join(["gemmfp16 --a_w 256 --a_h 128 --b_w 256 --transB 1", "# comment", "",
                            "gemmfp16 --a_w 256 --a_h 128 --b_w 256",     # B stored [K, N]: one transposing copy
                            shlex.join(MM_HALF), shlex.join(SDPA_128),
                            "gemm --a_w 64 --a_h 64 --b_w 64",            # fp32: not covered by the kernels
                            "no-such-command"]))
    out = tmp_path / "o.csv"
    rc = driver.main(["--commands-file", str(f), f"--csv={out}", "--backend", "mi355", "--backend", "torch", "--iter", "3"])
    assert rc == 1  # the last two commands fail
    rows = _rows(out, ["mi355", "torch"])
    assert len(rows) == 6
    assert [r["mi355 num_dispatches"] for r in rows[:4]] == ["3", "6", "3", "3"]   # MM_HALF's b is a transposed view
    assert all(float(r["torch mean"]) > 0 for r in rows[:5])
    assert rows[4]["mi355 mean"] == "N.A." and rows[4]["torch num_dispatches"] == "3"
    assert rows[5]["mi355 min"] == "N.A."


@pytest.mark.parametrize("cmd", [["gemmfp16", "--a_w", "512", "--a_h", "1024", "--b_w", "256", "--transB", "1"],
                                 ["gemmfp16", "--a_w", "96", "--a_h", "40", "--b_w", "72", "--transA", "1"],
                                 MM_HALF, MM_BF16, SDPA_128, [a.replace("c10::Half", "c10::BFloat16") for a in SDPA_128]])
def test_numerics_verdict_passes(dev, cmd):
    from iree_turbine_amd.driver.numerics import format_verdict_verbose, verify_numerics

    announce(f"driver numerics {cmd[0]}")
    (v,) = verify_numerics([shlex.join(cmd)])
    assert v.passed, format_verdict_verbose(v)
    assert v.structured_test_passed is True and v.boo_gpu_err.num_samples >= 1000
    assert v.boo_gpu_err.stddev <= 1e-5 + 1.2 * v.pytorch_gpu_err.stddev


def test_numerics_csv_columns_and_failures(dev, tmp_path):
    from iree_turbine_amd.driver import driver
    from iree_turbine_amd.driver.numerics import verify_numerics

    announce("driver numerics csv")
    out = tmp_path / "n.csv"
    cmd = ["gemmfp16", "--a_w", "128", "--a_h", "64", "--b_w", "128", "--transB", "1", "--iter", "2"]
    assert driver.main([f"--csv={out}", "--verify-numerics"] + cmd) == 0
    (row,) = _rows(out, ["mi355"])
    assert row["numerics_pass"] == "PASS" and row["structured_test"] == "PASS"
    assert float(row["boo_vs_ref_stddev"]) > 0 and float(row["boo_vs_pytorch_max"]) >= 0
    bad, unparsed = verify_numerics(["gemm --a_w 64 --a_h 64 --b_w 64", "conv -n 1"])
    assert not bad.passed and bad.failure_reasons == ["Execution error"] and "fp16" in bad.error_message
    assert not unparsed.passed and unparsed.failure_reasons == ["Parse error"]
