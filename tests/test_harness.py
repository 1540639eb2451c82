"""The TensorFlow-free C++ op shell and its standalone harness (tf-approximate_amd/shell/)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "tf-approximate_amd", "axconv_harness")


def run(*args, timeout=120):
    if not os.path.exists(HARNESS):
        pytest.fail("axconv_harness is not built: run `python tf-approximate_amd/build.py`")
    return subprocess.run([HARNESS, *args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout)


def test_help_runs_without_gpu():
    r = run("--help")
    assert r.returncode == 0 and "--layer" in r.stdout


def test_attribute_validation_matches_reference_messages():
    # InitApproxConv2DParameters, tf2/src/approx_nn_conv_ops.cpp:266-303
    r = run("--selftest")
    assert r.returncode == 0, r.stdout
    assert "MISMATCH" not in r.stdout


def test_unknown_flag_is_an_error():
    assert run("--nonsense").returncode == 2


@pytest.mark.gpu
@pytest.mark.parametrize("layer", ["config1", "dw"])
def test_exact_table_matches_fp64_convolution(layer):
    # the reference's own test criterion (tf2/test/test_table_approx_conv_2d.py:62): Linf ~1e-6, bound 1e-5
    r = run("--layer", layer, "--reps", "3")
    assert r.returncode == 0, r.stdout
    assert "max-normalized Linf" in r.stdout and r.stdout.strip().endswith("OK")


@pytest.mark.gpu
def test_table_from_file_and_missing_file(golden_dir):
    r = run("--layer", "config1", "--reps", "2", "--table", os.path.join(golden_dir, "tables", "mul8u_L40.bin"))
    assert r.returncode == 0, r.stdout
    r = run("--layer", "config1", "--reps", "0", "--table", os.path.join(golden_dir, "tables", "no_such_table.bin"))
    assert r.returncode == 2 and "op construction failed" in r.stdout
