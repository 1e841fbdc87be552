"""Runs futhark_amd/bin/capi-harness (tests/c/capi_harness.c): a C program
against include/segops.h with the call sequences of the reference's own C
harnesses (tests_lib/c/test_{c,index,raw,f,e,g}.c)."""
import os
import subprocess
from pathlib import Path

import pytest

HARNESS = Path(__file__).resolve().parent.parent / "futhark_amd" / "bin" / "capi-harness"


def test_harness_without_device_reports_through_get_error():
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    proc = subprocess.run([str(HARNESS), "--no-device"], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0, proc.stderr
    assert proc.stdout.startswith("ok no_device: ")


@pytest.mark.gpu
def test_harness_on_the_gpu():
    proc = subprocess.run([str(HARNESS)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    lines = proc.stdout.split()
    for name in ("lifecycle", "index", "raw", "threads", "errors_are_not_sticky",
                 "two_results_and_report", "all"):
        assert name in lines, proc.stdout
