"""Runs the C++ adapter's own test program (gufo-npu_amd/host/hip_projections_test.cpp):
HipProjections, the class that takes GgufProjections' place behind the reference's
`Projections` interface, against the CPU checker."""
import os
import subprocess

import pytest

from conftest import ROOT

BINARY = ROOT / "gufo-npu_amd" / "lib" / "hip_projections_test"


def run(*args):
    if not BINARY.exists():
        pytest.fail(f"{BINARY} is not built: run __graft_entry__.build()")
    return subprocess.run([str(BINARY), *args], capture_output=True, text=True, timeout=300)


def test_adapter_reports_missing_device():
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    done = run("--no-device")
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    assert "throws std::runtime_error ok" in done.stdout


@pytest.mark.gpu
def test_adapter_against_cpu_checker():
    done = run()
    print(done.stdout[-4000:], flush=True)
    assert done.returncode == 0, done.stdout[-3000:] + done.stderr[-2000:]
    assert done.stdout.strip().endswith("PASS")
    assert "FAIL" not in done.stdout
