"""Runs the C++ tests of the host mirror (flexflow-train_amd/host/test/test_host.cc):
the reference's entry-point signatures over the C ABI, checked against the
oracle.  One process per mode."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "flexflow-train_amd", "host", "build", "test_host")


def _run(mode):
    assert os.path.exists(EXE), "build the host mirror first: make -C flexflow-train_amd/host"
    proc = subprocess.run([EXE, mode], capture_output=True, text=True, timeout=300)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout[-3000:]
    assert " 0 failed" in proc.stdout


def test_host_mirror_cpu_side():
    _run("--cpu")


@pytest.mark.gpu
def test_host_mirror_on_device():
    _run("--gpu")
