"""Runs the C++ tests of the host mirror (flexflow-train_amd/host/test/test_host.cc):
the reference's entry-point signatures over the C ABI, checked against the
oracle.  The binary runs once per mode (one process on the GPU); every
TEST_CASE of its output is a pytest item of its own, so a failing case does
not hide the ones after it."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "flexflow-train_amd", "host", "build", "test_host")
SRC = os.path.join(ROOT, "flexflow-train_amd", "host", "test", "test_host.cc")


def _case_names():
    """TEST_CASE names per mode, from the source text (no binary needed to collect)."""
    text = open(SRC).read()
    cpu_at, gpu_at = text.index("static void cpu_tests()"), text.index("static void gpu_tests()")
    names = {"--cpu": [], "--gpu": []}
    for m in re.finditer(r'^\s*run\("((?:[^"\\]|\\.)*)"', text, re.M):
        if m.start() > cpu_at:
            names["--gpu" if m.start() > gpu_at else "--cpu"].append(m.group(1).replace('\\"', '"'))
    return names


CASES = _case_names()
_results = {}


def _run(mode):
    if mode not in _results:
        assert os.path.exists(EXE), "build the host mirror first: make -C flexflow-train_amd/host"
        proc = subprocess.run([EXE, mode], capture_output=True, text=True, timeout=300)
        cases, name, lines = {}, None, []
        for line in proc.stdout.splitlines():
            if line.startswith("TEST_CASE "):
                name, lines = line[len("TEST_CASE "):], []
            elif line.startswith("CASE_RESULT ") and name is not None:
                cases[name] = (line.split()[1] == "ok", "\n".join(lines))
                name = None
            else:
                lines.append(line)
        _results[mode] = (proc, cases, name)
    return _results[mode]


def _check_case(mode, case):
    proc, cases, unfinished = _run(mode)
    if case not in cases:
        why = "the process ended inside this case" if unfinished == case else "the case did not run"
        pytest.fail("%s (exit code %d)\n%s\n%s" % (why, proc.returncode, proc.stdout[-2000:], proc.stderr[-2000:]))
    ok, text = cases[case]
    print(text)
    assert ok, text


@pytest.mark.parametrize("case", CASES["--cpu"])
def test_host_mirror_cpu_side(case):
    _check_case("--cpu", case)


def test_host_mirror_cpu_side_exit_code():
    proc, cases, _ = _run("--cpu")
    assert proc.returncode == 0 and " 0 failed" in proc.stdout, proc.stdout[-3000:]
    assert set(cases) == set(CASES["--cpu"])


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES["--gpu"])
def test_host_mirror_on_device(case):
    _check_case("--gpu", case)


@pytest.mark.gpu
def test_host_mirror_on_device_exit_code():
    proc, cases, _ = _run("--gpu")
    assert proc.returncode == 0 and " 0 failed" in proc.stdout, proc.stdout[-3000:]
    assert set(cases) == set(CASES["--gpu"])
