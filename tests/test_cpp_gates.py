"""Runs the C++ gate executables built from tests/cpp (by __graft_entry__.build()
or `make -C tests/cpp`): the host suite and the entry-contract suite need no
GPU; the device suite is marked gpu."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "build")


def _run(name, timeout):
    exe = os.path.join(BUILD, name)
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "tests", "cpp"), os.path.join("..", "..", "build", name)])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=timeout)
    tail = "\n".join(r.stdout.splitlines()[-15:])
    assert r.returncode == 0, f"{name} exit {r.returncode}\n{tail}\n{r.stderr[-2000:]}"
    return r.stdout


def test_host_headers_against_reference_gates_and_oracle():
    out = _run("test_host", 600)
    assert " 0 failures" in out


def test_entry_contracts_throw_before_touching_the_device():
    out = _run("test_contracts", 120)
    assert " 0 failures" in out


@pytest.mark.gpu
def test_device_gates_through_the_cpp_api():
    out = _run("test_device", 600)
    assert " 0 failures" in out
