"""The C++ host layer (glm53f-afd_amd/host: the counterpart of the reference's kernel.rs / device.rs) through its
test program, tests/host/host_tests.cc: argument checks without a GPU, launches against the oracle with one."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "tests", "host")
EXE = os.path.join(HOST, "host_tests")


def _exe():
    if not os.path.exists(EXE):
        subprocess.run(["make", "-s", "-C", HOST], check=True)
    return EXE


def test_host_argument_checks_without_a_gpu():
    r = subprocess.run([_exe(), "--cpu"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_host_wrappers_launch_and_match_the_oracle():
    r = subprocess.run([_exe(), "--gpu"], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
