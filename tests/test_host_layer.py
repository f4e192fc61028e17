"""The C++ host layer (glm53f-afd_amd/host: the counterpart of the reference's kernel.rs / device.rs and of the BF16
half of the forward crate's gemm.rs / cublas.rs and of the KDA layer's call site in forward.rs) through its test
programs, tests/host/host_tests.cc, gemm_tests.cc and kda_layer_tests.cc: argument checks and shape rules without a
GPU, launches against the oracle and against each other with one."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "tests", "host")
EXE = os.path.join(HOST, "host_tests")
GEMM_EXE = os.path.join(HOST, "gemm_tests")
LAYER_EXE = os.path.join(HOST, "kda_layer_tests")


def _exe(path=EXE):
    if not os.path.exists(path):
        subprocess.run(["make", "-s", "-C", HOST], check=True)
    return path


def test_host_argument_checks_without_a_gpu():
    r = subprocess.run([_exe(), "--cpu"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_host_wrappers_launch_and_match_the_oracle():
    r = subprocess.run([_exe(), "--gpu"], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr


def test_gemm_engine_policy_and_shape_rules_without_a_gpu():
    r = subprocess.run([_exe(GEMM_EXE), "--cpu"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_gemm_engine_dispatch_matches_exact_arithmetic():
    r = subprocess.run([_exe(GEMM_EXE), "--gpu"], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr


def test_kda_call_site_shapes_without_a_gpu():
    r = subprocess.run([_exe(LAYER_EXE), "--cpu"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_kda_call_site_verify_commit_and_prefill():
    r = subprocess.run([_exe(LAYER_EXE), "--gpu"], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
