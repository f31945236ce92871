"""The C++ classes (qmlp::FusedNetwork, Tensor, TmpMemory, ...) used the way the reference's
C++ tests use them: tests/cpp/test_cpp_api.cpp, linked against libqmlp.so. The host part runs
everywhere; the device part compares inference, forward and adjoint with a plain fp32
evaluation inside the test program (rel 1e-2 / abs 1e-3)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP_DIR = os.path.join(ROOT, "tests", "cpp")
BINARY = os.path.join(CPP_DIR, "test_cpp_api")
CACHE = os.path.join(ROOT, "quick-mlp_amd", ".kernel_cache")


def _run(*args):
    env = dict(os.environ, QMLP_CACHE_DIR=CACHE)
    return subprocess.run([BINARY, *args], env=env, capture_output=True, text=True, timeout=600)


def test_cpp_api_host_part():
    subprocess.run(["make", "-C", CPP_DIR], check=True, capture_output=True)
    r = _run("--host")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout


@pytest.mark.gpu
def test_cpp_api_on_the_device():
    if os.environ.get("QMLP_WARM_CACHE"):
        pytest.skip("the host part of the program has already compiled its kernels into the cache")
    assert os.path.exists(BINARY), "tests/cpp/test_cpp_api is missing: run __graft_entry__.build() first"
    r = _run()
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout
