"""The C++ host side (include/nextsycl_host.hpp) through its harness program: the library opened by name and every entry
point bound (CPU), then the engines' call sequence - store, route, scratch from the arena, attention - checked against
the oracle on the GPU (tests/host/host_harness.cpp)."""
import os
import subprocess

import pytest

import nextsycl_amd

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "host", "host_harness")


def harness(*args, timeout=300):
    # (make rebuilds the harness only where the host header, the oracle or its own source is newer than it)
    subprocess.run(["make", "-C", os.path.join(HERE, "host")], check=True, capture_output=True)
    env = dict(os.environ, NEXTSYCL_LIB=os.environ.get("NEXTSYCL_LIB") or nextsycl_amd.library_path())
    return subprocess.run([EXE] + list(args), env=env, capture_output=True, text=True, timeout=timeout)


def test_cpp_host_binds_every_entry_point():
    r = harness("--symbols")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "91 entry points bound" in r.stdout, r.stdout


def test_cpp_host_reports_a_missing_library():
    env = dict(os.environ, NEXTSYCL_LIB="/nonexistent/libnextsycl-llm.so")
    if not os.path.exists(EXE):
        subprocess.run(["make", "-C", os.path.join(HERE, "host")], check=True, capture_output=True)
    r = subprocess.run([EXE, "--symbols"], env=env, capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "opening /nonexistent/libnextsycl-llm.so" in r.stdout


@pytest.mark.gpu
def test_cpp_host_runs_the_engine_sequence():
    r = harness()
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout and "FAIL" not in r.stdout
