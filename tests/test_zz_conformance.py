"""Runs the C++ conformance binary (tests/cpp/conformance.cpp): the reference's own gtest cases and
decode example re-expressed against the C++ host classes, with the oracle as expected value."""
import os
import subprocess

import pytest


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "attention_amd", "lib", "ahpc_conformance")


def run(args, env=None):
    assert os.path.exists(BIN), f"{BIN} missing: run __graft_entry__.build()"
    r = subprocess.run([BIN] + args, capture_output=True, text=True, timeout=600, env=env)
    print(r.stdout[-6000:])
    print(r.stderr[-2000:])
    assert r.returncode == 0, "conformance failures:\n" + "\n".join(
        l for l in r.stdout.splitlines() if "FAIL" in l or "EXPECT" in l or "exception" in l)


def test_host_cases_without_gpu():
    run(["--no-gpu"])


def test_all_cases_on_the_cpu_executor():
    """Every case, GPU ones included, with the kernels executed lane by lane on the CPU: tests/simt builds the
    library's sources for the host under the real library's file name, and the loader is pointed at it."""
    from simt import simt
    simt.build()
    env = dict(os.environ)
    as_hip = os.path.join(ROOT, "tests", "simt", "as_hip")
    env["LD_LIBRARY_PATH"] = as_hip + (os.pathsep + env["LD_LIBRARY_PATH"] if env.get("LD_LIBRARY_PATH") else "")
    run([], env)


@pytest.mark.gpu
def test_forward_decode_and_pool_cases_on_gpu():
    run(["--skip", "Backward,WideGroups"])


@pytest.mark.gpu
def test_backward_cases_on_gpu():
    run(["Backward"])


@pytest.mark.gpu
def test_wide_group_decode_cases_on_gpu():
    run(["WideGroups"])
