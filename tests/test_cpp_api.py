"""Runs the C++ API test program (tests/cpp/test_api.cpp, built by __graft_entry__.build()): the reference's own
boundary is the C++ classes, so a user's C++ code must compile against include/*.hpp with a plain host compiler
and behave like the reference's unit tests expect."""
import os
import subprocess

import pytest

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "test_api")


def run(mode):
    if not os.path.exists(BINARY):
        pytest.fail("tests/cpp/test_api is not built (run __graft_entry__.build())")
    proc = subprocess.run([BINARY] + ([mode] if mode else []), stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True, timeout=600)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-2000:]
    assert " 0 failures" in proc.stdout


def test_cpp_api_host_part():
    run(None)


@pytest.mark.gpu
def test_cpp_api_on_the_gpu():
    run("gpu")
