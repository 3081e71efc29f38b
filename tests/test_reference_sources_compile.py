"""The C++ headers under include/ keep the reference's API: the reference's own unit-test sources must compile
against them as they are.  The sources are read where they lie (nothing is copied, nothing is linked or run), with one
name mapped: isCudaReady() is isHipReady() here.  Skipped where the reference is not mounted (the GPU box)."""
import glob
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
UNITTEST = "/root/reference/unittest"


@pytest.mark.skipif(not os.path.isdir(UNITTEST), reason="the reference's sources are not mounted here")
def test_the_references_unit_test_sources_compile_against_these_headers():
    sources = sorted(glob.glob(os.path.join(UNITTEST, "*", "test_*.cpp")))
    assert len(sources) >= 5
    for src in sources:
        proc = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I" + os.path.join(ROOT, "include"), "-I" + UNITTEST,
                               "-DisCudaReady=isHipReady", src], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert proc.returncode == 0 and proc.stdout.strip() == "", src + "\n" + proc.stdout[-3000:]
