"""The library's host code (kernel-string parser, binding, generator, run-time compiler front end) under
AddressSanitizer and UndefinedBehaviorSanitizer: acrotensor_amd/lib/asan/sanitize_generator (built by
`make -C acrotensor_amd/csrc asan`, part of __graft_entry__.build()) generates the kernels whose sources
tests/golden/codegen_hashes.json pins, which must come out as from the ordinary build, and some hundred seeded random
kernels and captures; any sanitizer report fails the run.  No device is needed."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(os.path.dirname(HERE), "acrotensor_amd", "lib", "asan", "sanitize_generator")
sys.path.insert(0, os.path.join(HERE, "golden"))


def run(*args):
    if not os.path.exists(BINARY):
        pytest.fail("acrotensor_amd/lib/asan/sanitize_generator is not built (run __graft_entry__.build())")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    for name in list(env):
        if name.startswith("ACRO_HIP_") and name != "ACRO_HIP_CACHE_DIR":
            del env[name]                                  # experiment switches change what is emitted
    proc = subprocess.run([BINARY] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=900, env=env)
    print(proc.stdout[-4000:])
    assert "AddressSanitizer" not in proc.stdout and "runtime error:" not in proc.stdout and "LeakSanitizer" not in proc.stdout
    assert proc.returncode == 0
    return proc.stdout


def fnv1a(text):
    h = 1469598103934665603
    for c in text.encode():
        h = ((h ^ c) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return "%016x" % h


def spec_of_the_pinned_kernels():
    """The kernels of tests/golden/make_codegen_hashes.py in the driver's input format."""
    import make_codegen_hashes as pinned
    lines = []
    for name, kernel, shapes in pinned.SINGLES:
        if name == "dsetup":
            continue                                       # binds one tensor to two operands: not expressible here
        lines.append("single %s | %s | %s" % (name, kernel, " ; ".join(",".join(str(d) for d in s) for s in shapes)))
    for name, (factory, E) in pinned.CHAINS.items():
        small = factory(E=2)
        axes = {}
        for k, out, ins in small.kernels:
            lhs, rhs = k.replace("+=", "=").split("=")
            for token, tensor in zip([lhs.split()[0]] + rhs.split(), [out] + list(ins)):
                axes[tensor] = token.split("_")[1:]
        for transient in (True, False):
            lines.append("chain %s_%s" % (name, "transient" if transient else "stored"))
            for tensor, arr in small.arrays.items():
                shape = list(arr.shape)
                if tensor in axes and "e" in axes[tensor]:
                    shape[axes[tensor].index("e")] = E
                lines.append("tensor %s %s" % (tensor, ",".join(str(d) for d in shape)))
            for tensor, (parent, idx) in small.slices.items():
                lines.append("slice %s %s %s" % (tensor, parent, ",".join(str(i) for i in idx)))
            if transient:
                lines += ["transient %s" % tensor for tensor in small.transient]
            for k, out, ins in small.kernels:
                lines.append("kernel %s | %s %s" % (k, out, " ".join(ins)))
            lines.append("end")
    return "\n".join(lines) + "\n"


def test_pinned_kernels_come_out_the_same_under_the_sanitizers(tmp_path, monkeypatch):
    for name in list(os.environ):
        if name.startswith("ACRO_HIP_") and name != "ACRO_HIP_CACHE_DIR":
            monkeypatch.delenv(name)
    import make_codegen_hashes as pinned
    spec = tmp_path / "pinned.spec"
    spec.write_text(spec_of_the_pinned_kernels())
    reported = dict(line.split() for line in run("spec", spec).splitlines() if len(line.split()) == 2)
    expected = {name: fnv1a(src) for name, src in pinned.all_sources().items() if name != "dsetup"}
    assert sorted(reported) == sorted(expected)
    assert [name for name in expected if reported[name] != expected[name]] == []


def test_random_kernels_and_captures_under_the_sanitizers():
    out = run("random", 300, 20261126)
    assert "random kernels 300" in out and "captures 30" in out
