"""The source that the generator emits for the five baseline configurations and for one kernel of every other
schedule is pinned by hash (host only: generating needs no device).  A refactoring of the generator must leave every
hash as it is; a deliberate change of an emitted kernel is recorded with tests/golden/make_codegen_hashes.py."""
import json
import os
import sys

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLDEN)


def test_emitted_sources_are_the_recorded_ones(monkeypatch):
    for name in list(os.environ):
        if name.startswith("ACRO_HIP_") and name != "ACRO_HIP_CACHE_DIR":
            monkeypatch.delenv(name)                  # experiment switches change what is emitted
    import make_codegen_hashes
    recorded = json.load(open(os.path.join(GOLDEN, "codegen_hashes.json")))
    emitted = make_codegen_hashes.all_hashes()
    assert sorted(emitted) == sorted(recorded)
    changed = [name for name in recorded if emitted[name] != recorded[name]]
    assert changed == [], "emitted kernels changed (run tests/golden/make_codegen_hashes.py if that is intended)"
