"""The oracle against the vectors it wrote once it had been pinned (tests/golden/adamw_regression.json):
a change of a single bit — in the oracle's source, its compiler flags or on another host CPU — fails here."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_reproduces_its_frozen_vectors(O):
    spec = importlib.util.spec_from_file_location("make_adamw_regression",
                                                  os.path.join(ROOT, "tests", "golden", "make_adamw_regression.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    want = json.load(open(os.path.join(ROOT, "tests", "golden", "adamw_regression.json")))
    got = json.loads(json.dumps(mod.run()))
    assert got == want
