"""bench.py's table of legs against the committed counter summary: every leg whose kernels the
table names has its bytes per call in profiles/hbm_traffic.json (a kernel renamed in the library
and not in the table drops out of that file silently, and its leg then reports no traffic)."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_every_leg_has_its_traffic_figure():
    legs = _bench().LEG_KERNELS
    with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
        per_call = json.load(f)["bytes_per_call"]
    missing = []
    for leg, spec in legs.items():
        for name in spec.get("split", [leg]):
            if not per_call.get(name):
                missing.append(name)
    assert not missing, missing
