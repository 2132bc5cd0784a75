"""The HBM-traffic record that bench.py quotes (profiles/hbm_traffic.json) belongs to the library
as built: its version must be this library's, and bench.py's guard must drop a figure whose
kernels are not the ones a run launched."""
import importlib.util
import json
import os

from dkernel_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_record_is_of_this_library_version():
    rec = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json")))
    assert rec["dk_version"] == _lib.lib().dk_version(), "kernels changed version: re-profile and rewrite the record"
    for leg in ("fwd", "bwd", "decode", "combine"):
        assert rec[leg]["kernels"].endswith("; ") and rec[leg]["fetch_bytes"] > 0 and rec[leg]["write_bytes"] >= 0


def test_guard_drops_figures_of_other_kernels_or_versions():
    bench = _bench()
    rec = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json")))
    v = rec["dk_version"]
    got, src = bench.quoted_traffic("fwd", rec["fwd"]["kernels"], v)
    assert got == rec["fwd"]["fetch_bytes"] + rec["fwd"]["write_bytes"] and "profiles/" in src
    got, why = bench.quoted_traffic("fwd", "generic_fwd_kernel<128>; ", v)
    assert got is None and "re-profile" in why
    got, why = bench.quoted_traffic("fwd", rec["fwd"]["kernels"].encode(), v + 1)
    assert got is None and "version" in why
    assert bench.quoted_traffic("prefill", "x", v)[0] is None
