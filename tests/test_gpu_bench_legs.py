"""GPU: the legs bench.py adds to its line for the configurations other than the headline one run to the end and
report no error.  bench.py starts each leg as a process of its own and reports a leg that fails under an `error` key
so that the headline survives; here such a key is a failure.  Each leg runs for two timed steps (eight for the
dynamic-expansion leg, which splits its steps between eager issue and a graph replay; the host-backed cache over a
small host table, so that the test does not pin 51 GB)."""
import importlib.util
import os

import pytest

pytestmark = pytest.mark.gpu


def _bench_module():
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")
    spec = importlib.util.spec_from_file_location("bench_under_test", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_every_leg_reports_a_line_with_a_roofline_and_no_error(monkeypatch):
    bench = _bench_module()
    names = [p[0] for p in bench.OTHER_CONFIG_PLAN]
    assert names == ["c1", "c3", "c4", "c5"]
    small = [(n, 8 if n == "c4" else 2, 1, ["--host-rows", "4000000"] if n == "c5" else [])
             for n, _, _, _ in bench.OTHER_CONFIG_PLAN]
    monkeypatch.setattr(bench, "OTHER_CONFIG_PLAN", small)
    out = bench.other_configs()
    assert out, "no leg reported"
    for d in out:
        assert "error" not in d, d
        r = d["roofline"]
        assert r["bound"] in ("hbm", "host link") and r["peak"] > 0 and 0 < r["frac"] < 1, d
        assert d["value"] > 0 and d["ms_per_step"] > 0
    assert {d["config"] for d in out} == {"C1", "C3", "C4", "C5"}


def test_a_leg_that_fails_is_reported_under_an_error_key(monkeypatch):
    bench = _bench_module()
    monkeypatch.setattr(bench, "OTHER_CONFIG_PLAN", [("c4", 2, 1, [])])       # too few steps for that leg: it raises
    out = bench.other_configs()
    assert len(out) == 1 and out[0]["config"] == "C4" and "error" in out[0]
