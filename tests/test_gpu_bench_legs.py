"""GPU: the legs bench.py adds to its line for the configurations other than the headline one run to the end and
report no error.  bench.py catches an exception of a leg and reports it under an `error` key so that the headline
survives; here such a key is a failure.  Each leg runs for two timed steps (eight for the dynamic-expansion leg,
which splits its steps between eager issue and a graph replay; the host-backed cache over a small host table, so
that the test does not pin 51 GB)."""
import importlib.util
import os

import pytest
import torch

from recsdk_amd import capi, config_bench, host, synth

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
    monkeypatch.setattr(bench, "OTHER_CONFIG_PLAN", [(n, f, 8 if n == "c4" else 2, 1) for n, f, _, _ in bench.OTHER_CONFIG_PLAN])
    real_defaults = config_bench.default_args

    def small_defaults(**kw):
        a = real_defaults(**kw)
        a.host_rows = 4_000_000
        return a

    monkeypatch.setattr(config_bench, "default_args", small_defaults)
    capi.lib()
    torch.cuda.set_device(0)
    out = bench.other_configs(torch, capi, host, synth)
    assert out, "no leg reported"
    for d in out:
        assert "error" not in d, d
        r = d["roofline"]
        assert r["bound"] in ("hbm", "host link") and r["peak"] > 0 and 0 < r["frac"] < 1, d
        assert d["value"] > 0 and d["ms_per_step"] > 0
    assert {d["config"] for d in out} == {"C1", "C3", "C4", "C5"}
