"""Host-side pieces of bench.py and of the synthetic graphs: what a profile summary under
profiles/ is allowed to tell the bench line, and that the generators do not depend on the
host's random-normal sampler."""
import importlib.util
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_profile_summary_is_used_only_for_the_workload_it_describes(tmp_path, monkeypatch, capsys):
    bench = load_bench()
    prof = tmp_path / "profiles"
    prof.mkdir()
    (prof / "k.txt").write_text("text\n@config 2\n@V 1000\n@E 200000\n@F 128\n@traffic_bytes 1000000\n@l2_hit_rate 0.5\n")
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    same = bench.read_profile("k.txt", {"V": 1000, "E": 200000, "F": 128})
    assert same is not None and float(same["traffic_bytes"]) == 1000000
    # an edge or two apart (another host's math library): accepted, the bytes follow the edges
    near = bench.read_profile("k.txt", {"V": 1000, "E": 200100, "F": 128})
    assert near is not None and abs(float(near["traffic_bytes"]) - 1000000 * 200100 / 200000) < 1e-6
    # another workload: not used, and the run goes on
    assert bench.read_profile("k.txt", {"V": 1000, "E": 210000, "F": 128}) is None
    assert bench.read_profile("k.txt", {"V": 1001, "E": 200000, "F": 128}) is None
    assert "not used" in capsys.readouterr().err
    assert bench.read_profile("missing.txt", {"V": 1}) is None
    r = bench.roofline("k.txt", {"V": 1000, "E": 210000, "F": 128}, "kernel", 1.0, 2_000_000, 500_000, "test")
    assert r["traffic"] is None and r["achieved_basis"].startswith("algorithmic")


def test_lognormal_degrees_come_from_uniform_draws_only():
    """The same seed gives the same graph, the degrees follow the requested mean, and the
    generator's own normal sampler (whose rejection step compares library logarithms) is not
    what the degrees are drawn from."""
    from jittorgeometric_amd import synthetic
    a = synthetic.lognormal_degree(20000, 30.0, sigma=1.0, seed=4)
    b = synthetic.lognormal_degree(20000, 30.0, sigma=1.0, seed=4)
    assert np.array_equal(a, b) and a.dtype == np.int32
    deg = np.bincount(a[0], minlength=20000)
    assert 27.0 < deg.mean() < 33.0 and deg.max() > 300
    assert not (a[0] == a[1]).any()
    rng = np.random.default_rng(4)
    u1, u2 = rng.random(20000), rng.random(20000)
    z = np.sqrt(-2.0 * np.log1p(-u1)) * np.cos(2.0 * np.pi * u2)
    want = np.maximum(np.rint(np.exp(np.log(30.0) - 0.5 + z)), 0).astype(np.int64)
    # self-loops are dropped afterwards: a node keeps its drawn degree or loses a few entries
    assert (deg <= want).all() and (want - deg).sum() < 100
