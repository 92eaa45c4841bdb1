"""The parameter search of decdec_amd.autotune on synthetic timing tables (no GPU)."""
import itertools

import pytest

from decdec_amd import autotune as A

DIMS = {"qkv": (4096, 6144), "o": (4096, 4096), "gu": (4096, 28672), "d": (14336, 4096)}


def table(base, fixed, slope, n_tbs=(4, 8, 16), ks=range(1, 13), tb_gain=0.0):
    """time(n_tb, k) = base + fixed + slope * k * (1 - tb_gain * log2(n_tb / 4))"""
    import math
    return base, {n: {k: base + fixed + slope * k * (1 - tb_gain * math.log2(n / 4)) for k in ks} for n in n_tbs}


def layer(res, dims, ks, n_tbs):
    """times of the chosen configuration"""
    return sum(res[m][0] if k == 0 else res[m][1][n][k] for m, k, n in zip(dims, ks, n_tbs))


def test_break_even_estimate_follows_the_reference_rule():
    # run_profile.py:26-30 with HBM 8000 GB/s and a 64 GB/s link: 3 / 125 / 4 * 1024
    assert A.k_chunk_estimate(3) == 6 and A.k_chunk_estimate(4) == 8


def test_global_then_fine_grained_search():
    res = {"qkv": table(10, 0.2, 0.5), "o": table(8, 0.2, 0.4), "gu": table(40, 0.2, 2.0), "d": table(20, 0.2, 1.0)}
    out = A.tune(res, 1.10, DIMS)
    budget = out["layer_baseline"] * 1.10
    assert out["layer_baseline"] == pytest.approx(78)
    # global search: uniform k = 1 costs 0.8 + 3.9 = 4.7, k = 2 costs 8.6 > 7.8  -> k = 1 everywhere, then the
    # cheapest +1 steps (o: 0.4, qkv: 0.5, d: 1.0, gu: 2.0) are added while the budget of 7.8 allows
    ks = dict(zip(DIMS, out["k_chunk_per_module"]))
    assert all(k >= 1 for k in ks.values())
    assert out["layer_time"] <= budget + 1e-9
    assert out["layer_time"] == pytest.approx(layer(res, DIMS, out["k_chunk_per_module"], out["threadblocks_per_module"]))
    # no single further step fits
    for m, k, n in zip(DIMS, out["k_chunk_per_module"], out["threadblocks_per_module"]):
        nxt = res[m][1][n].get(k + 1)
        assert nxt is None or out["layer_time"] - res[m][1][n][k] + nxt > budget
    # the cheap modules got more channels than the expensive one
    assert ks["o"] >= ks["qkv"] >= ks["gu"]


def test_more_workgroups_win_when_they_speed_up_the_fetch():
    res = {m: table(b, 0.1, s, tb_gain=0.3) for m, (b, s) in
           {"qkv": (10, 0.5), "o": (8, 0.4), "gu": (40, 2.0), "d": (20, 1.0)}.items()}
    out = A.tune(res, 1.10, DIMS)
    assert out["best_max_n_tb"] == 16
    # brute force over uniform k and caps reproduces the global phase's k
    best = 0
    for cap, k in itertools.product((4, 8, 16), range(1, 13)):
        if sum(res[m][1][cap][k] for m in DIMS) <= out["layer_baseline"] * 1.10:
            best = max(best, k)
    assert min(out["k_chunk_per_module"]) >= best >= 1


def test_modules_are_excluded_smallest_first_when_nothing_fits():
    # DEC has a fixed cost of 6 us per module: with a 10 % budget on a 78 us layer (7.8 us) only one module can
    # be compensated at all, and the search keeps the largest one
    res = {"qkv": table(10, 6.0, 0.1), "o": table(8, 6.0, 0.1), "gu": table(40, 6.0, 0.1), "d": table(20, 6.0, 0.1)}
    out = A.tune(res, 1.10, DIMS)
    ks = dict(zip(DIMS, out["k_chunk_per_module"]))
    assert ks["o"] == 0 and ks["qkv"] == 0 and ks["d"] == 0 and ks["gu"] >= 1
    assert out["layer_time"] <= out["layer_baseline"] * 1.10 + 1e-9
    # and with a fixed cost no budget covers, nothing is compensated and the layer keeps its baseline time
    res = {m: table(b, 100.0, 0.1) for m, b in {"qkv": 10, "o": 8, "gu": 40, "d": 20}.items()}
    out = A.tune(res, 1.025, DIMS)
    assert out["k_chunk_per_module"] == [0, 0, 0, 0] and out["best_max_n_tb"] is None
    assert out["layer_time"] == pytest.approx(78)


@pytest.mark.gpu
def test_measure_and_tune_on_a_small_model():
    dims = {"qkv": (2048, 1536), "o": (2048, 1024)}
    res = A.measure(dims, "anyprec", 3, [4, 8], [1, 2, 4], reps=3, iters=3)
    for m in dims:
        base, tab = res[m]
        assert base > 0 and set(tab) == {4, 8} and all(t > 0 for n in tab for t in tab[n].values())
    out = A.tune(res, 3.0, dims)
    assert out["layer_time"] <= out["layer_baseline"] * 3.0
