"""Slice planner (tp_plan_slices, host code: runs without a GPU) against the oracle's restatement of
latency_model.py:97-152 and against exhaustive enumeration on tiny grids.  Every test is collected twice, once
unmarked and once marked `gpu`, so that both the CPU run and the run on the GPU box include it (the planner is
host code of the same shared library on either machine)."""
import math

import numpy as np
import pytest

from oracle import planner_oracle as po
from terapipe_amd import latency_model as lm


BOTH_RUNS = pytest.mark.parametrize("run", [pytest.param("cpu-run"), pytest.param("gpu-box-run", marks=pytest.mark.gpu)])


def _grid(B, N, seed, kind="smooth"):
    rng = np.random.default_rng(seed)
    g = np.full((B + 1, N + 1, N + 1), np.inf)
    for b in range(1, B + 1):
        for s in range(1, N + 1):
            for c in range(0, N + 1 - s):
                if kind == "smooth":      # fixed cost per slice + work terms, like a measured grid
                    g[b, s, c] = 0.3 + 0.05 * b * s + 0.01 * b * s * c + 0.02 * b * c
                else:
                    g[b, s, c] = rng.uniform(0.1, 2.0)
    return g


@BOTH_RUNS
@pytest.mark.parametrize("B,N,pipe,kind,seed", [(1, 5, 1, "random", 0), (2, 5, 4, "random", 1), (3, 6, 8, "smooth", 2),
                                                (2, 7, 3, "random", 3), (1, 8, 24, "smooth", 4)])
def test_planner_matches_oracle_and_brute_force(B, N, pipe, kind, seed, run):
    g = _grid(B, N, seed, kind)
    lat = np.sort(np.unique(g[np.isfinite(g)]))
    for max_latency in (math.inf, float(lat[len(lat) // 2]), float(lat[len(lat) // 4]), float(lat[0]) * 0.5):
        final, scheme = lm.planning(g, B, N * lm.STEP_GAP, pipe, max_latency)
        final_o, scheme_o = po.planning(g.tolist(), B, N, pipe, max_latency)
        assert (scheme is None) == (scheme_o is None)
        if scheme is None:
            assert math.isinf(final) and math.isinf(final_o)
            assert math.isinf(po.brute_force_best(g.tolist(), B, N, pipe, max_latency))
            continue
        assert final == pytest.approx(final_o, rel=1e-12)
        assert [(b, [s // lm.STEP_GAP for s in sl]) for b, sl in scheme] == scheme_o      # same plan, same tie-breaking
        # Note: the DP minimises the SUM first and carries the maximum along; it is the exact optimum of
        # sum + (pipe - 1) * max only together with the outer sweep over max_latency (best_plan below).
        assert sum(b for b, _ in scheme) == B and all(sum(sl) == N * lm.STEP_GAP for _, sl in scheme)
        in_order = [(b, list(reversed(sl))) for b, sl in scheme]
        assert lm.evaluate_split(g, in_order, pipe) == pytest.approx(final, rel=1e-12)
        assert final >= po.brute_force_best(g.tolist(), B, N, pipe, max_latency) - 1e-12


@BOTH_RUNS
@pytest.mark.parametrize("B,N,pipe,kind,seed", [(2, 5, 4, "random", 5), (2, 6, 6, "smooth", 6), (1, 7, 12, "random", 7)])
def test_best_plan_sweep_reaches_the_exhaustive_optimum(B, N, pipe, kind, seed, run):
    g = _grid(B, N, seed, kind)
    scheme, latency = lm.best_plan(g, B, N * lm.STEP_GAP, pipe, gap=0.0)
    assert latency == pytest.approx(po.brute_force_best(g.tolist(), B, N, pipe, math.inf), rel=1e-12)
    assert lm.evaluate_split(g, scheme, pipe) == pytest.approx(latency, rel=1e-12)


@BOTH_RUNS
def test_fit_latency_grid_reproduces_a_linear_model(run):
    B, S = 2, 64
    truth = lambda b, s, c: 1e-3 + 2e-5 * b * s + (3e-7 * b * s + 1e-7 * b * c + 5e-9 * b * s * c if c else 0.0)
    samples = {(b, s, c): truth(b, s, c) for b in (1, 2) for s in (8, 16, 32, 64) for c in (0, 8, 24, 48) if s + c <= S}
    grid = lm.fit_latency_grid(samples, B, S)
    for b in (1, 2):
        for s in (8, 24, 40):
            for c in (0, 16):
                assert grid[b, s // 8, c // 8] == pytest.approx(truth(b, s, c), rel=1e-6)
