"""Host logic of the operator benchmark and launch-shape sweep (no GPU): the enumeration of
the settings, the slope estimate, the choice of the best setting, the CSV."""
import csv
import itertools

import pytest

from msd_pytorch_amd import benchmark_ops as bo
from msd_pytorch_amd.bench import TimeitResult, bench, format_time


def test_every_swept_knob_is_known_to_the_library():
    from msd_pytorch_amd import _native
    lib = _native.load()
    for op, ranks in bo.SWEEP_GRID.items():
        for ndim, grid in ranks.items():
            for key in list(grid) + list(bo.ORDER_KNOB):
                assert lib.msd_set_tuning(key.encode(), -1) == 0, (op, ndim, key)


def test_enumeration_is_the_full_grid_with_the_default_first():
    for op, ranks in bo.SWEEP_GRID.items():
        for ndim, grid in ranks.items():
            settings = bo.enumerate_settings(op, ndim)
            assert settings[0] == {}
            want = 1
            for values in grid.values():
                want *= len(values)
            assert len(settings) == want + 1
            assert len({bo.setting_name(s) for s in settings}) == len(settings)
            assert all(set(s) == set(grid) for s in settings[1:])
            with_order = bo.enumerate_settings(op, ndim, with_order=True)
            assert len(with_order) == 2 * want + 1
    assert len(bo.enumerate_settings("forward", 2, limit=5)) == 6
    assert bo.setting_name({}) == "default"
    assert bo.setting_name({"fwd.vec2d": 4, "fwd.rows2d": 5}) == "fwd.vec2d=4;fwd.rows2d=5"


def test_slope_estimate_removes_the_fixed_cost():
    # wall time = 50 us of fixed cost + 7 us per call: the slope is the per-call time
    now = [0.0]

    def run(n):
        now[0] += 50e-6 + 7e-6 * n

    slope, (low, high) = bo.slope_time(run, counts=(1, 2, 4, 8), trials=3, clock=lambda: now[0])
    assert slope == pytest.approx(7e-6, rel=1e-9)
    assert low <= slope <= high and high - low < 1e-12
    # with noise the interval opens and still covers the truth
    noise = itertools.cycle([3e-6, -2e-6, 1e-6, -3e-6, 2e-6])

    def noisy(n):
        now[0] += 50e-6 + 7e-6 * n + next(noise)

    slope, (low, high) = bo.slope_time(noisy, counts=(1, 2, 4, 8), trials=4, clock=lambda: now[0])
    assert low < 7e-6 < high and high - low > 1e-7
    assert bo._t_quantile_95(10) == pytest.approx(1.8125, abs=2e-3)


class FakeLib:
    def __init__(self):
        self.state = {}

    def msd_set_tuning(self, key, value):
        if value < 0:
            self.state.pop(key.decode(), None)
        else:
            self.state[key.decode()] = value
        return 0


class FakeProblem:
    ndim, batch, c_in, width, dilation, spatial, nvox = 2, 1, 10, 1, 3, (64, 64), 4096
    row = bo.Problem.row


def test_sweep_cell_applies_each_setting_and_picks_the_best(tmp_path):
    lib = FakeLib()
    seen = []

    def measure(problem, op, trials):
        seen.append(dict(lib.state))
        t = 10e-6
        if lib.state.get("fwd.vec2d") == 4 and lib.state.get("fwd.rows2d") == 5:
            t = 6e-6                       # clearly faster
        elif lib.state.get("fwd.vec2d") == 2:
            t = 9.9e-6                     # faster only within the noise
        return t, (t - 0.3e-6, t + 0.3e-6)

    settings = bo.enumerate_settings("forward", 2)
    rows = bo.sweep_cell(FakeProblem(), "forward", settings, 3, lib, measure=measure)
    assert lib.state == {}                                  # every setting was undone
    assert seen[0] == {} and seen[1:] == settings[1:]
    default, best = bo.best_of(rows)
    assert default["setting"] == "default" and default["us"] == pytest.approx(10.0)
    assert best["us"] == pytest.approx(6.0) and "fwd.vec2d=4" in best["setting"] and "fwd.rows2d=5" in best["setting"]
    # a gain inside the confidence intervals is no recommendation
    near = [r for r in rows if r["us"] > 9.0]
    assert bo.best_of(near)[1] is near[0]
    path = tmp_path / "sweep.csv"
    bo.write_csv(str(path), rows)
    back = list(csv.DictReader(open(path)))
    assert len(back) == len(rows) and list(back[0]) == bo.CSV_FIELDS
    assert back[0]["setting"] == "default" and float(back[0]["GBps"]) == pytest.approx(rows[0]["GBps"])
    nbytes = bo.algorithmic_bytes("forward", 2, 4096, 10, 1)
    assert nbytes == (10 + 1) * 4096 * 4 + 10 * 9 * 4
    assert rows[0]["frac_hbm"] == pytest.approx(nbytes / 10e-6 / 8e12)


def test_timeit_helper():
    calls = []
    result = bench("append", lambda: calls.append(1), repeat=3, min_time=0.001)
    assert isinstance(result, TimeitResult) and result.repeat == 3 and len(result.all_runs) == 3
    assert result.loops in (10 ** p for p in range(10)) and len(calls) >= 3 * result.loops
    assert result.best <= result.average <= result.worst and result.stdev >= 0
    assert "per loop" in str(result) and str(result).startswith("append:")
    synced = []
    bench("synced", lambda: None, repeat=2, sync=lambda: synced.append(1), min_time=0.0)
    assert len(synced) >= 2 * 2 + 2          # two per run, at least the calibration run and two repeats
    assert format_time(1.5e-3) == "1.5 ms" and format_time(2.5e-7) == "250 ns" and format_time(125) == "2 min 5 s"


def test_algorithmic_bytes_of_the_paired_3d_chain():
    # workload D, depth 50: pairs (49, 48) ... (1, 0); the upper layer over the one channel the
    # lower one wrote (4 planes), then one read-modify-write pass over the channels below
    import bench
    per_layer, _, n = bench.algorithmic_work("D", False, kpairs=True, chainpairs=False)
    paired, flops, _ = bench.algorithmic_work("D", False, kpairs=True, chainpairs=True)
    expect = 3 * n * 4                                    # the top layer's mask pass
    for upper in range(49, 0, -2):
        lower = upper - 1
        expect += 4 * n * 4 + 27 * 4
        if lower > 0:                                     # layer 0's pass would only serve the block's input
            channels = 1 + lower
            expect += (2 * channels + 2) * n * 4 + 2 * channels * 27 * 4
    assert paired["backward_x"] == expect
    assert 0.5 < paired["backward_x"] / per_layer["backward_x"] < 0.55
    assert paired["backward_kb"] == per_layer["backward_kb"] and paired["forward"] == per_layer["forward"]
    assert flops["backward_x"] > 0
