"""The measurement helpers without a GPU: the rule that says when the clock has settled, the summary of
the readings inside a timed window, step times kept apart by the kind of step, and markers that are
no-ops outside a profiler."""

from __future__ import annotations

import itertools

import pytest

import time

import numpy as np

from miniserve_amd.measurement import GpuMonitor, gpu_now, mark, measured_region
from miniserve_amd.measurement.offline import run_to_completion
from miniserve_amd.measurement.sidecar import COLUMNS, throttled_share


def readings(clocks, power=None, t0=100.0, dt=0.1, polls=1):
    """Rows in the monitor's column order: time, shader clock, memory clock, power, two temperatures, two
    activities, the firmware's stamp of the refresh. Every refresh is read ``polls`` times in a row."""
    return [(t0 + (i * polls + k) * dt / polls, c, 2000.0, None if power is None else power[i], 40.0, 35.0, 99.0, 10.0, 7000 + i)
            for i, c in enumerate(clocks) for k in range(polls)]


def monitor_with(rows, **kw):
    g = GpuMonitor(**kw)
    g.load(rows)
    return g


def test_a_reading_without_a_gpu_says_unknown_not_zero():
    s = gpu_now()
    assert set(s) == set(COLUMNS[1:-1]) and "power_w" in s and "mclk_mhz" in s and "refresh" not in s
    assert all(v is None or v >= 0 for v in s.values())


def test_the_clock_is_steady_when_two_runs_of_readings_agree():
    assert monitor_with(readings([2400, 2400, 2400])).steady(readings=4) is None, "fewer than two runs of readings decide nothing"
    falling = monitor_with(readings([2400, 2300, 2100, 1900, 1750, 1720, 1700, 1700]))  # 2175 against 1717
    assert falling.steady(readings=4) is False
    flat = monitor_with(readings([2400, 2300, 2100, 1900, 1710, 1700, 1705, 1695, 1700, 1702, 1698, 1700]))
    assert flat.steady(readings=4) is True  # the last four against the four before them: within 2 %
    step = monitor_with(readings([1700] * 4 + [1740] * 4))  # 2.3 % apart
    assert step.steady(readings=4) is False and step.steady(readings=4, tolerance=0.03) is True
    assert monitor_with(readings([None] * 20)).steady() is None, "a clock that cannot be read settles nothing"
    gaps = monitor_with(readings([1700, None, 1700, 1700, None, 1700, 1700, 1700, 1700, 1700]))  # unknown readings are skipped
    assert gaps.steady(readings=4) is True
    # what counts are the firmware's refreshes, however often each is read: two refreshes polled ten times each decide
    # what two refreshes decide, not what twenty readings would
    polled = monitor_with(readings([2400, 2300, 1700, 1700], polls=10))
    assert len(polled.readings()) == 40 and len(polled.refreshes()) == 4
    assert polled.steady(readings=1) is True and polled.steady(readings=2) is False and polled.steady(readings=4) is None
    assert polled.window()["samples"] == 4 and polled.window()["sclk_mhz"]["mean"] == 2025.0


def test_the_window_covers_the_timed_span_only():
    g = monitor_with(readings([2400, 2000, 1800, 1700, 1700, 2400], power=[100, 600, 900, 1000, 1000, 120]))
    whole = g.window()
    assert whole["samples"] == 6 and whole["sclk_mhz"] == {"min": 1700, "max": 2400, "mean": 2000.0}
    inside = g.window(since=100.15, until=100.45)  # readings 2, 3 and 4
    assert inside["samples"] == 3 and inside["sclk_mhz"] == {"min": 1700, "max": 1800, "mean": 1733.3}
    assert inside["power_w"] == {"min": 900, "max": 1000, "mean": 966.7} and inside["mclk_mhz"]["mean"] == 2000.0
    empty = g.window(since=200.0)
    assert empty["samples"] == 0 and all(empty[c] is None for c in COLUMNS[1:-1])
    g = monitor_with(readings([None, None]))
    assert g.window()["sclk_mhz"] is None and g.window()["temp_c"]["mean"] == 40.0


def test_the_ring_keeps_the_latest_readings_in_order():
    g = monitor_with(readings(range(1000, 1010)), capacity=4)
    assert g.column("sclk_mhz").tolist() == [1006, 1007, 1008, 1009]
    assert np.all(np.diff(g.column("t")) > 0)


def test_the_monitor_thread_collects_and_stops():
    with GpuMonitor(interval_s=0.01) as g:
        first = g.read_now()
        while len(g.readings()) < 3:
            pass
    n = len(g.readings())
    times = g.column("t")
    assert n >= 3 and first in times and np.all(np.diff(times) >= 0)
    time.sleep(0.03)
    assert len(g.readings()) == n, "no reading after the with block has ended"


def test_warming_waits_for_a_steady_clock_between_a_least_and_a_most_time():
    """``work`` stands for a few decode steps; the readings are fed by the test instead of a thread."""
    g = GpuMonitor()
    clocks = iter([2400, 2300, 2200, 2100, 2000, 1900, 1800] + [1700] * 200)
    stamp = iter(range(10**6))

    def work():
        g._append([time.monotonic(), next(clocks), 2000.0, 900.0, 50.0, 40.0, 100.0, 20.0, next(stamp)])
        time.sleep(0.004)

    out = g.warm_until_steady(work, least_s=0.02, most_s=2.0, readings=3)
    # falling for seven refreshes, then flat: steady once the last three and the three before them agree
    assert out["steady"] is True and 0.02 <= out["seconds"] < 1.0 and 10 <= out["calls"] < 100 and out["refreshes"] >= 6
    falling = iter(range(2400, 0, -20))
    g2 = GpuMonitor()

    def cooling():
        g2._append([time.monotonic(), next(falling), 2000.0, 900.0, 50.0, 40.0, 100.0, 20.0, next(stamp)])
        time.sleep(0.004)

    out = g2.warm_until_steady(cooling, least_s=0.01, most_s=0.15, readings=3)
    assert out["steady"] is False and out["seconds"] >= 0.15, "a clock that keeps moving ends the wait at the most time, and says so"
    # the first refresh after the warm-up began mixes what came before with the load and does not count:
    # idle, then the load's clock twice, is steady at the third refresh and not at the second
    g4 = GpuMonitor()
    seen = iter([(900, 1), (900, 1), (2000, 2), (2000, 2), (2000, 3)] + [(2000, 3)] * 100)

    def slow_firmware():
        c, s = next(seen)
        g4._append([time.monotonic(), c, 2000.0, 900.0, 50.0, 40.0, 100.0, 20.0, 5000 + s])
        time.sleep(0.004)

    out = g4.warm_until_steady(slow_firmware, least_s=0.0, most_s=1.0)
    assert out == {"calls": 5, "seconds": out["seconds"], "refreshes": 2, "steady": True}
    # and a load kept up until the firmware reports once more
    g5 = GpuMonitor()
    ticks = iter([4, 4, 4, 5, 5])
    g5._append([time.monotonic(), 2000, 2000.0, 900.0, 50.0, 40.0, 100.0, 20.0, 4])
    assert g5.hold_until_refresh(lambda: g5._append([time.monotonic(), 2000, 2000.0, 900.0, 50.0, 40.0, 100.0, 20.0, next(ticks)])) is True
    assert len(g5.refreshes()) == 2 and len(g5.readings()) == 5
    assert g5.hold_until_refresh(lambda: time.sleep(0.01), most_s=0.03) is False
    g3 = GpuMonitor()
    out = g3.warm_until_steady(lambda: time.sleep(0.002), least_s=0.01, most_s=0.03)
    assert out["steady"] is None and out["seconds"] >= 0.03, "a clock that cannot be read decides nothing"
    stale = monitor_with(readings([1700] * 40, t0=time.monotonic() - 100))
    out = stale.warm_until_steady(lambda: time.sleep(0.002), least_s=0.01, most_s=0.03)
    assert out["steady"] is None, "readings from before the warm-up do not count"


def test_the_share_of_time_held_back_is_a_difference_of_counters():
    before = {"all": 1000.0, "power": 100.0, "socket_temperature": 0.0, "hot_spot": 0.0, "regulator_temperature": 0.0, "memory_temperature": float("nan")}
    after = {"all": 3000.0, "power": 600.0, "socket_temperature": 0.0, "hot_spot": 20.0, "regulator_temperature": 0.0, "memory_temperature": float("nan")}
    share = throttled_share(before, after)
    assert share == {"power": 0.25, "socket_temperature": 0.0, "hot_spot": 0.01, "regulator_temperature": 0.0, "memory_temperature": None}
    assert throttled_share(None, after) is None and throttled_share(before, before) is None  # the counter did not run


def test_markers_do_nothing_outside_a_profiler():
    with measured_region("timed"):
        with mark("step"):
            pass
    with pytest.raises(ZeroDivisionError):  # an exception passes through and the ranges are closed
        with measured_region("timed"):
            with mark("step"):
                1 / 0
    with mark("after"):
        pass


class _Batch:
    def __init__(self, phase, rows, tokens):
        self.phase, self.rows, self.num_tokens = phase, [None] * rows, tokens


class _Engine:
    """Returns the given batches one per step (None: a step whose tokens are not due yet)."""

    def __init__(self, batches):
        self._it = iter(batches)
        self._left = len(batches)

    @property
    def has_unfinished(self):
        return self._left > 0

    def step(self):
        self._left -= 1
        return next(self._it)


def test_step_times_are_kept_apart_by_the_kind_of_step():
    from miniserve_amd.engine.scheduler import Phase

    batches = [None, _Batch(Phase.PREFILL, 2, 40), _Batch(Phase.MIXED, 3, 18), _Batch(Phase.MIXED, 5, 22)]
    batches += [_Batch(Phase.DECODE, 4, 4) for _ in range(6)]
    out = run_to_completion(_Engine(batches))
    assert out["steps"] == 10 and out["seconds"] > 0
    assert out["prefill"]["steps"] == 1 and out["prefill"]["mean_tokens"] == 40 and out["prefill"]["mean_rows"] == 2
    assert out["mixed"]["steps"] == 2 and out["mixed"]["mean_tokens"] == 20 and out["mixed"]["mean_rows"] == 4
    assert out["decode"]["steps"] == 6 and out["decode"]["mean_rows"] == 4 and out["decode"]["median_ms"] >= 0
    assert out["decode"]["median_ms"] <= out["decode"]["mean_ms"] * 6
    stopped = run_to_completion(_Engine(list(itertools.repeat(_Batch(Phase.DECODE, 1, 1), 50))), max_steps=7)
    assert stopped["steps"] == 7 and stopped["decode"]["steps"] == 7 and stopped["mixed"] == {"steps": 0}
