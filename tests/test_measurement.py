"""The measurement helpers without a GPU: the rule that says when the clock has settled, the summary of
the readings inside a timed window, step times kept apart by the kind of step, and markers that are
no-ops outside a profiler."""

from __future__ import annotations

import itertools

import pytest

from miniserve_amd.measurement import GpuSampler, mark, measured_region, sample_gpu
from miniserve_amd.measurement.offline import run_to_completion


def readings(clocks, power=None, t0=100.0, dt=0.1):
    return [{"t": t0 + i * dt, "sclk_mhz": c, "power_w": None if power is None else power[i], "temp_c": 40.0, "util_pct": 99.0}
            for i, c in enumerate(clocks)]


def test_a_reading_without_a_gpu_says_unknown_not_zero():
    s = sample_gpu()
    assert set(s) == {"t", "sclk_mhz", "power_w", "temp_c", "util_pct"} and s["t"] > 0
    assert all(s[k] is None or s[k] >= 0 for k in ("sclk_mhz", "power_w", "temp_c", "util_pct"))


def test_the_clock_has_settled_when_two_windows_agree():
    g = GpuSampler()
    g.samples = readings([2400, 2400, 2400])
    assert g.settled() is None, "fewer than two windows of readings decide nothing"
    g.samples = readings([2400, 2300, 2100, 1900, 1750, 1720, 1700, 1700])  # still falling: 2175 against 1717
    assert g.settled() is False
    g.samples = readings([2400, 2300, 2100, 1900, 1710, 1700, 1705, 1695, 1700, 1702, 1698, 1700])
    assert g.settled() is True  # the last four against the four before them: within 2 %
    g.samples = readings([1700] * 4 + [1740] * 4)  # 2.3 % apart
    assert g.settled() is False and g.settled(tol=0.03) is True
    g.samples = readings([None] * 20)
    assert g.settled() is None, "a clock that cannot be read settles nothing"
    g.samples = readings([1700, None, 1700, 1700, None, 1700, 1700, 1700, 1700, 1700])  # unknown readings are skipped
    assert g.settled() is True


def test_the_summary_covers_the_timed_window_only():
    g = GpuSampler()
    g.samples = readings([2400, 2000, 1800, 1700, 1700, 2400], power=[100, 600, 900, 1000, 1000, 120])
    whole = g.summary()
    assert whole["samples"] == 6 and whole["sclk_mhz"] == {"min": 1700, "max": 2400, "mean": 2000.0}
    inside = g.summary(since=100.15, until=100.45)  # readings 2, 3 and 4
    assert inside["samples"] == 3 and inside["sclk_mhz"] == {"min": 1700, "max": 1800, "mean": 1733.3}
    assert inside["power_w"] == {"min": 900, "max": 1000, "mean": 966.7}
    assert g.summary(since=200.0) == {"samples": 0, "sclk_mhz": None, "power_w": None, "temp_c": None}
    g.samples = readings([None, None])
    assert g.summary()["sclk_mhz"] is None and g.summary()["temp_c"]["mean"] == 40.0


def test_the_sampler_thread_collects_and_stops():
    with GpuSampler(interval_s=0.01) as g:
        first = g.sample_now()
        while len(g.snapshot()) < 3:
            pass
    n = len(g.snapshot())
    assert n >= 3 and first in [s["t"] for s in g.snapshot()]
    times = [s["t"] for s in g.snapshot()]
    assert times == sorted(times)
    assert len(g.snapshot()) == n, "no reading after the with block has ended"


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
