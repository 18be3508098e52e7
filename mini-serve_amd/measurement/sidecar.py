"""The record that stands beside a measured number: what the GPU's clocks, power and temperatures did
while it was taken, what limits it ran under, and the software underneath. The reference writes such a
record beside every row of its results and warms up until the clock has settled
(bench/sidecar.py:117-260, bench/offline.py:449-528). Here the device is read through AMD's management
library (``amdsmi``, one metrics call of a third of a millisecond per reading); readings are rows of one
numpy array, unknown values are NaN and are reported as None, never as a guess.

The firmware refreshes the figures it hands out about once a second (measured: every source of the
library shows the same values for a second, then the next), and stamps each refresh with its own clock.
Polling faster finds a refresh sooner but learns nothing more, so everything below counts *refreshes*:
the first reading of each firmware time stamp. A statement about the clock therefore takes seconds, not
tenths: the first refresh after a load begins still mixes idle and load, the two after it can agree.

``GpuMonitor`` keeps a ring of readings filled by a background thread. ``window(since, until)`` condenses
the refreshes of a time span; ``steady()`` says whether the shader clock has stopped moving;
``warm_until_steady(work, least_s, most_s)`` runs ``work()`` again and again until it has;
``hold_until_refresh(work, most_s)`` keeps the load up until the firmware has reported on it once more.
"""

from __future__ import annotations

import threading
import time

import numpy as np

# One reading: monotonic time, shader and memory clock (MHz), socket power (W), hot-spot and memory
# temperature (C), shader and memory-controller activity (%), and the firmware's time stamp of the refresh
# the figures come from (its own units; only equality is used).
COLUMNS = ("t", "sclk_mhz", "mclk_mhz", "power_w", "temp_c", "mem_temp_c", "busy_pct", "mem_busy_pct", "refresh")
REPORTED = COLUMNS[1:-1]  # what summaries name
_METRIC_KEYS = {"refresh": "firmware_timestamp", "sclk_mhz": "current_gfxclk", "mclk_mhz": "current_uclk", "power_w": "current_socket_power",
                "temp_c": "temperature_hotspot", "mem_temp_c": "temperature_mem", "busy_pct": "average_gfx_activity",
                "mem_busy_pct": "average_umc_activity"}
_NAN = float("nan")


def _number(v) -> float:
    """The management library writes "N/A" where a figure does not exist on this device."""
    return float(v) if isinstance(v, (int, float)) and not isinstance(v, bool) else _NAN


class _Device:
    """The management library's handle of one GPU, or nothing where the library or the device is absent."""

    def __init__(self, index: int):
        self.smi = self.handle = None
        try:
            import amdsmi

            amdsmi.amdsmi_init()
            handles = amdsmi.amdsmi_get_processor_handles()
            if index < len(handles):
                self.smi, self.handle = amdsmi, handles[index]
        except Exception:  # noqa: BLE001  (no library, no driver, no permission: every reading is unknown)
            pass

    def read(self) -> list[float]:
        row = [time.monotonic()] + [_NAN] * (len(COLUMNS) - 1)
        if self.handle is not None:
            try:
                m = self.smi.amdsmi_get_gpu_metrics_info(self.handle)
                for i, col in enumerate(COLUMNS[1:], 1):
                    row[i] = _number(m.get(_METRIC_KEYS[col]))
            except Exception:  # noqa: BLE001
                pass
        return row

    def limits(self) -> dict:
        """What bounds the clocks: the socket's power limit (W) and the shader and memory clock ranges (MHz)."""
        out = {"power_limit_w": None, "sclk_range_mhz": None, "mclk_range_mhz": None}
        if self.handle is None:
            return out
        smi = self.smi
        try:
            cap = _number(smi.amdsmi_get_power_cap_info(self.handle).get("power_cap"))  # microwatts
            out["power_limit_w"] = None if cap != cap else round(cap / 1e6, 1)
        except Exception:  # noqa: BLE001
            pass
        for key, kind in (("sclk_range_mhz", "GFX"), ("mclk_range_mhz", "MEM")):
            try:
                c = smi.amdsmi_get_clock_info(self.handle, getattr(smi.AmdSmiClkType, kind))
                lo, hi = _number(c.get("min_clk")), _number(c.get("max_clk"))
                out[key] = None if lo != lo or hi != hi else [lo, hi]
            except Exception:  # noqa: BLE001
                pass
        return out

    def throttle_counters(self) -> dict | None:
        """The firmware's running counts of time spent held back, by cause (the call takes 0.1 s: made at the
        edges of a run, never per reading)."""
        if self.handle is None:
            return None
        try:
            v = self.smi.amdsmi_get_violation_status(self.handle)
        except Exception:  # noqa: BLE001
            return None
        keys = {"all": "acc_counter", "power": "acc_ppt_pwr", "socket_temperature": "acc_socket_thrm",
                "hot_spot": "acc_prochot_thrm", "regulator_temperature": "acc_vr_thrm", "memory_temperature": "acc_hbm_thrm"}
        return {name: _number(v.get(k)) for name, k in keys.items()}


def throttled_share(before: dict | None, after: dict | None) -> dict | None:
    """Share of the firmware's counting intervals between two ``throttle_counters`` in which each cause held
    the device back (None where a counter is missing or did not run)."""
    if not before or not after:
        return None
    ticks = after["all"] - before["all"]
    if not ticks > 0:
        return None
    out = {}
    for name in before:
        if name != "all":
            d = after[name] - before[name]
            out[name] = None if d != d else round(d / ticks, 4)
    return out


class GpuMonitor:
    """Readings of one GPU in a ring of ``capacity`` rows, taken every ``interval_s`` seconds by a thread
    between ``start()`` and ``stop()`` (or inside a ``with`` block), and on demand by ``read_now()``."""

    def __init__(self, device: int = 0, interval_s: float = 0.05, capacity: int = 1 << 16):
        self.interval_s = interval_s
        self._dev = _Device(device)
        self._rows = np.full((capacity, len(COLUMNS)), np.nan)
        self._count = 0
        self._guard = threading.Lock()
        self._halt = threading.Event()
        self._worker = None
        self._throttle_at_start = None

    # -- collecting

    def _append(self, row) -> None:
        with self._guard:
            self._rows[self._count % len(self._rows)] = row
            self._count += 1

    def read_now(self) -> float:
        """One reading right away (the edges of a timed span); returns its time."""
        row = self._dev.read()
        self._append(row)
        return row[0]

    def load(self, rows) -> None:
        """Replace the ring's content by ``rows`` (sequences in ``COLUMNS`` order; None = unknown)."""
        with self._guard:
            self._rows[:] = np.nan
            self._count = 0
        for r in rows:
            self._append([_NAN if v is None else float(v) for v in r])

    def _loop(self) -> None:
        while not self._halt.is_set():
            self._append(self._dev.read())
            self._halt.wait(self.interval_s)

    def start(self) -> "GpuMonitor":
        self._throttle_at_start = self._dev.throttle_counters()
        self._halt.clear()
        self._worker = threading.Thread(target=self._loop, daemon=True, name="miniserve-gpu-monitor")
        self._worker.start()
        return self

    def stop(self) -> None:
        if self._worker is not None:
            self._halt.set()
            self._worker.join()
            self._worker = None

    __enter__ = start

    def __exit__(self, *exc) -> bool:
        self.stop()
        return False

    # -- reading back

    def readings(self) -> np.ndarray:
        """The rows held, oldest first (a copy)."""
        with self._guard:
            n, cap = self._count, len(self._rows)
            rows = self._rows[:n].copy() if n <= cap else np.roll(self._rows, -(n % cap), axis=0).copy()
        return rows[np.argsort(rows[:, 0], kind="stable")]

    def refreshes(self, since: float | None = None, until: float | None = None) -> np.ndarray:
        """The first reading of every refresh of the firmware's figures within the span (every reading,
        where the firmware's time stamp is unknown)."""
        rows = self.readings()
        stamp = rows[:, COLUMNS.index("refresh")]
        if len(rows) and not np.isnan(stamp).all():
            rows = rows[np.concatenate(([True], stamp[1:] != stamp[:-1])) & ~np.isnan(stamp)]
        t = rows[:, 0]
        return rows[(t >= (-np.inf if since is None else since)) & (t <= (np.inf if until is None else until))]

    def column(self, name: str) -> np.ndarray:
        return self.readings()[:, COLUMNS.index(name)]

    def window(self, since: float | None = None, until: float | None = None) -> dict:
        """Count of refreshes, and per figure lowest, highest and mean of the known ones, of the span."""
        rows = self.refreshes(since, until)
        out = {"samples": int(len(rows))}
        for col in REPORTED:
            v = rows[:, COLUMNS.index(col)]
            known = v[~np.isnan(v)]
            out[col] = None if known.size == 0 else {"min": float(known.min()), "max": float(known.max()),
                                                     "mean": round(float(known.mean()), 1)}
        return out

    @staticmethod
    def _agree(clock: np.ndarray, readings: int, tolerance: float) -> bool | None:
        clock = clock[~np.isnan(clock)]
        if clock.size < 2 * readings:
            return None
        latest, earlier = clock[-readings:].mean(), clock[-2 * readings : -readings].mean()
        return bool(latest > 0 and abs(latest - earlier) <= tolerance * latest)

    def steady(self, readings: int = 1, tolerance: float = 0.02, since: float | None = None) -> bool | None:
        """Whether the shader clock has stopped moving: the mean of its latest ``readings`` refreshes lies
        within ``tolerance`` of the mean of the ``readings`` before them (the reference's rule,
        bench/sidecar.py:187-196, over refreshes instead of samples). None while fewer than twice
        ``readings`` are known."""
        return self._agree(self.refreshes(since)[:, COLUMNS.index("sclk_mhz")], readings, tolerance)

    def warm_until_steady(self, work, least_s: float, most_s: float, readings: int = 1, tolerance: float = 0.02) -> dict:
        """Call ``work()`` (which must leave the device busy and return when its work is done) until at
        least ``least_s`` have passed and the clock is steady, or ``most_s`` have passed. Of the refreshes
        since the call began the first does not count: it mixes what came before with the load. Returns
        what happened: calls, seconds, refreshes seen, and ``steady`` (None when the clock could not be read
        often enough to tell)."""
        began = time.monotonic()
        calls, verdict, seen = 0, None, 0
        while True:
            work()
            calls += 1
            spent = time.monotonic() - began
            if spent < least_s:
                continue
            clock = self.refreshes(began)[1:, COLUMNS.index("sclk_mhz")]
            seen = int(clock.size)
            verdict = self._agree(clock, readings, tolerance)
            if verdict or spent >= most_s:
                return {"calls": calls, "seconds": round(spent, 3), "refreshes": seen, "steady": verdict}

    def hold_until_refresh(self, work, most_s: float = 1.5) -> bool:
        """Call ``work()`` until the firmware has refreshed its figures once more (so that a span too short
        to hold a refresh is followed by one taken under the same load), or ``most_s`` have passed."""
        began = time.monotonic()
        before = len(self.refreshes())
        while time.monotonic() - began < most_s:
            work()
            if len(self.refreshes()) > before:
                return True
        return False

    def conditions(self) -> dict:
        """What the run was bounded by: limits, and the share of time the firmware held the device back
        since ``start()``."""
        out = self._dev.limits()
        out["throttled_share"] = throttled_share(self._throttle_at_start, self._dev.throttle_counters())
        return out


def gpu_now(device: int = 0) -> dict:
    """One reading as a dictionary (None = unknown), without its time."""
    row = _Device(device).read()
    return {c: (None if v != v else v) for c, v in zip(COLUMNS, row) if c in REPORTED}


def sidecar(engine=None) -> dict:
    """The software and device record, one reading of the GPU, and the engine's effective configuration."""
    from ..engine.describe import engine_description, runtime_description

    out = {"runtime": runtime_description(), "gpu_now": gpu_now()}
    if engine is not None:
        out["engine"] = engine_description(engine)
    return out
