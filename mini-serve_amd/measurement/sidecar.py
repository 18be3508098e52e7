"""The record that stands beside a measured number: device, clocks, power and temperature while it was
taken, software versions, the commit. The reference writes such a sidecar beside every row of its
results and warms up until the clock has settled (bench/sidecar.py:117-260, bench/offline.py:449-528);
here the GPU is read through torch's device-management calls (AMD SMI underneath), and whatever does
not answer is recorded as None rather than guessed."""

from __future__ import annotations

import threading
import time


def sample_gpu(device: int = 0) -> dict:
    """One reading of the GPU: time, shader clock (MHz), power (torch.cuda.power_draw's milliwatts / 1000),
    temperature (C), utilisation (%), each as torch's device-management calls report them."""
    import torch

    out = {"t": time.monotonic()}
    for key, fn, scale in (("sclk_mhz", "clock_rate", 1.0), ("power_w", "power_draw", 1e-3), ("temp_c", "temperature", 1.0),
                           ("util_pct", "utilization", 1.0)):
        try:
            out[key] = round(float(getattr(torch.cuda, fn)(device)) * scale, 1)
        except Exception:  # noqa: BLE001  (the management library is missing or refuses: recorded as unknown)
            out[key] = None
    return out


class GpuSampler:
    """Reads the GPU every ``interval_s`` seconds in a background thread while it is loaded."""

    def __init__(self, device: int = 0, interval_s: float = 0.1):
        self.device, self.interval_s = device, interval_s
        self.samples: list[dict] = []
        self._stop = threading.Event()
        self._lock = threading.Lock()
        self._thread = None

    def __enter__(self):
        self._stop.clear()
        self._thread = threading.Thread(target=self._run, daemon=True, name="gpu-sampler")
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()
        return False

    def _run(self):
        while not self._stop.is_set():
            s = sample_gpu(self.device)
            with self._lock:
                self.samples.append(s)
            self._stop.wait(self.interval_s)

    def sample_now(self) -> float:
        """Take one reading right away (the edges of a timed window); returns its time."""
        s = sample_gpu(self.device)
        with self._lock:
            self.samples.append(s)
        return s["t"]

    def snapshot(self) -> list[dict]:
        with self._lock:
            return sorted(self.samples, key=lambda x: x["t"])

    def settled(self, window: int = 4, tol: float = 0.02):
        """Whether the mean clock of the last ``window`` readings is within ``tol`` of the ``window``
        before them (the reference's rule, bench/sidecar.py:187-196); None when the clock cannot be read."""
        clocks = [s["sclk_mhz"] for s in self.snapshot() if s["sclk_mhz"] is not None]
        if len(clocks) < 2 * window:
            return None
        earlier = sum(clocks[-2 * window : -window]) / window
        recent = sum(clocks[-window:]) / window
        return bool(recent > 0 and abs(recent - earlier) <= tol * recent)

    def summary(self, since: float | None = None, until: float | None = None) -> dict:
        s = [x for x in self.snapshot() if (since is None or x["t"] >= since) and (until is None or x["t"] <= until)]
        out = {"samples": len(s)}
        for key in ("sclk_mhz", "power_w", "temp_c"):
            vals = [x[key] for x in s if x[key] is not None]
            out[key] = None if not vals else {"min": min(vals), "max": max(vals), "mean": round(sum(vals) / len(vals), 1)}
        return out


def sidecar(engine=None) -> dict:
    """Runtime description, one idle reading of the GPU, and the engine's effective configuration."""
    from ..engine.describe import engine_description, runtime_description

    out = {"runtime": runtime_description(), "gpu_now": {k: v for k, v in sample_gpu().items() if k != "t"}}
    if engine is not None:
        out["engine"] = engine_description(engine)
    return out
