"""What a measurement needs beside the engine: the record of the conditions it ran under (sidecar),
and range markers that let a profiler keep to the measured steps."""

from .markers import measured_region, mark
from .sidecar import GpuMonitor, gpu_now, sidecar

__all__ = ["GpuMonitor", "gpu_now", "sidecar", "measured_region", "mark"]
