"""What a measurement needs beside the engine: the record of the conditions it ran under (sidecar),
and range markers that let a profiler keep to the measured steps."""

from .markers import measured_region, mark
from .sidecar import GpuSampler, sample_gpu, sidecar

__all__ = ["GpuSampler", "sample_gpu", "sidecar", "measured_region", "mark"]
