"""Hand-written HIP kernels for gfx950 and their Python entry points."""
