"""How close the engine must be to the plain implementation. Fixed from the arithmetic, never
widened to pass.

float32: unit roundoff 2^-24 = 6e-8. A logit is the end of a chain of a few hundred sums per layer;
with every sum in float32 the error stays below about 1e-5 of the logits' scale. The bound allows
1e-4 of the largest absolute logit.

bfloat16: activations between kernels are rounded to 8 significant bits (half-ulp 2^-9 = 2e-3), about
ten roundings per layer on the path of a value, accumulating like a random walk; the residual sum
and all reductions stay in float32. The bound allows 5e-2 of the largest absolute logit at the worst
element and 1.2e-2 root-mean-square. A formula mistake (norm in the wrong place, wrong pairing,
a key too many) moves logits by the order of their scale.
"""

import numpy as np

F32_REL = 1e-4
BF16_REL_MAX = 5e-2
BF16_REL_RMS = 1.2e-2


def check_logits(got: np.ndarray, want: np.ndarray, dtype: str, what: str = "") -> None:
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    scale = float(np.abs(want).max())
    diff = np.abs(got.astype(np.float64) - want)
    worst = float(diff.max())
    if dtype == "float32":
        assert worst <= F32_REL * scale, f"{what}: float32 max |diff| {worst:.3e} > {F32_REL * scale:.3e} (scale {scale:.3f})"
    else:
        rms = float(np.sqrt((diff**2).mean()))
        assert worst <= BF16_REL_MAX * scale, f"{what}: bfloat16 max |diff| {worst:.3e} > {BF16_REL_MAX * scale:.3e}"
        assert rms <= BF16_REL_RMS * scale, f"{what}: bfloat16 rms diff {rms:.3e} > {BF16_REL_RMS * scale:.3e}"
