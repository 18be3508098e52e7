"""Interfaces of the parts a layer is put together from.

A part is built from a ``PartSpec`` (its sizes and constants) and a ``Runtime`` (compute dtype,
device, kernels); it declares the tensors it needs under its own prefix and receives exactly
those. No part knows which model it is in. The kinds:

* ``Norm``            ``forward(x_f32, rows=None, add=None) -> y``  (residual stream in, compute dtype out)
* ``PositionEncoding`` ``rotation(batch) -> Rotation | None``       (what a mixer's q/k are turned by in this step)
* ``Mixer``           ``forward(x, batch, cache, state, residual) -> pending`` (``state``: name -> tensor)
* ``FeedForward``     ``forward(x, residual) -> pending``
* ``Block``           ``forward(residual, batch, cache, state, pending) -> pending`` (where norms and sums sit)
* ``Embedding``       ``forward(token_ids) -> residual``            (float32 ``[T, width]``)
* ``Head``            ``forward(x) -> logits``                      (float32 ``[rows, vocab]``)

The residual stream is float32 in every compute dtype: sums of layer outputs are never rounded
to bfloat16. Mixers and feed-forwards do not return their output: they either add it into
``residual`` themselves (a matrix product can do that in its epilogue) and return None, or return a
*pending* sum (``ops.SplitSum``: partial sums that still have to be added to ``residual``). Whoever
reads the residual stream next takes the pending sum along: a norm adds it while it normalises
(``add=``), anything else calls ``ops.add_pending`` first.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import TYPE_CHECKING, Any, Mapping

from ..config.spec import PartSpec

if TYPE_CHECKING:  # pragma: no cover
    import torch


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part expects in the checkpoint. ``kind``: ``"float"`` tensors follow the compute
    dtype (a tensor stored in 32-bit stays 32-bit); ``"int"`` tables are kept as int32.

    ``init`` says how the random-weights mode draws it: ``"normal"`` N(0, std) (matrices, embeddings),
    ``"ones"`` a scale around one (norm weights: all one, or uniform in the range the caller gives),
    ``"uniform"`` U(-std, std), ``"zeros"`` (a bias that starts switched off); integer tables are
    drawn uniformly from ``[0, high)``."""

    shape: tuple[int, ...]
    kind: str = "float"
    init: str = "normal"
    high: int | None = None

    def __post_init__(self):
        if self.kind not in ("float", "int"):
            raise ValueError(f"unknown tensor kind {self.kind!r}")
        if self.kind == "float" and self.init not in ("normal", "ones", "uniform", "zeros"):
            raise ValueError(f"unknown init {self.init!r}")
        if self.kind == "int" and (self.high is None or self.high < 1):
            raise ValueError("an integer table needs ``high``: its entries are drawn from [0, high)")


@dataclass(frozen=True)
class CachePlane:
    """One thing a mixer keeps per token in the paged cache: ``heads`` vectors of ``width`` elements.
    Within a page a plane lies ``[page_size, width]`` per head, or, ``token_minor``, ``[width,
    page_size]`` (the tokens of one element side by side: what a product over tokens reads)."""

    name: str
    heads: int
    width: int
    token_minor: bool = False


@dataclass(frozen=True)
class KVNeed:
    """What a mixer keeps per token, as a list of planes (keys and values of equal or different
    widths, one latent vector, ...). ``window == 0`` keeps every token, ``window > 0`` only the last
    ``window`` (older pages may be given back)."""

    planes: tuple[CachePlane, ...]
    window: int = 0

    def __post_init__(self):
        names = [p.name for p in self.planes]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"cache planes need distinct names, got {names}")

    @classmethod
    def keys_values(cls, num_kv_heads: int, head_dim: int, window: int = 0) -> "KVNeed":
        """Keys ``[page_size, head_dim]`` and values ``[head_dim, page_size]`` per KV head: what the
        attention kernels read."""
        return cls((CachePlane("k", num_kv_heads, head_dim), CachePlane("v", num_kv_heads, head_dim, token_minor=True)), window)

    @property
    def elements_per_token(self) -> int:
        return sum(p.heads * p.width for p in self.planes)


@dataclass(frozen=True)
class StateTensor:
    """One tensor of a mixer's per-request state: shape per request and torch dtype name."""

    name: str
    shape: tuple[int, ...]
    dtype: str = "float32"


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size a mixer keeps: one or several named tensors."""

    tensors: tuple[StateTensor, ...]

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"state tensors need distinct names, got {names}")

    @classmethod
    def single(cls, shape, dtype: str = "float32", name: str = "state") -> "StateNeed":
        return cls((StateTensor(name, tuple(shape), dtype),))


@dataclass(frozen=True)
class Rotation:
    """Rotary position encoding as a mixer's kernels need it: the first ``dim`` elements of each
    head are turned in pairs by the step's angles, whose cosines and sines are the two halves of a row
    of ``table`` (pair ``j`` by angle ``j``). ``pairing`` says which elements make pair ``j``:
    ``"halves"`` (j, j + dim/2), ``"adjacent"`` (2j, 2j + 1); the kernels name the pairings they know
    (``ops.ROTATION_PAIRINGS``) and refuse any other."""

    dim: int
    table: Any  # float32 device tensor [tokens of the step, dim]: cosines, then sines
    pairing: str = "halves"


class Runtime:
    """What every part is built with: the compute dtype, the device and the kernel library."""

    def __init__(self, dtype, device, ops):
        self.dtype = dtype  # torch.float32 or torch.bfloat16
        self.device = device
        self.ops = ops


class Part:
    """Base of all parts. Subclasses override ``tensors`` (static: needs no device) and ``bind``."""

    kind: str = ""

    def __init__(self, spec: PartSpec, rt: Runtime | None):
        self.spec = spec
        self.rt = rt

    @classmethod
    def tensors(cls, spec: PartSpec) -> dict[str, TensorSpec]:
        """Checkpoint tensors of this part, named relative to the layer prefix (or absolutely
        for parts outside layers)."""
        return {}

    @classmethod
    def aliases(cls, spec: PartSpec) -> dict[str, str]:
        """Tensors this part reads that are stored under another name: ``{name: source}``, ``name``
        relative like the names of ``tensors`` (and never among them), ``source`` the full name of a
        tensor some part declares. The part receives the source's tensor under ``name`` (the same memory,
        no copy); a tensor stored under ``name`` itself is a duplicate and is dropped."""
        return {}

    def bind(self, tensors: Mapping[str, "torch.Tensor"]) -> None:
        """Receive the tensors declared by ``tensors`` and ``aliases`` (same names), already on the device."""

    def parameters_bytes(self) -> int:
        """Bytes of weights a decode step reads from this part (for the bandwidth model)."""
        return 0

    def flops(self, rows) -> int:
        """Floating-point operations of one pass over ``rows``: a list of ``(new tokens, tokens already in
        the cache)`` per request; a multiply-add counts two. What a measurement divides by its time."""
        return 0


class Norm(Part):
    def forward(self, x, rows=None, add=None):
        """Normalise rows of the float32 ``x`` plus ``add`` (a pending sum). Without ``rows``, ``x`` is
        also brought up to date in place; with ``rows`` the stream is not read again and stays as it is."""
        raise NotImplementedError


class PositionEncoding(Part):
    def rotation(self, batch) -> Rotation | None:
        """What the mixer turns q and k by in this step. Anything computed from the step's positions
        alone belongs in ``batch.memo`` (a dict that lives as long as the step), under a key that names
        the encoding's constants, so that layers with equal constants compute it once."""
        return None


class Mixer(Part):
    def kv_need(self) -> KVNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    def forward(self, x, batch, cache, state, residual):
        """Add the mixer's output to ``residual``, or return it as a pending sum."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x, residual):
        """Add the feed-forward's output to ``residual``, or return it as a pending sum."""
        raise NotImplementedError


class Block(Part):
    def __init__(self, spec: PartSpec, rt, mixer: Mixer, feed_forward: FeedForward):
        super().__init__(spec, rt)
        self.mixer = mixer
        self.feed_forward = feed_forward

    def forward(self, residual, batch, cache, state, pending=None):
        """Run the layer on ``residual`` (to which ``pending`` still has to be added); returns what is
        pending afterwards."""
        raise NotImplementedError


class Embedding(Part):
    def forward(self, token_ids):
        raise NotImplementedError


class Head(Part):
    def forward(self, x):
        raise NotImplementedError
