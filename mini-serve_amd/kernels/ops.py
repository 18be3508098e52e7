"""The kernel library as Python calls: every function checks shapes, dtypes and contiguity on the
host, then launches hand-written HIP kernels on torch's current stream. There is no fallback:
without a GPU or without the built library these calls raise.

Tensors are torch tensors used as plain device buffers; no torch operator computes anything here.
"""

from __future__ import annotations

import ctypes

import torch

from . import build

_lib = None

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32
_c_void, _c_int, _c_float, _c_ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong

_ERRORS = {1: "bad argument", 2: "unsupported size", 3: "kernel launch failed"}

_SIGNATURES = {
    "ms_embed": [_c_void, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void],
    "ms_feed_tokens": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
    "ms_rmsnorm": [_c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_int, _c_int, _c_float, _c_void, _c_int, _c_ll, _c_void],
    "ms_act_mul": [_c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_act_mul_parts": [_c_void, _c_int, _c_ll, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gemm_bf16_gated": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_cast": [_c_void, _c_int, _c_void, _c_int, _c_ll, _c_void],
    "ms_rope_table": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
    "ms_qk_norm_rope_store": [_c_void, _c_void, _c_int, _c_ll, _c_void, _c_int, _c_int, _c_void, _c_void, _c_void,
                              _c_int, _c_float, _c_void, _c_int, _c_int, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int,
                              _c_void],
    "ms_gemm_f32": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gemm_bf16": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gemm_bf16_tile_splits": [_c_int, _c_int, _c_int],
    "ms_gemm_bf16_tile_shape": [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int],
    "ms_gemm_bf16_small": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_gemm_bf16_small_splits": [_c_int, _c_int, _c_int],
    "ms_gemm_bf16_small_tile_cols": [_c_int, _c_int],
    "ms_splitk_reduce": [_c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_paged_attention_generic": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void,
                                   _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void],
    "ms_attention_decode_bf16": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void,
                                 _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void],
    "ms_attention_decode_fused_bf16": [_c_void, _c_int, _c_ll, _c_void, _c_void, _c_float, _c_void, _c_int, _c_int, _c_void, _c_void,
                                       _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int,
                                       _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_void],
    "ms_attention_merge_project": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    "ms_attention_merge_project_splits": [_c_int, _c_int, _c_int, _c_int, _c_int],
    "ms_attention_prefill_bf16": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_int, _c_int,
                                  _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void],
    "ms_attention_prefill_parts_bf16": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void,
                                        _c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_float,
                                        _c_void],
    "ms_attention_prefill_tile_tokens": [_c_int, _c_int],
    "ms_sample_rows": [_c_void, _c_int, _c_int, _c_ll, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void],
    "ms_sample_scratch_bytes": [_c_int],
    "ms_sample_rows_static": [_c_void, _c_int, _c_int, _c_ll, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void],
    "ms_sample_rows_static_max_rows": [],
    "ms_measure_read": [_c_void, _c_ll, _c_int, _c_void, _c_void],
    "ms_measure_copy": [_c_void, _c_void, _c_ll, _c_int, _c_void],
}


class KernelLibraryMissing(RuntimeError):
    pass


def library():
    """The loaded kernel library; built first if no build of the current sources exists."""
    global _lib
    if _lib is None:
        if not torch.cuda.is_available():
            raise KernelLibraryMissing("no GPU is visible: the engine runs on HIP kernels only and has no CPU fallback")
        try:
            path = build.build_kernels()
            lib = ctypes.CDLL(str(path))
        except Exception as e:  # noqa: BLE001
            raise KernelLibraryMissing(f"the HIP kernel library could not be built or loaded: {e}") from e
        for name, args in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = _c_int
        _lib = lib
    return _lib


def library_path() -> str:
    return str(build.build_kernels())


_pinned_stream: int | None = None


def _stream() -> int:
    return _pinned_stream if _pinned_stream is not None else torch.cuda.current_stream().cuda_stream


class stream_scope:
    """Looks the current HIP stream up once for all kernel launches inside the ``with`` block (the
    lookup costs several microseconds, a model pass makes hundreds). The stream must not be switched
    inside the block."""

    def __enter__(self):
        global _pinned_stream
        self._before = _pinned_stream
        _pinned_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self._before
        return False


def _check(code: int, what: str) -> None:
    if code:
        raise RuntimeError(f"{what}: {_ERRORS.get(code, code)}")


def _dev(t: torch.Tensor, name: str, dtypes, ndim: int | None = None) -> None:
    """A contiguous tensor on the GPU of one of ``dtypes`` (and of ``ndim`` dimensions). A model pass
    makes hundreds of these checks: what is right passes in three calls; what is wrong is looked at
    again, slowly, for the message."""
    try:
        if t.is_cuda and t.is_contiguous() and (t.dtype is dtypes or t.dtype in dtypes) and (ndim is None or t.dim() == ndim):
            return
    except (AttributeError, TypeError):
        pass
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name} must be a tensor on the GPU")
    if t.dtype not in (dtypes if isinstance(dtypes, tuple) else (dtypes,)):
        raise TypeError(f"{name} has dtype {t.dtype}, expected {dtypes}")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name} has {t.dim()} dimensions, expected {ndim}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


class SplitSum:
    """A matrix that exists only as partial sums: its value is ``parts.sum(0)`` (float32
    ``[splits, M, N]``, to be added in ascending split order). The small-M matrix product leaves its
    result in this form so that the kernel that consumes it does the summing and no kernel of its own
    is spent on it. ``accumulate`` marks a sum that still has to be added to the residual stream."""

    __slots__ = ("parts",)

    def __init__(self, parts: torch.Tensor):
        self.parts = parts

    @property
    def shape(self):
        return tuple(self.parts.shape[1:])

    @property
    def splits(self) -> int:
        return self.parts.shape[0]

    @property
    def stride(self) -> int:
        return self.parts.shape[1] * self.parts.shape[2]


def _check_split(v: SplitSum, name: str, shape) -> None:
    _dev(v.parts, name, F32, 3)
    if v.shape != tuple(shape):
        raise ValueError(f"{name} holds partial sums of a {v.shape} matrix, expected {tuple(shape)}")


# ------------------------------------------------------------------------------------- elementwise


def embed(token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """``float32 [T, width]`` rows of ``table`` (float32 or bfloat16). Ids must be in range (the
    caller checks them on the host before they are uploaded)."""
    _dev(token_ids, "token_ids", I32, 1)
    _dev(table, "table", (F32, BF16), 2)
    out = torch.empty((token_ids.shape[0], table.shape[1]), dtype=F32, device=table.device)
    _check(library().ms_embed(token_ids.data_ptr(), table.data_ptr(), int(table.dtype == BF16), out.data_ptr(),
                              token_ids.shape[0], table.shape[1], _stream()), "embed")
    return out


def feed_tokens(token_ids: torch.Tensor, row_start: torch.Tensor | None, feed: torch.Tensor, source: torch.Tensor) -> None:
    """In place: the last token of row ``i`` of ``token_ids`` becomes ``source[feed[i]]`` where
    ``feed[i] >= 0``. ``row_start``: ``rows + 1`` offsets of the rows in ``token_ids`` (None: one token
    per row). For tokens that were sampled on the device and not yet read back."""
    _dev(token_ids, "token_ids", I32, 1)
    _dev(feed, "feed", I32, 1)
    _dev(source, "source", I32, 1)
    rows = feed.shape[0]
    if row_start is not None:
        _dev(row_start, "row_start", I32, 1)
        if row_start.shape[0] != rows + 1:
            raise ValueError("row_start must hold one offset more than there are rows")
    elif token_ids.shape[0] < rows:
        raise ValueError("fewer tokens than rows")
    _check(library().ms_feed_tokens(token_ids.data_ptr(), _ptr(row_start), feed.data_ptr(), source.data_ptr(), rows,
                                    source.shape[0], _stream()), "feed_tokens")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype, rows: torch.Tensor | None = None,
            add: SplitSum | None = None) -> torch.Tensor:
    """RMSNorm of the float32 rows of ``x`` (all, or those named by ``rows``). ``add``: a pending sum that
    is added to the rows first; without ``rows`` also into ``x`` itself (in place), with ``rows`` (which
    may name a row twice) ``x`` is left unchanged."""
    _dev(x, "x", F32, 2)
    _dev(weight, "weight", (F32, BF16), 1)
    if weight.shape[0] != x.shape[1]:
        raise ValueError(f"norm weight has {weight.shape[0]} elements for width {x.shape[1]}")
    if out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    n = x.shape[0]
    if rows is not None:
        _dev(rows, "rows", I32, 1)
        n = rows.shape[0]
    parts, splits, stride = None, 0, 0
    if add is not None:
        _check_split(add, "add", x.shape)
        parts, splits, stride = add.parts.data_ptr(), add.splits, add.stride
    out = torch.empty((n, x.shape[1]), dtype=out_dtype, device=x.device)
    _check(library().ms_rmsnorm(x.data_ptr(), weight.data_ptr(), int(weight.dtype == BF16), out.data_ptr(),
                                int(out_dtype == BF16), _ptr(rows), n, x.shape[1], float(eps), parts, splits, stride,
                                _stream()), "rmsnorm")
    return out


GATE_BLOCK = 16  # rows per run of gate / up rows in an interleaved gate-up weight


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``[2 I, K]`` with alternating runs of ``GATE_BLOCK`` gate rows and ``GATE_BLOCK`` up rows: the
    order in which the matrix kernels hold gate and up of one output in one lane. ``I`` must be a
    multiple of ``GATE_BLOCK``."""
    i, k = gate.shape
    if up.shape != gate.shape or i % GATE_BLOCK:
        raise ValueError(f"gate {tuple(gate.shape)} and up {tuple(up.shape)} cannot be interleaved in runs of {GATE_BLOCK}")
    both = torch.stack((gate.view(i // GATE_BLOCK, GATE_BLOCK, k), up.view(i // GATE_BLOCK, GATE_BLOCK, k)), dim=1)
    return both.reshape(2 * i, k).contiguous()


# Activations of the gated feed-forward and the numbers the kernels know them by (MS_ACT_* in csrc/common.h):
# silu(x) = x sigmoid(x); gelu_tanh(x) = x / 2 (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))).
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def _activation(name: str) -> int:
    try:
        return ACTIVATIONS[name]
    except KeyError:
        raise NotImplementedError(f"activation {name!r}: the kernels know {sorted(ACTIVATIONS)}") from None


def act_mul(gu, activation: str = "silu", out_dtype=None, block: int = 0) -> torch.Tensor:
    """``act(gate) * up`` for ``gu [T, 2 I]``, a tensor or a ``SplitSum`` (then ``out_dtype`` names the
    result's dtype). ``block == 0``: the row holds the ``I`` gates, then the ``I`` ups; ``block > 0``:
    alternating runs of ``block`` gates and ``block`` ups (see ``interleave_gate_up``)."""
    act = _activation(activation)
    if isinstance(gu, SplitSum):
        _dev(gu.parts, "gu", F32, 3)
        t, width = gu.shape
        if width % 2 or out_dtype not in (F32, BF16) or (block and (width // 2) % block):
            raise ValueError("gate/up partial sums need an even width (whole runs) and an output dtype")
        out = torch.empty((t, width // 2), dtype=out_dtype, device=gu.parts.device)
        for t0 in range(0, t, 32768):
            n = min(32768, t - t0)
            _check(library().ms_act_mul_parts(gu.parts[:, t0:].data_ptr(), gu.splits, gu.stride, out[t0:].data_ptr(),
                                              int(out_dtype == BF16), n, width // 2, int(block), act, _stream()), "act_mul")
        return out
    _dev(gu, "gu", (F32, BF16), 2)
    if gu.shape[1] % 2 or (block and (gu.shape[1] // 2) % block):
        raise ValueError("gate/up buffer needs an even width (whole runs)")
    inter = gu.shape[1] // 2
    out = torch.empty((gu.shape[0], inter), dtype=gu.dtype, device=gu.device)
    # grid.y carries the token index: split very long batches
    for t0 in range(0, gu.shape[0], 32768):
        n = min(32768, gu.shape[0] - t0)
        _check(library().ms_act_mul(gu[t0:].data_ptr(), out[t0:].data_ptr(), int(gu.dtype == BF16), n, inter, int(block), act,
                                    _stream()), "act_mul")
    return out


def gated_linear(x: torch.Tensor, gate_up: torch.Tensor, activation: str = "silu", out_dtype=None, block: int = 0):
    """``act(x gate^T) * (x up^T)`` for ``gate_up [2 I, K]`` laid out as ``act_mul`` describes. With
    interleaved bfloat16 weights the activation runs in the matrix kernel's epilogue where a kernel
    for the shape exists (few rows: no partial sums leave the kernel; many rows: the gate/up matrix is
    never written); otherwise the product and the activation are two kernels."""
    act = _activation(activation)
    _dev(x, "x", (F32, BF16), 2)
    _dev(gate_up, "gate_up", (F32, BF16), 2)
    m, k = x.shape
    if gate_up.shape[1] != k or gate_up.shape[0] % 2:
        raise ValueError(f"gated_linear: x is [{m}, {k}], gate_up is {tuple(gate_up.shape)}")
    inter = gate_up.shape[0] // 2
    if block == GATE_BLOCK and gate_up.dtype == BF16 and out_dtype == BF16 and m > 0:
        xa = cast(x, BF16)
        out = torch.empty((m, inter), dtype=BF16, device=x.device)
        rc = library().ms_gemm_bf16_gated(xa.data_ptr(), gate_up.data_ptr(), out.data_ptr(), m, inter, k, k, act, _stream())
        if rc == 0:
            return out
        if rc != 2:  # 2: no fused kernel for this shape
            _check(rc, "gemm_bf16_gated")
    gu = linear(x, gate_up, out_dtype=out_dtype, defer=True)
    return act_mul(gu, activation, out_dtype=out_dtype, block=block)


def cast(x: torch.Tensor, dtype) -> torch.Tensor:
    if x.dtype == dtype:
        return x
    _dev(x, "x", (F32, BF16))
    if dtype not in (F32, BF16):
        raise TypeError(f"unsupported dtype {dtype}")
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _check(library().ms_cast(x.data_ptr(), int(x.dtype == BF16), out.data_ptr(), int(dtype == BF16), x.numel(), _stream()),
           "cast")
    return out


# ------------------------------------------------------------------------------------- matrix products

SMALL_M = 64  # rows up to which the split-K weight-streaming kernel runs
MAX_STEP_TOKENS = 65535  # rows one launch of the matrix and elementwise kernels takes (a grid dimension)


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype=None, accumulate_into: torch.Tensor | None = None,
           defer: bool = False):
    """``x [M, K] @ weight [N, K]^T``. Either returns a new ``[M, N]`` tensor of ``out_dtype``, or adds
    the product into the float32 tensor ``accumulate_into`` (the residual stream) and returns None.
    The weight's dtype picks the arithmetic: float32 weights run the true 32-bit kernel (``x`` is
    widened first if needed), bfloat16 weights the matrix-core kernels with float32 accumulation.

    ``defer=True`` allows the result to come back as a ``SplitSum`` (partial sums that the consuming
    kernel adds up) where the small-M kernel produced it in that form; with ``accumulate_into`` the
    returned ``SplitSum`` is what still has to be added to that tensor."""
    _dev(x, "x", (F32, BF16), 2)
    _dev(weight, "weight", (F32, BF16), 2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise ValueError(f"linear: x is [{m}, {k}], weight is {tuple(weight.shape)}")
    if accumulate_into is not None:
        _dev(accumulate_into, "accumulate_into", F32, 2)
        if tuple(accumulate_into.shape) != (m, n):
            raise ValueError(f"linear: accumulator is {tuple(accumulate_into.shape)}, expected {(m, n)}")
    elif out_dtype not in (F32, BF16):
        raise TypeError(f"unsupported output dtype {out_dtype}")
    lib = library()
    if weight.dtype == BF16 and m <= SMALL_M:
        xa = cast(x, BF16)
        splits = lib.ms_gemm_bf16_small_splits(m, n, k)
        if splits == 1 and accumulate_into is None and out_dtype == F32:
            out = torch.empty((m, n), dtype=F32, device=x.device)  # the single partial sum is the result
            _check(lib.ms_gemm_bf16_small(xa.data_ptr(), weight.data_ptr(), out.data_ptr(), None, 1, 0, m, n, k, k, n,
                                          _stream()), "gemm_bf16_small")
            return out
        parts = torch.empty((splits, m, n), dtype=F32, device=x.device)
        if defer:
            _check(lib.ms_gemm_bf16_small(xa.data_ptr(), weight.data_ptr(), parts.data_ptr(), None, 1, 0, m, n, k, k, n,
                                          _stream()), "gemm_bf16_small")
            return SplitSum(parts)
        out = accumulate_into if accumulate_into is not None else torch.empty((m, n), dtype=out_dtype, device=x.device)
        mode = 2 if accumulate_into is not None else (1 if out.dtype == F32 else 0)
        _check(lib.ms_gemm_bf16_small(xa.data_ptr(), weight.data_ptr(), parts.data_ptr(), out.data_ptr(), mode, 1, m, n, k,
                                      k, n, _stream()), "gemm_bf16_small")
        return None if accumulate_into is not None else out
    if weight.dtype == BF16 and defer:
        splits = lib.ms_gemm_bf16_tile_splits(m, n, k)
        if splits > 1:  # few output tiles: split K over the grid and leave the sum to the consumer
            xa = cast(x, BF16)
            parts = torch.empty((splits, m, n), dtype=F32, device=x.device)
            _check(lib.ms_gemm_bf16(xa.data_ptr(), weight.data_ptr(), parts.data_ptr(), 1, m, n, k, k, n, splits, _stream()),
                   "gemm_bf16")
            return SplitSum(parts)
    out = accumulate_into if accumulate_into is not None else torch.empty((m, n), dtype=out_dtype, device=x.device)
    if weight.dtype == F32:
        xa = cast(x, F32)
        mode = 1 if accumulate_into is not None else (0 if out.dtype == F32 else 2)
        _check(lib.ms_gemm_f32(xa.data_ptr(), weight.data_ptr(), out.data_ptr(), mode, m, n, k, k, n, _stream()), "gemm_f32")
    else:
        xa = cast(x, BF16)
        mode = 2 if accumulate_into is not None else (1 if out.dtype == F32 else 0)
        _check(lib.ms_gemm_bf16(xa.data_ptr(), weight.data_ptr(), out.data_ptr(), mode, m, n, k, k, n, 1, _stream()), "gemm_bf16")
    return None if accumulate_into is not None else out


def tile_shape(m: int, n: int, k: int, splits: int = 1, gated: bool = False) -> tuple[int, int] | None:
    """``(rows, columns)`` of the tile that ``linear`` (or, with ``gated``, ``gated_linear`` with ``n = 2 I``)
    runs a bfloat16 product of more than ``SMALL_M`` contiguous rows with; None where the shape takes the
    kernel that stages its slabs through registers."""
    code = library().ms_gemm_bf16_tile_shape(m, n, k, k, splits, int(gated))
    return divmod(code, 1000) if code else None


def add_pending(residual: torch.Tensor, pending: SplitSum | None) -> None:
    """``residual += pending`` for callers whose next kernel cannot take a pending sum itself."""
    if pending is None:
        return
    _dev(residual, "residual", F32, 2)
    _check_split(pending, "pending", residual.shape)
    m, n = residual.shape
    _check(library().ms_splitk_reduce(pending.parts.data_ptr(), residual.data_ptr(), 2, pending.splits, m, n, n, _stream()),
           "splitk_reduce")


# ------------------------------------------------------------------------------------- attention


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """Cosines and sines of the rotation angles ``float32(position) * inv_freq[j]`` of a step's tokens:
    float32 ``[T, 2 * len(inv_freq)]``, a row holding the cosines, then the sines. Made once per step
    and shared by all layers that rotate by the same frequencies."""
    _dev(positions, "positions", I32, 1)
    _dev(inv_freq, "inv_freq", F32, 1)
    t, half = positions.shape[0], inv_freq.shape[0]
    out = torch.empty((t, 2 * half), dtype=F32, device=positions.device)
    _check(library().ms_rope_table(positions.data_ptr(), inv_freq.data_ptr(), out.data_ptr(), t, half, _stream()), "rope_table")
    return out


# Which elements of a head make pair j of a rotation, and the numbers the kernels know the pairings by (MS_ROPE_* in
# csrc/common.h): "halves" (j, j + dim/2), "adjacent" (2j, 2j + 1).
ROTATION_PAIRINGS = {"halves": 0, "adjacent": 1}


def _pairing(name: str) -> int:
    try:
        return ROTATION_PAIRINGS[name]
    except KeyError:
        raise NotImplementedError(f"rotation pairing {name!r}: the kernels know {sorted(ROTATION_PAIRINGS)}") from None


def qk_norm_rope_store(qkv, slots, q_weight, k_weight, eps, rope, k_cache, v_cache,
                       num_heads, num_kv_heads, head_dim, out_dtype=None, pairing: str = "halves") -> torch.Tensor:
    """From ``qkv [T, (Hq + 2 Hkv) D]`` (a tensor, or a ``SplitSum`` of it): per-head RMSNorm of q and k
    (if weights are given), rotation of the first ``rope.shape[1]`` elements of each head, in pairs as
    ``pairing`` names them, by the angles
    of ``rope`` (a ``rope_table`` of these tokens; None: no rotation), k and v stored into the cache
    pages at ``slots`` (skipped when ``slots`` is None). Returns the tensor that holds the finished
    queries in its first ``Hq * D`` columns: ``qkv`` itself (written in place), or for a ``SplitSum`` a
    new ``[T, Hq D]`` tensor of ``out_dtype``."""
    width = (num_heads + 2 * num_kv_heads) * head_dim
    if isinstance(qkv, SplitSum):
        _dev(qkv.parts, "qkv", F32, 3)
        t = qkv.shape[0]
        if qkv.shape[1] != width or out_dtype not in (F32, BF16):
            raise ValueError(f"qkv partial sums have width {qkv.shape[1]}, expected {width}, and need an output dtype")
        dtype = out_dtype
        q_out = torch.empty((t, num_heads * head_dim), dtype=dtype, device=qkv.parts.device)
        src, parts, splits, stride = None, qkv.parts.data_ptr(), qkv.splits, qkv.stride
    else:
        _dev(qkv, "qkv", (F32, BF16), 2)
        t = qkv.shape[0]
        if qkv.shape[1] != width:
            raise ValueError(f"qkv has width {qkv.shape[1]}, expected {width}")
        dtype = qkv.dtype
        q_out = qkv
        src, parts, splits, stride = qkv.data_ptr(), None, 0, 0
    if head_dim > 256 or head_dim < 1:
        raise ValueError(f"head_dim {head_dim} is outside the kernels' range 1..256")
    w_bf16 = 0
    if q_weight is not None:
        for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
            _dev(w, nm, (F32, BF16), 1)
            if w.shape[0] != head_dim:
                raise ValueError(f"{nm} weight has {w.shape[0]} elements for head_dim {head_dim}")
        if q_weight.dtype != k_weight.dtype:
            raise TypeError("q_norm and k_norm weights differ in dtype")
        w_bf16 = int(q_weight.dtype == BF16)
    page_size = 1
    if slots is not None:
        _dev(slots, "slots", I32, 1)
        if slots.shape[0] != t:
            raise ValueError("one slot per token is needed")
        page_size = _check_caches(k_cache, v_cache, dtype, num_kv_heads, head_dim)
    rot_dim, pair = 0, _pairing(pairing)
    if rope is not None:
        _dev(rope, "rope", F32, 2)
        rot_dim = rope.shape[1]
        if rope.shape[0] != t or rot_dim % 2 or rot_dim > head_dim or rot_dim < 2:
            raise ValueError(f"rotation table is {tuple(rope.shape)}; {t} tokens and an even width up to {head_dim} are needed")
    _check(library().ms_qk_norm_rope_store(
        src, parts, splits, stride, q_out.data_ptr(), q_out.shape[1], int(dtype == BF16), _ptr(slots),
        _ptr(q_weight), _ptr(k_weight), w_bf16, float(eps), _ptr(rope), int(rot_dim), pair,
        _ptr(k_cache) if slots is not None else None, _ptr(v_cache) if slots is not None else None, t, num_heads,
        num_kv_heads, head_dim, page_size, _stream()), "qk_norm_rope_store")
    return q_out


def _check_caches(k_cache, v_cache, dtype, num_kv_heads, head_dim) -> int:
    """Keys ``[pages, Hkv, page, D]``, values ``[pages, Hkv, D, page]``; returns the page size."""
    _dev(k_cache, "k_cache", dtype, 4)
    _dev(v_cache, "v_cache", dtype, 4)
    page = k_cache.shape[2]
    if tuple(k_cache.shape[1:]) != (num_kv_heads, page, head_dim):
        raise ValueError(f"k_cache is {tuple(k_cache.shape)}, expected [pages, {num_kv_heads}, page, {head_dim}]")
    if tuple(v_cache.shape) != (k_cache.shape[0], num_kv_heads, head_dim, page):
        raise ValueError(f"v_cache is {tuple(v_cache.shape)}, expected [{k_cache.shape[0]}, {num_kv_heads}, {head_dim}, {page}]")
    return page


PREFILL_BIG_BLOCKS = 640  # from this many 128-row blocks on, the prefill attention runs 128-row blocks
DECODE_TARGET_BLOCKS = 512  # workgroups the split decode kernel aims for
DECODE_MIN_CHUNKS = 4  # 32-token chunks a split should at least hold


def decode_splits(rows: int, num_kv_heads: int, max_kv_len: int) -> int:
    """How many ways the keys of each sequence are split in the decode kernel: enough workgroups to
    fill the chip, but no split shorter than a few chunks."""
    by_fill = -(-DECODE_TARGET_BLOCKS // max(1, rows * num_kv_heads))
    by_len = max(1, -(-max_kv_len // 32) // DECODE_MIN_CHUNKS)
    return max(1, min(by_fill, by_len))


def decode_attention_fusable(qkv, batch, q_weight, k_weight, rope, k_cache, v_cache, num_heads, num_kv_heads, head_dim,
                             pairing: str = "halves") -> bool:
    """Whether ``decode_attention_fused`` takes this step: every row brings one token, the qkv
    projection comes as partial sums, bfloat16 cache with 16-token pages, a head size of 64 or 128, at
    most 16 query heads per KV head, bfloat16 norm weights (or none), rotation over the whole head in
    pairs (j, j + D/2) (or none)."""
    return (isinstance(qkv, SplitSum) and (rope is None or pairing == "halves") and batch.is_decode and batch.decode_tokens is None
            and k_cache.dtype == BF16 and v_cache.dtype == BF16 and k_cache.dim() == 4 and k_cache.shape[2] == 16
            and head_dim in (64, 128) and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16
            and qkv.stride % 4 == 0
            and (q_weight is None) == (k_weight is None) and (q_weight is None or (q_weight.dtype == BF16 and k_weight.dtype == BF16))
            and (rope is None or rope.shape[1] == head_dim))


MERGE_PROJECT_MAX_ROWS = 16  # rows up to which the splits' reduction and the output projection are one kernel
MERGE_PROJECT_MAX_SPLITS = 64


def decode_attention_fused(qkv, q_weight, k_weight, eps, rope, store, k_cache, v_cache, block_table, batch,
                           num_heads, num_kv_heads, head_dim, scale, window, project: torch.Tensor | None = None):
    """``qk_norm_rope_store`` and ``paged_attention`` of a step of single tokens in one kernel, from the
    partial sums ``qkv`` (a ``SplitSum`` of ``[T, (Hq + 2 Hkv) D]``): the queries never go to memory,
    and with ``store`` the new token's key and value are written to the cache by the block that uses
    them first. Returns bfloat16 ``[T, Hq * D]``. ``decode_attention_fusable`` says when this applies.

    ``project``: the output projection's weight ``[N, Hq * D]`` (bfloat16). Where the keys were split
    (they are whenever the step has few rows) and the step has up to ``MERGE_PROJECT_MAX_ROWS`` rows,
    the reduction of the splits and that projection run as one kernel and a ``SplitSum`` of
    ``[T, N]`` is returned instead of the attention's output: no reduction kernel, and the attention's
    output never goes to memory."""
    if not decode_attention_fusable(qkv, batch, q_weight, k_weight, rope, k_cache, v_cache, num_heads, num_kv_heads, head_dim):
        raise ValueError("this step cannot run the fused decode attention")
    _dev(qkv.parts, "qkv", F32, 3)
    t = qkv.shape[0]
    if qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
        raise ValueError(f"qkv partial sums have width {qkv.shape[1]}, expected {(num_heads + 2 * num_kv_heads) * head_dim}")
    page = _check_caches(k_cache, v_cache, BF16, num_kv_heads, head_dim)
    if not scale > 0:
        raise ValueError(f"the attention scale must be positive, not {scale}")
    if q_weight is not None:
        for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
            _dev(w, nm, BF16, 1)
            if w.shape[0] != head_dim:
                raise ValueError(f"{nm} weight has {w.shape[0]} elements for head_dim {head_dim}")
    if rope is not None:
        _dev(rope, "rope", F32, 2)
        if rope.shape[0] != t:
            raise ValueError("one row of the rotation table per token is needed")
    _dev(block_table, "block_table", I32, 2)
    _dev(batch.token_row, "token_row", I32, 1)
    _dev(batch.positions, "positions", I32, 1)
    if batch.token_row.shape[0] != t or batch.positions.shape[0] != t or block_table.shape[0] < batch.num_rows:
        raise ValueError("batch metadata does not match the number of tokens or rows")
    dev = qkv.parts.device
    lib = library()
    splits = decode_splits(t, num_kv_heads, batch.max_kv_len)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty((t * num_heads * splits * head_dim,), dtype=F32, device=dev)
        part_ml = torch.empty((t * num_heads * splits * 2,), dtype=F32, device=dev)
    merged = None  # partial sums of the projection, where one kernel reduces the splits and projects
    if (project is not None and MERGE_PROJECT_MAX_ROWS > 0 and 1 < splits <= MERGE_PROJECT_MAX_SPLITS
            and t <= MERGE_PROJECT_MAX_ROWS):
        _dev(project, "project", BF16, 2)
        n = project.shape[0]
        out_splits = lib.ms_attention_merge_project_splits(t, num_heads, head_dim, splits, n)
        if project.shape[1] == num_heads * head_dim and out_splits >= 1:
            merged = torch.empty((out_splits, t, n), dtype=F32, device=dev)
    out = None if merged is not None else torch.empty((t, num_heads * head_dim), dtype=BF16, device=dev)
    _check(lib.ms_attention_decode_fused_bf16(
        qkv.parts.data_ptr(), qkv.splits, qkv.stride, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(rope),
        ROTATION_PAIRINGS["halves"], int(bool(store)),
        k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1], None,
        batch.token_row.data_ptr(), batch.positions.data_ptr(), _ptr(out), _ptr(part_o), _ptr(part_ml), t, splits,
        num_heads, num_kv_heads, head_dim, page, float(scale), int(window), int(merged is None), _stream()),
        "attention_decode_fused")
    if merged is None:
        return out
    _check(lib.ms_attention_merge_project(part_o.data_ptr(), part_ml.data_ptr(), project.data_ptr(), merged.data_ptr(), t,
                                          num_heads, head_dim, splits, merged.shape[2], _stream()), "attention_merge_project")
    return SplitSum(merged)


def paged_attention(qkv, k_cache, v_cache, block_table, batch, num_heads, num_kv_heads, head_dim, scale, window):
    """Attention of the batch's new tokens over the cache. ``qkv [T, >= Hq D]`` holds the queries
    in its first ``Hq * D`` columns. Returns ``[T, Hq * D]``.

    bfloat16 with 16-token pages and a head size of 64 or 128: rows that bring one token run the
    split decode kernel, rows that bring several the tiled prefill kernel. Everything else (float32,
    other head sizes or page sizes) runs the generic kernel."""
    _dev(qkv, "qkv", (F32, BF16), 2)
    t = qkv.shape[0]
    page = _check_caches(k_cache, v_cache, qkv.dtype, num_kv_heads, head_dim)
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise ValueError(f"head_dim {head_dim} is not supported: the attention kernels take multiples of 16 up to 256")
    if num_heads % num_kv_heads:
        raise ValueError(f"{num_heads} query heads are no multiple of {num_kv_heads} KV heads")
    if qkv.shape[1] < num_heads * head_dim:
        raise ValueError("qkv is narrower than the query heads")
    if not scale > 0:
        raise ValueError(f"the attention scale must be positive, not {scale}")  # the kernels scale masked scores too
    _dev(block_table, "block_table", I32, 2)
    _dev(batch.token_row, "token_row", I32, 1)
    _dev(batch.positions, "positions", I32, 1)
    if batch.token_row.shape[0] != t or batch.positions.shape[0] != t or block_table.shape[0] < batch.num_rows:
        raise ValueError("batch metadata does not match the number of tokens or rows")
    out = torch.empty((t, num_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    lib = library()
    common = (block_table.data_ptr(), block_table.shape[1])
    meta = (batch.token_row.data_ptr(), batch.positions.data_ptr(), out.data_ptr())
    n_dec = batch.num_decode_tokens
    fast = (qkv.dtype == BF16 and page == 16 and head_dim in (64, 128) and num_heads // num_kv_heads <= 16
            and qkv.shape[1] % 8 == 0)
    if not fast:
        _check(lib.ms_paged_attention_generic(
            qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), int(qkv.dtype == BF16), *common, None,
            *meta, t, num_heads, num_kv_heads, head_dim, page, float(scale), int(window), _stream()), "paged_attention")
        return out
    if n_dec:
        splits = decode_splits(n_dec, num_kv_heads, batch.max_kv_len)
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty((n_dec * num_heads * splits * head_dim,), dtype=F32, device=qkv.device)
            part_ml = torch.empty((n_dec * num_heads * splits * 2,), dtype=F32, device=qkv.device)
        _check(lib.ms_attention_decode_bf16(
            qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common, _ptr(batch.decode_tokens), *meta,
            _ptr(part_o), _ptr(part_ml), n_dec, splits, num_heads, num_kv_heads, head_dim, page, float(scale), int(window),
            _stream()), "attention_decode")
    if n_dec < t:
        if block_table.shape[1] % 4:  # the prefill kernel reads four page ids at once
            wide = torch.zeros((block_table.shape[0], -(-block_table.shape[1] // 4) * 4), dtype=I32, device=block_table.device)
            wide[:, : block_table.shape[1]] = block_table
            block_table = wide
            common = (block_table.data_ptr(), block_table.shape[1])
        group = num_heads // num_kv_heads
        # 128 query rows per block read K and V least often; 64 (each wave takes half of every key tile)
        # give short chains and more blocks. The latter until 128-row blocks alone fill the chip twice over.
        n_prefill = t - n_dec
        rows = 128 if (group > 64 or -(-n_prefill // (128 // group)) * num_kv_heads >= PREFILL_BIG_BLOCKS) else 64
        tile_tokens = lib.ms_attention_prefill_tile_tokens(group, rows)
        plan = _prefill_parts_plan(batch, tile_tokens, num_kv_heads, rows * head_dim * 4) if window == 0 else None
        if plan is not None:
            part_o = torch.empty((plan.slots * num_kv_heads * rows * head_dim,), dtype=F32, device=qkv.device)
            part_ml = torch.empty((plan.slots * num_kv_heads * rows * 2,), dtype=F32, device=qkv.device)
            _check(lib.ms_attention_prefill_parts_bf16(
                qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common, plan.table.data_ptr(),
                plan.entries, plan.merges, part_o.data_ptr(), part_ml.data_ptr(), rows, *meta, num_heads, num_kv_heads,
                head_dim, page, float(scale), _stream()), "attention_prefill_parts")
            return out
        first, count, tiles = batch.prefill_tiles(tile_tokens)
        _check(lib.ms_attention_prefill_bf16(
            qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), *common, first.data_ptr(), count.data_ptr(),
            tiles, rows, *meta, num_heads, num_kv_heads, head_dim, page, float(scale), int(window), _stream()),
            "attention_prefill")
    return out


def build_prefill_tiles(row_lens, row_starts, tile_tokens: int, device):
    """Tiles of at most ``tile_tokens`` consecutive new tokens of the rows that bring several tokens:
    ``(first flat token index [n], token count [n], n)`` on the device, the tile deepest into its
    sequence (the most keys to visit) first."""
    tiles = []
    t = 0
    for n, s in zip(row_lens, row_starts):
        if n > 1:
            for a in range(0, n, tile_tokens):
                tiles.append((s + min(n, a + tile_tokens), t + a, min(tile_tokens, n - a)))
        t += n
    tiles.sort(key=lambda x: -x[0])
    host = torch.tensor([[f for _, f, _ in tiles], [c for _, _, c in tiles]], dtype=I32)
    dev = host.to(device, non_blocking=True)
    return dev[0], dev[1], len(tiles)


PREFILL_KEY_TILE = 64        # keys per iteration of the prefill attention kernel
PREFILL_RESIDENT_BLOCKS = 512  # blocks of it the chip holds at once (two per CU)
PREFILL_MIN_PART = 4         # key tiles: no part is made shorter than this
PREFILL_PARTS_LAUNCH_US = 8.0  # what the merge kernel costs beside the bytes it moves
PREFILL_PARTS_MARGIN = 1.5   # parts are made where they save this many times what they cost


class PrefillPartsPlan:
    """Tiles of new tokens whose keys are handed out in parts. ``table``: int32 on the device, per entry
    first token, token count, first key tile, end key tile, slot (-1: a whole tile), heaviest entry
    first; then per merged tile first token, token count, first slot, number of parts."""

    __slots__ = ("table", "entries", "merges", "slots")

    def __init__(self, table, entries, merges, slots):
        self.table, self.entries, self.merges, self.slots = table, entries, merges, slots


def plan_prefill_parts(row_lens, row_starts, tile_tokens: int, kv_heads: int, part_bytes: int = 64 * 128 * 4):
    """Host part of ``PrefillPartsPlan``: ``(entries, merges)`` as lists of tuples, or None where
    whole tiles do as well. A step takes as long as its deepest tile's chain of key tiles (about 1.2 us
    each for a block on its own) or as long as all key tiles take the chip (about 2.4 us for each
    resident block's), whichever is longer. Where the chain is the longer by far (a short portion
    deep into a long sequence), the keys of tiles deeper than the chip's fair share (all key tiles /
    resident blocks) are cut into equal parts no longer than that share. The parts cost a second
    kernel and ``part_bytes`` written and read per part and KV head, so whole tiles stay unless the
    shorter chain saves half as much again as that (measured: one 2,048-token prompt is slower in
    parts, a 512-token portion behind 16,000 cached tokens a quarter faster)."""
    tiles = []
    t = 0
    for n, s in zip(row_lens, row_starts):
        if n > 1:
            for a in range(0, n, tile_tokens):
                c = min(tile_tokens, n - a)
                tiles.append(((s + a + c - 1) // PREFILL_KEY_TILE + 1, t + a, c))
        t += n
    if not tiles or len(tiles) * kv_heads >= 2 * PREFILL_RESIDENT_BLOCKS:
        return None
    total = sum(d for d, _, _ in tiles) * kv_heads
    share = max(PREFILL_MIN_PART, -(-total // PREFILL_RESIDENT_BLOCKS))
    deepest = max(d for d, _, _ in tiles)
    if deepest <= share:
        return None
    slots = sum(-(-d // share) for d, _, _ in tiles if d > share)
    busy_us = 2.4 * total / PREFILL_RESIDENT_BLOCKS
    saved_us = 1.2 * deepest - max(1.2 * share, busy_us)
    cost_us = PREFILL_PARTS_LAUNCH_US + 2 * slots * kv_heads * part_bytes / 3e6
    if saved_us <= PREFILL_PARTS_MARGIN * cost_us:
        return None
    entries, merges, slot = [], [], 0
    for depth, first, count in tiles:
        parts = -(-depth // share)
        if parts == 1:
            entries.append((first, count, 0, depth, -1))
            continue
        per = -(-depth // parts)
        parts = -(-depth // per)
        merges.append((first, count, slot, parts))
        for p in range(parts):
            entries.append((first, count, p * per, min(depth, (p + 1) * per), slot))
            slot += 1
    entries.sort(key=lambda e: e[2] - e[3])  # most key tiles first
    return entries, merges


def _prefill_parts_plan(batch, tile_tokens: int, kv_heads: int, part_bytes: int):
    memo = getattr(batch, "memo", None)
    key = ("prefill_parts", tile_tokens, kv_heads, part_bytes)
    if memo is not None and key in memo:
        return memo[key]
    plan = None
    made = plan_prefill_parts(batch.row_lens, batch.row_starts_host, tile_tokens, kv_heads, part_bytes)
    if made is not None:
        entries, merges = made
        flat = [e[i] for i in range(5) for e in entries] + [m[i] for i in range(4) for m in merges]
        table = torch.tensor(flat, dtype=I32).to(batch.positions.device, non_blocking=True)
        plan = PrefillPartsPlan(table, len(entries), len(merges), sum(m[3] for m in merges))
    if memo is not None:
        memo[key] = plan
    return plan


# ------------------------------------------------------------------------------------- sampling


def sample_rows(logits, temperature=None, top_p=None, seed=None, counter=None) -> torch.Tensor:
    """``int32 [rows]`` token ids from float32 ``logits [rows, vocab]``. Without ``temperature`` every
    row takes the first maximal index; with it, rows whose temperature is 0 still do."""
    _dev(logits, "logits", F32, 2)
    rows, vocab = logits.shape
    if temperature is not None:
        _dev(temperature, "temperature", F32, 1)
        _dev(seed, "seed", I32, 1)
        _dev(counter, "counter", I32, 1)
        if top_p is not None:
            _dev(top_p, "top_p", F32, 1)
        for v in (temperature, seed, counter) + ((top_p,) if top_p is not None else ()):
            if v.shape[0] != rows:
                raise ValueError("one sampling parameter per row is needed")
    out = torch.empty((rows,), dtype=I32, device=logits.device)
    lib = library()
    need = lib.ms_sample_scratch_bytes(rows)
    if need < 0:
        raise ValueError(f"sample_rows: {rows} rows are more than one call takes")
    scratch = torch.empty((need,), dtype=torch.uint8, device=logits.device)
    _check(lib.ms_sample_rows(logits.data_ptr(), rows, vocab, vocab, _ptr(temperature), _ptr(top_p), _ptr(seed),
                              _ptr(counter), scratch.data_ptr(), out.data_ptr(), _stream()), "sample_rows")
    return out


def sample_rows_static(logits, out, temperature=None, top_p=None, seed=None, counter=None) -> torch.Tensor:
    """``sample_rows`` into the caller's ``out`` (int32 ``[rows]``) without allocating anything: the
    candidates between the two kernels lie in an array inside the library, one per GPU, instead of
    in a scratch tensor. For callers that cannot allocate (under graph capture, say). At most
    ``ms_sample_rows_static_max_rows()`` rows; calls that overlap on one GPU race for the array."""
    _dev(logits, "logits", F32, 2)
    _dev(out, "out", I32, 1)
    rows, vocab = logits.shape
    if out.shape[0] != rows:
        raise ValueError("one output element per row is needed")
    lib = library()
    most = lib.ms_sample_rows_static_max_rows()
    if rows > most:
        raise ValueError(f"sample_rows_static takes at most {most} rows, got {rows}: use sample_rows")
    if temperature is not None:
        _dev(temperature, "temperature", F32, 1)
        _dev(seed, "seed", I32, 1)
        _dev(counter, "counter", I32, 1)
        if top_p is not None:
            _dev(top_p, "top_p", F32, 1)
        for v in (temperature, seed, counter) + ((top_p,) if top_p is not None else ()):
            if v.shape[0] != rows:
                raise ValueError("one sampling parameter per row is needed")
    _check(lib.ms_sample_rows_static(logits.data_ptr(), rows, vocab, vocab, _ptr(temperature), _ptr(top_p), _ptr(seed),
                                     _ptr(counter), out.data_ptr(), _stream()), "sample_rows_static")
    return out


# ------------------------------------------------------------------------------------- measurement


def measure_read(buffer: torch.Tensor, blocks: int = 4096) -> torch.Tensor:
    """Streams ``buffer`` (contiguous, a multiple of 16 bytes) through ``blocks`` blocks once and
    returns their checksums ``int32 [blocks]``: the read half of the memory system's rate."""
    if not buffer.is_cuda or not buffer.is_contiguous():
        raise ValueError("measure_read takes a contiguous tensor on the GPU")
    out = torch.empty((blocks,), dtype=I32, device=buffer.device)
    _check(library().ms_measure_read(buffer.data_ptr(), buffer.numel() * buffer.element_size(), blocks, out.data_ptr(),
                                     _stream()), "measure_read")
    return out


def measure_copy(src: torch.Tensor, dst: torch.Tensor, blocks: int = 4096) -> None:
    """``dst[:] = src`` as a streaming copy of ``blocks`` blocks (both contiguous, same size, a multiple
    of 16 bytes)."""
    if not (src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("measure_copy takes contiguous tensors on the GPU")
    n = src.numel() * src.element_size()
    if n != dst.numel() * dst.element_size():
        raise ValueError("source and destination differ in size")
    _check(library().ms_measure_copy(src.data_ptr(), dst.data_ptr(), n, blocks, _stream()), "measure_copy")
