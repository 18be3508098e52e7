"""The C++ block core behind the same interface as the Python allocator and table. Built from
``csrc/block_core.cpp`` on first use; raises the same exception types as the Python classes, so
callers and tests cannot tell the backends apart (miniserve/cache/backend.py:46-94)."""

from __future__ import annotations

import ctypes
from collections.abc import Iterable

import numpy as np

from ..kernels import build
from .allocator import OutOfBlocks
from .table import NO_BLOCK

_lib = None
_I = ctypes.c_int
_P = ctypes.c_void_p
_IP = ctypes.POINTER(ctypes.c_int)


def _library():
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(str(build.build_core()))
        sigs = {
            "msb_allocator_new": ([_I, _I], _P), "msb_allocator_delete": ([_P], None),
            "msb_allocator_num_free": ([_P], _I), "msb_allocator_refcount": ([_P, _I, _IP], _I),
            "msb_allocator_allocate": ([_P, _I, _P], _I), "msb_allocator_incref": ([_P, _P, _I], _I),
            "msb_allocator_free": ([_P, _P, _I], _I), "msb_allocator_check": ([_P], _I),
            "msb_table_new": ([_P, _P, _I, _IP], _P), "msb_table_delete": ([_P], None),
            "msb_table_num_tokens": ([_P], _I), "msb_table_num_blocks": ([_P], _I), "msb_table_first_live": ([_P], _I),
            "msb_table_blocks_needed": ([_P, _I], _I), "msb_table_append": ([_P, _I, _P, _I, _IP], _I),
            "msb_table_slot": ([_P, _I, _IP], _I), "msb_table_tail_slots": ([_P, _I, _P], _I),
            "msb_table_rewind": ([_P, _I], _I), "msb_table_release_before": ([_P, _I, _IP], _I),
            "msb_table_release": ([_P], _I), "msb_table_blocks": ([_P, _P, _I], _I),
            "msb_pack_tables": ([_P, _I, _P, _I, _I, _I, _I, _IP], _I),
        }
        for name, (args, res) in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = args, res
        _lib = lib
    return _lib


def _raise(status: int, what: str):
    if status == 0:
        return
    if status == 1:
        raise OutOfBlocks(what)
    if status in (3, 6):
        raise IndexError(what)
    if status == 7:
        raise AssertionError(what)
    raise ValueError(f"{what} (status {status})")


def _ints(values) -> np.ndarray:
    return np.ascontiguousarray(values, dtype=np.int32)


class NativeBlockAllocator:
    backend = "cpp"

    def __init__(self, num_blocks: int, block_size: int):
        if num_blocks < 1 or block_size < 1:
            raise ValueError(f"num_blocks and block_size must be positive, got {num_blocks}, {block_size}")
        self._lib = _library()
        self._h = self._lib.msb_allocator_new(num_blocks, block_size)
        self.num_blocks = num_blocks
        self.block_size = block_size

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.msb_allocator_delete(self._h)
            self._h = None

    @property
    def num_free(self) -> int:
        return self._lib.msb_allocator_num_free(self._h)

    @property
    def num_used(self) -> int:
        return self.num_blocks - self.num_free

    def can_allocate(self, n: int) -> bool:
        return 0 <= n <= self.num_free

    def refcount(self, block: int) -> int:
        out = _I()
        _raise(self._lib.msb_allocator_refcount(self._h, block, ctypes.byref(out)), f"block id {block} out of range")
        return out.value

    def allocate(self, n: int) -> list[int]:
        if n < 0:
            raise ValueError(f"cannot allocate {n} blocks")
        out = np.empty(max(n, 1), dtype=np.int32)
        _raise(self._lib.msb_allocator_allocate(self._h, n, out.ctypes.data), f"requested {n} blocks, {self.num_free} free")
        return out[:n].tolist()

    def incref(self, blocks: Iterable[int]) -> None:
        a = _ints(list(blocks))
        _raise(self._lib.msb_allocator_incref(self._h, a.ctypes.data, len(a)), f"incref of {a.tolist()}")

    def free(self, blocks: Iterable[int]) -> None:
        a = _ints(list(blocks))
        _raise(self._lib.msb_allocator_free(self._h, a.ctypes.data, len(a)), f"free of {a.tolist()}")

    def new_table(self, prefix_blocks: Iterable[int] = ()):
        return NativeBlockTable(self, list(prefix_blocks))

    def check_invariants(self) -> None:
        _raise(self._lib.msb_allocator_check(self._h) and 7, "free stack disagrees with holder counts")


class NativeBlockTable:
    def __init__(self, allocator: NativeBlockAllocator, prefix_blocks=()):
        self.allocator = allocator
        self.block_size = allocator.block_size
        self._lib = allocator._lib
        a = _ints(list(prefix_blocks))
        st = _I()
        self._h = self._lib.msb_table_new(allocator._h, a.ctypes.data, len(a), ctypes.byref(st))
        if not self._h:
            if st.value == 9:
                raise ValueError(f"duplicate block in prefix {a.tolist()}")
            _raise(st.value, f"prefix {a.tolist()}")

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.msb_table_delete(self._h)
            self._h = None

    @property
    def num_tokens(self) -> int:
        return self._lib.msb_table_num_tokens(self._h)

    @property
    def num_blocks(self) -> int:
        return self._lib.msb_table_num_blocks(self._h)

    @property
    def first_live(self) -> int:
        return self._lib.msb_table_first_live(self._h)

    @property
    def num_held(self) -> int:
        return self.num_blocks - self.first_live

    @property
    def capacity(self) -> int:
        return self.num_blocks * self.block_size

    @property
    def last_block_len(self) -> int:
        n = self.num_tokens
        return 0 if n == 0 else n - (self.num_blocks - 1) * self.block_size

    @property
    def blocks(self) -> list[int]:
        n = self.num_blocks
        out = np.empty(max(n, 1), dtype=np.int32)
        _raise(self._lib.msb_table_blocks(self._h, out.ctypes.data, n), "blocks")
        return out[:n].tolist()

    def blocks_needed(self, n: int) -> int:
        if n < 0:
            raise ValueError(f"cannot append {n} tokens")
        return self._lib.msb_table_blocks_needed(self._h, n)

    def append_tokens(self, n: int) -> list[int]:
        k = self.blocks_needed(n)
        out = np.empty(max(k, 1), dtype=np.int32)
        got = _I()
        _raise(self._lib.msb_table_append(self._h, n, out.ctypes.data, len(out), ctypes.byref(got)),
               f"requested {k} blocks, {self.allocator.num_free} free")
        return out[: got.value].tolist()

    def slot(self, pos: int) -> int:
        out = _I()
        _raise(self._lib.msb_table_slot(self._h, pos, ctypes.byref(out)), f"position {pos} out of range or given back")
        return out.value

    def tail_slots(self, n: int) -> list[int]:
        out = np.empty(max(n, 1), dtype=np.int32)
        self.tail_slots_into(n, out)
        return out[:n].tolist()

    def tail_slots_into(self, n: int, out: np.ndarray) -> None:
        if n < 0 or len(out) < n or out.dtype != np.int32 or not out.flags.c_contiguous:
            raise IndexError(f"tail of {n} tokens does not fit the buffer")
        _raise(self._lib.msb_table_tail_slots(self._h, n, out.ctypes.data), f"tail of {n} tokens out of range")

    def rewind(self, n: int) -> None:
        _raise(self._lib.msb_table_rewind(self._h, n), f"cannot rewind {n} tokens")

    def release_before(self, pos: int) -> int:
        out = _I()
        _raise(self._lib.msb_table_release_before(self._h, pos, ctypes.byref(out)), "release_before")
        return out.value

    def release(self) -> None:
        _raise(self._lib.msb_table_release(self._h), "release")


def pack_native(tables, out: np.ndarray, pad_rows: int, pad_block: int) -> int:
    rows, width = out.shape
    handles = (ctypes.c_void_p * max(len(tables), 1))(*[t._h for t in tables])
    total = _I()
    st = _library().msb_pack_tables(handles, len(tables), out.ctypes.data, rows, width, pad_rows, pad_block, ctypes.byref(total))
    if st == 8:
        raise ValueError(f"packing buffer too small: {out.shape} for {len(tables)} tables + {pad_rows} padding rows")
    _raise(st, "pack_tables")
    return total.value


__all__ = ["NativeBlockAllocator", "NativeBlockTable", "pack_native", "NO_BLOCK"]
