"""The C++ block core behind the same interface as the Python allocator and table (``cache/pages.py``). Built from
``csrc/block_core.cpp`` on first use; raises the same exception types as the Python classes, so
callers and tests cannot tell the backends apart (miniserve/cache/backend.py:46-94)."""

from __future__ import annotations

import ctypes
from collections.abc import Iterable

import numpy as np

from ..kernels import build
from .pages import NO_PAGE, OutOfBlocks

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
    if not isinstance(values, np.ndarray):
        values = list(values)
    return np.ascontiguousarray(values, dtype=np.int32).reshape(-1)


class NativePageAllocator:
    backend = "cpp"

    def __init__(self, num_pages: int, page_size: int):
        if num_pages < 1 or page_size < 1:
            raise ValueError(f"a group needs at least one page of at least one token, got {num_pages} x {page_size}")
        self._lib = _library()
        self._h = self._lib.msb_allocator_new(num_pages, page_size)
        self.num_pages = num_pages
        self.page_size = page_size

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.msb_allocator_delete(self._h)
            self._h = None

    @property
    def num_free(self) -> int:
        return self._lib.msb_allocator_num_free(self._h)

    @property
    def num_used(self) -> int:
        return self.num_pages - self.num_free

    def holders_of(self, page: int) -> int:
        out = _I()
        _raise(self._lib.msb_allocator_refcount(self._h, page, ctypes.byref(out)), f"page {page} does not exist")
        return out.value

    def take(self, n: int) -> list[int]:
        if n < 0:
            raise ValueError(f"cannot take {n} pages")
        out = np.empty(max(n, 1), dtype=np.int32)
        _raise(self._lib.msb_allocator_allocate(self._h, n, out.ctypes.data), f"{n} pages wanted, {self.num_free} free")
        return out[:n].tolist()

    def hold(self, pages: Iterable[int]) -> None:
        a = _ints(pages)
        _raise(self._lib.msb_allocator_incref(self._h, a.ctypes.data, len(a)), f"cannot share pages {a.tolist()}")

    def give_back(self, pages: Iterable[int]) -> None:
        a = _ints(pages)
        _raise(self._lib.msb_allocator_free(self._h, a.ctypes.data, len(a)), f"cannot give back pages {a.tolist()}")

    def new_table(self, shared: Iterable[int] = ()):
        return NativePageTable(self, shared)

    def check_invariants(self) -> None:
        _raise(self._lib.msb_allocator_check(self._h) and 7, "the free stack and the holder counts disagree")


class NativePageTable:
    def __init__(self, allocator: NativePageAllocator, shared=()):
        self.allocator = allocator
        self.page_size = allocator.page_size
        self._lib = allocator._lib
        a = _ints(shared)
        st = _I()
        self._h = self._lib.msb_table_new(allocator._h, a.ctypes.data, len(a), ctypes.byref(st))
        if not self._h:
            if st.value == 9:
                raise ValueError(f"duplicate page in the shared prefix {a.tolist()}")
            _raise(st.value, f"shared prefix {a.tolist()}")

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.msb_table_delete(self._h)
            self._h = None

    @property
    def num_tokens(self) -> int:
        return self._lib.msb_table_num_tokens(self._h)

    @property
    def num_entries(self) -> int:
        return self._lib.msb_table_num_blocks(self._h)

    @property
    def first_live(self) -> int:
        return self._lib.msb_table_first_live(self._h)

    @property
    def num_held(self) -> int:
        return self.num_entries - self.first_live

    @property
    def entries(self) -> np.ndarray:
        n = self.num_entries
        out = np.empty(max(n, 1), dtype=np.int32)
        _raise(self._lib.msb_table_blocks(self._h, out.ctypes.data, n), "entries")
        return out[:n]

    @property
    def pages(self) -> list[int]:
        return self.entries.tolist()

    def pages_needed(self, n: int) -> int:
        if n < 0:
            raise ValueError(f"cannot append {n} tokens")
        return self._lib.msb_table_blocks_needed(self._h, n)

    def append(self, n: int) -> list[int]:
        k = self.pages_needed(n)
        out = np.empty(max(k, 1), dtype=np.int32)
        got = _I()
        _raise(self._lib.msb_table_append(self._h, n, out.ctypes.data, len(out), ctypes.byref(got)),
               f"{k} pages wanted, {self.allocator.num_free} free")
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


def pack_native(tables, out: np.ndarray, pad_rows: int, pad_page: int) -> int:
    rows, width = out.shape
    handles = (ctypes.c_void_p * max(len(tables), 1))(*[t._h for t in tables])
    total = _I()
    st = _library().msb_pack_tables(handles, len(tables), out.ctypes.data, rows, width, pad_rows, pad_page, ctypes.byref(total))
    if st == 8:
        raise ValueError(f"the packing buffer is {out.shape}; {len(tables)} tables + {pad_rows} padding rows do not fit")
    _raise(st, "pack_tables")
    return total.value


__all__ = ["NativePageAllocator", "NativePageTable", "pack_native", "NO_PAGE"]
