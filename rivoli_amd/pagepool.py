"""ctypes view of the host page allocator (rivoli_amd/csrc/pagepool.cpp, C ABI in
include/rivoli_pagepool.h). It owns which page every token of every sequence lives in and
hands the kernels their block tables and slot mappings; it never touches device memory."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from .build import HOST_LIB_PATH

_LIB = None


class PoolExhausted(RuntimeError):
    """The pool cannot supply the pages asked for (-1005); the caller must free a sequence."""


def lib() -> C.CDLL:
    global _LIB
    if _LIB is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise FileNotFoundError(f"{HOST_LIB_PATH} is missing: run `python -m rivoli_amd.build`")
        h = C.CDLL(HOST_LIB_PATH)
        ip = C.POINTER(C.c_int)
        h.rivoli_pagepool_create.restype = C.c_void_p
        h.rivoli_pagepool_create.argtypes = [C.c_int, C.c_int]
        h.rivoli_pagepool_destroy.restype = None
        h.rivoli_pagepool_destroy.argtypes = [C.c_void_p]
        for name, args in {
            "seq_create": [C.c_void_p], "seq_free": [C.c_void_p, C.c_int],
            "seq_extend": [C.c_void_p, C.c_int, C.c_int, ip], "seq_len": [C.c_void_p, C.c_int],
            "seq_blocks": [C.c_void_p, C.c_int], "block_table": [C.c_void_p, C.c_int, ip, C.c_int],
            "pages_free": [C.c_void_p], "pages_owned": [C.c_void_p], "frontier": [C.c_void_p],
        }.items():
            fn = getattr(h, "rivoli_pagepool_" + name)
            fn.restype, fn.argtypes = C.c_int, args
        _LIB = h
    return _LIB


EXPORTED = ["rivoli_pagepool_" + n for n in (
    "create", "destroy", "seq_create", "seq_free", "seq_extend", "seq_len", "seq_blocks",
    "block_table", "pages_free", "pages_owned", "frontier")]


class PagePool:
    def __init__(self, n_pages: int, page_tokens: int = 64):
        self._h = lib().rivoli_pagepool_create(n_pages, page_tokens)
        if not self._h:
            raise ValueError("page pool: invalid size")
        self.n_pages, self.page_tokens = n_pages, page_tokens

    def __del__(self):
        if getattr(self, "_h", None):
            lib().rivoli_pagepool_destroy(self._h)
            self._h = None

    @staticmethod
    def _check(r: int, what: str) -> int:
        if r == -1005:
            raise PoolExhausted(what)
        if r < 0:
            raise ValueError(f"page pool: {what} refused ({r})")
        return r

    def seq_create(self) -> int:
        return self._check(lib().rivoli_pagepool_seq_create(self._h), "seq_create")

    def seq_free(self, seq: int) -> int:
        return self._check(lib().rivoli_pagepool_seq_free(self._h, seq), "seq_free")

    def seq_extend(self, seq: int, n_tokens: int) -> np.ndarray:
        slots = np.empty(n_tokens, np.int32)
        self._check(lib().rivoli_pagepool_seq_extend(
            self._h, seq, n_tokens, slots.ctypes.data_as(C.POINTER(C.c_int))), "seq_extend")
        return slots

    def seq_len(self, seq: int) -> int:
        return self._check(lib().rivoli_pagepool_seq_len(self._h, seq), "seq_len")

    def block_table(self, seq: int) -> np.ndarray:
        n = self._check(lib().rivoli_pagepool_seq_blocks(self._h, seq), "seq_blocks")
        out = np.empty(n, np.int32)
        lib().rivoli_pagepool_block_table(self._h, seq, out.ctypes.data_as(C.POINTER(C.c_int)), n)
        return out

    @property
    def pages_free(self) -> int:
        return lib().rivoli_pagepool_pages_free(self._h)

    @property
    def pages_owned(self) -> int:
        return lib().rivoli_pagepool_pages_owned(self._h)

    @property
    def frontier(self) -> int:
        return lib().rivoli_pagepool_frontier(self._h)
