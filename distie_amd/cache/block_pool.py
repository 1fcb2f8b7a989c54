"""ctypes face of the native id pool (distie_amd/csrc/block_pool.cpp).

Errors follow the reference's binding (core/python/bindings.cpp:11-21): asking for more
ids than are free raises `OutOfBlocks` (a RuntimeError), an invalid free raises ValueError;
both leave the pool unchanged."""

from __future__ import annotations

import ctypes
from typing import List, Sequence

from ..csrc import build

_lib = None


class OutOfBlocks(RuntimeError):
    """The pool has fewer free ids than were asked for."""


def _library():
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(str(build.ensure("core")))
        lib.distie_pool_create.restype = ctypes.c_void_p
        lib.distie_pool_create.argtypes = [ctypes.c_int64]
        lib.distie_pool_destroy.argtypes = [ctypes.c_void_p]
        lib.distie_pool_take.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.POINTER(ctypes.c_int32)]
        lib.distie_pool_give.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int32), ctypes.c_int64,
                                         ctypes.c_char_p, ctypes.c_int64]
        for name in ("distie_pool_size", "distie_pool_free_count"):
            getattr(lib, name).restype = ctypes.c_int64
            getattr(lib, name).argtypes = [ctypes.c_void_p]
        lib.distie_pool_is_held.argtypes = [ctypes.c_void_p, ctypes.c_int32]
        _lib = lib
    return _lib


class BlockPool:
    def __init__(self, num_blocks: int) -> None:
        if num_blocks < 1:
            raise ValueError("num_blocks must be > 0")
        self._lib = _library()
        self._handle = self._lib.distie_pool_create(int(num_blocks))
        if not self._handle:
            raise ValueError(f"cannot make a pool of {num_blocks} ids")
        self.num_blocks = int(num_blocks)

    def allocate(self, count: int) -> List[int]:
        if count < 0:
            raise ValueError("count must be >= 0")
        if count == 0:
            return []
        out = (ctypes.c_int32 * count)()
        if self._lib.distie_pool_take(self._handle, count, out) != 0:
            raise OutOfBlocks(f"out of blocks: requested {count}, free {self.num_free}")
        return list(out)

    def free(self, ids: Sequence[int]) -> None:
        ids = [int(i) for i in ids]
        if not ids:
            return
        array = (ctypes.c_int32 * len(ids))(*ids)
        why = ctypes.create_string_buffer(128)
        if self._lib.distie_pool_give(self._handle, array, len(ids), why, 128) != 0:
            raise ValueError(why.value.decode())

    @property
    def num_free(self) -> int:
        return int(self._lib.distie_pool_free_count(self._handle))

    @property
    def num_used(self) -> int:
        return self.num_blocks - self.num_free

    @property
    def utilization(self) -> float:
        return self.num_used / self.num_blocks

    def is_held(self, block_id: int) -> bool:
        return self._lib.distie_pool_is_held(self._handle, int(block_id)) == 1

    def __del__(self) -> None:
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            self._lib.distie_pool_destroy(handle)
