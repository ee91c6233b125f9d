"""Block tables of one group of layers, all in one int32 array: a row per live request (the row is the request's
state slot), so that the native step layout (csrc/host/host_core.cpp) reads them where they lie. ``BlockTable`` is
what the cache manager holds per request and group: it behaves like the list of page ids it replaces (-1 = a page
that was given back).
"""
from __future__ import annotations

from typing import Iterator, List

import numpy as np


class TableArena:
    def __init__(self, rows: int, cols: int = 16):
        self.data = np.zeros((rows, max(1, cols)), np.int32)
        self.lens = np.zeros(rows, np.int32)

    def table(self, row: int) -> "BlockTable":
        self.lens[row] = 0
        return BlockTable(self, row)

    def _room(self, cols: int) -> None:
        if cols > self.data.shape[1]:
            grown = np.zeros((self.data.shape[0], max(cols, 2 * self.data.shape[1])), np.int32)
            grown[:, :self.data.shape[1]] = self.data
            self.data = grown


class BlockTable:
    __slots__ = ("arena", "row")

    def __init__(self, arena: TableArena, row: int):
        self.arena = arena
        self.row = row

    def __len__(self) -> int:
        return int(self.arena.lens[self.row])

    def __bool__(self) -> bool:
        return bool(self.arena.lens[self.row] > 0)

    def tolist(self) -> List[int]:
        return self.arena.data[self.row, :self.arena.lens[self.row]].tolist()

    def __iter__(self) -> Iterator[int]:
        return iter(self.tolist())

    def __getitem__(self, i):
        if isinstance(i, slice):
            return self.tolist()[i]
        n = len(self)
        if i < 0:
            i += n
        if not 0 <= i < n:
            raise IndexError("block table index out of range")
        return int(self.arena.data[self.row, i])

    def __setitem__(self, i: int, page: int) -> None:
        n = len(self)
        if i < 0:
            i += n
        if not 0 <= i < n:
            raise IndexError("block table index out of range")
        self.arena.data[self.row, i] = page

    def append(self, page: int) -> None:
        n = len(self)
        self.arena._room(n + 1)
        self.arena.data[self.row, n] = page
        self.arena.lens[self.row] = n + 1

    def pop(self) -> int:
        n = len(self)
        if n == 0:
            raise IndexError("pop from an empty block table")
        self.arena.lens[self.row] = n - 1
        return int(self.arena.data[self.row, n - 1])

    def clear(self) -> None:
        self.arena.lens[self.row] = 0

    def __eq__(self, other) -> bool:
        if isinstance(other, BlockTable):
            other = other.tolist()
        return self.tolist() == other

    __hash__ = None

    def __repr__(self) -> str:
        return f"BlockTable({self.tolist()})"
