"""A request's block table for one cache group.

It is a plain list of page ids (logical page index -> page id, or ``PAD_PAGE`` for a page a
window has passed) for everything that reads or compares it.  The step function needs the same
numbers as int32 every step, and converting a list of hundreds of Python ints per request per
step costs more host time than all the rest of a decode step's preparation; so the list keeps
an int32 mirror that is extended as pages are appended and rebuilt only when an existing entry
was overwritten (which the owner reports with :meth:`entry_changed`).
"""

from __future__ import annotations

from collections.abc import Sequence

import numpy as np


class PageTable(list):
    """``list[int]`` with :meth:`as_array`."""

    def __init__(self, pages: Sequence[int] = ()) -> None:
        super().__init__(pages)
        self._mirror = np.empty(max(16, len(self)), dtype=np.int32)
        self._mirrored = 0  # leading entries of the mirror that are current

    def entry_changed(self, index: int) -> None:
        """The owner overwrote entry ``index`` (appending needs no report)."""
        self._mirrored = min(self._mirrored, index)

    def as_array(self) -> np.ndarray:
        """The table as an int32 array (a view, valid until the table changes next)."""
        count = len(self)
        if count > self._mirror.size:
            grown = np.empty(max(count, 2 * self._mirror.size), dtype=np.int32)
            grown[: self._mirrored] = self._mirror[: self._mirrored]
            self._mirror = grown
        if self._mirrored > count:  # entries were removed: nothing promises the rest is current
            self._mirrored = 0
        if self._mirrored < count:
            self._mirror[self._mirrored:count] = self[self._mirrored:count]
            self._mirrored = count
        return self._mirror[:count]


def table_array(table: Sequence[int]) -> np.ndarray:
    """int32 array of any block table: the mirror of a :class:`PageTable`, a conversion otherwise."""
    if isinstance(table, PageTable):
        return table.as_array()
    return np.asarray(table, dtype=np.int32)
