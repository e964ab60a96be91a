"""A small least-recently-used table for device workspaces keyed by call shape.

Workspaces are sized by the number of tokens of a call; a server that sees many distinct
prefill lengths would otherwise keep one set of buffers per length for the life of the
process.  Dropping an entry only drops this table's reference: buffers still in use by queued
kernels are kept alive by the caller's own references and, once those go, returned to the
allocator in stream order."""
from __future__ import annotations

import os
from collections import OrderedDict
from typing import Any, Callable, Hashable


class LruTable:
    def __init__(self, limit: int) -> None:
        if limit < 1:
            raise ValueError("an LRU table holds at least one entry")
        self.limit = int(limit)
        self._items: "OrderedDict[Hashable, Any]" = OrderedDict()

    @classmethod
    def from_env(cls, name: str, default: int) -> "LruTable":
        return cls(max(1, int(os.environ.get(name, default))))

    def __len__(self) -> int:
        return len(self._items)

    def __contains__(self, key: Hashable) -> bool:
        return key in self._items

    def keys(self):
        return list(self._items)

    def get_or_make(self, key: Hashable, make: Callable[[], Any]) -> Any:
        item = self._items.get(key)
        if item is None:
            item = make()
            self._items[key] = item
            while len(self._items) > self.limit:
                self._items.popitem(last=False)
        else:
            self._items.move_to_end(key)
        return item

    def clear(self) -> None:
        self._items.clear()
