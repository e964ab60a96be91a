"""A small least-recently-used table for device workspaces keyed by call shape.

Workspaces are sized by the number of tokens of a call; a server that sees many distinct
prefill lengths would otherwise keep one set of buffers per length for the life of the
process.  Dropping an entry only drops this table's reference: buffers still in use by queued
kernels are kept alive by the caller's own references and, once those go, returned to the
allocator in stream order.

A captured HIP graph is different: it holds raw pointers into the buffers of the entry it was
captured on and no Python reference.  An entry that is looked up while the current stream is
capturing is therefore pinned: it is never dropped by the size limit (only by ``clear()``, which
the owner of the graphs calls once they are gone), and pinned entries do not count against the
limit."""
from __future__ import annotations

import os
from collections import OrderedDict
from typing import Any, Callable, Hashable, Optional, Set


def _stream_is_capturing() -> bool:
    try:
        import torch
        return bool(torch.cuda.is_available() and torch.cuda.is_current_stream_capturing())
    except Exception:  # noqa: BLE001 -- no device, or a build without graph support
        return False


class LruTable:
    def __init__(self, limit: int, capturing: Optional[Callable[[], bool]] = None) -> None:
        if limit < 1:
            raise ValueError("an LRU table holds at least one entry")
        self.limit = int(limit)
        self._items: "OrderedDict[Hashable, Any]" = OrderedDict()
        self._pinned: Set[Hashable] = set()
        self._capturing = capturing if capturing is not None else _stream_is_capturing

    @classmethod
    def from_env(cls, name: str, default: int) -> "LruTable":
        return cls(max(1, int(os.environ.get(name, default))))

    def __len__(self) -> int:
        return len(self._items)

    def __contains__(self, key: Hashable) -> bool:
        return key in self._items

    def keys(self):
        return list(self._items)

    def pinned(self):
        return set(self._pinned)

    def pin(self, key: Hashable) -> None:
        """Keep ``key`` for good (a graph captured on it may be replayed at any time)."""
        if key in self._items:
            self._pinned.add(key)

    def get_or_make(self, key: Hashable, make: Callable[[], Any]) -> Any:
        item = self._items.get(key)
        if item is None:
            item = make()
            self._items[key] = item
        else:
            self._items.move_to_end(key)
        if self._capturing():
            self._pinned.add(key)
        # drop the least recently used entries no graph points into
        excess = len(self._items) - len(self._pinned) - self.limit
        if excess > 0:
            for old in [k for k in self._items if k not in self._pinned and k != key][:excess]:
                del self._items[old]
        return item

    def clear(self) -> None:
        self._items.clear()
        self._pinned.clear()
