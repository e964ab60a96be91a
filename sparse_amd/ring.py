"""The staging ring of one offloaded layer: a fixed set of HBM slot indices that forecast
copies are written into, outside the resident cache.

The ring is the only object the scoring thread and the layer's own thread share.  Its
positions hold slot indices of the layer's slab and go round three states:

    idle --open()--> held --publish()--> lent --give_back()--> idle

``open`` starts a *window* for one decode step of the layer and holds some idle positions for
it; ``publish`` (scoring thread) queues one copy into the next held position; ``seal`` (layer
thread, at the layer's executor) ends the window: it hands the filled positions to the layer,
lets the unfilled ones go, and every later ``publish`` for that window is declined.  All three
run under one lock, so a copy is either queued before the seal and seen by the layer, or never
queued -- nothing has to be joined or cancelled.  The reference reaches the same guarantee with
a per-step job object that owns a transfer dict and a closed flag (utils/rs_staging.py:23-49);
here the slots themselves carry the state and the window is just a ticket.

A lent position comes back with the event that must pass before its slot may be overwritten,
and possibly with another slot index: when the layer keeps a staged expert it keeps the slot
too and gives the ring the slot of the expert it evicted.
"""
from __future__ import annotations

import threading
from typing import Any, Callable, Hashable, List, Optional, Sequence, Tuple

IDLE, HELD, LENT = "idle", "held", "lent"

Filled = Tuple[int, int, Any]     # (expert, ring position, copy event)


class StagingRing:
    def __init__(self, slots: Sequence[int]) -> None:
        self.slots: List[int] = [int(s) for s in slots]
        self.state: List[str] = [IDLE] * len(self.slots)
        self.fence: List[Any] = [None] * len(self.slots)
        self.lock = threading.Lock()
        self.cursor = 0                         # where the next window starts looking
        self.ticket: Optional[Hashable] = None  # the open window, None while sealed
        self.held: List[int] = []               # positions of the open window without a copy yet
        self.filled: List[Filled] = []
        self.chosen: Optional[int] = None       # how many experts the scorer picked; None = not scored
        self.worker: Any = None                 # the scoring task of the last window (never joined here)

    def __len__(self) -> int:
        return len(self.slots)

    def is_open(self) -> bool:
        return self.ticket is not None

    def all_idle(self) -> bool:
        return self.ticket is None and all(s == IDLE for s in self.state)

    def open(self, ticket: Hashable, want: int, passed: Callable[[Any], bool]) -> int:
        """Start a window with up to ``want`` positions whose last use is over (``passed`` asks
        an event without blocking).  Returns how many it holds; 0 leaves the ring sealed."""
        with self.lock:
            assert self.ticket is None and not self.held and not self.filled, "one window per layer at a time"
            n = len(self.slots)
            for step in range(n):
                if len(self.held) >= want:
                    break
                pos = (self.cursor + step) % n
                if self.state[pos] == IDLE and (self.fence[pos] is None or passed(self.fence[pos])):
                    self.state[pos], self.fence[pos] = HELD, None
                    self.held.append(pos)
            if self.held:
                self.ticket, self.chosen = ticket, None
                self.cursor = (self.held[-1] + 1) % n
            return len(self.held)

    def note_chosen(self, ticket: Hashable, count: int) -> None:
        with self.lock:
            if self.ticket == ticket:
                self.chosen = int(count)

    def publish(self, ticket: Hashable, expert: int, copy: Callable[[int, int], Any]) -> bool:
        """Queue the copy of ``expert`` into the window's next position and make it visible to
        the seal, or decline: the window is over, another one is open, or it is full.
        ``copy(slot, position)`` must only enqueue into storage that already exists and return
        the event behind the copy."""
        with self.lock:
            if ticket is None or self.ticket != ticket or not self.held:
                return False
            assert all(e != int(expert) for e, _p, _ev in self.filled), "an expert is staged once per window"
            pos = self.held.pop(0)
            event = copy(self.slots[pos], pos)
            self.state[pos] = LENT
            self.filled.append((int(expert), pos, event))
            return True

    def seal(self) -> Tuple[Optional[Hashable], List[Filled], Optional[int]]:
        """End the window.  Returns ``(ticket, filled, chosen)``; waits only for a ``publish``
        that is inside the lock right now."""
        with self.lock:
            ticket, self.ticket = self.ticket, None
            for pos in self.held:
                self.state[pos] = IDLE
            self.held = []
            filled, self.filled = self.filled, []
            chosen, self.chosen = self.chosen, None
            return ticket, filled, chosen

    def give_back(self, pos: int, fence: Any, slot: Optional[int] = None) -> None:
        """Return a lent position; ``slot`` replaces the index it holds when the layer kept the
        old one."""
        with self.lock:
            assert self.state[pos] == LENT
            if slot is not None:
                self.slots[pos] = int(slot)
            self.state[pos], self.fence[pos] = IDLE, fence
