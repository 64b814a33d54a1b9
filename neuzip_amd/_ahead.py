"""Which dense weights to decode together: the order of the requests, learned.

A model asks for its weights in the same order pass after pass (forwards through
the blocks, backwards through them in training, once more from the update hooks).
``RequestOrder`` learns that order as "at this place came c next", a place being
(the handle asked for before the current one, the current handle, how many times
in a row it has been asked for now, whether anything was written since the
request before) - enough to keep the forward walk, the backward walk, the
repeated requests of an update hook and the read-update-write loop of an
optimizer apart - and, for a
request that finds nothing waiting, names the handles to decode in the same
launch; the decoded weights of the others wait here for their requests.

Pure bookkeeping: no device code and no tensors are touched here.  The owner
passes in how to decode (``decode_one``, ``decode_many``) and how large a stored
tensor is (``size_of``), and tells the cache about every write (``written``).
What a request gets back always equals a decode at the time of the request,
because a write drops whatever waits for its handle.
"""
from __future__ import annotations

from typing import Callable, Dict, Hashable, List, Optional, Sequence, Tuple


class RequestOrder:
    def __init__(self, decode_one: Callable[[Hashable], object],
                 decode_many: Callable[[Sequence[Hashable]], Optional[List[object]]],
                 size_of: Callable[[Hashable], int], fill: int, most: int = 16):
        """``decode_many(handles)`` -> one decoded object per handle (a handle may
        appear twice), or None when the launch could not be made; ``fill``: total
        size at which a launch is large enough; ``most``: handles per launch."""
        self.decode_one, self.decode_many, self.size_of = decode_one, decode_many, size_of
        self.fill, self.most = int(fill), int(most)
        self.enabled = True
        self.hits = self.waste = 0          # objects decoded ahead that were asked for / dropped unused, ever
        self._recent = [0, 0]               # the same two over the last thousand or so
        self._pause = 0                     # requests still to be served one by one: the order did not repeat itself
        self._pause_next = 256              # ... and for how many the next time it does not
        self._next: Dict[tuple, tuple] = {}     # place -> (the handle that was asked for next, after a write?)
        self._at: tuple = (None, None, 0, False)  # the place of the last request
        self._wrote = False                     # has anything been written since that request?
        # handle -> [(decoded object, where the walk that decoded it began, its place in that walk)]
        self._waiting: Dict[Hashable, List[Tuple[object, tuple, int]]] = {}
        self._rewritten = set()  # handles whose waiting object a write has dropped
        # A walk that begins at `start` takes at most _limit[start] handles: the last time, what
        # came after was written before it was asked for (the update hooks of a backward pass
        # rewrite the layers one by one: a walk that runs on into the next forward pass would
        # decode weights that are about to change).  A walk that loses nothing may be one longer
        # the next time.
        self._limit: Dict[tuple, int] = {}
        self._cut: Dict[tuple, int] = {}  # start -> the first place a write has dropped since the walk

    # -- what the owner reports ------------------------------------------------
    def written(self, handle) -> None:
        """``handle`` is about to hold other values: what waits for it is dropped"""
        self._wrote = True
        for _, start, at in self._waiting.pop(handle, ()):
            self._cut[start] = min(at, self._cut.get(start, at))
            self._rewritten.add(handle)
            self.waste += 1
            self._recent[1] += 1

    def clear(self) -> None:
        """drop everything that waits (nothing is counted)"""
        self._waiting.clear()
        self._rewritten.clear()

    def forget_position(self) -> None:
        """the next request is not taken as the successor of the last ones"""
        self._at = (None, None, 0, False)

    @property
    def paused(self) -> bool:
        """no walks at the moment: the order of the requests has not been repeating itself"""
        return self._pause > 0

    def waiting(self):
        """the handles something waits for"""
        return set(self._waiting)

    # -- a request ---------------------------------------------------------------
    def request(self, handle):
        """-> (decoded object, whether it was decoded ahead of this request)"""
        if self._at[1] is not None:
            self._next[self._at] = (handle, self._wrote)
        start = self._at = self._step(self._at, handle, self._wrote)
        self._wrote = False
        queue = self._waiting.get(handle)
        if queue:
            obj = queue.pop(0)[0]
            if not queue:
                del self._waiting[handle]
            self.hits += 1
            self._recent[0] += 1
            if self._recent[0] + self._recent[1] > 1024:
                self._recent = [self._recent[0] // 2, self._recent[1] // 2]
            return obj, True
        if self._waiting:
            if handle in self._rewritten:
                # its object did wait and a write has dropped it since: the others stay
                self._rewritten.discard(handle)
                return self._decode_walk(start, self._walk(start, self._waiting)), False
            # not what was expected next
            lost = sum(len(q) for q in self._waiting.values())
            self.waste += lost
            self._recent[1] += lost
            self._waiting.clear()
            if self._recent[1] > 64 and self._recent[1] > self._recent[0]:
                # the requests do not come in the order they came in before: no walks for a
                # while (the order is still being learned), twice as long every time it happens
                self._pause, self._pause_next = self._pause_next, min(2 * self._pause_next, 1 << 16)
                self._recent = [0, 0]
        self._rewritten.clear()
        if self._pause:
            self._pause -= 1
            return self.decode_one(handle), False
        if not self.enabled:
            return self.decode_one(handle), False
        return self._decode_walk(start, self._walk(start)), False

    def _decode_walk(self, start: tuple, walk: list):
        """decode the handles of ``walk``; the first is handed out, the others wait"""
        if len(walk) == 1:
            return self.decode_one(walk[0])
        objs = self.decode_many(walk)
        if objs is None:
            return self.decode_one(walk[0])
        for at in range(1, len(walk)):
            self._waiting.setdefault(walk[at], []).append((objs[at], start, at))
        return objs[0]

    @staticmethod
    def _step(place: tuple, handle, wrote: bool) -> tuple:
        """the place after ``handle`` has been asked for at ``place``"""
        before, current, times, _ = place
        return (before, current, times + 1, wrote) if handle == current else (current, handle, 1, wrote)

    def _walk(self, start: tuple, stop_at=()) -> list:
        """the handles to decode with the request that led to the place ``start``
        (the walk ends in front of a handle of ``stop_at``)"""
        cut = self._cut.pop(start, None)
        if cut is not None:
            self._limit[start] = cut
        elif start in self._limit:
            self._limit[start] += 1
            if self._limit[start] >= self.most:
                del self._limit[start]
        most = self._limit.get(start, self.most)
        place = start
        walk, total, seen = [start[1]], self.size_of(start[1]), {start}
        # follow the links until the launch is full or the walk comes back to where it has been
        while len(walk) < most and total < self.fill:
            nxt, wrote = self._next.get(place, (None, False))
            if nxt is None or nxt in stop_at:
                break
            place = self._step(place, nxt, wrote)
            if place in seen:
                break
            seen.add(place)
            try:
                total += self.size_of(nxt)
            except (KeyError, RuntimeError):
                break  # no longer stored
            walk.append(nxt)
        return walk
