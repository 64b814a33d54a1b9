"""Host logic of the decode-ahead: neuzip_amd/_ahead.py, with decoders that only count.

The one property everything else rests on: whatever the order of requests and
writes, a request is answered with the value its handle holds at that moment.
"""
import importlib.util
import os
import random

import pytest

_spec = importlib.util.spec_from_file_location(
    "nz_ahead", os.path.join(os.path.dirname(__file__), "..", "neuzip_amd", "_ahead.py"))
_ahead = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(_ahead)  # no torch, no device library needed


class Store:
    """handles with version numbers; a decode returns (handle, version at the time of the launch)"""

    def __init__(self, sizes, fill=1 << 30, most=16, fail_many=False):
        self.sizes = dict(sizes)
        self.version = {h: 0 for h in self.sizes}
        self.launches = []
        self.fail_many = fail_many
        self.order = _ahead.RequestOrder(self._one, self._many, self._size, fill, most)

    def _size(self, h):
        return self.sizes[h]  # KeyError for a handle that is gone

    def _one(self, h):
        self.launches.append([h])
        return (h, self.version[h])

    def _many(self, hs):
        if self.fail_many:
            return None
        self.launches.append(list(hs))
        return [(h, self.version[h]) for h in hs]

    def request(self, h):
        obj, ahead = self.order.request(h)
        assert obj == (h, self.version[h]), f"stale or foreign value for {h}: {obj} at version {self.version[h]}"
        return ahead

    def write(self, h):
        self.order.written(h)  # before the store changes, as the backend does
        self.version[h] += 1


def test_a_repeating_forward_order_is_served_by_a_few_launches():
    s = Store({k: 100 for k in range(24)})
    per_pass = []
    for rep in range(4):
        s.launches.clear()
        for k in range(24):
            s.request(k)
        per_pass.append([len(l) for l in s.launches])
    assert per_pass[0] == [1] * 24            # nothing known yet
    assert len(per_pass[2]) <= 2 and len(per_pass[3]) <= 2  # launches of 16 that run on into the next pass
    assert s.order.waste == 0 and s.order.hits >= 60


def test_a_launch_stops_at_the_fill_and_at_sixteen_handles():
    s = Store({k: 100 for k in range(40)}, fill=450)
    for rep in range(3):
        s.launches.clear()
        for k in range(40):
            s.request(k)
    assert max(len(l) for l in s.launches) == 5  # 5 x 100 >= 450
    s = Store({k: 1 for k in range(40)})
    for rep in range(3):
        s.launches.clear()
        for k in range(40):
            s.request(k)
    assert max(len(l) for l in s.launches) == 16


def test_forward_and_backward_walks_are_kept_apart():
    s = Store({k: 100 for k in range(10)})
    for rep in range(5):
        s.launches.clear()
        for k in range(10):
            s.request(k)
        for k in reversed(range(10)):
            s.request(k)
    assert len(s.launches) <= 3 and s.order.waste == 0


def test_update_hooks_in_the_backward_pass():
    """every layer: asked for by the backward pass, again by its update hook, then written"""
    s = Store({k: 100 for k in range(8)})
    per_step = []
    for step in range(12):
        s.launches.clear()
        wasted = s.order.waste
        for k in range(8):
            s.request(k)
        for k in reversed(range(8)):
            s.request(k)
            s.request(k)
            s.write(k)
        per_step.append((len(s.launches), s.order.waste - wasted))
    # once the walks have learned where the writes cut them: two launches for the 24 requests
    # of a step, and at most one weight decoded for nothing (the probe that lets walks grow again)
    assert all(l <= 2 and w <= 1 for l, w in per_step[6:]), per_step


def test_read_update_write_loop_after_the_backward_pass():
    """the reference's explicit loop: write(read(h).add_(g), h) for every parameter"""
    s = Store({k: 100 for k in range(20)})
    for step in range(6):
        s.launches.clear()
        wasted = s.order.waste
        for k in range(20):
            s.request(k)
        for k in reversed(range(20)):
            s.request(k)
        for k in range(20):
            s.request(k)
            s.write(k)
    assert len(s.launches) <= 5 and s.order.waste == wasted


def test_a_write_drops_what_waits_and_the_others_stay():
    s = Store({k: 100 for k in range(6)})
    for rep in range(2):
        for k in range(6):
            s.request(k)
    s.request(0)                       # hit or miss, then a walk over what follows
    s.request(1)
    assert s.order.waiting() >= {2, 3, 4}
    s.write(3)
    assert 3 not in s.order.waiting() and {2, 4} <= s.order.waiting()
    assert s.request(2) is True
    assert s.request(3) is False       # decoded again: the new value (checked inside request)
    assert s.request(4) is True        # ... and what waited behind it was kept


def test_an_unforeseen_request_drops_everything_that_waits():
    s = Store({k: 100 for k in range(7)})
    for rep in range(2):
        for k in range(6):
            s.request(k)
    s.request(0), s.request(1)
    n = len(s.order.waiting())
    assert n >= 3
    assert s.request(4) is True        # out of order, but it was waiting: taken
    wasted = s.order.waste
    assert s.request(6) is False       # never seen before
    assert s.order.waste == wasted + n - 1 and not s.order.waiting()


def test_requests_without_a_repeating_order_are_served_one_by_one_for_a_while():
    rng = random.Random(4)
    s = Store({k: 100 for k in range(6)})
    pauses = 0
    for rep in range(400):
        order = list(range(6))
        rng.shuffle(order)
        was = s.order.paused
        for k in order:
            s.request(k)
        pauses += s.order.paused and not was
    assert pauses >= 2 and s.order.paused     # again and again, each pause twice as long as the one before
    s.launches.clear()
    for k in range(6):
        s.request(k)
    assert s.launches == [[k] for k in range(6)]
    # the order settles: once the pause is over the walks are back
    for rep in range(2000):
        for k in range(6):
            s.request(k)
    assert not s.order.paused
    s.launches.clear()
    for rep in range(4):
        for k in range(6):
            s.request(k)
    assert len(s.launches) <= 5


@pytest.mark.parametrize("seed", range(12))
def test_every_request_gets_the_current_value_whatever_happens(seed):
    """requests, writes, handles that disappear, launches that fail: random mixtures of
    repeating passes and noise; Store.request checks every answer"""
    rng = random.Random(seed)
    n = rng.choice([3, 7, 20])
    s = Store({k: rng.choice([1, 50, 400]) for k in range(n)}, fill=rng.choice([300, 2000, 1 << 30]),
              most=rng.choice([2, 5, 16]))
    base = list(range(n))
    for rep in range(60):
        mode = rng.random()
        if mode < 0.5:
            seq = [("r", k) for k in base]
        elif mode < 0.7:
            seq = [("r", k) for k in base] + [x for k in reversed(base) for x in (("r", k), ("r", k), ("w", k))]
        elif mode < 0.85:
            seq = [(rng.choice("rw"), rng.randrange(n)) for _ in range(2 * n)]
        else:
            seq = [("r", k) for k in base for _ in range(rng.choice([1, 2, 3]))]
        s.fail_many = rng.random() < 0.1
        for op, k in seq:
            if k not in s.sizes:
                continue
            if op == "r":
                s.request(k)
            else:
                s.write(k)
        if rep == 30 and n > 3:  # a handle goes away: walks end in front of it
            gone = base.pop(rng.randrange(len(base)))
            s.order.written(gone)
            del s.sizes[gone]
    assert s.order.hits + s.order.waste >= 0


def test_clear_and_forget_position():
    s = Store({k: 100 for k in range(5)})
    for rep in range(3):
        for k in range(5):
            s.request(k)
    s.request(0), s.request(1)
    assert s.order.waiting()
    wasted = s.order.waste
    s.order.clear()
    assert not s.order.waiting() and s.order.waste == wasted
    s.order.forget_position()
    s.launches.clear()
    s.request(3)  # no known place: nothing is learned from, or predicted for, this request
    assert s.launches == [[3]]
