"""A small executable model of the work queue of the persistent move kernel (deepep-ascend_amd/csrc/dispatch.hip:
`dispatch_cast_queue_kernel`, `queue_word`), run under thousands of random interleavings on the CPU.

What is modelled: every workgroup owns its first chunks by index; a feeder keeps the workgroup's ring of chunk words one
chunk ahead of its ticket counter, asking one global counter for chunks whose size shrinks towards the end, and posts a
chunk of size zero when the counter has run past the last item; it then reports to a wrapping counter, and the last
feeder to report puts the global counter back to zero.  A mover draws a ticket, waits until the ring shows the ticket's
chunk, and takes item `first + offset`, draws again if the offset lies past the chunk's size, or leaves at a chunk of
size zero.  Every atomic operation is one step; the scheduler picks the next actor at random.

What must hold for every schedule: every item is taken exactly once; every actor ends; no mover ever finds a later
chunk in the ring slot of the chunk it waits for; both counters are back at zero after the launch, so that the next
launch (modelled too) starts clean.  The same checker finds the failure of a ring that is too short, so it is not
vacuous."""
import random

import pytest

SLOT = 16           # tickets per chunk (kQueueSlot)
STATIC = 2          # chunks a workgroup owns by index (kQueueStatic)


class Violation(Exception):
    pass


class Device:
    def __init__(self):
        self.counter = 0        # the global item counter
        self.done = 0           # the wrapping counter the feeders report to


class Workgroup:
    def __init__(self, index, total, ring_slots):
        self.ticket = 0
        self.ring = [None] * ring_slots          # (chunk number, size, first item)
        for c in range(STATIC):
            base = (index * STATIC + c) * SLOT
            self.ring[c] = (c, min(SLOT, total - base) if base < total else 0, base)


def feeder(dev, wg, index, workgroups, total):
    posted = STATIC
    ended = (index * STATIC + STATIC - 1) * SLOT >= total
    size = SLOT
    static_items = workgroups * STATIC * SLOT
    while not ended:
        drawing = wg.ticket // SLOT
        yield
        if posted > drawing + 1:
            continue
        got = dev.counter
        dev.counter += size                                           # one atomic
        yield
        base = static_items + got
        if base >= total:
            wg.ring[posted % len(wg.ring)] = (posted, 0, total)
            ended = True
        else:
            wg.ring[posted % len(wg.ring)] = (posted, min(size, total - base), base)
            posted += 1
            left = total - base
            size = 16 if left > total // 4 else 8 if left > total // 16 else 4
        yield
    before = dev.done
    dev.done = 0 if before == workgroups - 1 else before + 1          # atomicInc with wrap
    yield
    if before == workgroups - 1:
        dev.counter = 0


def mover(wg, total, taken):
    def draw():
        while True:
            n = wg.ticket
            wg.ticket += 1                                             # one atomic
            yield None
            c, o = divmod(n, SLOT)
            spins = 0
            while True:
                word = wg.ring[c % len(wg.ring)]
                if word is not None and word[0] == c:
                    break
                if word is not None and word[0] > c:
                    raise Violation(f"chunk {c} was overwritten by chunk {word[0]} before a mover had read it")
                spins += 1
                if spins > 100000:
                    raise Violation("a mover waits for a chunk that is never posted")
                yield None
            if word[1] == 0:
                yield ("item", None)
                return
            if o < word[1]:
                yield ("item", word[2] + o)
                return

    def next_item():
        for step in draw():
            if step is None:
                yield None
            else:
                yield step

    def take(gen):
        item = None
        for step in gen:
            if step is None:
                yield
            else:
                item = step[1]
        return item

    work = yield from take(next_item())
    while work is not None:
        following = yield from take(next_item())
        if work >= total or taken[work]:
            raise Violation(f"item {work} taken twice or out of range")
        taken[work] = True
        yield
        work = following


def run_launch(dev, rng, total, workgroups, movers, ring_slots):
    if dev.counter != 0 or dev.done != 0:
        raise Violation("a launch starts with counters that are not zero")
    taken = [False] * total
    actors = []
    for index in range(workgroups):
        wg = Workgroup(index, total, ring_slots)
        actors.append(feeder(dev, wg, index, workgroups, total))
        actors.extend(mover(wg, total, taken) for _ in range(movers))
    steps = 0
    while actors:
        steps += 1
        if steps > 2000000:
            raise Violation("no progress")
        actor = rng.choice(actors)
        try:
            next(actor)
        except StopIteration:
            actors.remove(actor)
    if not all(taken):
        raise Violation(f"{taken.count(False)} items were never taken")
    if dev.counter != 0 or dev.done != 0:
        raise Violation("a counter did not return to zero")


def test_every_item_once_under_random_schedules():
    for seed in range(40):
        rng = random.Random(seed)
        dev = Device()
        for _ in range(3):                                             # launches share the counters
            workgroups = rng.randint(1, 5)
            total = rng.choice([0, 1, 15, 16, 17, 31, 33, rng.randint(34, 900)])
            # the launcher starts no more workgroups than there are pairs of static chunks to own
            workgroups = max(1, min(workgroups, -(-total // (SLOT * STATIC))))
            run_launch(dev, rng, total, workgroups, movers=rng.randint(1, 4), ring_slots=16)


def test_the_model_catches_a_ring_that_is_too_short():
    """With two ring slots the feeder posts a chunk into the slot of a chunk some mover holds a ticket for but has not
    looked up yet: some schedule shows it."""
    caught = 0
    for seed in range(200):
        rng = random.Random(seed)
        dev = Device()
        try:
            run_launch(dev, rng, total=700, workgroups=2, movers=4, ring_slots=2)
        except Violation:
            caught += 1
    assert caught > 0
