"""A small executable model of the hand-off inside a single-launch dispatch (deepep-ascend_amd/csrc/dispatch.hip:
`launch_tag`, `await_tagged_words`, `settle_gate`, `finish_hand_off`, `publisher_is_done_with_the_tag`), run under
thousands of random interleavings on the CPU.

What is modelled: every workgroup reads the generation word once, at its start, and derives the launch's tag from it
(generation + 1).  Counting workgroups store tagged words (chunk totals, position words; for the expanded layout also
the expert chunk totals the publisher reads).  The publisher of an expanded dispatch reads those, stores the tagged expert
bases, waits for its stores and reports as a party.  A mover polls the words it needs until they carry its tag, then
advances its gate (a counter that wraps when all movers of the gate have passed); the last mover of a gate reports the
gate as a party.  The party that completes the count clears the tagged tables if the launch used the last tag of the
period, and then advances the generation.  Stores land an arbitrary time after they were issued; a workgroup only knows
that its own have landed after waiting for them.

What must hold for every schedule: all workgroups of a launch see the same generation; a mover only ever consumes a word
written by its own launch; when the tables are cleared no tagged store is still on its way; counters are back at zero
after the launch; the generation advances by exactly one per launch.  The same checker finds the failure when the
publisher is left out of the party count (the gap a late publisher could slip through), so it is not vacuous."""
import random

import pytest

PERIOD = 5          # tags 1 .. PERIOD (the kernels: 16383); small, so that many wraps are exercised
GATES = 3           # the kernels: 256


class Violation(Exception):
    pass


class Memory:
    def __init__(self):
        self.generation = 0
        self.tagged = {}            # word -> (tag, launch that wrote it)
        self.in_flight = []         # issued, not yet landed: (owner, word, tag, launch)
        self.gates = [0] * GATES
        self.gates_finished = 0
        self.chunk_done = {}

    def land(self, rng, owner=None, everything=False):
        """Some (or all) stores in flight become visible; with `owner`, all stores of that workgroup (it waited)."""
        rest = []
        for entry in self.in_flight:
            who, word, tag, launch = entry
            if everything or who == owner or (owner is None and rng.random() < 0.5):
                self.tagged[word] = (tag, launch)
            else:
                rest.append(entry)
        self.in_flight = rest


def counting_workgroup(mem, launch, c, tokens_of_chunk, expanded, seen):
    generation = mem.generation
    seen.append(generation)
    tag = generation + 1
    yield
    words = [("total", c)] + [("pos", t) for t in tokens_of_chunk] + ([("expert_total", c)] if expanded else [])
    for w in words:
        mem.in_flight.append((("count", c), w, tag, launch))
        yield
    yield ("wait_own", ("count", c))
    mem.chunk_done[c] = 1
    yield


def publisher(mem, launch, chunks, experts, expanded, count_publisher, seen, rng, finish):
    generation = mem.generation
    if expanded:
        seen.append(generation)     # only the publisher of an expanded dispatch uses the tag it derives from it
    tag = generation + 1
    yield
    while not all(mem.chunk_done.get(c, 0) for c in range(chunks)):
        yield
    for c in range(chunks):
        mem.chunk_done[c] = 0
    if not expanded:
        return
    for c in range(chunks):                     # the tagged expert totals of every chunk
        while mem.tagged.get(("expert_total", c), (0, None)) != (tag, launch):
            got = mem.tagged.get(("expert_total", c), (0, None))
            if got[0] == tag and got[1] != launch:
                raise Violation("publisher took a stale expert total for this launch's")
            yield
    for e in range(experts):
        mem.in_flight.append(("publisher", ("base", e), tag, launch))
        yield
    if count_publisher:
        yield ("wait_own", "publisher")
        yield from finish(tag)


def mover(mem, launch, m, token, chunks, needs_base, seen, finish, movers_of_gate):
    generation = mem.generation
    seen.append(generation)
    tag = generation + 1
    yield
    wanted = [("total", c) for c in range(chunks)] + [("pos", token)] + ([("base", needs_base)] if needs_base is not None else [])
    for w in wanted:
        while True:
            got = mem.tagged.get(w, (0, None))
            if got[0] == tag:
                if got[1] != launch:
                    raise Violation(f"mover {m} consumed {w} of launch {got[1]} in launch {launch}")
                break
            yield
    gate = m % GATES
    before = mem.gates[gate]
    mem.gates[gate] = 0 if before == movers_of_gate[gate] - 1 else before + 1        # atomicInc with wrap
    yield
    if before == movers_of_gate[gate] - 1:
        yield from finish(tag)


def run_launch(mem, launch, rng, chunks, movers, experts, expanded, count_publisher=True):
    tokens = list(range(movers))                # one mover per token
    tokens_of_chunk = [[t for t in tokens if t % chunks == c] for c in range(chunks)]
    gates_in_use = min(movers, GATES)
    movers_of_gate = [len([m for m in range(movers) if m % GATES == g]) for g in range(GATES)]
    parties = gates_in_use + (1 if expanded and count_publisher else 0)
    start_generation = mem.generation
    seen = []

    def finish(tag):
        before = mem.gates_finished
        mem.gates_finished = 0 if before == parties - 1 else before + 1               # atomicInc with wrap
        yield
        if before != parties - 1:
            return
        nxt = tag
        if nxt == PERIOD:
            if any(entry[2] != 0 for entry in mem.in_flight):
                raise Violation("tagged tables cleared while a tagged store was still on its way")
            for w in list(mem.tagged):
                mem.tagged[w] = (0, None)
            yield
            nxt = 0
        mem.generation = nxt
        yield

    actors = [counting_workgroup(mem, launch, c, tokens_of_chunk[c], expanded, seen) for c in range(chunks)]
    actors.append(publisher(mem, launch, chunks, experts, expanded, count_publisher, seen, rng, finish))
    for m in range(movers):
        base = rng.randrange(experts) if expanded and rng.random() < 0.7 else None      # some movers need no base at all
        actors.append(mover(mem, launch, m, tokens[m], chunks, base, seen, finish, movers_of_gate))
    live = list(actors)
    steps = 0
    while live:
        steps += 1
        if steps > 200000:
            raise Violation("no progress")
        actor = rng.choice(live)
        try:
            what = next(actor)
        except StopIteration:
            live.remove(actor)
            continue
        if isinstance(what, tuple) and what[0] == "wait_own":
            mem.land(rng, owner=what[1])
        elif rng.random() < 0.3:
            mem.land(rng)
    mem.land(rng, everything=True)              # the kernel boundary
    if len(set(seen)) != 1:
        raise Violation(f"workgroups of one launch read different generations: {sorted(set(seen))}")
    if mem.generation != (start_generation + 1) % PERIOD:
        raise Violation(f"generation went from {start_generation} to {mem.generation}")
    if any(mem.gates) or mem.gates_finished:
        raise Violation("a counter did not return to zero")


@pytest.mark.parametrize("expanded", [False, True], ids=["compact", "expanded"])
def test_hand_off_holds_under_random_schedules(expanded):
    for seed in range(60):
        rng = random.Random(seed)
        mem = Memory()
        for launch in range(1, 4 * PERIOD + 2):          # several tag periods
            run_launch(mem, launch, rng, chunks=rng.randint(1, 3), movers=rng.randint(1, 8), experts=rng.randint(1, 4),
                       expanded=expanded)


def test_the_model_catches_a_publisher_that_is_not_a_party():
    """Leave the publisher of an expanded dispatch out of the count, as the protocol once did: some schedule lets the
    generation advance before the publisher has read it, or clears the tables under its stores."""
    caught = 0
    for seed in range(300):
        rng = random.Random(seed)
        mem = Memory()
        try:
            for launch in range(1, 3 * PERIOD + 1):
                run_launch(mem, launch, rng, chunks=1, movers=rng.randint(1, 3), experts=2, expanded=True,
                           count_publisher=False)
        except Violation:
            caught += 1
    assert caught > 0
