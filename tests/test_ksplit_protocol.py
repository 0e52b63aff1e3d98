"""A host model of the counting protocol that the K split of the prefill kernel uses to hand partial sums
between the workgroups of one output tile (tk_gemm32_kernel, KSPLIT): every slice (1) publishes its partial
sums, (2) counts its arrival with one atomic increment that returns the old value, and (3) only the slice
that reads `slices - 1` adds the others' sums to its own, resets the counter and writes the output. The model
walks EVERY interleaving of those steps over the slices and checks what the kernel relies on: exactly one
slice finishes a launch, it sees every other slice's sums, nothing ever waits, and the counter is zero again
for the next launch -- also when two launches follow each other without anything clearing it."""
import itertools


def _interleavings(n_slices):
    """Every order of the 2*n steps (publish, arrive) in which a slice publishes before it arrives."""
    steps = [(s, phase) for s in range(n_slices) for phase in (0, 1)]
    for order in itertools.permutations(steps):
        pos = {st: i for i, st in enumerate(order)}
        if all(pos[(s, 0)] < pos[(s, 1)] for s in range(n_slices)):
            yield order


def _run(order, n_slices, partial, counter):
    """One launch of one tile. Returns (finished slices, their totals, counter afterwards)."""
    published = {}
    finished, totals = [], []
    for s, phase in order:
        if phase == 0:
            published[s] = partial[s]        # agent-scope stores, acknowledged before the arrival below
        else:
            old = counter                    # fetch_add returns the old value
            counter += 1
            if old == n_slices - 1:          # by construction the last to arrive
                assert set(published) == set(range(n_slices)), "the finisher would read sums not yet published"
                finished.append(s)
                totals.append(sum(published.values()))
                counter = 0                  # reset for the next launch
    return finished, totals, counter


def test_every_interleaving_has_one_finisher_that_sees_all_sums():
    for n in (2, 3, 4):
        partial = [10 ** s for s in range(n)]
        for order in _interleavings(n):
            finished, totals, counter = _run(order, n, partial, 0)
            assert len(finished) == 1 and totals == [sum(partial)] and counter == 0


def test_back_to_back_launches_need_no_clearing():
    n = 3
    counter = 0
    for launch in range(4):
        partial = [launch * 100 + s for s in range(n)]
        for order in itertools.islice(_interleavings(n), launch, None, 7):
            finished, totals, counter = _run(order, n, partial, counter)
            assert len(finished) == 1 and totals == [sum(partial)] and counter == 0


def test_a_stale_counter_is_why_a_failed_launch_clears_it():
    """If a launch were cut short after one arrival, the counter would stay at 1 and the next launch's second
    arrival would wrongly finish with a sum missing: the host therefore clears the counters after a failed
    launch (kcount_stale in tk_api.hip)."""
    n = 3
    order = next(_interleavings(n))
    try:
        _run(order, n, [1, 2, 3], 1)
    except AssertionError:
        return
    raise AssertionError("a stale counter went unnoticed")
