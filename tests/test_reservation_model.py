"""Host-side model of how the single-sweep step's chunks reserve room for
their records in a shared segment (``k_fused_spec``, csrc/fused_step.hip).

A chunk with ``cnt`` records does ONE ``base = atomicAdd(&count, cnt)`` and
keeps ``[base, base + cnt)`` when that lies inside the segment's capacity;
otherwise its records go to the overflow list, the reservation is NOT taken
back, and the chunk leaves ``base`` in the segment's fail word when ``base``
is still inside the capacity.  The check kernel then takes the segment's
records to be ``[0, count)`` while ``count <= cap`` and ``[0, fail base)``
afterwards.  The model runs every order of the atomic operations of a few
chunks and checks that this range is exactly tiled by the reservations that
were kept -- and that the protocol this one replaced (a failed reservation
subtracts itself again) is not safe, which is why it was dropped."""
import itertools


def _never_take_back(cnts, cap, order):
    """One atomic op per chunk; ``order`` is the order in which they land."""
    count, fail, kept = 0, None, []
    for w in order:
        base = count
        count += cnts[w]
        if base + cnts[w] <= cap:
            kept.append((base, base + cnts[w]))
        elif base <= cap:
            fail = base if fail is None else min(fail, base)
    valid = count if count <= cap else fail
    return valid, kept


def _take_back(cnts, cap, ops):
    """The replaced protocol: ``ops`` is a sequence of (chunk, phase) events,
    phase 0 the atomicAdd, phase 1 the atomicSub a failed chunk issues later."""
    count, kept, failed = 0, [], set()
    for w, phase in ops:
        if phase == 0:
            base = count
            count += cnts[w]
            if base + cnts[w] <= cap:
                kept.append((base, base + cnts[w]))
            else:
                failed.add(w)
        elif w in failed:
            count -= cnts[w]
    return count, kept


def _tiles(valid, kept):
    at = 0
    for a, b in sorted(kept):
        if a != at:
            return False
        at = b
    return at == valid


def test_never_taking_back_leaves_exactly_the_kept_records():
    for cap in (8, 13):
        for cnts in itertools.product((1, 3, 5, 8, 10), repeat=4):
            for order in itertools.permutations(range(4)):
                valid, kept = _never_take_back(cnts, cap, order)
                assert valid is not None and valid <= cap
                assert _tiles(valid, kept), (cap, cnts, order, valid, kept)


def test_taking_back_can_count_slots_nobody_wrote():
    """cap - 5 taken; A adds 10 (over), B adds 3 (over, base cap + 5), A
    subtracts, C adds 2 at base cap - 2 and fits, B subtracts: the count ends
    at cap - 3 with C's records outside it and two counted slots unwritten."""
    cap = 20
    cnts = {"pre": cap - 5, "A": 10, "B": 3, "C": 2}
    ops = [("pre", 0), ("A", 0), ("B", 0), ("A", 1), ("C", 0), ("B", 1)]
    count, kept = _take_back(cnts, cap, ops)
    assert count == cap - 3 and (cap - 2, cap) in kept
    assert not _tiles(count, kept)
    # the same chunks in the same order under the protocol in use
    valid, kept = _never_take_back(cnts, cap, ["pre", "A", "B", "C"])
    assert valid == cap - 5 and _tiles(valid, kept)
