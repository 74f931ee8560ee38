"""MonotonicCascadeTrie against stored answers.

The scenario table restates, as data, the known answers the reference keeps for this class in its own
tests/test_trie.py (shape, the failures fed in, then what must and must not be pruned, the antichain left over,
which prefixes are dead); the enumeration orders further down are hand-derived from the centre-out rule.
"""
import pytest

from tritonix_amd.utils.pruners import MonotonicCascadeTrie
from tritonix_amd.utils.spaces import Choice, SpaceConfig


def trie_of(shape, failures=()):
    trie = MonotonicCascadeTrie(SpaceConfig({f"d{i}": Choice(range(n)) for i, n in enumerate(shape)}))
    for failure in failures:
        trie.prune(failure)
    return trie


# shape, failures in arrival order, expectations
SCENARIOS = {
    "untouched space": dict(
        shape=(4, 4, 3), failures=[], alive=[(2, 2, 1)], antichain=[]),
    "a failure rules out what is at least as large, nothing else": dict(
        shape=(4, 4, 4, 4), failures=[(2, 2, 0, 0)],
        dead=[(2, 2, 0, 0), (3, 3, 3, 3)], alive=[(2, 1, 3, 3)]),
    "a smaller failure replaces the larger one it implies": dict(
        shape=(4, 4, 4, 4), failures=[(2, 2, 2, 2), (1, 1, 1, 1)], antichain=[(1, 1, 1, 1)]),
    "failures outside the index range still reduce to an antichain": dict(
        shape=(4, 4, 4, 4), failures=[(1, 4, 4, 1), (3, 3, 3, 0), (0, 4, 0, 1), (1, 3, 0, 0)],
        antichain={(1, 3, 0, 0), (0, 4, 0, 1)}),
    "incomparable points survive": dict(
        shape=(4, 4, 3), failures=[(2, 1, 0)], alive=[(1, 3, 2), (3, 0, 1)]),
    "two incomparable failures": dict(
        shape=(4, 4, 3), failures=[(2, 1, 0), (1, 2, 1)], alive=[(1, 2, 0)], dead=[(1, 3, 1)]),
    "a third failure swallows the second": dict(
        shape=(4, 4, 3), failures=[(2, 1, 0), (1, 2, 1), (1, 2, 0)], dead=[(1, 2, 1)],
        holds=[(1, 2, 0)], dropped=[(1, 2, 1)]),
    "prefix with a live completion": dict(
        shape=(4, 4, 4, 4), failures=[(1, 2, 0, 1)], open_prefixes=[(1, 2), (1, 2, 0), ()]),
    "prefix whose zero completion is dead": dict(
        shape=(4, 4, 4, 4), failures=[(1, 2, 0, 1), (1, 2, 0, 0)],
        dead_prefixes=[(1, 2), (1, 2, 0)], open_prefixes=[(1, 1), ()]),
}


@pytest.mark.parametrize("name", sorted(SCENARIOS))
def test_scenario(name):
    want = SCENARIOS[name]
    trie = trie_of(want["shape"], want["failures"])
    assert trie.shape == want["shape"] and trie.dimensions == len(want["shape"])
    for idx in want.get("dead", []):
        assert trie.is_pruned(idx), idx
    for idx in want.get("alive", []):
        assert not trie.is_pruned(idx), idx
    if "antichain" in want:
        kept = trie._minimal_failures
        assert (set(kept) == want["antichain"]) if isinstance(want["antichain"], set) else (kept == want["antichain"])
    for idx in want.get("holds", []):
        assert idx in trie._minimal_failures
    for idx in want.get("dropped", []):
        assert idx not in trie._minimal_failures
    for prefix in want.get("dead_prefixes", []):
        assert trie._is_prefix_doomed(prefix), prefix
    for prefix in want.get("open_prefixes", []):
        assert not trie._is_prefix_doomed(prefix), prefix


def test_malformed_input():
    with pytest.raises(ValueError):
        trie_of((4, 0, 3))                    # a parameter without values
    with pytest.raises(ValueError):
        trie_of((3, 3)).is_pruned((1,))       # index tuple of the wrong length


def test_enumeration_counts_and_order():
    trie = trie_of((3, 3, 3), [(1, 1, 0)])
    left = list(trie.generate_all_unpruned())
    assert len(left) == 27 - 2 * 2 * 3
    assert left == sorted(left)
    assert {(1, 0, 2), (0, 2, 1)} <= set(left) and not {(1, 1, 0), (2, 2, 2)} & set(left)
    other = trie_of((4, 3, 3), [(2, 1, 1), (1, 2, 2)])
    assert set(other.generate_all_unpruned()) == set(other.generate_all_unpruned_midpoint())
    assert len(set(other.generate_all_unpruned())) == 36 - (2 * 2 * 2 + 3 * 1 * 1 - 2 * 1 * 1)


def test_random_pick_is_a_survivor_and_exhaustion_gives_none():
    trie = trie_of((4, 4, 3), [(2, 1, 0), (1, 2, 0)])
    for _ in range(20):
        pick = trie.get_random_unpruned()
        assert pick is not None and not trie.is_pruned(pick)
    empty = trie_of((2, 2), [(0, 0)])
    assert empty.get_random_unpruned() is None and empty.get_mid_point_unpruned() is None
    assert list(empty.generate_all_unpruned()) == [] and list(empty.generate_all_unpruned_midpoint()) == []


# ---- hand-derived centre-out orders (tests/golden/hand_traces.json) -------------------------------------------
def test_centre_out_orders(traces):
    want = traces["midpoint_3x2"]
    trie = trie_of((3, 2))
    assert [list(c) for c in trie.generate_all_unpruned_midpoint()] == want["none"]
    assert trie.get_mid_point_unpruned() == (1, 1)
    trie.prune((1, 1))
    assert [list(c) for c in trie.generate_all_unpruned_midpoint()] == want["after_prune_1_1"]
    trie.prune((1, 0))
    assert [list(c) for c in trie.generate_all_unpruned_midpoint()] == want["after_prune_1_1_and_1_0"]
    assert [c[0] for c in trie_of((4,)).generate_all_unpruned_midpoint()] == traces["midpoint_order_size4"]


def test_generators_are_lazy():
    """A failure recorded between two items changes what comes next: the tuner prunes while it iterates."""
    trie = trie_of((3, 2))
    walk = trie.generate_all_unpruned_midpoint()
    assert next(walk) == (1, 1)
    trie.prune((1, 0))                         # takes (1,0), (2,0), (2,1) with it
    assert list(walk) == [(0, 1), (0, 0)]
